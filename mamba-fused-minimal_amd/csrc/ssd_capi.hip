// extern "C" entry points of libssd_gfx950.so: argument validation, kernel-family selection, launch.
#include "../../include/ssd_gfx950.h"
#include "ssd_params.h"
#include "ssd_cost.h"

#include <stdlib.h>
#include <string.h>

#include <atomic>

namespace {

using ssd::Params;
using ssd::PassParams;

// ssd_set_token_split: 0 = choose, 1 = four-tile kernel, 2 / 4 = token-split kernels.  A process-wide test and tuning
// hook: atomic, so that setting it while another thread launches is a race on the choice only, never on memory.
std::atomic<int> g_forced_split{0};

bool dtype_ok(int dt) { return dt == SSD_F32 || dt == SSD_BF16 || dt == SSD_F16; }

// Device check, cached per device ordinal: the kernels are gfx950 code objects only.  A cache entry is written
// once with its final value (0 = unknown, else 1 = gfx950 / 2 = another device, plus the compute-unit count
// shifted left by 8), so concurrent first calls at worst query the device twice.
std::atomic<int> g_device_cache[64];

int device_info()
{
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0) return 0;
    if (dev < 64) {
        const int c = g_device_cache[dev].load(std::memory_order_acquire);
        if (c) return c;
    }
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, dev) != hipSuccess) return 0;
    const bool ok = strncmp(prop.gcnArchName, "gfx950", 6) == 0;
    const int c = (ok ? 1 : 2) | (prop.multiProcessorCount << 8);
    if (dev < 64) g_device_cache[dev].store(c, std::memory_order_release);
    return c;
}

int check_device() { return (device_info() & 255) == 1 ? SSD_OK : SSD_ERR_DEVICE; }

int compute_units() { return device_info() >> 8; }

int check_dims(const ssd_dims *d)
{
    if (!d) return SSD_ERR_NULL;
    if (d->batch <= 0 || d->seqlen <= 0 || d->nheads <= 0 || d->headdim <= 0 || d->dstate <= 0 || d->ngroups <= 0 ||
        d->chunk_size <= 0 || d->nchunks <= 0)
        return SSD_ERR_SHAPE;
    if (d->nheads % d->ngroups) return SSD_ERR_SHAPE;
    if (d->nchunks != (d->seqlen + d->chunk_size - 1) / d->chunk_size) return SSD_ERR_SHAPE;
    return SSD_OK;
}

bool present(const ssd_tensor *t) { return t && t->data; }

// A dimension of size one is only ever indexed with zero, so whatever stride the caller reports for it (frameworks
// keep arbitrary ones on such dimensions of views) must not decide alignment checks or kernel choice: zero them.
void drop_unit_strides(Params &p)
{
    if (p.batch == 1) p.sx_b = p.sB_b = p.sdt_b = p.sda_b = p.ssq_b = p.sin_b = p.sst_b = p.so_b = p.sf_b = 0;
    if (p.nheads == 1) p.sx_h = p.sdt_h = p.sda_h = p.sin_h = p.sst_h = p.so_h = p.sf_h = 0;
    if (p.ngroups == 1) p.sB_g = 0;
    if (p.C == 1) p.sdt_c = p.sda_c = p.sst_c = p.so_c = 0;
}

// Fills the part of Params common to the chunk-state and fused calls.
int fill_common(Params &p, const ssd_tensor *x, const ssd_tensor *B, const ssd_tensor *dt, const ssd_tensor *dacs,
                const ssd_tensor *seq, const ssd_tensor *states, const ssd_dims *d, int clamp)
{
    int rc = check_dims(d);
    if (rc) return rc;
    if (!present(x) || !present(B) || !present(dt) || !present(dacs)) return SSD_ERR_NULL;
    if (!dtype_ok(x->dtype) || x->dtype != B->dtype) return SSD_ERR_DTYPE;
    if (dt->dtype != SSD_F32 || dacs->dtype != SSD_F32) return SSD_ERR_DTYPE;
    if (x->stride[3] != 1 || B->stride[3] != 1) return SSD_ERR_STRIDE;
    memset(&p, 0, sizeof(p));
    p.x = x->data; p.B = B->data; p.dt = (const float *)dt->data; p.dacs = (const float *)dacs->data;
    p.batch = d->batch; p.seqlen = d->seqlen; p.nheads = d->nheads; p.headdim = d->headdim; p.dstate = d->dstate;
    p.ngroups = d->ngroups; p.Q = d->chunk_size; p.C = d->nchunks;
    p.sx_b = x->stride[0]; p.sx_l = x->stride[1]; p.sx_h = x->stride[2];
    p.sB_b = B->stride[0]; p.sB_l = B->stride[1]; p.sB_g = B->stride[2];
    p.sdt_b = dt->stride[0]; p.sdt_h = dt->stride[1]; p.sdt_c = dt->stride[2]; p.sdt_k = dt->stride[3];
    p.sda_b = dacs->stride[0]; p.sda_h = dacs->stride[1]; p.sda_c = dacs->stride[2]; p.sda_k = dacs->stride[3];
    p.dt_in = x->dtype;
    p.clamp = clamp ? 1 : 0;
    if (present(seq)) {
        p.seq = (const int32_t *)seq->data;
        p.ssq_b = seq->stride[0]; p.ssq_l = seq->stride[1];
    }
    if (present(states)) {
        if (!dtype_ok(states->dtype)) return SSD_ERR_DTYPE;
        if (states->stride[4] != 1) return SSD_ERR_STRIDE;
        p.states = states->data; p.dt_states = states->dtype;
        p.sst_b = states->stride[0]; p.sst_c = states->stride[1]; p.sst_h = states->stride[2]; p.sst_p = states->stride[3];
    }
    drop_unit_strides(p);
    return SSD_OK;
}

// The recurrence over `states` as the stand-alone kernel sees it: the (headdim, dstate) plane of a head flattened,
// dA_chunk = the last column of dA_cumsum.
PassParams pass_params_of(const Params &p)
{
    PassParams q;
    memset(&q, 0, sizeof(q));
    q.states = p.states; q.dt_states = p.dt_states;
    q.sst_b = p.sst_b; q.sst_c = p.sst_c; q.sst_h = p.sst_h;
    q.da = p.dacs + (int64_t)(p.Q - 1) * p.sda_k;
    q.sda_b = p.sda_b; q.sda_h = p.sda_h; q.sda_c = p.sda_c;
    q.init = p.init; q.dt_init = p.dt_init; q.sin_b = p.sin_b; q.sin_h = p.sin_h;
    q.seq = p.seq; q.ssq_b = p.ssq_b; q.ssq_l = p.ssq_l;
    q.out = p.out; q.dt_out = p.dt_out; q.so_b = p.so_b; q.so_c = p.so_c; q.so_h = p.so_h;
    q.fin = p.fin; q.sf_b = p.sf_b; q.sf_h = p.sf_h;
    q.batch = p.batch; q.C = p.C; q.nheads = p.nheads; q.dim = p.headdim * p.dstate;
    q.seqlen = p.seqlen; q.Q = p.Q;
    return q;
}

// Fused call with `states`: can it run as the chunk-state launch of the four-tile kernel + the recurrence?
bool pair_supported(const Params &p)
{
    if (!p.states || !p.out || !p.fin) return false;
    if (p.dt_states != ssd::DT_F32) return false;      // the recurrence would start from rounded states
    // the recurrence walks a head's plane as one row
    if (p.sst_p != p.dstate || p.so_p != p.dstate || p.sf_p != p.dstate || (p.init && p.sin_p != p.dstate)) return false;
    Params cs = p;
    cs.out = nullptr; cs.fin = nullptr; cs.init = nullptr;
    return ssd::quad_chunk_state_supported(cs);
}

// chunk states into p.states, then the recurrence over them into p.out / p.fin (which may be the same buffer)
hipError_t launch_pair(const Params &p, hipStream_t s, bool generic = false)
{
    Params cs = p;
    cs.out = nullptr; cs.fin = nullptr; cs.init = nullptr;
    const hipError_t e = generic ? ssd::launch_generic(cs, false, s) : ssd::launch_quad_chunk_state(cs, s);
    return e == hipSuccess ? ssd::launch_state_passing(pass_params_of(p), s) : e;
}

// The same for arguments only the plain FMA kernel takes (other element types, odd sizes): as a fused launch that
// kernel has one workgroup per 16 x 64 piece of a state walk the whole sequence, as a chunk-state launch one per piece
// and chunk -- batch 1 x 1024 tokens x 8 heads, fp32: 122 us fused, 28 + 17 us as chunk states + recurrence; 4096
// tokens: 479 against 30 + 17.
bool generic_pair_supported(const Params &p)
{
    if (!p.states || !p.out || !p.fin || p.C < 2) return false;
    if (p.dt_states != ssd::DT_F32) return false;      // the recurrence would start from rounded states
    return p.sst_p == p.dstate && p.so_p == p.dstate && p.sf_p == p.dstate && (!p.init || p.sin_p == p.dstate);
}

// the fused call's arguments with `out` doubling as the `states` buffer
Params with_states_in_out(const Params &p)
{
    Params q = p;
    q.states = p.out; q.dt_states = p.dt_out;
    q.sst_b = p.so_b; q.sst_c = p.so_c; q.sst_h = p.so_h; q.sst_p = p.so_p;
    return q;
}

// What a call runs.  The values are those of ssd_fused_plan::family.
enum Family { F_GENERIC = SSD_FAMILY_GENERIC, F_TOKEN_SPLIT = SSD_FAMILY_TOKEN_SPLIT, F_FOUR_TILE = SSD_FAMILY_FOUR_TILE,
              F_PAIR = SSD_FAMILY_PAIR, F_CHAIN = SSD_FAMILY_CHAIN };
struct Choice {
    int family;
    bool states_in_out;      // chunk-state launch + recurrence: `out` doubles as the place for the chunk states
    bool generic_pair;       // F_GENERIC as chunk-state launch + recurrence
};

// The kernel family of a call without a workspace.
Choice choose(const Params &p, bool fused, int64_t n_cu)
{
    // Fused launch: with at least two state tiles per compute unit the four-tiles-per-workgroup kernel wins (B is
    // fetched once per four tiles and the state never leaves the accumulators); with fewer, the token-split
    // kernel, which puts four waves on every tile, has the shorter chunk.
    const int tiles = p.batch * p.nheads * (p.headdim / 32);
    const int forced = g_forced_split.load(std::memory_order_relaxed);      // one value for the whole choice
    if (fused && (forced == 1 || (forced == 0 && tiles >= 2 * n_cu)) && ssd::quad_supported(p)) return {F_FOUR_TILE, false, false};
    // Few state tiles, many chunks, fp32 `out`: the chunk-state launch keeps every compute unit busy where the
    // fused kernels have one workgroup per tile.  It writes the chunk states into `out`, and the streaming
    // recurrence turns them into the passed states in place (b=1 L=32768 H=80: 330 us against 425 us).
    if (fused && !p.states && forced == 0 && tiles < 2 * n_cu && (int64_t)tiles * p.C >= 32 * n_cu &&
        p.dt_out == ssd::DT_F32 && pair_supported(with_states_in_out(p)))
        return {F_PAIR, true, false};
    // The caller wants the per-chunk states as well: the chunk-state launch of the four-tile kernel, which keeps
    // every compute unit busy whatever the number of tiles, then the streaming recurrence over what it wrote
    // (b=1 L=32768 H=80: 336 us against 496 us for the token-split kernel doing both at once).
    if (fused && p.states && (forced == 1 || (forced == 0 && (int64_t)tiles * p.C >= 32 * n_cu)) && pair_supported(p))
        return {F_PAIR, false, false};
    if (!fused && (forced == 1 || (forced == 0 && (int64_t)tiles * p.C >= 8 * n_cu)) && ssd::quad_chunk_state_supported(p))
        return {F_FOUR_TILE, false, false};
    if (ssd::mfma_supported(p)) return {F_TOKEN_SPLIT, false, false};
    if (fused && forced == 0 && !p.states && p.dt_out == ssd::DT_F32 && generic_pair_supported(with_states_in_out(p)))
        return {F_GENERIC, true, true};
    if (fused && forced == 0 && p.states && generic_pair_supported(p)) return {F_GENERIC, false, true};
    return {F_GENERIC, false, false};
}

int run(const Params &p_in, bool fused, void *stream)
{
    int rc = check_device();
    if (rc) return rc;
    Params p = p_in;
    p.n_cu = compute_units();
    hipStream_t s = (hipStream_t)stream;
    const Choice c = choose(p, fused, p.n_cu > 0 ? p.n_cu : 256);
    hipError_t e;
    switch (c.family) {
        case F_FOUR_TILE: e = fused ? ssd::launch_quad(p, s) : ssd::launch_quad_chunk_state(p, s); break;
        case F_PAIR: e = launch_pair(c.states_in_out ? with_states_in_out(p) : p, s); break;
        case F_TOKEN_SPLIT: e = ssd::launch_mfma(p, fused, s); break;
        default:
            e = c.generic_pair ? launch_pair(c.states_in_out ? with_states_in_out(p) : p, s, true) : ssd::launch_generic(p, fused, s);
            break;
    }
    return (int)e;
}

// Scratch for ssd_fused_chunk_state_passing_fwd_static: ticket counters, error word and flags of the chain kernel in
// device memory that belongs to the library's code object -- every GPU the library runs on holds its own copy, at its
// own address, until the process ends.  The name is a host-side handle, not a device address: the address is asked
// for once per device (scratch_pointer) and only that pointer is handed to kernels.
constexpr int kStaticScratchInts = 1 << 18;     // 1 MiB: header + one flag per (state tile, chunk)
static __device__ __align__(256) int g_static_scratch[kStaticScratchInts];

std::atomic<int *> g_scratch_ptr[64];

// device address of g_static_scratch on the current device (nullptr + error code on failure)
hipError_t scratch_pointer(int **ptr)
{
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev >= 0 && dev < 64) {
        int *cached = g_scratch_ptr[dev].load(std::memory_order_acquire);
        if (cached) { *ptr = cached; return hipSuccess; }
    }
    void *sym = nullptr;
    e = hipGetSymbolAddress(&sym, HIP_SYMBOL(g_static_scratch));
    if (e != hipSuccess) return e;
    if (!sym) return hipErrorInvalidSymbol;
    if (dev >= 0 && dev < 64) g_scratch_ptr[dev].store((int *)sym, std::memory_order_release);
    *ptr = (int *)sym;
    return hipSuccess;
}

// The fused problem as the cost model sees it.
ssd::cost::Problem problem_of(const Params &p, int n_cu)
{
    ssd::cost::Problem q;
    q.units = (int64_t)p.batch * p.nheads * (p.headdim / 32) / 4;
    q.chunks = p.C; q.chunk_size = p.Q; q.dstate = p.dstate;
    q.n_cu = n_cu > 0 ? n_cu : 256;
    return q;
}

// Estimate for the family `c` (what the call would run without a workspace); a family the model does not cover
// counts as slower than anything.
double estimate_us(const ssd::cost::Problem &q, const Choice &c)
{
    switch (c.family) {
        case F_FOUR_TILE: return ssd::cost::four_tile_us(q);
        case F_PAIR: return ssd::cost::pair_us(q);
        case F_TOKEN_SPLIT: return ssd::cost::token_split_us(q);
        default: return 1e30;
    }
}

// Whether the ticket / flag-chain kernel is the better fused kernel for a problem it covers: it keeps every compute
// unit busy whatever the number of state tiles, at the price of its start, of reading each passed state back once per
// item and of a link per item.
bool chain_preferred(const Params &p, int n_cu)
{
    const ssd::cost::Problem q = problem_of(p, n_cu);
    double chain = 0.;
    ssd::cost::chain_chunks_per_item(q, &chain);
    // within the model's error the chain kernel gets the call: its time follows the amount of work, the others'
    // depends on how their workgroups happen to fall on the compute units
    return chain < 1.05 * estimate_us(q, choose(p, true, q.n_cu));
}

// Whether a fused call runs on the ticket / flag-chain kernel: a usable workspace came with it and that kernel is
// asked for or estimated to be the faster one.  Returns a status (a kernel forced where it cannot run).
int chain_decision(const Params &p, const ssd_dims *dims, const ssd_fused_opts *opts, bool *use)
{
    *use = false;
    if (opts && opts->used_workspace) *opts->used_workspace = 0;
    const int kernel = opts ? opts->kernel : SSD_KERNEL_AUTO;
    if (kernel < SSD_KERNEL_AUTO || kernel > SSD_KERNEL_CHAIN_GLOBAL) return SSD_ERR_SHAPE;
    // bf16 out (or none): the workspace also holds the fp32 states that cross between items, as many as the launch will
    // have items (the forced number of chunks per item, or the one the launch would choose)
    const bool out16 = ssd::chain_needs_carry(p);
    const int forced_r = opts ? opts->chunks_per_item : 0;
    const int r = out16 ? ssd::chain_chunks_per_item(p, compute_units(), forced_r) : 0;
    const uint64_t need = out16 ? ssd::chain_workspace_bytes_out16(dims->batch, dims->nheads, dims->headdim, dims->dstate, dims->nchunks, r)
                                : ssd::chain_workspace_bytes(dims->batch, dims->nheads, dims->headdim, dims->nchunks);
    const bool have_ws = opts && opts->workspace && ((uintptr_t)opts->workspace % (out16 ? 16 : 4)) == 0 &&
                         opts->workspace_bytes >= need && !(out16 && r < 2);
    // with the scan's state half asked for, the chain kernel is the only one that computes it in the same launch
    if (have_ws && ssd::chain_supported(p) &&
        (kernel != SSD_KERNEL_AUTO || p.y || (g_forced_split.load(std::memory_order_relaxed) == 0 && chain_preferred(p, compute_units())))) {
        *use = true;
        if (opts->used_workspace) *opts->used_workspace = 1;
        return check_device();
    }
    return kernel != SSD_KERNEL_AUTO ? SSD_ERR_SCRATCH : SSD_OK;     // forced, but no workspace or not a shape it covers
}

int run_chain(Params &p, const ssd_fused_opts *opts, void *stream)
{
    p.ws = (int *)opts->workspace;
    p.epoch = opts->epoch > 0 ? opts->epoch : 0;
    p.spin_limit = opts->spin_limit;
    p.n_seg = opts->chunks_per_item == 1 || opts->chunks_per_item == 2 || opts->chunks_per_item == 4 ? opts->chunks_per_item : 0;
    return (int)ssd::launch_chain(p, compute_units(),
                                  opts->kernel == SSD_KERNEL_CHAIN_LOCAL ? 1 : opts->kernel == SSD_KERNEL_CHAIN_GLOBAL ? 2 : 0,
                                  (hipStream_t)stream);
}

// Arguments of the dt preparation as its kernel takes them.
int fill_cumsum(ssd::CumsumParams &p, const ssd_tensor *dt, const ssd_tensor *A, const ssd_tensor *dt_bias,
                const ssd_tensor *dt_out, const ssd_tensor *dA_cumsum, int32_t batch, int32_t seqlen, int32_t nheads,
                int32_t chunk_size, int dt_softplus, float dt_min, float dt_max)
{
    if (!present(dt) || !present(A) || !present(dt_out) || !present(dA_cumsum)) return SSD_ERR_NULL;
    if (batch <= 0 || seqlen <= 0 || nheads <= 0 || chunk_size <= 0) return SSD_ERR_SHAPE;
    if (!dtype_ok(dt->dtype) || !dtype_ok(A->dtype) || dt_out->dtype != SSD_F32 || dA_cumsum->dtype != SSD_F32)
        return SSD_ERR_DTYPE;
    memset(&p, 0, sizeof(p));
    p.dt = dt->data; p.dt_type = dt->dtype;
    p.sdt_b = dt->stride[0]; p.sdt_l = dt->stride[1]; p.sdt_h = dt->stride[2];
    p.A = A->data; p.A_type = A->dtype; p.sA = A->stride[0];
    if (present(dt_bias)) {
        if (!dtype_ok(dt_bias->dtype)) return SSD_ERR_DTYPE;
        p.dt_bias = dt_bias->data; p.dt_bias_type = dt_bias->dtype; p.sbias = dt_bias->stride[0];
    }
    p.dt_out = (float *)dt_out->data;
    p.so_b = dt_out->stride[0]; p.so_h = dt_out->stride[1]; p.so_c = dt_out->stride[2]; p.so_k = dt_out->stride[3];
    p.dacs = (float *)dA_cumsum->data;
    p.sa_b = dA_cumsum->stride[0]; p.sa_h = dA_cumsum->stride[1]; p.sa_c = dA_cumsum->stride[2]; p.sa_k = dA_cumsum->stride[3];
    p.batch = batch; p.seqlen = seqlen; p.nheads = nheads; p.Q = chunk_size;
    p.C = (seqlen + chunk_size - 1) / chunk_size;
    p.softplus = dt_softplus ? 1 : 0; p.dt_min = dt_min; p.dt_max = dt_max;
    return ssd::chunk_cumsum_supported(p) ? SSD_OK : SSD_ERR_SHAPE;
}

}  // namespace

extern "C" {

int ssd_version(void) { return SSD_ABI_VERSION; }

const char *ssd_status_string(int status)
{
    switch (status) {
        case SSD_OK: return "ok";
        case SSD_ERR_NULL: return "a required pointer is NULL";
        case SSD_ERR_SHAPE: return "inconsistent problem sizes";
        case SSD_ERR_DTYPE: return "unsupported element type";
        case SSD_ERR_STRIDE: return "innermost stride must be 1";
        case SSD_ERR_DEVICE: return "no gfx950 device is current";
        case SSD_ERR_SCRATCH: return "workspace missing or too small for the requested kernel";
        case SSD_ERR_CHAIN_TIMEOUT: return "a wave of the flag-chain kernel gave up waiting for its predecessor";
        case SSD_ERR_CHAIN_XCD: return "workgroups of two XCDs drew from one ticket counter of the flag-chain kernel";
        case SSD_ERR_CHAIN_INCOMPLETE: return "a ticket counter of the flag-chain kernel was never served: outputs are missing";
        case SSD_ERR_CHAIN_WORKSPACE: return "the workspace was not in the state the epoch of the call promised";
        default: break;
    }
    if (status > 0) return hipGetErrorString((hipError_t)status);
    return "unknown status";
}

int ssd_chunk_state_fwd(const ssd_tensor *x, const ssd_tensor *B, const ssd_tensor *dt, const ssd_tensor *dA_cumsum,
                        const ssd_tensor *seq_idx, const ssd_tensor *states, const ssd_dims *dims, int clamp,
                        void *stream)
{
    if (!present(states)) return SSD_ERR_NULL;
    Params p;
    int rc = fill_common(p, x, B, dt, dA_cumsum, seq_idx, states, dims, clamp);
    if (rc) return rc;
    return run(p, false, stream);
}

// Fills Params for a fused call (chunk state + state passing).  out_optional: `out` may be absent.
static int fill_fused(Params &p, const ssd_tensor *x, const ssd_tensor *B, const ssd_tensor *dt, const ssd_tensor *dA_cumsum,
                      const ssd_tensor *seq_idx, const ssd_tensor *initial_states, const ssd_tensor *states,
                      const ssd_tensor *out, const ssd_tensor *final_states, const ssd_dims *dims, int clamp,
                      bool out_optional = false)
{
    if ((!present(out) && !out_optional) || !present(final_states)) return SSD_ERR_NULL;
    int rc = fill_common(p, x, B, dt, dA_cumsum, seq_idx, states, dims, clamp);
    if (rc) return rc;
    if (final_states->dtype != SSD_F32) return SSD_ERR_DTYPE;
    if (final_states->stride[3] != 1) return SSD_ERR_STRIDE;
    if (present(out)) {
        if (!dtype_ok(out->dtype)) return SSD_ERR_DTYPE;
        if (out->stride[4] != 1) return SSD_ERR_STRIDE;
        p.out = out->data; p.dt_out = out->dtype;
        p.so_b = out->stride[0]; p.so_c = out->stride[1]; p.so_h = out->stride[2]; p.so_p = out->stride[3];
    }
    p.fin = (float *)final_states->data;
    p.sf_b = final_states->stride[0]; p.sf_h = final_states->stride[1]; p.sf_p = final_states->stride[2];
    if (present(initial_states)) {
        if (!dtype_ok(initial_states->dtype)) return SSD_ERR_DTYPE;
        if (initial_states->stride[3] != 1) return SSD_ERR_STRIDE;
        p.init = initial_states->data; p.dt_init = initial_states->dtype;
        p.sin_b = initial_states->stride[0]; p.sin_h = initial_states->stride[1]; p.sin_p = initial_states->stride[2];
    }
    drop_unit_strides(p);
    return SSD_OK;
}

int ssd_fused_chunk_state_passing_fwd(const ssd_tensor *x, const ssd_tensor *B, const ssd_tensor *dt,
                                      const ssd_tensor *dA_cumsum, const ssd_tensor *seq_idx,
                                      const ssd_tensor *initial_states, const ssd_tensor *states,
                                      const ssd_tensor *out, const ssd_tensor *final_states, const ssd_dims *dims,
                                      int clamp, void *stream)
{
    Params p;
    int rc = fill_fused(p, x, B, dt, dA_cumsum, seq_idx, initial_states, states, out, final_states, dims, clamp);
    if (rc) return rc;
    return run(p, true, stream);
}

uint64_t ssd_fused_workspace_bytes(const ssd_dims *dims)
{
    if (check_dims(dims)) return 0;
    return ssd::chain_workspace_bytes(dims->batch, dims->nheads, dims->headdim, dims->nchunks);
}

uint64_t ssd_fused_workspace_bytes_for(const ssd_dims *dims, int out_dtype, int chunks_per_item)
{
    if (check_dims(dims)) return 0;
    if (out_dtype == SSD_F32) return ssd::chain_workspace_bytes(dims->batch, dims->nheads, dims->headdim, dims->nchunks);
    if (out_dtype != SSD_BF16) return 0;
    Params p;
    memset(&p, 0, sizeof(p));
    p.batch = dims->batch; p.nheads = dims->nheads; p.headdim = dims->headdim; p.dstate = dims->dstate;
    p.C = dims->nchunks; p.Q = dims->chunk_size; p.dt_out = ssd::DT_BF16;
    const int r = ssd::chain_chunks_per_item(p, compute_units(), chunks_per_item);
    if (r < 2) return 0;
    return ssd::chain_workspace_bytes_out16(dims->batch, dims->nheads, dims->headdim, dims->dstate, dims->nchunks, r);
}

int ssd_fused_chunk_state_passing_fwd_ws(const ssd_tensor *x, const ssd_tensor *B, const ssd_tensor *dt,
                                         const ssd_tensor *dA_cumsum, const ssd_tensor *seq_idx,
                                         const ssd_tensor *initial_states, const ssd_tensor *states,
                                         const ssd_tensor *out, const ssd_tensor *final_states, const ssd_dims *dims,
                                         int clamp, const ssd_fused_opts *opts, void *stream)
{
    Params p;
    int rc = fill_fused(p, x, B, dt, dA_cumsum, seq_idx, initial_states, states, out, final_states, dims, clamp);
    if (rc) return rc;
    bool chain = false;
    rc = chain_decision(p, dims, opts, &chain);
    if (rc) return rc;
    return chain ? run_chain(p, opts, stream) : run(p, true, stream);
}

int ssd_fused_chunk_state_passing_fwd_static(const ssd_tensor *x, const ssd_tensor *B, const ssd_tensor *dt,
                                             const ssd_tensor *dA_cumsum, const ssd_tensor *seq_idx,
                                             const ssd_tensor *initial_states, const ssd_tensor *out,
                                             const ssd_tensor *final_states, const ssd_dims *dims, int clamp,
                                             void *stream)
{
    Params p;
    int rc = fill_fused(p, x, B, dt, dA_cumsum, seq_idx, initial_states, nullptr, out, final_states, dims, clamp);
    if (rc) return rc;
    // only the kernel that needs scratch is offered here, and its fp32 `out` only (the scratch has no room for the
    // states that bf16 `out` makes it keep in fp32 as well)
    if (!ssd::chain_supported(p) || p.dt_out != ssd::DT_F32) return SSD_ERR_SHAPE;
    if (ssd_fused_workspace_bytes(dims) > sizeof(int) * (uint64_t)kStaticScratchInts) return SSD_ERR_SCRATCH;
    rc = check_device();
    if (rc) return rc;
    int *scratch = nullptr;
    const hipError_t e = scratch_pointer(&scratch);
    if (e != hipSuccess) return (int)e;
    p.ws = scratch;
    return (int)ssd::launch_chain(p, compute_units(), 0, (hipStream_t)stream);
}

int ssd_fused_static_status(void *stream)
{
    int rc = check_device();
    if (rc) return rc;
    int *scratch = nullptr;
    const hipError_t e = scratch_pointer(&scratch);
    if (e != hipSuccess) return (int)e;
    return ssd_fused_workspace_status(scratch, stream);
}

int ssd_fused_workspace_status(const void *workspace, void *stream)
{
    if (!workspace) return SSD_ERR_NULL;
    int rc = check_device();
    if (rc) return rc;
    int32_t header[SSD_WORKSPACE_HEADER_INTS];
    memset(header, 0, sizeof(header));
    hipError_t e = hipMemcpyAsync(header, workspace, sizeof(header), hipMemcpyDeviceToHost, (hipStream_t)stream);
    if (e == hipSuccess) e = hipStreamSynchronize((hipStream_t)stream);
    if (e != hipSuccess) return (int)e;
    return ssd_fused_workspace_status_of(header);
}

int ssd_fused_workspace_status_of(const int32_t *header)
{
    static_assert(SSD_WORKSPACE_HEADER_INTS == ssd::kChainWsHeaderInts, "the header as the kernel lays it out");
    static_assert(SSD_ERR_CHAIN_TIMEOUT == -7 && SSD_ERR_CHAIN_XCD == -8 && SSD_ERR_CHAIN_INCOMPLETE == -9 &&
                  SSD_ERR_CHAIN_WORKSPACE == -10, "values chain_status_of_header returns");
    if (!header) return SSD_ERR_NULL;
    return ssd::chain_status_of_header(header);
}

int ssd_fused_cumsum_chunk_state_passing_fwd(const ssd_tensor *x, const ssd_tensor *B, const ssd_tensor *dt_raw,
                                             const ssd_tensor *A, const ssd_tensor *dt_bias, const ssd_tensor *seq_idx,
                                             const ssd_tensor *initial_states, const ssd_tensor *dt_out,
                                             const ssd_tensor *dA_cumsum, const ssd_tensor *out,
                                             const ssd_tensor *final_states, const ssd_dims *dims, int dt_softplus,
                                             float dt_min, float dt_max, int clamp, void *stream)
{
    return ssd_fused_cumsum_chunk_state_passing_fwd_ws(x, B, dt_raw, A, dt_bias, seq_idx, initial_states, dt_out, dA_cumsum, out,
                                                       final_states, dims, dt_softplus, dt_min, dt_max, clamp, nullptr, stream);
}

int ssd_fused_cumsum_chunk_state_passing_fwd_ws(const ssd_tensor *x, const ssd_tensor *B, const ssd_tensor *dt_raw,
                                                const ssd_tensor *A, const ssd_tensor *dt_bias, const ssd_tensor *seq_idx,
                                                const ssd_tensor *initial_states, const ssd_tensor *dt_out,
                                                const ssd_tensor *dA_cumsum, const ssd_tensor *out,
                                                const ssd_tensor *final_states, const ssd_dims *dims, int dt_softplus,
                                                float dt_min, float dt_max, int clamp, const ssd_fused_opts *opts,
                                                void *stream)
{
    Params p;
    int rc = fill_fused(p, x, B, dt_out, dA_cumsum, seq_idx, initial_states, nullptr, out, final_states, dims, clamp);
    if (rc) return rc;
    ssd::CumsumParams cp;
    rc = fill_cumsum(cp, dt_raw, A, dt_bias, dt_out, dA_cumsum, dims->batch, dims->seqlen, dims->nheads, dims->chunk_size,
                     dt_softplus, dt_min, dt_max);
    if (rc) return rc;
    bool chain = false;
    rc = chain_decision(p, dims, opts, &chain);
    if (rc) return rc;
    rc = check_device();
    if (rc) return rc;
    // Two launches on the caller's stream: the producer, which also clears the chain kernel's workspace on its way
    // when that kernel follows, and the fused kernel.  Computing dt / dA_cumsum inside the fused kernels was built and
    // measured for both of them and lost both times (batch 4 x 8192 tokens x 80 heads: 270 against 240 microseconds in
    // the four-tile kernel, 232 against 197 in the chain kernel): their workgroups take two heads each and have to
    // gather those two columns out of the token-major dt rows, a cache line per token, where the producer reads the
    // rows whole.
    if (chain && opts->epoch <= 0) {
        cp.clear = (int *)opts->workspace;
        cp.n_clear = (int)(ssd::chain_workspace_bytes(dims->batch, dims->nheads, dims->headdim, dims->nchunks) / sizeof(int));
        p.ws_cleared = 1;
    }
    const hipError_t e = ssd::launch_chunk_cumsum(cp, (hipStream_t)stream);
    if (e != hipSuccess) return (int)e;
    return chain ? run_chain(p, opts, stream) : run(p, true, stream);
}

int ssd_state_passing_fwd(const ssd_tensor *states, const ssd_tensor *dA_chunk, const ssd_tensor *initial_states,
                          const ssd_tensor *seq_idx, const ssd_tensor *out, const ssd_tensor *final_states,
                          int32_t batch, int32_t nchunks, int32_t nheads, int32_t dim, int32_t seqlen,
                          int32_t chunk_size, void *stream)
{
    if (!present(states) || !present(dA_chunk) || !present(out) || !present(final_states)) return SSD_ERR_NULL;
    if (batch <= 0 || nchunks <= 0 || nheads <= 0 || dim <= 0) return SSD_ERR_SHAPE;
    if (!dtype_ok(states->dtype) || !dtype_ok(out->dtype) || dA_chunk->dtype != SSD_F32 || final_states->dtype != SSD_F32)
        return SSD_ERR_DTYPE;
    if (states->stride[3] != 1 || out->stride[3] != 1 || final_states->stride[2] != 1) return SSD_ERR_STRIDE;
    PassParams p;
    memset(&p, 0, sizeof(p));
    p.states = states->data; p.dt_states = states->dtype;
    p.sst_b = states->stride[0]; p.sst_c = states->stride[1]; p.sst_h = states->stride[2];
    p.da = (const float *)dA_chunk->data;
    p.sda_b = dA_chunk->stride[0]; p.sda_h = dA_chunk->stride[1]; p.sda_c = dA_chunk->stride[2];
    p.out = out->data; p.dt_out = out->dtype;
    p.so_b = out->stride[0]; p.so_c = out->stride[1]; p.so_h = out->stride[2];
    p.fin = (float *)final_states->data;
    p.sf_b = final_states->stride[0]; p.sf_h = final_states->stride[1];
    p.batch = batch; p.C = nchunks; p.nheads = nheads; p.dim = dim;
    if (present(initial_states)) {
        if (!dtype_ok(initial_states->dtype)) return SSD_ERR_DTYPE;
        if (initial_states->stride[2] != 1) return SSD_ERR_STRIDE;
        p.init = initial_states->data; p.dt_init = initial_states->dtype;
        p.sin_b = initial_states->stride[0]; p.sin_h = initial_states->stride[1];
    }
    if (present(seq_idx)) {
        if (seqlen <= 0 || chunk_size <= 0) return SSD_ERR_SHAPE;
        p.seq = (const int32_t *)seq_idx->data;
        p.ssq_b = seq_idx->stride[0]; p.ssq_l = seq_idx->stride[1];
        p.seqlen = seqlen; p.Q = chunk_size;
    }
    int rc = check_device();
    if (rc) return rc;
    return (int)ssd::launch_state_passing(p, (hipStream_t)stream);
}

int ssd_query_path(const ssd_tensor *x, const ssd_tensor *B, const ssd_dims *dims)
{
    Params p;
    ssd_tensor f32 = {(void *)16, SSD_F32, 0, {0, 0, 0, 1, 0}};
    int rc = fill_common(p, x, B, &f32, &f32, nullptr, nullptr, dims, 1);
    if (rc) return rc;
    return ssd::mfma_supported(p) ? 1 : 0;
}

int ssd_query_fused_plan(const ssd_dims *dims, int has_workspace, int compute_units, ssd_fused_plan *plan)
{
    if (!plan) return SSD_ERR_NULL;
    int rc = check_dims(dims);
    if (rc) return rc;
    if (compute_units < 0) return SSD_ERR_SHAPE;
    // plain tensors of these sizes at a made-up, well-aligned address: only sizes, strides and types are looked at
    const int64_t L = dims->seqlen, H = dims->nheads, P = dims->headdim, N = dims->dstate,
                  G = dims->ngroups, Q = dims->chunk_size, C = dims->nchunks;
    void *const somewhere = (void *)(uintptr_t)4096;
    const ssd_tensor x = {somewhere, SSD_BF16, 0, {L * H * P, H * P, P, 1, 0}};
    const ssd_tensor B = {somewhere, SSD_BF16, 0, {L * G * N, G * N, N, 1, 0}};
    const ssd_tensor dt = {somewhere, SSD_F32, 0, {H * C * Q, C * Q, Q, 1, 0}};
    const ssd_tensor out = {somewhere, SSD_F32, 0, {C * H * P * N, H * P * N, P * N, N, 1}};
    const ssd_tensor fin = {somewhere, SSD_F32, 0, {H * P * N, P * N, N, 1, 0}};
    Params p;
    rc = fill_fused(p, &x, &B, &dt, &dt, nullptr, nullptr, nullptr, &out, &fin, dims, 1);
    if (rc) return rc;
    const int n_cu = compute_units > 0 ? compute_units : 256;
    p.n_cu = n_cu;
    memset(plan, 0, sizeof(*plan));
    const ssd::cost::Problem q = problem_of(p, n_cu);
    const Choice c = choose(p, true, n_cu);
    if (ssd::mfma_supported(p)) plan->estimate_us[SSD_FAMILY_TOKEN_SPLIT] = (float)ssd::cost::token_split_us(q);
    if (ssd::quad_supported(p)) plan->estimate_us[SSD_FAMILY_FOUR_TILE] = (float)ssd::cost::four_tile_us(q);
    if (pair_supported(with_states_in_out(p))) plan->estimate_us[SSD_FAMILY_PAIR] = (float)ssd::cost::pair_us(q);
    plan->family = c.family;
    if (ssd::chain_supported(p)) {
        double us = 0.;
        const int r = ssd::cost::chain_chunks_per_item(q, &us);
        plan->estimate_us[SSD_FAMILY_CHAIN] = (float)us;
        if (has_workspace && g_forced_split.load(std::memory_order_relaxed) == 0 && us < 1.05 * estimate_us(q, c)) {
            plan->family = SSD_FAMILY_CHAIN;
            plan->chunks_per_item = r;
        }
    }
    return SSD_OK;
}

int ssd_chunk_cumsum_fwd(const ssd_tensor *dt, const ssd_tensor *A, const ssd_tensor *dt_bias, const ssd_tensor *dt_out,
                         const ssd_tensor *dA_cumsum, int32_t batch, int32_t seqlen, int32_t nheads, int32_t chunk_size,
                         int dt_softplus, float dt_min, float dt_max, void *stream)
{
    ssd::CumsumParams p;
    int rc = fill_cumsum(p, dt, A, dt_bias, dt_out, dA_cumsum, batch, seqlen, nheads, chunk_size, dt_softplus, dt_min, dt_max);
    if (rc) return rc;
    rc = check_device();
    if (rc) return rc;
    return (int)ssd::launch_chunk_cumsum(p, (hipStream_t)stream);
}

uint64_t ssd_fused_scan_workspace_bytes(const ssd_dims *dims, int with_out, int chunks_per_item)
{
    if (check_dims(dims)) return 0;
    if (with_out) return ssd::chain_workspace_bytes(dims->batch, dims->nheads, dims->headdim, dims->nchunks);
    Params p;
    memset(&p, 0, sizeof(p));
    p.batch = dims->batch; p.nheads = dims->nheads; p.headdim = dims->headdim; p.dstate = dims->dstate;
    p.C = dims->nchunks; p.Q = dims->chunk_size; p.y = (void *)16;
    const int r = ssd::chain_chunks_per_item(p, compute_units(), chunks_per_item);
    return ssd::chain_workspace_bytes_out16(dims->batch, dims->nheads, dims->headdim, dims->dstate, dims->nchunks, r);
}

int ssd_fused_chunk_state_passing_scan_fwd(const ssd_tensor *x, const ssd_tensor *B, const ssd_tensor *C, const ssd_tensor *dt,
                                           const ssd_tensor *dA_cumsum, const ssd_tensor *seq_idx,
                                           const ssd_tensor *initial_states, const ssd_tensor *out,
                                           const ssd_tensor *final_states, const ssd_tensor *y, const ssd_dims *dims,
                                           int clamp, int accumulate, const ssd_fused_opts *opts, void *stream)
{
    if (!present(C) || !present(y)) return SSD_ERR_NULL;
    Params p;
    int rc = fill_fused(p, x, B, dt, dA_cumsum, seq_idx, initial_states, nullptr, out, final_states, dims, clamp, true);
    if (rc) return rc;
    if (!dtype_ok(C->dtype) || !dtype_ok(y->dtype)) return SSD_ERR_DTYPE;
    if (C->stride[3] != 1 || y->stride[3] != 1) return SSD_ERR_STRIDE;
    Params q = p;
    q.Cm = C->data; q.sC_b = C->stride[0]; q.sC_l = C->stride[1]; q.sC_g = C->stride[2];
    q.y = y->data; q.dt_y = y->dtype; q.sy_b = y->stride[0]; q.sy_l = y->stride[1]; q.sy_h = y->stride[2];
    q.y_accumulate = accumulate ? 1 : 0;
    if (q.batch == 1) q.sC_b = q.sy_b = 0;
    if (q.ngroups == 1) q.sC_g = 0;
    if (q.nheads == 1) q.sy_h = 0;
    bool chain = false;
    // With `out` asked for as well, the one-launch kernel writes as many bytes as the two calls below and runs work
    // items of two chunks where they run four: measured slower (batch 4 x 8192 tokens x 80 heads, fp32 y: 424 against
    // 181 + 208 microseconds), so it serves such a call only where it is insisted on.
    const bool wanted = !present(out) || (opts && opts->kernel != SSD_KERNEL_AUTO);
    if (C->dtype == x->dtype && wanted) {
        rc = chain_decision(q, dims, opts, &chain);
        if (rc && present(out)) { rc = SSD_OK; chain = false; }      // forced, but not possible: the two calls below still are
        if (rc) return rc;
    } else if (opts && opts->used_workspace) {
        *opts->used_workspace = 0;
    }
    if (chain) return run_chain(q, opts, stream);
    // Elsewhere the passed states have to exist in memory: the fused call as it would run without y, then the
    // stand-alone consumer over its `out`.
    if (!present(out)) return SSD_ERR_SCRATCH;
    bool plain_chain = false;
    rc = chain_decision(p, dims, opts, &plain_chain);
    if (rc) { rc = SSD_OK; plain_chain = false; }
    rc = plain_chain ? run_chain(p, opts, stream) : run(p, true, stream);
    if (rc) return rc;
    return ssd_chunk_scan_states_fwd(C, out, dA_cumsum, seq_idx, y, dims, accumulate, stream);
}

int ssd_chunk_scan_states_fwd(const ssd_tensor *C, const ssd_tensor *prev_states, const ssd_tensor *dA_cumsum,
                              const ssd_tensor *seq_idx, const ssd_tensor *y, const ssd_dims *dims, int accumulate,
                              void *stream)
{
    if (!present(C) || !present(prev_states) || !present(dA_cumsum) || !present(y) || !dims) return SSD_ERR_NULL;
    const ssd_dims &d = *dims;
    if (d.batch <= 0 || d.seqlen <= 0 || d.nheads <= 0 || d.headdim <= 0 || d.dstate <= 0 || d.ngroups <= 0 ||
        d.chunk_size <= 0 || d.nheads % d.ngroups != 0 || d.nchunks != (d.seqlen + d.chunk_size - 1) / d.chunk_size)
        return SSD_ERR_SHAPE;
    if (!dtype_ok(C->dtype) || !dtype_ok(prev_states->dtype) || !dtype_ok(y->dtype) || dA_cumsum->dtype != SSD_F32)
        return SSD_ERR_DTYPE;
    if (C->stride[3] != 1 || prev_states->stride[4] != 1 || y->stride[3] != 1) return SSD_ERR_STRIDE;
    ssd::ScanParams p;
    memset(&p, 0, sizeof(p));
    p.Cm = C->data; p.dt_C = C->dtype;
    p.sC_b = C->stride[0]; p.sC_l = C->stride[1]; p.sC_g = C->stride[2];
    p.states = prev_states->data; p.dt_states = prev_states->dtype;
    p.sst_b = prev_states->stride[0]; p.sst_c = prev_states->stride[1]; p.sst_h = prev_states->stride[2];
    p.sst_p = prev_states->stride[3];
    p.dacs = (const float *)dA_cumsum->data;
    p.sda_b = dA_cumsum->stride[0]; p.sda_h = dA_cumsum->stride[1]; p.sda_c = dA_cumsum->stride[2];
    p.sda_k = dA_cumsum->stride[3];
    if (present(seq_idx)) {
        p.seq = (const int32_t *)seq_idx->data;
        p.ssq_b = seq_idx->stride[0]; p.ssq_l = seq_idx->stride[1];
    }
    p.out = y->data; p.dt_out = y->dtype;
    p.so_b = y->stride[0]; p.so_l = y->stride[1]; p.so_h = y->stride[2];
    p.batch = d.batch; p.seqlen = d.seqlen; p.nheads = d.nheads; p.headdim = d.headdim; p.dstate = d.dstate;
    p.ngroups = d.ngroups; p.Q = d.chunk_size; p.C = d.nchunks;
    p.accumulate = accumulate ? 1 : 0;
    int rc = check_device();
    if (rc) return rc;
    return (int)ssd::launch_scan_states(p, (hipStream_t)stream);
}

int ssd_set_scan_kernel(int kernel)
{
    if (kernel < 0 || kernel > 2) return SSD_ERR_SHAPE;
    return ssd::set_scan_kernel(kernel);
}

int ssd_measure_traffic_floor_part(const ssd_tensor *x, const ssd_tensor *B, const ssd_tensor *dt, const ssd_tensor *dA_cumsum,
                                   const ssd_tensor *out, const ssd_tensor *final_states, const ssd_dims *dims, int part,
                                   void *stream)
{
    if (part < 0 || part > 2) return SSD_ERR_SHAPE;
    Params p;
    int rc = fill_fused(p, x, B, dt, dA_cumsum, nullptr, nullptr, nullptr, out, final_states, dims, 1);
    if (rc) return rc;
    if (!ssd::chain_supported(p) || p.dt_out != ssd::DT_F32) return SSD_ERR_SHAPE;
    rc = check_device();
    if (rc) return rc;
    const int n_cu = compute_units();
    return (int)ssd::launch_mover(p, n_cu > 0 ? n_cu : 256, part, (hipStream_t)stream);
}

int ssd_measure_traffic_floor(const ssd_tensor *x, const ssd_tensor *B, const ssd_tensor *dt, const ssd_tensor *dA_cumsum,
                              const ssd_tensor *out, const ssd_tensor *final_states, const ssd_dims *dims, void *stream)
{
    return ssd_measure_traffic_floor_part(x, B, dt, dA_cumsum, out, final_states, dims, 0, stream);
}

int ssd_set_chain_xcds(int xcds)
{
    if (xcds < 0 || xcds > ssd::kChainMaxXcd) return SSD_ERR_SHAPE;
    return ssd::set_chain_xcds(xcds);
}

int ssd_set_segment_chunks(int chunks)
{
    if (chunks < 0) return SSD_ERR_SHAPE;
    return ssd::set_quad_segment_chunks(chunks);
}

int ssd_set_token_split(int waves)
{
    if (waves < 0 || waves > 4 || waves == 3) return SSD_ERR_SHAPE;
    const int old = g_forced_split.exchange(waves);
    ssd::set_token_split(waves == 2 || waves == 4 ? waves : 0);
    return old;
}

}  // extern "C"
