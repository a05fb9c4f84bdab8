// Host side of the ticket / flag-chain fused kernel (ssd_chain_kernel.h): workspace layout and sizes, what the kernel
// covers, the choice of its variant for a launch, and the launch itself.
#include "ssd_chain_kernel.h"

namespace ssd {

namespace chain {

// workspace cleared before every launch: ticket counter, error word and flags; the tag says that the error word is
// this kernel's (a workspace may hold anything before its first launch)
__global__ void __launch_bounds__(256) clear_kernel(int *ws, int n)
{
    for (int i = blockIdx.x * 256 + threadIdx.x; i < n; i += gridDim.x * 256) ws[i] = chain_workspace_clear(i, n);
}

static bool aligned(const void *ptr, size_t a) { return ((uintptr_t)ptr % a) == 0; }

static bool rows_ok(const void *ptr, int64_t strides_or, int64_t row_stride, int headdim)
{
    return aligned(ptr, 16) && strides_or % 4 == 0 && (int64_t)headdim * row_stride < (1LL << 28);
}

// LOCAL reads passed states back with plain loads, which the per-CU cache may serve: safe as long as a compute unit
// never holds a line that another wave's tile shares, i.e. as long as every row that is read back (of fp32 `out`, or
// of the fp32 slots of the workspace when `out` is 16-bit) starts and ends on 128-byte line boundaries.
static bool local_lines_ok(const Params &p)
{
    if (chain_needs_carry(p)) return aligned(p.ws, 128);      // slots: 256-byte offset, 32 x dstate x 4 bytes each
    const int64_t strides_or = p.so_b | p.so_c | p.so_h | p.so_p | p.dstate;
    return aligned(p.out, 128) && (strides_or * 4) % 128 == 0;
}

static std::atomic<int> g_forced_xcds{0};

}  // namespace chain

int set_chain_xcds(int n) { return chain::g_forced_xcds.exchange(n); }

// the state that crosses between work items goes through fp32 slots of the workspace unless `out` is an fp32 tensor
// to read it back from
bool chain_needs_carry(const Params &p) { return !p.out || p.dt_out != DT_F32; }

// bit 2 first: with a workspace that is not what the epoch promised, the other words mean nothing
int chain_status_of_header(const int *h)
{
    if (h[kChainWsTagWord] != kChainWsTag) return 0;       // the chain kernel has not run on this memory
    const int bank = h[kChainWsEpochWord] & 1, err = h[kChainWsErrWord + bank];
    if (err & kChainErrWorkspace) return -10;
    if (err & kChainErrXcd) return -8;
    for (int s = 0; s < kChainMaxXcd; ++s)
        if (h[kChainWsBankStride * bank + s] < h[kChainWsBankStride * bank + kChainWsTotalOffset + s]) return -9;
    return (err & kChainErrTimeout) ? -7 : 0;
}

size_t chain_workspace_bytes(int batch, int nheads, int headdim, int nchunks)
{
    const int64_t tiles = (int64_t)batch * nheads * ((headdim + 31) / 32);
    return (size_t)(chain::kWsHeaderInts + tiles * nchunks) * sizeof(int);
}

// ints in front of the fp32 carry slots: header and flags, rounded up to 256 bytes
static int64_t carry_offset_ints(int64_t tiles, int nchunks)
{
    return (chain::kWsHeaderInts + tiles * nchunks + 63) / 64 * 64;
}

size_t chain_workspace_bytes_out16(int batch, int nheads, int headdim, int dstate, int nchunks, int chunks_per_item)
{
    const int64_t tiles = (int64_t)batch * nheads * ((headdim + 31) / 32);
    const int r = chunks_per_item > 0 ? chunks_per_item : 1;
    const int64_t items = (nchunks + r - 1) / r;
    return (size_t)(carry_offset_ints(tiles, nchunks) * (int64_t)sizeof(int) + tiles * items * 32 * dstate * (int64_t)sizeof(float));
}

// Chunks per item: four (what the register file holds parked) unless the estimate says that the compute units end up
// with too few or too unequal numbers of items that large.  With bf16 `out` at least two: with one, the fp32 copies
// of the passed states would be a whole fp32 `out`.
int chain_chunks_per_item(const Params &p, int n_cu, int forced)
{
    if (p.y) return 2;        // the variant that also computes the scan's state half: what the register file holds
    if (forced == 1 || forced == 2 || forced == 4) return forced;
    cost::Problem q;
    q.units = (p.batch * p.nheads * (p.headdim / 32)) >> 2; q.chunks = p.C; q.chunk_size = p.Q; q.dstate = p.dstate;
    q.n_cu = n_cu > 0 ? n_cu : 256;
    const int r = cost::chain_chunks_per_item(q, nullptr);
    return chain_needs_carry(p) && r < 2 ? 2 : r;
}

// fp32 initial_states / final_states, fp32 or bf16 out, no `states` output, and what the four-tile kernel asks of the
// inputs
bool chain_supported(const Params &p)
{
    using namespace chain;
    if (p.states || !p.fin) return false;
    if (!p.out && !p.y) return false;          // passed states that nobody receives and nobody consumes
    if (!quad_inputs_supported(p)) return false;
    if (p.init && p.dt_init != DT_F32) return false;
    if (p.out && p.dt_out != DT_F32 && p.dt_out != DT_BF16) return false;
    if (p.out && !rows_ok(p.out, p.so_b | p.so_c | p.so_h | p.so_p, p.so_p, p.headdim)) return false;
    if (p.y) {
        // the scan variant: C rows like B rows, y rows of 16 bytes per lane, fp32 passed states or none
        if (p.out && p.dt_out != DT_F32) return false;
        if (p.dt_y != DT_F32 && p.dt_y != DT_BF16) return false;
        if (!p.Cm || !aligned(p.Cm, 16) || (p.sC_b | p.sC_l | p.sC_g) % 8 != 0 || p.sC_l * 2 * p.Q >= (1LL << 31)) return false;
        if (!aligned(p.y, 16) || (p.sy_b | p.sy_l | p.sy_h) % 8 != 0 || p.sy_l * 4 * p.Q >= (1LL << 31)) return false;
    }
    if (!rows_ok(p.fin, p.sf_b | p.sf_h | p.sf_p, p.sf_p, p.headdim)) return false;
    if (p.init && !rows_ok(p.init, p.sin_b | p.sin_h | p.sin_p, p.sin_p, p.headdim)) return false;
    if ((int64_t)p.batch * p.nheads * (p.headdim / 32) * p.C >= (1LL << 30)) return false;     // flag index, tickets
    return true;
}

template <int NT, int SPC, int R, bool SEQ, bool LOCAL, bool OUT16>
static hipError_t launch_chain_k(const Params &p, int n_wg, hipStream_t s)
{
    return chain::launch_kernel<NT, SPC, R, SEQ, LOCAL, OUT16 ? 1 : 0, false>(p, n_wg, s);
}

template <int R, bool SEQ, bool LOCAL, bool OUT16>
static hipError_t launch_chain_r(const Params &p, int n_wg, hipStream_t s)
{
    const int nt = p.dstate / 16, spc = p.Q / 32;
    if (nt == 8 && spc == 8) return launch_chain_k<8, 8, R, SEQ, LOCAL, OUT16>(p, n_wg, s);
    if (nt == 8 && spc == 4) return launch_chain_k<8, 4, R, SEQ, LOCAL, OUT16>(p, n_wg, s);
    if (nt == 4 && spc == 8) return launch_chain_k<4, 8, R, SEQ, LOCAL, OUT16>(p, n_wg, s);
    return launch_chain_k<4, 4, R, SEQ, LOCAL, OUT16>(p, n_wg, s);
}

template <bool SEQ, bool LOCAL>
static hipError_t launch_chain_t(const Params &p, int r, int n_wg, hipStream_t s)
{
    if (p.dt_out != DT_F32) {       // bf16 out: items of one chunk are not offered (chain_chunks_per_item)
        if (r >= 4) return launch_chain_r<4, SEQ, LOCAL, true>(p, n_wg, s);
        return launch_chain_r<2, SEQ, LOCAL, true>(p, n_wg, s);
    }
    if (r >= 4) return launch_chain_r<4, SEQ, LOCAL, false>(p, n_wg, s);
    if (r >= 2) return launch_chain_r<2, SEQ, LOCAL, false>(p, n_wg, s);
    return launch_chain_r<1, SEQ, LOCAL, false>(p, n_wg, s);
}

// p.ws: at least chain_workspace_bytes(...) of device memory, 4-byte aligned (bf16 out: chain_workspace_bytes_out16(...)
// for the chunks per item that chain_chunks_per_item(p, n_cu, p.n_seg) gives, 16-byte aligned); the launch clears what
// it uses.
// n_cu: compute units of the device.  mode: 0 = choose, 1 = LOCAL, 2 = GLOBAL.
hipError_t launch_chain(const Params &p_in, int n_cu, int mode, hipStream_t s)
{
    Params p = p_in;
    p.n_items = p.batch * p.nheads * (p.headdim / 32);
    if (p.n_items <= 0 || p.C <= 0) return hipSuccess;
    if (p.spin_limit <= 0) p.spin_limit = 1 << 22;
    const int64_t n_ws = chain::kWsHeaderInts + (int64_t)p.n_items * p.C;
    hipError_t e = hipSuccess;
    // epoch <= 0: the workspace may hold anything: cleared here (or by the launch in front), and this is launch 1 on it
    const bool clear = p.epoch <= 0;
    if (clear) p.epoch = 1;
    if (clear && !p.ws_cleared) {
        hipLaunchKernelGGL(chain::clear_kernel, dim3((unsigned)((n_ws + 255) / 256 < 1024 ? (n_ws + 255) / 256 : 1024)), dim3(256), 0, s,
                           p.ws, (int)n_ws);
        e = hipGetLastError();
        if (e != hipSuccess) return e;
    }
    // An XCD is 32 compute units on this part.  Units are dealt to the XCDs in contiguous ranges; LOCAL pays when
    // the fullest XCD holds at most an eighth more than its fair share of them.
    const int n_units = p.n_items >> 2;
    p.n_xcd = n_cu >= 32 ? n_cu / 32 : 1;
    const int forced_xcds = chain::g_forced_xcds.load(std::memory_order_relaxed);
    if (forced_xcds > 0) p.n_xcd = forced_xcds;      // test hook: a wrong count is what the kernel's checks are for
    if (p.n_xcd > chain::kMaxXcd) p.n_xcd = chain::kMaxXcd;
    // LOCAL when the units spread evenly over the XCDs and each has a few of its own: producer and consumer of a passed
    // state then share an L2 (no read-back from memory), and an XCD only fetches the B rows of its own units' groups
    // (b=1 L=131072 H=128 G=8: 5.3 GB of HBM traffic instead of 6.5 GB for 4.7 GB algorithmic, 1.15 ms
    // against 1.17 ms).  With few units per XCD most of its workgroups sit in a few chains, and where all units share
    // one (batch, group) every XCD fetches all of B anyway: eight units per XCD is where LOCAL starts to pay (five, at
    // b=1 L=32768 H=80 in 16 packed sequences: 208 us against 204 us with one counter; eight, at b=1 L=131072 H=128 G=8:
    // 1.065 against 1.068 ms; twenty, at b=4 L=8192 H=80: 179 against 186 us).
    const int fullest = (n_units + p.n_xcd - 1) / p.n_xcd;
    bool local = mode == 1 || (mode == 0 && n_units >= 8 * p.n_xcd && (int64_t)fullest * p.n_xcd * 8 <= (int64_t)n_units * 9);
    // Chunks per item: four (what the register file holds parked) unless the estimate says that the compute units
    // end up with too few or too unequal numbers of items that large.  p.n_seg > 0 forces a value.
    const int r = chain_chunks_per_item(p, n_cu, p.n_seg);
    if (chain_needs_carry(p)) {
        if (r < 2) return hipErrorInvalidValue;
        p.carry = (float *)(p.ws + carry_offset_ints(p.n_items, p.C));
    }
    // buffers whose tiles share cache lines (an `out` view at an odd offset): through memory, also where LOCAL was asked for
    if (local && !chain::local_lines_ok(p)) local = false;
    const int64_t total = (int64_t)n_units * ((p.C + r - 1) / r);
    int n_wg = (int)(total < n_cu ? total : n_cu);
    // LOCAL: a workgroup only works on the units of the XCD it finds itself on, so every XCD needs one.  Workgroups go
    // to the XCDs in turn, but not starting from XCD 0 (the turn carries over from the launch before): a whole number
    // of rounds, at least one, reaches them all; workgroups without work leave at once.
    if (local) n_wg = (n_wg + p.n_xcd - 1) / p.n_xcd * p.n_xcd;
    if (p.y) return launch_chain_scan(p, r, local, n_wg, s);
    if (p.seq) return local ? launch_chain_t<true, true>(p, r, n_wg, s) : launch_chain_t<true, false>(p, r, n_wg, s);
    return local ? launch_chain_t<false, true>(p, r, n_wg, s) : launch_chain_t<false, false>(p, r, n_wg, s);
}

}  // namespace ssd
