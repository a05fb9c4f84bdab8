// Internal kernel-argument block shared by the HIP kernels and the C-ABI dispatcher.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <atomic>
#include <utility>

namespace ssd {

enum : int { DT_F32 = 0, DT_BF16 = 1, DT_F16 = 2 };

// All strides are in elements of the tensor they index; innermost strides of x, B, states, out,
// init and fin are 1 (checked on the host).
struct Params {
    const void *x;        // (b, L, H, P)
    const void *B;        // (b, L, G, N)
    const float *dt;      // (b, H, C, Q)
    const float *dacs;    // (b, H, C, Q)
    const int32_t *seq;   // (b, L) or null
    const void *init;     // (b, H, P, N) or null
    void *states;         // (b, C, H, P, N) or null
    void *out;            // (b, C, H, P, N)           (fused only)
    float *fin;           // (b, H, P, N)              (fused only)
    int batch, seqlen, nheads, headdim, dstate, ngroups, Q, C;
    int64_t sx_b, sx_l, sx_h;
    int64_t sB_b, sB_l, sB_g;
    int64_t sdt_b, sdt_h, sdt_c, sdt_k;
    int64_t sda_b, sda_h, sda_c, sda_k;
    int64_t ssq_b, ssq_l;
    int64_t sin_b, sin_h, sin_p;
    int64_t sst_b, sst_c, sst_h, sst_p;
    int64_t so_b, so_c, so_h, so_p;
    int64_t sf_b, sf_h, sf_p;
    int dt_in, dt_states, dt_out, dt_init;
    int clamp;
    int n_items;          // work items of the launch
    int n_seg;            // segments the chunks are split into (chunk-state launch of the four-tile kernel)
    int *ws;              // ticket counter, error word and flags of the ticket / flag-chain kernel
    int spin_limit;       // polls after which a wave of that kernel stops waiting for a flag
    int n_xcd;            // XCDs (L2 caches) the units of that kernel are dealt to
    int n_cu;             // compute units of the device (0: not known, the launchers then assume 256 in 8 XCDs)
    int ws_cleared;       // the launch in front of that kernel has cleared `ws` already (chain_workspace_clear below)
    int epoch;            // of this launch on `ws` (below); <= 0: contents unknown, the launcher clears it and takes 1
    float *carry;         // inside `ws`, behind the flags: the fp32 states that cross between items when `out` is 16-bit or absent
    // the scan's state half inside the chain kernel (null y: not wanted)
    const void *Cm;       // (b, L, G, N), the element type of x
    void *y;              // (b, L, H, P)
    int64_t sC_b, sC_l, sC_g;
    int64_t sy_b, sy_l, sy_h;
    int dt_y, y_accumulate;
};

// State passing on a flattened state axis.
struct PassParams {
    const void *states;   // (b, C, H, dim)
    const float *da;      // (b, H, C)
    const void *init;     // (b, H, dim) or null
    const int32_t *seq;   // (b, L) or null
    void *out;            // (b, C, H, dim)
    float *fin;           // (b, H, dim)
    int batch, C, nheads, dim, seqlen, Q;
    int64_t sst_b, sst_c, sst_h;
    int64_t sda_b, sda_h, sda_c;
    int64_t sin_b, sin_h;
    int64_t ssq_b, ssq_l;
    int64_t so_b, so_c, so_h;
    int64_t sf_b, sf_h;
    int dt_states, dt_out, dt_init;
};

// dt preparation + per-chunk cumulative sum.
struct CumsumParams {
    const void *dt;        // (b, L, H), any of the three element types
    const void *A;         // (H)
    const void *dt_bias;   // (H) or null
    float *dt_out;         // (b, H, C, Q)
    float *dacs;           // (b, H, C, Q)
    int batch, seqlen, nheads, Q, C;
    int64_t sdt_b, sdt_l, sdt_h, sA, sbias;
    int64_t so_b, so_h, so_c, so_k;
    int64_t sa_b, sa_h, sa_c, sa_k;
    int dt_type, A_type, dt_bias_type;
    int softplus;
    float dt_min, dt_max;
    int *clear;            // a chain workspace to clear on the way (the kernel behind this one is the chain kernel), or null
    int n_clear;           // ints of it
};

// State-consuming half of the chunk scan: y = scale * (C . prev_states).
struct ScanParams {
    const void *Cm;        // (b, L, G, N)
    const void *states;    // (b, C, H, P, N): the state entering each chunk
    const float *dacs;     // (b, H, C, Q)
    const int32_t *seq;    // (b, L) or null
    void *out;             // (b, L, H, P)
    int batch, seqlen, nheads, headdim, dstate, ngroups, Q, C;
    int64_t sC_b, sC_l, sC_g;
    int64_t sst_b, sst_c, sst_h, sst_p;
    int64_t sda_b, sda_h, sda_c, sda_k;
    int64_t ssq_b, ssq_l;
    int64_t so_b, so_l, so_h;
    int dt_C, dt_states, dt_out;
    int accumulate;        // add to what out holds instead of overwriting it
};

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t hbits) { return __builtin_bit_cast(float, hbits << 16); }

__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f)
{
    return __builtin_bit_cast(uint16_t, (__bf16)f);   // round to nearest even
}

__device__ __forceinline__ float load_as_f32(const void *base, int64_t idx, int dt)
{
    if (dt == DT_F32) return ((const float *)base)[idx];
    if (dt == DT_BF16) return bf16_bits_to_f32(((const uint16_t *)base)[idx]);
    return (float)((const _Float16 *)base)[idx];
}

__device__ __forceinline__ void store_from_f32(void *base, int64_t idx, int dt, float v)
{
    if (dt == DT_F32) ((float *)base)[idx] = v;
    else if (dt == DT_BF16) ((uint16_t *)base)[idx] = f32_to_bf16_bits(v);
    else ((_Float16 *)base)[idx] = (_Float16)v;
}

// Inclusive sum over the 64 lanes of a wave with data-parallel-primitive moves (no LDS traffic): shifts by 1, 2, 4, 8
// inside each row of 16 lanes, then lane 15 of a row added to the whole next row, then lane 31 to the upper half.
__device__ __forceinline__ float wave_inclusive_sum(float x)
{
#if defined(__HIP_DEVICE_COMPILE__)
    auto shifted = [](float v, auto ctrl, auto rows) {
        return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), decltype(ctrl)::value,
                                                                     decltype(rows)::value, 0xf, true));
    };
    using std::integral_constant;
    x += shifted(x, integral_constant<int, 0x111>{}, integral_constant<int, 0xf>{});     // row_shr:1
    x += shifted(x, integral_constant<int, 0x112>{}, integral_constant<int, 0xf>{});     // row_shr:2
    x += shifted(x, integral_constant<int, 0x114>{}, integral_constant<int, 0xf>{});     // row_shr:4
    x += shifted(x, integral_constant<int, 0x118>{}, integral_constant<int, 0xf>{});     // row_shr:8
    x += shifted(x, integral_constant<int, 0x142>{}, integral_constant<int, 0xa>{});     // row_bcast:15 into rows 1, 3
    x += shifted(x, integral_constant<int, 0x143>{}, integral_constant<int, 0xc>{});     // row_bcast:31 into rows 2, 3
#endif
    return x;
}

// A launch that asks for more than 64 KB of LDS needs hipFuncAttributeMaxDynamicSharedMemorySize set on the kernel
// first, once per device.  `done` (one per kernel instantiation) has a bit per device ordinal, set after the call
// succeeded: threads that launch a kernel for the first time together set the attribute twice, which is harmless.
inline hipError_t ensure_dynamic_lds(const void *kernel, int bytes, std::atomic<uint64_t> &done)
{
    if (bytes <= 65536) return hipSuccess;
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    const uint64_t bit = dev >= 0 && dev < 64 ? 1ull << dev : 0;
    if (bit && (done.load(std::memory_order_acquire) & bit)) return hipSuccess;
    e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e == hipSuccess && bit) done.fetch_or(bit, std::memory_order_release);
    return e;
}

// Launchers implemented in the .hip files; each returns the hipError_t of its launch.
hipError_t launch_mfma(const Params &p, bool fused, hipStream_t s);
hipError_t launch_generic(const Params &p, bool fused, hipStream_t s);
hipError_t launch_state_passing(const PassParams &p, hipStream_t s);
bool mfma_supported(const Params &p);
hipError_t launch_quad(const Params &p, hipStream_t s);     // fused, four state tiles per workgroup sharing B in LDS
bool quad_supported(const Params &p);
hipError_t launch_quad_chunk_state(const Params &p, hipStream_t s);     // chunk states only, same kernel
bool quad_chunk_state_supported(const Params &p);
bool quad_inputs_supported(const Params &p);     // what the four-tile kernel asks of x, B, dt, dA_cumsum and the shape
int set_quad_segment_chunks(int n);     // 0 = automatic; chunks per workgroup of the above; returns the old value
// fused, work items drawn by ticket and chained by flags: every compute unit busy whatever the number of tiles
hipError_t launch_chain(const Params &p, int n_cu, int mode, hipStream_t s);
bool chain_supported(const Params &p);
bool chain_needs_carry(const Params &p);      // the workspace also holds the fp32 states that cross between items
// the variant of the chain kernel that also computes the scan's state half (p.y); the launch plan is launch_chain's
hipError_t launch_chain_scan(const Params &p, int chunks_per_item, bool local, int n_wg, hipStream_t s);
size_t chain_workspace_bytes(int batch, int nheads, int headdim, int nchunks);
// ... and with room for the fp32 states that cross between items of `chunks_per_item` chunks when `out` is bf16
size_t chain_workspace_bytes_out16(int batch, int nheads, int headdim, int dstate, int nchunks, int chunks_per_item);
int chain_chunks_per_item(const Params &p, int n_cu, int forced);     // what launch_chain takes (forced: 0, 1, 2 or 4)

// Layout of a chain workspace (ints).  A launch carries an epoch, one more than that of the launch before it on the
// same workspace.  Everything a launch must find in a known state is either tagged with the epoch or kept twice:
//   [32 b + slot]  ticket counters, one bank b = epoch & 1 per parity, a slot per XCD (16).  The workgroups that draw
//                  ticket 0 of a slot zero the other bank, the other error word and record the epoch: the next
//                  launch finds its counters at zero without a fill launch in between.
//   [32 b + 16 + slot]  work items each slot has to hand out in the launch with parity b (written with the above): a
//                  slot whose counter ends below it was never served (ssd_fused_workspace_status)
//   [64 + b]       error word of the launch with parity b (bit 0: a flag wait ran out, bit 1: two XCDs drew from one
//                  slot, bit 2: the workspace is not in the state the epoch promises);  [66] epoch of the last launch;
//                  [67] a tag that says a chain launch has cleared this memory at least once (without it the words
//                  above mean nothing);  [68] ints cleared by the last clearing (flags beyond hold anything)
//   [96 + slot]    hardware id (+1) of the XCD that drew from each slot
//   [128 ...]      flags, one per (state tile, chunk): raised = holds the epoch of the launch (older values, from
//                  launches before, and the zeros of a clearing never equal it)
//   behind the flags, from the next multiple of 64 ints: 32 x dstate fp32 per (state tile, item) when `out` is bf16;
//                  written before it is read in every launch, never cleared
constexpr int kChainWsHeaderInts = 128, kChainWsBankStride = 32, kChainWsTotalOffset = 16, kChainWsErrWord = 64,
              kChainWsEpochWord = 66, kChainWsTagWord = 67, kChainWsClearedWord = 68, kChainWsOwnerWord = 96,
              kChainWsTag = 0x53534443, kChainMaxXcd = 16;
enum : int { kChainErrTimeout = 1, kChainErrXcd = 2, kChainErrWorkspace = 4 };
// The value a clearing of the first n ints of a chain workspace leaves at int i: zero, except for the tag and the
// record of n itself.  Any kernel that runs in front of the chain kernel on the same stream may do the clearing (the
// stand-alone producer of dt / dA_cumsum does when both are launched by one call); Params::ws_cleared then keeps the
// chain kernel's own fill launch away.
__host__ __device__ constexpr int chain_workspace_clear(int i, int n)
{
    return i == kChainWsTagWord ? kChainWsTag : i == kChainWsClearedWord ? n : 0;
}
// What the first kChainWsHeaderInts ints of a workspace say about the last chain launch on it: 0, or the most
// serious of the conditions above as a negative ssd_status.  Host logic.
int chain_status_of_header(const int *header);
int set_chain_xcds(int n);        // 0 = from the device's compute units; a test hook; returns the old value
// measurement only: the fused call's x / B reads and `out` writes with nothing else (ssd_mover.hip); overwrites p.out
hipError_t launch_mover(const Params &p, int n_cu, int part, hipStream_t s);
hipError_t launch_chunk_cumsum(const CumsumParams &p, hipStream_t s);
bool chunk_cumsum_supported(const CumsumParams &p);
hipError_t launch_scan_states(const ScanParams &p, hipStream_t s);
bool scan_states_mfma_supported(const ScanParams &p);
int set_scan_kernel(int k);       // 0 = automatic; 1 = one workgroup per head; 2 = runs of heads; returns the old value
int set_token_split(int wv);      // 0 = automatic; 2 or 4 forces the token split of the MFMA kernels; returns the old value

}  // namespace ssd
