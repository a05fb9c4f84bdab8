// A measurement kernel, not part of the path: the memory traffic of the fused chunk-state + state-passing call with
// every arithmetic instruction, every dependency between chunks and every wait on another workgroup taken away.  What
// it takes is the floor that this device's memory system sets for the path's access pattern -- x rows read once (64
// bytes per token and state tile), B rows read once per four state tiles (from L2 after the first reader), one
// 32 x dstate fp32 tile written per (state tile, chunk) -- against which the fused kernels are priced (bench.py).
// The reference has no counterpart (its kernels are kernels/fused_globalbar.py:16-198, kernels/fused_concurrent.py:17-252).
//
// One persistent workgroup per compute unit, four waves, one state tile stream per wave as in the fused kernels
// (ssd_chain.hip): per 32-token step a wave requests its 32 x rows (two requests of 16 rows x 64 bytes) and a quarter of
// the step's B tile straight into LDS, kDepth steps ahead, and at the end of a chunk stores a tile of 32 x dstate fp32
// in the fused kernels' store pattern (16 bytes per lane, four adjacent lanes per 64-byte run).  Nothing is read back
// from LDS and the stored values are a register that holds zeros: `out` is scratch to this kernel.  `part` leaves one
// side out: 1 = the loads only, 2 = the stores only (how the two share the memory system: bench.py times all three).
#include "ssd_tile.h"

namespace ssd {

namespace mover {

using namespace tile;

constexpr int kDepth = 7;       // steps of requests in flight per wave, the fused chain kernel's distance

template <int NT, int SPC>
__global__ void __launch_bounds__(256, 1) mover_kernel(const Params p, const int part)
{
    constexpr int Q = 32 * SPC, NTW = NT / 4, kPerStep = 2 + NTW, kSlot = kPerStep * 1024;
    extern __shared__ __attribute__((aligned(16))) char lds[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    char *mine = lds + wave * (kDepth + 1) * kSlot;
    const int n_units = p.n_items >> 2, total = n_units * p.C, n_pt = p.headdim >> 5;
    const int64_t xrb = 2 * p.sx_l, Brb = 2 * p.sB_l;
    const int xlane = (int)((lane >> 2) * xrb) + 16 * (lane & 3);
    const int Blane = (int)((lane >> 2) * Brb) + 16 * (lane & 3);
    const u32x4 zero = {0u, 0u, 0u, 0u};

    struct Work { __amdgpu_buffer_rsrc_t rsx, rsB, rso; int p0, valid; };
    // item i (chunk-major: chunk i / units of unit i % units) as this wave sees it
    auto decode = [&](int i) {
        Work w;
        w.valid = i < total;
        const int iv = w.valid ? i : 0;
        const int c = iv / n_units, tile_ = 4 * (iv - c * n_units) + wave;
        const int r1 = tile_ / n_pt, b = r1 / p.nheads, h = r1 - b * p.nheads;
        const int g = h / (p.nheads / p.ngroups);
        w.p0 = 32 * (tile_ - r1 * n_pt);
        const int64_t rows = w.valid ? p.seqlen - c * Q : 0;
        w.rsx = make_rsrc((const char *)p.x + 2 * (b * p.sx_b + h * p.sx_h) + (int64_t)c * Q * xrb, rows * xrb);
        w.rsB = make_rsrc((const char *)p.B + 2 * (b * p.sB_b + g * p.sB_g) + (int64_t)c * Q * Brb, rows * Brb);
        w.rso = make_rsrc((const float *)p.out + b * p.so_b + c * p.so_c + h * p.so_h + (int64_t)w.p0 * p.so_p,
                          w.valid ? (31 * p.so_p + p.dstate) * 4 : 0);
        return w;
    };
    auto request = [&](const Work &w, int s, int slot) {
#if defined(__HIP_DEVICE_COMPILE__)
        typedef __attribute__((address_space(3))) void *lds_ptr;
        char *dst = mine + slot * kSlot;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(w.rsx, (lds_ptr)dst, 16, xlane + 2 * w.p0, (int)((32 * s) * xrb), 0, 0);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(w.rsx, (lds_ptr)(dst + 1024), 16, xlane + 2 * w.p0, (int)((32 * s + 16) * xrb), 0, 0);
#pragma unroll
        for (int k = 0; k < NTW; ++k) {
            const int bi = wave * NTW + k, th = bi / (NT / 2), pair = bi % (NT / 2);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(w.rsB, (lds_ptr)(dst + 2048 + k * 1024), 16, Blane,
                                                     (int)((32 * s + 16 * th) * Brb) + 64 * pair, 0, 0);
        }
#else
        (void)w; (void)s; (void)slot; (void)xlane; (void)Blane;
#endif
    };
    auto store_tile = [&](const Work &w) {
        const int pitch = (int)p.so_p, row = 2 * (lane >> 2), col = 4 * (lane & 3);
#pragma unroll
        for (int k = 0; k < 2 * NT; ++k) store4_f32(w.rso, row * pitch + col, (k & 1) * pitch + 16 * (k >> 1), __builtin_bit_cast(f32x4, zero), 0);
    };

    // the stream of steps of this workgroup's items: item j of the workgroup is blockIdx.x + j * gridDim.x
    int i_req = blockIdx.x, s_req = 0;       // the step to request next
    Work w_req = decode(i_req);
    auto advance_req = [&]() {
        if (++s_req == SPC) { s_req = 0; i_req += gridDim.x; w_req = decode(i_req); }
    };
    int n = 0;
#pragma unroll 1
    for (; n < kDepth; ++n) { if (part != 2) request(w_req, s_req, n % (kDepth + 1)); advance_req(); }
    Work w_cur = decode(blockIdx.x);
#pragma unroll 1
    for (int i = blockIdx.x; i < total; i += gridDim.x) {
#pragma unroll 1
        for (int s = 0; s < SPC; ++s, ++n) {
            if (part != 2) request(w_req, s_req, n % (kDepth + 1));       // past the end: empty descriptors, nothing fetched
            advance_req();
            // the oldest step has landed once only the kDepth newer ones are outstanding (stores issued since count
            // as well, which makes the wait shorter than needed at the first step of a chunk: nothing reads the data)
            __builtin_amdgcn_s_waitcnt(vmcnt_imm(kDepth * kPerStep > 63 ? 63 : kDepth * kPerStep));
            __builtin_amdgcn_s_barrier();                  // the fused kernels share a step's B tile: one barrier per step
        }
        if (part != 1) store_tile(w_cur);
        w_cur = decode(i + gridDim.x);
    }
}

template <int NT, int SPC>
static hipError_t launch_k(const Params &p, int n_wg, int part, hipStream_t s)
{
    constexpr int lds = 4 * (kDepth + 1) * (2 + NT / 4) * 1024;
    static std::atomic<uint64_t> configured{0};
    const hipError_t e = ensure_dynamic_lds((const void *)mover_kernel<NT, SPC>, lds, configured);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL((mover_kernel<NT, SPC>), dim3(n_wg), dim3(256), lds, s, p, part);
    return hipGetLastError();
}

}  // namespace mover

// p: x, B, out and the sizes of a fused call that the chain kernel covers (chain_supported); `out` is overwritten.
hipError_t launch_mover(const Params &p_in, int n_cu, int part, hipStream_t s)
{
    Params p = p_in;
    p.n_items = p.batch * p.nheads * (p.headdim / 32);
    const int64_t total = (int64_t)(p.n_items >> 2) * p.C;
    if (total <= 0) return hipSuccess;
    const int n_wg = (int)(total < n_cu ? total : n_cu);
    const int nt = p.dstate / 16, spc = p.Q / 32;
    if (nt == 8 && spc == 8) return mover::launch_k<8, 8>(p, n_wg, part, s);
    if (nt == 8 && spc == 4) return mover::launch_k<8, 4>(p, n_wg, part, s);
    if (nt == 4 && spc == 8) return mover::launch_k<4, 8>(p, n_wg, part, s);
    return mover::launch_k<4, 4>(p, n_wg, part, s);
}

}  // namespace ssd
