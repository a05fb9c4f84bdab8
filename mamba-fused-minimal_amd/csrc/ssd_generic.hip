// Generic FMA kernel for the SSD chunk-state contraction (optionally fused with the recurrence): any element
// type (f32 / bf16 / f16), any headdim, dstate and chunk size.  It is the path for fp32 inputs and for shapes the
// MFMA tiling does not cover; all arithmetic is fp32 FMA, so fp32 inputs keep fp32 accuracy.
//
// One workgroup owns a 16 (headdim) x 64 (dstate) state tile of one (batch, head) and, in fused mode, walks the
// chunks serially with the state in registers (4 values per thread).  Tokens are staged 32 at a time through
// LDS: x already multiplied by the per-token weight, B widened to fp32.
//
// Reference semantics: kernels/ssd_chunk_state.py:97-173, kernels/ssd_state_passing.py:27-84.
#include "ssd_params.h"

namespace ssd {

constexpr int GP = 16, GN = 64, GK = 32;

template <bool FUSED>
__global__ void __launch_bounds__(256) generic_kernel(const Params p)
{
    __shared__ float xs[GK][GP];
    __shared__ float Bs[GK][GN];
    const int tid = threadIdx.x;
    const int pl = tid >> 4, nl = (tid & 15) * 4;

    const int n_pt = (p.headdim + GP - 1) / GP, n_nt = (p.dstate + GN - 1) / GN;
    int item = blockIdx.x;
    const int nt = item % n_nt; item /= n_nt;
    const int pt = item % n_pt; item /= n_pt;
    const int h = item % p.nheads; item /= p.nheads;
    int b, c_begin, c_end;
    if (FUSED) { b = item; c_begin = 0; c_end = p.C; }
    else { b = item / p.C; c_begin = item - b * p.C; c_end = c_begin + 1; }

    const int L = p.seqlen, Q = p.Q;
    const int g = h / (p.nheads / p.ngroups);
    const int prow = pt * GP + pl, ncol = nt * GN + nl;
    const bool prow_ok = prow < p.headdim;
    const int64_t x_base = b * p.sx_b + h * p.sx_h;
    const int64_t B_base = b * p.sB_b + g * p.sB_g;
    const float *dtb = p.dt + b * p.sdt_b + h * p.sdt_h;
    const float *dab = p.dacs + b * p.sda_b + h * p.sda_h;
    const int32_t *sqb = p.seq ? p.seq + b * p.ssq_b : nullptr;

    float st[4] = {0.f, 0.f, 0.f, 0.f};
    if (FUSED) {
        if (p.init && prow_ok)
            for (int j = 0; j < 4; ++j)
                if (ncol + j < p.dstate)
                    st[j] = load_as_f32(p.init, b * p.sin_b + h * p.sin_h + (int64_t)prow * p.sin_p + ncol + j, p.dt_init);
        if (prow_ok)
            for (int j = 0; j < 4; ++j)
                if (ncol + j < p.dstate)
                    store_from_f32(p.out, b * p.so_b + h * p.so_h + (int64_t)prow * p.so_p + ncol + j, p.dt_out, st[j]);
    }
    int32_t prev_id = 0;

    for (int c = c_begin; c < c_end; ++c) {
        const float last = dab[c * p.sda_c + (int64_t)(Q - 1) * p.sda_k];
        const int lim_end = min((c + 1) * Q, L);
        const int32_t id_last = sqb ? sqb[(int64_t)(lim_end - 1) * p.ssq_l] : 0;
        float acc[4] = {0.f, 0.f, 0.f, 0.f};
        for (int k0 = 0; k0 < Q; k0 += GK) {
            __syncthreads();
            // stage x * w: GK x GP values, 2 per thread
            for (int e = tid; e < GK * GP; e += 256) {
                const int kk = e / GP, pp = e % GP;
                const int k = k0 + kk, t = c * Q + k;
                float v = 0.f;
                if (k < Q && t < L && pt * GP + pp < p.headdim) {
                    float ex = last - dab[c * p.sda_c + (int64_t)k * p.sda_k];
                    if (p.clamp) ex = fminf(ex, 0.f);
                    float w = __expf(ex) * dtb[c * p.sdt_c + (int64_t)k * p.sdt_k];
                    if (sqb && sqb[(int64_t)t * p.ssq_l] != id_last) w = 0.f;
                    v = load_as_f32(p.x, x_base + (int64_t)t * p.sx_l + pt * GP + pp, p.dt_in) * w;
                }
                xs[kk][pp] = v;
            }
            for (int e = tid; e < GK * GN; e += 256) {
                const int kk = e / GN, nn = e % GN;
                const int k = k0 + kk, t = c * Q + k;
                float v = 0.f;
                if (k < Q && t < L && nt * GN + nn < p.dstate)
                    v = load_as_f32(p.B, B_base + (int64_t)t * p.sB_l + nt * GN + nn, p.dt_in);
                Bs[kk][nn] = v;
            }
            __syncthreads();
#pragma unroll 8
            for (int kk = 0; kk < GK; ++kk) {
                const float xv = xs[kk][pl];
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[j] = fmaf(xv, Bs[kk][nl + j], acc[j]);
            }
        }
        if (p.states && prow_ok)
            for (int j = 0; j < 4; ++j)
                if (ncol + j < p.dstate)
                    store_from_f32(p.states, b * p.sst_b + c * p.sst_c + h * p.sst_h + (int64_t)prow * p.sst_p + ncol + j,
                                   p.dt_states, acc[j]);
        if (FUSED) {
            float sc = __expf(last);
            if (sqb) {
                if (id_last != prev_id) sc = 0.f;
                prev_id = id_last;
            }
            for (int j = 0; j < 4; ++j) st[j] = sc * st[j] + acc[j];
            if (prow_ok)
                for (int j = 0; j < 4; ++j)
                    if (ncol + j < p.dstate) {
                        if (c < p.C - 1)
                            store_from_f32(p.out, b * p.so_b + (c + 1) * p.so_c + h * p.so_h + (int64_t)prow * p.so_p + ncol + j,
                                           p.dt_out, st[j]);
                        else
                            p.fin[b * p.sf_b + h * p.sf_h + (int64_t)prow * p.sf_p + ncol + j] = st[j];
                    }
        }
    }
}

hipError_t launch_generic(const Params &p_in, bool fused, hipStream_t s)
{
    Params p = p_in;
    const int64_t n_pt = (p.headdim + GP - 1) / GP, n_nt = (p.dstate + GN - 1) / GN;
    const int64_t items = (int64_t)p.batch * p.nheads * n_pt * n_nt * (fused ? 1 : p.C);
    if (items <= 0) return hipSuccess;
    if (items > 0x7fffffffLL) return hipErrorInvalidValue;
    p.n_items = (int)items;
    dim3 grid((unsigned)items), block(256);
    if (fused) hipLaunchKernelGGL(generic_kernel<true>, grid, block, 0, s, p);
    else hipLaunchKernelGGL(generic_kernel<false>, grid, block, 0, s, p);
    return hipGetLastError();
}

}  // namespace ssd
