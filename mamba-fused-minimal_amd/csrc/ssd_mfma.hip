// bf16 MFMA kernel for the SSD chunk-state contraction, optionally fused with the inter-chunk recurrence.
//
// Work decomposition (gfx950, 64-wide waves, v_mfma_f32_16x16x32_bf16):
//   * one workgroup (4 waves) owns a (batch, head, 32-row slice of headdim) x all of dstate state tile and,
//     in fused mode, walks the chunks of that unit serially, so the running state never leaves registers and
//     no workgroup ever waits for another one;
//   * inside a chunk the 4 waves split the tokens (the contraction index): wave w contracts tokens
//     [w*Q/4, (w+1)*Q/4).  Each wave therefore streams its own rows of x and B straight from global memory
//     into MFMA operand registers -- no operand goes through LDS:
//       - lane (i = lane%16, kg = lane/16) loads, for 8 consecutive tokens 8kg..8kg+7 of a 32-token step,
//         one dword of x (headdim rows 2i, 2i+1) and NB consecutive bf16 of B (dstate columns NB*i .. NB*i+NB-1);
//       - x is widened to fp32, multiplied by the per-token weight w_k and split into bf16 hi + bf16 lo, so that
//         the two MFMAs hi*B + lo*B carry ~16 mantissa bits of x*w (a single bf16 rounding of the scaled operand,
//         which is what the reference does, is not accurate enough for an fp32 comparison);
//       - the 2x2 16-bit transposes that turn "8 tokens x 2 values" into the token-contiguous MFMA operand
//         layout are one v_cvt_pk_bf16_f32 (x side, free with the rounding) or one v_perm_b32 (B side) per dword;
//       - MFMA tile (jp, jn) covers headdim rows {2i+jp} and dstate columns {NB*i+jn}: the row/column
//         permutation makes every lane own NB consecutive dstate values of one row, so results are stored
//         with 128-bit stores and each 16-lane group writes one full, contiguous row of the state;
//   * the four token-partial tiles are summed through LDS (48 KB for dstate 128): wave w ends up owning the
//     rows with (row/2)%4 == w, applies s = exp(dA_chunk)*s + partial sum, and stores out / states.
//
// Reference semantics: kernels/ssd_chunk_state.py:97-173, kernels/ssd_state_passing.py:27-84,
// kernels/fused_globalbar.py:16-198 (same math, one launch).
#include "ssd_params.h"

namespace ssd {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi)
{
    bf16x2 v = {(__bf16)lo, (__bf16)hi};
    return __builtin_bit_cast(uint32_t, v);
}

__device__ __forceinline__ void lds_barrier()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

template <int NBD> __device__ __forceinline__ void load_brow(const uint16_t *ptr, uint32_t (&o)[NBD]);
template <> __device__ __forceinline__ void load_brow<2>(const uint16_t *ptr, uint32_t (&o)[2])
{
    u32x2 v = *(const u32x2 *)ptr;
    o[0] = v.x; o[1] = v.y;
}
template <> __device__ __forceinline__ void load_brow<4>(const uint16_t *ptr, uint32_t (&o)[4])
{
    u32x4 v = *(const u32x4 *)ptr;
    o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w;
}

// Store NB consecutive state values of one row (fp32, bf16 or f16 destination).
template <int NB> __device__ __forceinline__ void store_row(void *base, int dt, int64_t off, const float (&v)[NB])
{
    if (dt == DT_F32) {
        float *d = (float *)base + off;
#pragma unroll
        for (int u = 0; u < NB / 4; ++u) {
            f32x4 q = {v[4 * u], v[4 * u + 1], v[4 * u + 2], v[4 * u + 3]};
            *(f32x4 *)(d + 4 * u) = q;
        }
    } else {
        uint32_t w[NB / 2];
#pragma unroll
        for (int u = 0; u < NB / 2; ++u) {
            if (dt == DT_BF16) {
                w[u] = pack_bf16(v[2 * u], v[2 * u + 1]);
            } else {
                typedef __attribute__((ext_vector_type(2))) _Float16 h2;
                h2 hv = {(_Float16)v[2 * u], (_Float16)v[2 * u + 1]};
                w[u] = __builtin_bit_cast(uint32_t, hv);
            }
        }
        uint32_t *d = (uint32_t *)((uint16_t *)base + off);
        if constexpr (NB == 8) {
            u32x4 q = {w[0], w[1], w[2], w[3]};
            *(u32x4 *)d = q;
        } else {
            u32x2 q = {w[0], w[1]};
            *(u32x2 *)d = q;
        }
    }
}

// Token-split reduction through LDS.  Wave W keeps accumulator component r == W of every tile (headdim rows
// 2*(4kg+W)+jp) and hands the other three components to their owners.
template <int W, int NB>
__device__ __forceinline__ void exchange_write(const f32x4 (&acc)[2][NB], f32x4 *red, int lane)
{
    constexpr int NU = NB / 4;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        if (r == W) continue;
        const int slot = W < r ? W : W - 1;
#pragma unroll
        for (int jp = 0; jp < 2; ++jp)
#pragma unroll
            for (int u = 0; u < NU; ++u) {
                f32x4 v = {acc[jp][4 * u][r], acc[jp][4 * u + 1][r], acc[jp][4 * u + 2][r], acc[jp][4 * u + 3][r]};
                red[((r * 3 + slot) * (2 * NU) + jp * NU + u) * 64 + lane] = v;
            }
    }
}

template <int W, int NB>
__device__ __forceinline__ void exchange_read(const f32x4 (&acc)[2][NB], const f32x4 *red, int lane,
                                              float (&sum)[2][NB])
{
    constexpr int NU = NB / 4;
#pragma unroll
    for (int jp = 0; jp < 2; ++jp)
#pragma unroll
        for (int u = 0; u < NU; ++u) {
            f32x4 t = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < 4; ++s) {       // fixed summation order over the four token quarters
                f32x4 part;
                if (s == W) {
                    part = (f32x4){acc[jp][4 * u][W], acc[jp][4 * u + 1][W], acc[jp][4 * u + 2][W], acc[jp][4 * u + 3][W]};
                } else {
                    const int slot = s < W ? s : s - 1;
                    part = red[((W * 3 + slot) * (2 * NU) + jp * NU + u) * 64 + lane];
                }
                t = (s == 0) ? part : t + part;
            }
            sum[jp][4 * u] = t.x; sum[jp][4 * u + 1] = t.y; sum[jp][4 * u + 2] = t.z; sum[jp][4 * u + 3] = t.w;
        }
}

// NB = dstate / 16 (4 or 8); KS = 32-token steps per wave per chunk (chunk_size = 128 * KS).
template <int NB, int KS, bool HAS_SEQ, bool FUSED>
__global__ void __launch_bounds__(256, 2) mfma_kernel(const Params p)
{
    constexpr int NBD = NB / 2, NU = NB / 4, QW = 32 * KS;
    __shared__ f32x4 red[12 * 2 * NU * 64];
    __shared__ __attribute__((aligned(16))) float wbuf[4 * QW];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, i16 = lane & 15, kg = lane >> 4;

    // Work item -> (batch, [chunk,] head, row slice).  Consecutive items share B (same batch, same group) and
    // are placed on the same XCD (workgroups are dealt round-robin over the 8 XCDs), so that B tiles and the
    // two row slices of one head meet in one L2.
    const int per_xcd = (p.n_items + 7) >> 3;
    const int item = (int)(blockIdx.x & 7) * per_xcd + (int)(blockIdx.x >> 3);
    if (item >= p.n_items) return;
    const int n_pt = p.headdim >> 5;
    const int pt = item % n_pt;
    const int r1 = item / n_pt;
    const int h = r1 % p.nheads;
    const int r2 = r1 / p.nheads;
    int b, c_begin, c_end;
    if (FUSED) { b = r2; c_begin = 0; c_end = p.C; }
    else { b = r2 / p.C; c_begin = r2 - b * p.C; c_end = c_begin + 1; }

    const int L = p.seqlen, Q = p.Q;
    const int g = h / (p.nheads / p.ngroups);
    const int p0 = pt * 32;
    const uint16_t *xb = (const uint16_t *)p.x + b * p.sx_b + h * p.sx_h + p0 + 2 * i16;
    const uint16_t *Bb = (const uint16_t *)p.B + b * p.sB_b + g * p.sB_g + NB * i16;
    const float *dtb = p.dt + b * p.sdt_b + h * p.sdt_h;
    const float *dab = p.dacs + b * p.sda_b + h * p.sda_h;
    const int32_t *sqb = HAS_SEQ ? p.seq + b * p.ssq_b : nullptr;

    // flat step index over (chunk, 32-token step) for the register prefetch
    const int n_steps = (c_end - c_begin) * KS;
    auto load_x = [&](int gstep, uint32_t (&xo)[8]) {
        const int c = c_begin + gstep / KS, s = gstep % KS;
        const int t0 = c * Q + wave * QW + 32 * s + 8 * kg;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int t = min(t0 + j, L - 1);
            xo[j] = *(const uint32_t *)(xb + (int64_t)t * p.sx_l);
        }
    };
    auto load_B = [&](int gstep, uint32_t (&bo)[8][NBD]) {
        const int c = c_begin + gstep / KS, s = gstep % KS;
        const int t0 = c * Q + wave * QW + 32 * s + 8 * kg;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int t = min(t0 + j, L - 1);
            load_brow<NBD>(Bb + (int64_t)t * p.sB_l, bo[j]);
        }
    };

    uint32_t x0[8], x1[8], x2[8], b0[8][NBD], b1[8][NBD];
    load_x(0, x0);
    load_B(0, b0);
    if (n_steps > 1) load_x(1, x1);

    // owner rows of this lane after the token reduction
    const int prow = p0 + 2 * (4 * kg + wave);
    float st[2][NB];
    if (FUSED) {
#pragma unroll
        for (int jp = 0; jp < 2; ++jp) {
            if (p.init) {
                const int64_t off = b * p.sin_b + h * p.sin_h + (int64_t)(prow + jp) * p.sin_p + NB * i16;
#pragma unroll
                for (int jn = 0; jn < NB; ++jn) st[jp][jn] = load_as_f32(p.init, off + jn, p.dt_init);
            } else {
#pragma unroll
                for (int jn = 0; jn < NB; ++jn) st[jp][jn] = 0.f;
            }
            // out[:, 0] = initial state (kernels/ssd_state_passing.py:66)
            store_row<NB>(p.out, p.dt_out, b * p.so_b + h * p.so_h + (int64_t)(prow + jp) * p.so_p + NB * i16, st[jp]);
        }
    }
    int32_t prev_id = 0;

    int gstep = 0;
    for (int c = c_begin; c < c_end; ++c) {
        // ---- per-token weights of this wave's token quarter (kernels/ssd_chunk_state.py:134-156)
        const float last = dab[c * p.sda_c + (int64_t)(Q - 1) * p.sda_k];
        const int lim_end = min((c + 1) * Q, L);          // one past the last valid token of the chunk
        if (lane < QW) {
            const int k = wave * QW + lane;
            const int t = c * Q + k;
            const float dtv = dtb[c * p.sdt_c + k * p.sdt_k];
            const float cs = dab[c * p.sda_c + k * p.sda_k];
            float e = last - cs;
            if (p.clamp) e = fminf(e, 0.f);
            float wv = __expf(e) * dtv;
            if (t >= L) wv = 0.f;
            if (HAS_SEQ) {
                const int32_t id = sqb[(int64_t)min(t, L - 1) * p.ssq_l];
                const int32_t id_last = sqb[(int64_t)(lim_end - 1) * p.ssq_l];
                if (id != id_last) wv = 0.f;
            }
            wbuf[wave * QW + lane] = wv;
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront", "local");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront", "local");

        f32x4 acc[2][NB];
#pragma unroll
        for (int jp = 0; jp < 2; ++jp)
#pragma unroll
            for (int jn = 0; jn < NB; ++jn) acc[jp][jn] = (f32x4){0.f, 0.f, 0.f, 0.f};

#pragma unroll
        for (int s = 0; s < KS; ++s, ++gstep) {
            // prefetch: B one step ahead, x two steps ahead
            if (gstep + 1 < n_steps) load_B(gstep + 1, b1);
            if (gstep + 2 < n_steps) load_x(gstep + 2, x2);

            const f32x4 wlo = *(const f32x4 *)&wbuf[wave * QW + 32 * s + 8 * kg];
            const f32x4 whi = *(const f32x4 *)&wbuf[wave * QW + 32 * s + 8 * kg + 4];
            const float wv[8] = {wlo.x, wlo.y, wlo.z, wlo.w, whi.x, whi.y, whi.z, whi.w};

            // x * w in fp32, split into bf16 hi + bf16 lo, packed along the token axis
            uint32_t ahi[2][4], alo[2][4];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
#pragma unroll
                for (int jp = 0; jp < 2; ++jp) {
                    const uint32_t r0 = x0[2 * q], r1_ = x0[2 * q + 1];
                    const float v0 = __builtin_bit_cast(float, jp ? (r0 & 0xffff0000u) : (r0 << 16)) * wv[2 * q];
                    const float v1 = __builtin_bit_cast(float, jp ? (r1_ & 0xffff0000u) : (r1_ << 16)) * wv[2 * q + 1];
                    const uint32_t hp = pack_bf16(v0, v1);
                    const float h0 = __builtin_bit_cast(float, hp << 16);
                    const float h1 = __builtin_bit_cast(float, hp & 0xffff0000u);
                    ahi[jp][q] = hp;
                    alo[jp][q] = pack_bf16(v0 - h0, v1 - h1);
                }
            }
            bf16x8 Ahi[2], Alo[2];
#pragma unroll
            for (int jp = 0; jp < 2; ++jp) {
                Ahi[jp] = __builtin_bit_cast(bf16x8, (u32x4){ahi[jp][0], ahi[jp][1], ahi[jp][2], ahi[jp][3]});
                Alo[jp] = __builtin_bit_cast(bf16x8, (u32x4){alo[jp][0], alo[jp][1], alo[jp][2], alo[jp][3]});
            }
#pragma unroll
            for (int jn = 0; jn < NB; ++jn) {
                const uint32_t sel = (jn & 1) ? 0x07060302u : 0x05040100u;
                u32x4 f;
                f.x = __builtin_amdgcn_perm(b0[1][jn >> 1], b0[0][jn >> 1], sel);
                f.y = __builtin_amdgcn_perm(b0[3][jn >> 1], b0[2][jn >> 1], sel);
                f.z = __builtin_amdgcn_perm(b0[5][jn >> 1], b0[4][jn >> 1], sel);
                f.w = __builtin_amdgcn_perm(b0[7][jn >> 1], b0[6][jn >> 1], sel);
                const bf16x8 Bf = __builtin_bit_cast(bf16x8, f);
#pragma unroll
                for (int jp = 0; jp < 2; ++jp) {
                    acc[jp][jn] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(Ahi[jp], Bf, acc[jp][jn], 0, 0, 0);
                    acc[jp][jn] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(Alo[jp], Bf, acc[jp][jn], 0, 0, 0);
                }
            }
            // rotate the prefetch registers
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                x0[j] = x1[j]; x1[j] = x2[j];
#pragma unroll
                for (int d = 0; d < NBD; ++d) b0[j][d] = b1[j][d];
            }
        }

        // ---- sum the four token quarters
        lds_barrier();                      // previous chunk's exchange reads are done
        switch (wave) {
            case 0: exchange_write<0, NB>(acc, red, lane); break;
            case 1: exchange_write<1, NB>(acc, red, lane); break;
            case 2: exchange_write<2, NB>(acc, red, lane); break;
            default: exchange_write<3, NB>(acc, red, lane); break;
        }
        lds_barrier();
        float sum[2][NB];
        switch (wave) {
            case 0: exchange_read<0, NB>(acc, red, lane, sum); break;
            case 1: exchange_read<1, NB>(acc, red, lane, sum); break;
            case 2: exchange_read<2, NB>(acc, red, lane, sum); break;
            default: exchange_read<3, NB>(acc, red, lane, sum); break;
        }

        // ---- per-chunk states (side output) and the recurrence (kernels/ssd_state_passing.py:69-84)
        if (p.states) {
#pragma unroll
            for (int jp = 0; jp < 2; ++jp)
                store_row<NB>(p.states, p.dt_states,
                              b * p.sst_b + c * p.sst_c + h * p.sst_h + (int64_t)(prow + jp) * p.sst_p + NB * i16, sum[jp]);
        }
        if (FUSED) {
            float sc = __expf(last);
            if (HAS_SEQ) {
                const int32_t cur = sqb[(int64_t)(lim_end - 1) * p.ssq_l];
                if (cur != prev_id) sc = 0.f;
                prev_id = cur;
            }
#pragma unroll
            for (int jp = 0; jp < 2; ++jp) {
#pragma unroll
                for (int jn = 0; jn < NB; ++jn) st[jp][jn] = sc * st[jp][jn] + sum[jp][jn];
                if (c < p.C - 1)
                    store_row<NB>(p.out, p.dt_out,
                                  b * p.so_b + (c + 1) * p.so_c + h * p.so_h + (int64_t)(prow + jp) * p.so_p + NB * i16, st[jp]);
                else
                    store_row<NB>(p.fin, DT_F32, b * p.sf_b + h * p.sf_h + (int64_t)(prow + jp) * p.sf_p + NB * i16, st[jp]);
            }
        }
    }
}

static bool aligned(const void *ptr, size_t a) { return ((uintptr_t)ptr % a) == 0; }

bool mfma_supported(const Params &p)
{
    if (p.dt_in != DT_BF16) return false;
    if (p.headdim % 32 != 0) return false;
    if (p.dstate != 64 && p.dstate != 128) return false;
    if (p.Q != 128 && p.Q != 256) return false;
    const int nb = p.dstate / 16;
    if (!aligned(p.x, 4) || (p.sx_b | p.sx_l | p.sx_h) % 2) return false;
    if (!aligned(p.B, 2 * nb) || p.sB_b % nb || p.sB_l % nb || p.sB_g % nb) return false;
    auto ok16 = [](const void *q, int64_t a, int64_t b, int64_t c, int64_t d) {
        return q == nullptr || (aligned(q, 16) && a % 8 == 0 && b % 8 == 0 && c % 8 == 0 && d % 8 == 0);
    };
    if (!ok16(p.states, p.sst_b, p.sst_c, p.sst_h, p.sst_p)) return false;
    if (!ok16(p.out, p.so_b, p.so_c, p.so_h, p.so_p)) return false;
    if (!ok16(p.fin, p.sf_b, p.sf_h, p.sf_p, 0)) return false;
    return true;
}

template <int NB, int KS>
static hipError_t launch_nb_ks(const Params &p, bool fused, hipStream_t s)
{
    const int per_xcd = (p.n_items + 7) / 8;
    dim3 grid(per_xcd * 8), block(256);
    const bool seq = p.seq != nullptr;
    if (fused) {
        if (seq) hipLaunchKernelGGL((mfma_kernel<NB, KS, true, true>), grid, block, 0, s, p);
        else hipLaunchKernelGGL((mfma_kernel<NB, KS, false, true>), grid, block, 0, s, p);
    } else {
        if (seq) hipLaunchKernelGGL((mfma_kernel<NB, KS, true, false>), grid, block, 0, s, p);
        else hipLaunchKernelGGL((mfma_kernel<NB, KS, false, false>), grid, block, 0, s, p);
    }
    return hipGetLastError();
}

hipError_t launch_mfma(const Params &p_in, bool fused, hipStream_t s)
{
    Params p = p_in;
    const int n_pt = p.headdim / 32;
    p.n_items = fused ? p.batch * p.nheads * n_pt : p.batch * p.C * p.nheads * n_pt;
    if (p.n_items <= 0) return hipSuccess;
    const int nb = p.dstate / 16, ks = p.Q / 128;
    if (nb == 8 && ks == 2) return launch_nb_ks<8, 2>(p, fused, s);
    if (nb == 8 && ks == 1) return launch_nb_ks<8, 1>(p, fused, s);
    if (nb == 4 && ks == 2) return launch_nb_ks<4, 2>(p, fused, s);
    return launch_nb_ks<4, 1>(p, fused, s);
}

}  // namespace ssd
