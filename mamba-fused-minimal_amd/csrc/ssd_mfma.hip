// bf16 MFMA kernel for the SSD chunk-state contraction, optionally fused with the inter-chunk recurrence.
//
// Work decomposition (gfx950, 64-wide waves, v_mfma_f32_16x16x32_bf16):
//   * one workgroup owns a (batch, head, 32-row slice of headdim) x all of dstate state tile and, in fused mode,
//     walks the chunks of that unit serially, so the running state never leaves registers and no workgroup ever
//     waits for another one;
//   * inside a chunk the 4 contraction waves split the tokens (the contraction index): wave w contracts tokens
//     [w*Q/4, (w+1)*Q/4).  Each wave therefore streams its own rows of x and B straight from global memory into
//     MFMA operand registers -- no operand goes through LDS:
//       - lane (i = lane%16, kg = lane/16) loads, for the 8 consecutive tokens 8kg..8kg+7 of a 32-token step,
//         one dword of x (headdim rows 2i, 2i+1) and, per dstate half, HB consecutive bf16 of B;
//       - x is widened to fp32, multiplied by the per-token weight w_k and split into bf16 hi + bf16 lo, so that
//         the two MFMAs hi*B + lo*B carry ~16 mantissa bits of x*w (a single bf16 rounding of the scaled operand,
//         which is what the reference does, is not accurate enough for an fp32 comparison);
//       - the 2x2 16-bit transposes that turn "8 tokens x 2 values" into the token-contiguous MFMA operand
//         layout are one v_cvt_pk_bf16_f32 (x side, free with the rounding) or one v_perm_b32 (B side) per dword;
//       - MFMA tile (jp, half, jq) covers headdim rows {2i+jp} and dstate columns {half*N/2 + HB*i + jq}: the
//         row/column permutation makes every lane own HB consecutive dstate values of one row, so results leave
//         with 128-bit stores and each 16-lane group writes one contiguous 256-byte piece of a state row;
//   * the dstate halves are processed one after the other (all token steps of half 0, then of half 1), which
//     keeps only half of the accumulators and of the raw B rows live and lets three workgroups share a CU;
//   * after each half the four token-partial tiles are summed through LDS: wave w ends up owning the rows with
//     (row/2)%4 == w, applies s = exp(dA_chunk)*s + partial sum, and stores out / states;
//   * in fused mode an optional fifth wave computes nothing: it touches the x and B cache lines of the chunk two
//     ahead, so that the contraction waves (whose loads return in order and can only run a step or two ahead)
//     find them in L2.
//
// Reference semantics: kernels/ssd_chunk_state.py:97-173, kernels/ssd_state_passing.py:27-84,
// kernels/fused_globalbar.py:16-198 (same math, one launch).
#include "ssd_params.h"

namespace ssd {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

template <int HB> struct FVec;
template <> struct FVec<4> { typedef f32x4 type; };
template <> struct FVec<2> { typedef f32x2 type; };

__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi)
{
    bf16x2 v = {(__bf16)lo, (__bf16)hi};
    return __builtin_bit_cast(uint32_t, v);
}

// Workgroup barrier that only orders LDS traffic (global loads issued earlier stay in flight).
__device__ __forceinline__ void lds_barrier()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// Store HB consecutive state values of one row (fp32, bf16 or f16 destination) with a raw buffer store:
// scalar descriptor + scalar element offset `soff` + loop-invariant per-lane element offset `voff`.
template <int HB>
__device__ __forceinline__ void store_row(__amdgpu_buffer_rsrc_t rs, int dt, int voff, int soff, const float (&v)[HB])
{
    if (dt == DT_F32) {
        if constexpr (HB == 4) {
            const u32x4 q = {__builtin_bit_cast(uint32_t, v[0]), __builtin_bit_cast(uint32_t, v[1]),
                             __builtin_bit_cast(uint32_t, v[2]), __builtin_bit_cast(uint32_t, v[3])};
            __builtin_amdgcn_raw_buffer_store_b128(q, rs, 4 * voff, 4 * soff, 0);
        } else {
            const u32x2 q = {__builtin_bit_cast(uint32_t, v[0]), __builtin_bit_cast(uint32_t, v[1])};
            __builtin_amdgcn_raw_buffer_store_b64(q, rs, 4 * voff, 4 * soff, 0);
        }
    } else {
        uint32_t w[HB / 2];
#pragma unroll
        for (int u = 0; u < HB / 2; ++u) {
            if (dt == DT_BF16) {
                w[u] = pack_bf16(v[2 * u], v[2 * u + 1]);
            } else {
                typedef __attribute__((ext_vector_type(2))) _Float16 h2;
                h2 hv = {(_Float16)v[2 * u], (_Float16)v[2 * u + 1]};
                w[u] = __builtin_bit_cast(uint32_t, hv);
            }
        }
        if constexpr (HB == 4) {
            const u32x2 q = {w[0], w[1]};
            __builtin_amdgcn_raw_buffer_store_b64(q, rs, 2 * voff, 2 * soff, 0);
        } else {
            __builtin_amdgcn_raw_buffer_store_b32(w[0], rs, 2 * voff, 2 * soff, 0);
        }
    }
}

// Descriptor of one (headdim x dstate) state slice starting at element `first` of a tensor with `esize`-byte elements.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t slice_rsrc(void *base, int esize, int64_t first, int64_t extent_elems)
{
    const int64_t bytes = extent_elems * esize;
    return __builtin_amdgcn_make_buffer_rsrc((char *)base + first * esize, 0,
                                             (int)(bytes > 0x7fffffffLL ? 0x7fffffffLL : bytes), 0x00020000);
}

__device__ __forceinline__ int esize_of(int dt) { return dt == DT_F32 ? 4 : 2; }

// Token-split reduction through LDS.  Every wave rotates the headdim rows it feeds to the MFMA (see `rot` in the
// kernel) so that accumulator component r of wave w holds rows owned by wave (w + r) % 4: component 0 stays,
// components 1..3 go to the three other waves.  The code is the same for all waves; only addresses differ.
template <int HB>
__device__ __forceinline__ void exchange_write(const f32x4 (&acc)[2][HB], typename FVec<HB>::type *red, int wave, int lane)
{
#pragma unroll
    for (int r = 1; r < 4; ++r) {
        const int dst = (wave + r) & 3;
#pragma unroll
        for (int jp = 0; jp < 2; ++jp) {
            typename FVec<HB>::type v;
#pragma unroll
            for (int j = 0; j < HB; ++j) v[j] = acc[jp][j][r];
            red[((dst * 3 + (r - 1)) * 2 + jp) * 64 + lane] = v;
        }
    }
}

template <int HB>
__device__ __forceinline__ void exchange_read(const f32x4 (&acc)[2][HB], const typename FVec<HB>::type *red, int wave,
                                              int lane, float (&sum)[2][HB])
{
#pragma unroll
    for (int jp = 0; jp < 2; ++jp) {
        typename FVec<HB>::type t;
#pragma unroll
        for (int j = 0; j < HB; ++j) t[j] = acc[jp][j][0];
#pragma unroll
        for (int r = 1; r < 4; ++r)             // fixed order: own quarter, then the three others
            t += red[((wave * 3 + (r - 1)) * 2 + jp) * 64 + lane];
#pragma unroll
        for (int j = 0; j < HB; ++j) sum[jp][j] = t[j];
    }
}

constexpr int kPrefetchAhead = 2;   // chunks the fifth wave runs ahead of the contraction

// NB = dstate / 16 (4 or 8); KS = 32-token steps per wave per chunk (chunk_size = 128 * KS);
// PF = run the L2-prefetch wave (fused mode only; block = 320 threads instead of 256);
// ALL32 = initial states, states, out are all fp32 (or absent): element-type branches fold away.
template <int NB, int KS, bool HAS_SEQ, bool FUSED, bool PF, bool ALL32>
__global__ void __launch_bounds__(PF ? 320 : 256) __attribute__((amdgpu_waves_per_eu(3, 3))) mfma_kernel(const Params p)
{
    constexpr int HB = NB / 2;          // dstate columns per lane per half
    constexpr int HD = HB / 2;          // dwords of B per lane per row per half
    constexpr int QW = 32 * KS;
    typedef typename FVec<HB>::type fvec;
    __shared__ fvec red[2][12 * 2 * 64];                       // [half][(dst*3+slot)*2+jp][lane]
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
    const int dt_out = ALL32 ? (int)DT_F32 : p.dt_out, dt_states = ALL32 ? (int)DT_F32 : p.dt_states,
              dt_init = ALL32 ? (int)DT_F32 : p.dt_init;
    const int g = h / (p.nheads / p.ngroups);
    const int p0 = pt * 32;
    const float *dtb = p.dt + b * p.sdt_b + h * p.sdt_h;
    const float *dab = p.dacs + b * p.sda_b + h * p.sda_h;
    const int32_t *sqb = HAS_SEQ ? p.seq + b * p.ssq_b : nullptr;

    const char *xrow = (const char *)p.x + 2 * (b * p.sx_b + h * p.sx_h);
    const char *Brow = (const char *)p.B + 2 * (b * p.sB_b + g * p.sB_g);
    const int64_t xrb = 2 * p.sx_l, Brb = 2 * p.sB_l;            // row pitch in bytes

    if (PF && wave == 4) {
        // L2-prefetch wave: one dword per 128-byte line of the x rows (this row slice) and B rows of chunk c+2.
        // It takes part in the two workgroup barriers of every chunk, which paces it.  The loaded values are
        // ordinary compiler-visible loads folded into a dummy one chunk later, so the wave never waits on a
        // young load and no register is rewritten while a load into it is still in flight.
        constexpr int NXL = 2 * KS;                    // x: Q tokens, one 64-lane load covers 64 tokens
        constexpr int NBL = 2 * KS * (NB / 4);         // B: (2 * dstate / 128) lines per token
        constexpr int LINES = NB / 4;
        uint32_t v[NXL + NBL];
#pragma unroll
        for (int i = 0; i < NXL + NBL; ++i) v[i] = 0;
        uint32_t fold = 0;
        for (int c = c_begin; c < c_end; ++c) {
#pragma unroll
            for (int i = 0; i < NXL + NBL; ++i) fold ^= v[i];
            asm volatile("" ::"v"(fold));
            const int cp = c + kPrefetchAhead;
            if (cp < c_end) {
                const int t0 = cp * Q;
#pragma unroll
                for (int i = 0; i < NXL; ++i) {
                    const int t = t0 + 64 * i + lane;
                    v[i] = (t < L) ? *(const uint32_t *)(xrow + (int64_t)t * xrb + 2 * p0) : 0u;
                }
#pragma unroll
                for (int i = 0; i < NBL; ++i) {
                    const int e = 64 * i + lane;
                    const int t = t0 + e / LINES, piece = e % LINES;
                    v[NXL + i] = (t < L) ? *(const uint32_t *)(Brow + (int64_t)t * Brb + 128 * piece) : 0u;
                }
            }
            lds_barrier();
            lds_barrier();
        }
        return;
    }

    // x and B are read with raw buffer loads: a scalar resource descriptor per chunk (base = first token of the
    // chunk for this batch/head or group, extent = the tokens that exist), a loop-invariant 32-bit per-lane byte
    // offset and a scalar row offset.  No vector address arithmetic in the main loop, and rows past the end of a
    // ragged last chunk read as zero instead of being fetched.
    const int lane_tok = wave * QW + 8 * kg;                     // first token of this lane within step 0 of a chunk
    // MFMA row i of this wave is headdim row pair rot(i) = 4*(i/4) + (i%4 + wave)%4 (see exchange_write)
    const int rot = (i16 & ~3) | ((i16 + wave) & 3);
    const int xlane = (int)(lane_tok * xrb) + 2 * (p0 + 2 * rot);
    const int Blane = (int)(lane_tok * Brb) + 2 * HB * i16;
    // Prefetches are issued unconditionally -- a branch around a load makes the compiler wait for *all* loads
    // before the next use -- so a chunk past the end of this workgroup's range gets an empty extent instead:
    // every lane is then out of range and nothing is fetched.
    auto chunk_rsrc = [&](const char *base, int64_t pitch, int c) {
        int64_t extent = (int64_t)(L - c * Q) * pitch;           // bytes from the chunk's first token to the end
        extent = extent > 0x7fffffffLL ? 0x7fffffffLL : extent;
        const int cc = c < c_end ? c : c_begin;                  // keep the base inside the tensor
        return __builtin_amdgcn_make_buffer_rsrc((void *)(base + (int64_t)cc * Q * pitch), 0,
                                                 c < c_end ? (int)extent : 0, 0x00020000);
    };
    // x rows of one chunk (all KS steps of this wave)
    auto load_x = [&](int c, uint32_t (&xo)[KS][8]) {
        const auto rs = chunk_rsrc(xrow, xrb, c);
#pragma unroll
        for (int s = 0; s < KS; ++s)
#pragma unroll
            for (int j = 0; j < 8; ++j)
                xo[s][j] = __builtin_amdgcn_raw_buffer_load_b32(rs, xlane, (int)((32 * s + j) * xrb), 0);
    };
    // B rows of one (chunk, half, step) unit; units are numbered u = ((c - c_begin) * 2 + half) * KS + s
    auto load_B = [&](int u, uint32_t (&bo)[8][HD]) {
        const int s = u % KS, half = (u / KS) & 1, c = c_begin + u / (2 * KS);
        const auto rs = chunk_rsrc(Brow, Brb, c);
        const int col = half * p.dstate;                         // byte offset of the half: (N/2) * 2
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            if constexpr (HD == 2) {
                const u32x2 v = __builtin_amdgcn_raw_buffer_load_b64(rs, Blane, (int)((32 * s + j) * Brb) + col, 0);
                bo[j][0] = v.x; bo[j][1] = v.y;
            } else {
                bo[j][0] = __builtin_amdgcn_raw_buffer_load_b32(rs, Blane, (int)((32 * s + j) * Brb) + col, 0);
            }
        }
    };

    // Per-chunk scalars and per-token decay inputs, fetched one chunk ahead of their use.
    struct Meta { float dtv, cs, last; int32_t id, id_last; };
    auto load_meta = [&](int c) {
        Meta m;
        const int k = wave * QW + (lane & (QW - 1));
        m.dtv = dtb[c * p.sdt_c + k * p.sdt_k];
        m.cs = dab[c * p.sda_c + k * p.sda_k];
        m.last = dab[c * p.sda_c + (int64_t)(Q - 1) * p.sda_k];
        m.id = 0; m.id_last = 0;
        if (HAS_SEQ) {
            m.id = sqb[(int64_t)min(c * Q + k, L - 1) * p.ssq_l];
            m.id_last = sqb[(int64_t)(min((c + 1) * Q, L) - 1) * p.ssq_l];
        }
        return m;
    };

    uint32_t xraw[KS][8], bA[8][HD], bB[8][HD];
    Meta mcur = load_meta(c_begin), mnext = mcur;
    load_x(c_begin, xraw);
    load_B(0, bA);

    // owner rows of this lane after the token reduction
    const int prow = p0 + 2 * (4 * kg + wave);
    const int ncol = HB * i16;                                   // + half * N/2
    // per-lane element offsets inside one (headdim x dstate) slice of out / states / final, and the slice extents
    const int vo_out = prow * (int)p.so_p + ncol, vo_st = prow * (int)p.sst_p + ncol, vo_fin = prow * (int)p.sf_p + ncol;
    const int64_t slice_out = (int64_t)(p.headdim - 1) * p.so_p + p.dstate;
    const int64_t slice_st = (int64_t)(p.headdim - 1) * p.sst_p + p.dstate;
    const int64_t slice_fin = (int64_t)(p.headdim - 1) * p.sf_p + p.dstate;
    float st[2][2][HB];                                          // [half][jp][jq]
    if (FUSED) {
#pragma unroll
        for (int half = 0; half < 2; ++half)
#pragma unroll
            for (int jp = 0; jp < 2; ++jp) {
                const int n0 = half * (p.dstate >> 1) + ncol;
                if (p.init) {
                    const int64_t off = b * p.sin_b + h * p.sin_h + (int64_t)(prow + jp) * p.sin_p + n0;
                    if (dt_init == DT_F32) {
                        const fvec q = *(const fvec *)((const float *)p.init + off);
#pragma unroll
                        for (int j = 0; j < HB; ++j) st[half][jp][j] = q[j];
                    } else {
#pragma unroll
                        for (int j = 0; j < HB; ++j) st[half][jp][j] = load_as_f32(p.init, off + j, dt_init);
                    }
                } else {
#pragma unroll
                    for (int j = 0; j < HB; ++j) st[half][jp][j] = 0.f;
                }
                // out[:, 0] = initial state (kernels/ssd_state_passing.py:66)
                store_row<HB>(slice_rsrc(p.out, esize_of(dt_out), b * p.so_b + h * p.so_h, slice_out), dt_out,
                              vo_out, jp * (int)p.so_p + half * (p.dstate >> 1), st[half][jp]);
            }
    }
    int32_t prev_id = 0;
    int unit = 0;

    // MFMAs of one (half, step) unit: bc holds the unit's raw B rows, bn receives the next unit's.
    auto mma_unit = [&](f32x4 (&acc)[2][HB], const bf16x8 (&Ahi)[2], const bf16x8 (&Alo)[2],
                        uint32_t (&bc)[8][HD], uint32_t (&bn)[8][HD]) {
        load_B(unit + 1, bn);
        __builtin_amdgcn_sched_barrier(0);       // keep the prefetch ahead of this unit's waits
#pragma unroll
        for (int jq = 0; jq < HB; ++jq) {
            const uint32_t sel = (jq & 1) ? 0x07060302u : 0x05040100u;
            u32x4 f;
            f.x = __builtin_amdgcn_perm(bc[1][jq >> 1], bc[0][jq >> 1], sel);
            f.y = __builtin_amdgcn_perm(bc[3][jq >> 1], bc[2][jq >> 1], sel);
            f.z = __builtin_amdgcn_perm(bc[5][jq >> 1], bc[4][jq >> 1], sel);
            f.w = __builtin_amdgcn_perm(bc[7][jq >> 1], bc[6][jq >> 1], sel);
            const bf16x8 Bf = __builtin_bit_cast(bf16x8, f);
#pragma unroll
            for (int jp = 0; jp < 2; ++jp) {
                acc[jp][jq] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(Ahi[jp], Bf, acc[jp][jq], 0, 0, 0);
                acc[jp][jq] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(Alo[jp], Bf, acc[jp][jq], 0, 0, 0);
            }
        }
        ++unit;
    };

    for (int c = c_begin; c < c_end; ++c) {
        mnext = load_meta(min(c + 1, c_end - 1));

        // ---- per-token weights of this wave's token quarter (kernels/ssd_chunk_state.py:134-156)
        {
            float e = mcur.last - mcur.cs;
            if (p.clamp) e = fminf(e, 0.f);
            float wv = __expf(e) * mcur.dtv;
            if (c * Q + wave * QW + (lane & (QW - 1)) >= L) wv = 0.f;
            if (HAS_SEQ && mcur.id != mcur.id_last) wv = 0.f;
            wbuf[wave * QW + (lane & (QW - 1))] = wv;
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront", "local");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront", "local");

        // ---- x * w in fp32, split into bf16 hi + bf16 lo, packed along the token axis, for every step of the chunk
        bf16x8 Ahi[KS][2], Alo[KS][2];
#pragma unroll
        for (int s = 0; s < KS; ++s) {
            const f32x4 wlo = *(const f32x4 *)&wbuf[wave * QW + 32 * s + 8 * kg];
            const f32x4 whi = *(const f32x4 *)&wbuf[wave * QW + 32 * s + 8 * kg + 4];
            const float wv[8] = {wlo.x, wlo.y, wlo.z, wlo.w, whi.x, whi.y, whi.z, whi.w};
            uint32_t ahi[2][4], alo[2][4];
#pragma unroll
            for (int q = 0; q < 4; ++q)
#pragma unroll
                for (int jp = 0; jp < 2; ++jp) {
                    const uint32_t r0 = xraw[s][2 * q], r1_ = xraw[s][2 * q + 1];
                    const float v0 = __builtin_bit_cast(float, jp ? (r0 & 0xffff0000u) : (r0 << 16)) * wv[2 * q];
                    const float v1 = __builtin_bit_cast(float, jp ? (r1_ & 0xffff0000u) : (r1_ << 16)) * wv[2 * q + 1];
                    const uint32_t hp = pack_bf16(v0, v1);
                    const float h0 = __builtin_bit_cast(float, hp << 16);
                    const float h1 = __builtin_bit_cast(float, hp & 0xffff0000u);
                    ahi[jp][q] = hp;
                    alo[jp][q] = pack_bf16(v0 - h0, v1 - h1);
                }
#pragma unroll
            for (int jp = 0; jp < 2; ++jp) {
                Ahi[s][jp] = __builtin_bit_cast(bf16x8, (u32x4){ahi[jp][0], ahi[jp][1], ahi[jp][2], ahi[jp][3]});
                Alo[s][jp] = __builtin_bit_cast(bf16x8, (u32x4){alo[jp][0], alo[jp][1], alo[jp][2], alo[jp][3]});
            }
        }
        // the raw x registers are free again: fetch the next chunk's rows, a whole chunk ahead of their use
        load_x(c + 1, xraw);

        float sc = 0.f;
        if (FUSED) {
            sc = __expf(mcur.last);
            if (HAS_SEQ) {
                if (mcur.id_last != prev_id) sc = 0.f;
                prev_id = mcur.id_last;
            }
        }

#pragma unroll
        for (int half = 0; half < 2; ++half) {
            f32x4 acc[2][HB];
#pragma unroll
            for (int jp = 0; jp < 2; ++jp)
#pragma unroll
                for (int jq = 0; jq < HB; ++jq) acc[jp][jq] = (f32x4){0.f, 0.f, 0.f, 0.f};

            // 2*KS units per chunk: the raw B buffers alternate with a fixed parity per position
#pragma unroll
            for (int s = 0; s < KS; ++s) {
                if (((half * KS + s) & 1) == 0) mma_unit(acc, Ahi[s], Alo[s], bA, bB);
                else mma_unit(acc, Ahi[s], Alo[s], bB, bA);
            }

            // ---- sum the four token quarters of this half.  One barrier per half is enough: the write to
            // red[half] of the next chunk is separated from this chunk's reads by the other half's barrier.
            fvec *rd = red[half];
            exchange_write<HB>(acc, rd, wave, lane);
            lds_barrier();
            float sum[2][HB];
            exchange_read<HB>(acc, rd, wave, lane, sum);

            // ---- per-chunk states (side output) and the recurrence (kernels/ssd_state_passing.py:69-84)
            const int hcol = half * (p.dstate >> 1);
            if (p.states) {
                const auto rs = slice_rsrc(p.states, esize_of(dt_states), b * p.sst_b + c * p.sst_c + h * p.sst_h, slice_st);
#pragma unroll
                for (int jp = 0; jp < 2; ++jp)
                    store_row<HB>(rs, dt_states, vo_st, jp * (int)p.sst_p + hcol, sum[jp]);
            }
            if (FUSED) {
#pragma unroll
                for (int jp = 0; jp < 2; ++jp) {
#pragma unroll
                    for (int j = 0; j < HB; ++j) st[half][jp][j] = sc * st[half][jp][j] + sum[jp][j];
                    if (c < p.C - 1)
                        store_row<HB>(slice_rsrc(p.out, esize_of(dt_out), b * p.so_b + (c + 1) * p.so_c + h * p.so_h, slice_out),
                                      dt_out, vo_out, jp * (int)p.so_p + hcol, st[half][jp]);
                    else
                        store_row<HB>(slice_rsrc(p.fin, 4, b * p.sf_b + h * p.sf_h, slice_fin), DT_F32, vo_fin,
                                      jp * (int)p.sf_p + hcol, st[half][jp]);
                }
            }
        }
        mcur = mnext;
    }
}

static bool aligned(const void *ptr, size_t a) { return ((uintptr_t)ptr % a) == 0; }

bool mfma_supported(const Params &p)
{
    if (p.dt_in != DT_BF16) return false;
    if (p.headdim % 32 != 0) return false;
    if (p.dstate != 64 && p.dstate != 128) return false;
    if (p.Q != 128 && p.Q != 256) return false;
    const int hb = p.dstate / 32;                       // bf16 per lane per half
    if (!aligned(p.x, 4) || (p.sx_b | p.sx_l | p.sx_h) % 2) return false;
    if (!aligned(p.B, 2 * hb) || p.sB_b % hb || p.sB_l % hb || p.sB_g % hb) return false;
    // buffer addressing: per-lane offsets within a chunk must fit 31 bits
    if ((int64_t)p.Q * 2 * p.sx_l >= (1LL << 31) || (int64_t)p.Q * 2 * p.sB_l >= (1LL << 31)) return false;
    auto ok16 = [](const void *q, int64_t a, int64_t b, int64_t c, int64_t d) {
        return q == nullptr || (aligned(q, 16) && a % 4 == 0 && b % 4 == 0 && c % 4 == 0 && d % 4 == 0);
    };
    if (!ok16(p.states, p.sst_b, p.sst_c, p.sst_h, p.sst_p)) return false;
    if (!ok16(p.out, p.so_b, p.so_c, p.so_h, p.so_p)) return false;
    if (!ok16(p.fin, p.sf_b, p.sf_h, p.sf_p, 0)) return false;
    if (!ok16(p.init, p.sin_b, p.sin_h, p.sin_p, 0)) return false;
    return true;
}

static int g_prefetch_wave = 0;     // fused launches: 1 = run the fifth (L2-prefetch) wave
void set_prefetch_wave(int on) { g_prefetch_wave = on; }

template <int NB, int KS, bool SEQ, bool FUSED, bool PF>
static void launch_one(const Params &p, dim3 grid, dim3 block, hipStream_t s)
{
    const bool all32 = (!p.out || p.dt_out == DT_F32) && (!p.states || p.dt_states == DT_F32) &&
                       (!p.init || p.dt_init == DT_F32);
    if (all32) hipLaunchKernelGGL((mfma_kernel<NB, KS, SEQ, FUSED, PF, true>), grid, block, 0, s, p);
    else hipLaunchKernelGGL((mfma_kernel<NB, KS, SEQ, FUSED, PF, false>), grid, block, 0, s, p);
}

template <int NB, int KS>
static hipError_t launch_nb_ks(const Params &p, bool fused, hipStream_t s)
{
    const int per_xcd = (p.n_items + 7) / 8;
    const bool seq = p.seq != nullptr;
    const bool pf = fused && g_prefetch_wave && p.C > kPrefetchAhead;
    dim3 grid(per_xcd * 8), block(pf ? 320 : 256);
    if (fused && pf) {
        if (seq) launch_one<NB, KS, true, true, true>(p, grid, block, s);
        else launch_one<NB, KS, false, true, true>(p, grid, block, s);
    } else if (fused) {
        if (seq) launch_one<NB, KS, true, true, false>(p, grid, block, s);
        else launch_one<NB, KS, false, true, false>(p, grid, block, s);
    } else {
        if (seq) launch_one<NB, KS, true, false, false>(p, grid, block, s);
        else launch_one<NB, KS, false, false, false>(p, grid, block, s);
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
