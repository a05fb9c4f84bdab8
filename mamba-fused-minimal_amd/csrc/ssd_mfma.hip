// bf16 MFMA kernel for the SSD chunk-state contraction, optionally fused with the inter-chunk recurrence.
//
// Work decomposition (gfx950, 64-wide waves, v_mfma_f32_16x16x32_bf16):
//   * one workgroup (4 waves) owns a (batch, head, 32-row slice of headdim) x all of dstate state tile and, in
//     fused mode, walks the chunks of that unit serially, so the running state never leaves registers and no
//     workgroup ever waits for another one;
//   * inside a chunk the 4 waves split the tokens (the contraction index): wave w contracts tokens
//     [w*Q/4, (w+1)*Q/4) in steps of 32.  Each wave streams its own rows of x and B:
//       - B goes straight from global memory into MFMA operand registers: lane (i = lane%16, kg = lane/16)
//         loads, for the 8 consecutive tokens 8kg..8kg+7 of a step, NB consecutive bf16 (16 bytes for dstate
//         128); one v_perm_b32 per dword turns "8 tokens x 2 columns" into the token-contiguous operand layout;
//       - x is fetched with 16-byte loads too (4 lanes per token row of the slice, 16 rows per instruction --
//         the memory pipeline is limited by the number of vector-memory instructions, not by their width),
//         staged in a wave-private LDS area and read back in the operand layout (8 tokens x 2 headdim rows per
//         lane); it is then widened to fp32, multiplied by the per-token weight w_k and split into bf16 hi +
//         bf16 lo, so that the two MFMAs hi*B + lo*B carry ~16 mantissa bits of x*w (a single bf16 rounding of
//         the scaled operand, which is what the reference does, is not accurate enough for an fp32 comparison);
//       - MFMA tile (jp, jn) covers headdim rows {2i+jp} and dstate columns {NB*i+jn}: the row/column
//         permutation makes every lane own NB consecutive dstate values of one row, so results leave with
//         128-bit stores;
//       - all loads are raw buffer loads (scalar descriptor + loop-invariant lane offset + scalar row offset)
//         issued two steps (B) or one chunk (x, dt, dA_cumsum) ahead of their use;
//   * the four token-partial tiles are summed through LDS: wave w ends up owning the rows with
//     (row/2)%4 == w, applies s = exp(dA_chunk)*s + partial sum, and stores out / states.
//
// Reference semantics: kernels/ssd_chunk_state.py:97-173, kernels/ssd_state_passing.py:27-84,
// kernels/fused_globalbar.py:16-198 (same math, one launch).
#include "ssd_tile.h"

namespace ssd {

using namespace tile;      // register types, pack_bf16 (ssd_tile.h)

template <int HB> struct FVec;
template <> struct FVec<4> { typedef f32x4 type; };
template <> struct FVec<2> { typedef f32x2 type; };

// Workgroup barrier that only orders the LDS reads and writes made by ds instructions: global loads issued
// earlier -- including the ones that deposit x rows in LDS, which a release fence would wait for -- stay in
// flight.  s_waitcnt lgkmcnt(0) (vmcnt and expcnt fields left at their maxima) completes this wave's ds
// operations; the barrier intrinsic keeps the compiler from moving memory operations across it.
__device__ __forceinline__ void lds_barrier()
{
    __builtin_amdgcn_s_waitcnt(0xc07f);
    __builtin_amdgcn_s_barrier();
}

// Store HB consecutive state values of one row (fp32, bf16 or f16 destination) with a raw buffer store:
// scalar descriptor + scalar element offset `soff` + loop-invariant per-lane element offset `voff`.
// The data registers of a wide store are read out over several cycles after issue; when the compiler reuses the
// register tuple for the next store and writes it in the very next instruction, some lanes were seen to store the
// new value.  Each store is therefore followed by wait states that depend on its data registers.
template <int HB>
__device__ __forceinline__ void store_row(__amdgpu_buffer_rsrc_t rs, int dt, int voff, int soff, const float (&v)[HB])
{
    if (dt == DT_F32) {
        if constexpr (HB == 4) {
            const u32x4 q = {__builtin_bit_cast(uint32_t, v[0]), __builtin_bit_cast(uint32_t, v[1]),
                             __builtin_bit_cast(uint32_t, v[2]), __builtin_bit_cast(uint32_t, v[3])};
            __builtin_amdgcn_raw_buffer_store_b128(q, rs, 4 * voff, 4 * soff, 0);
            asm volatile("s_nop 3" ::"v"(q) : "memory");
        } else {
            const u32x2 q = {__builtin_bit_cast(uint32_t, v[0]), __builtin_bit_cast(uint32_t, v[1])};
            __builtin_amdgcn_raw_buffer_store_b64(q, rs, 4 * voff, 4 * soff, 0);
            asm volatile("s_nop 3" ::"v"(q) : "memory");
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
            asm volatile("s_nop 3" ::"v"(q) : "memory");
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

// Token-split reduction through LDS.  WV waves split the tokens of a chunk.  Every wave rotates the headdim rows it
// feeds to the MFMA (see `rot` in the kernel) so that accumulator component r = q*WV + d of wave w holds rows owned
// by wave (w + d) % WV: components with d == 0 stay, the others go to the WV-1 other waves, where they add to that
// wave's component q*WV.  The code is the same for all waves; only addresses differ.
// Layout of `red`: [destination wave][d-1][q][jp][unit][lane] of 16-byte units.
template <int NB, int WV>
__device__ __forceinline__ void exchange_write(const f32x4 (&acc)[2][NB], f32x4 *red, int wave, int lane)
{
    constexpr int NU = NB / 4, NOWN = 4 / WV;
#pragma unroll
    for (int d = 1; d < WV; ++d) {
        const int dst = (wave + d) & (WV - 1);
#pragma unroll
        for (int q = 0; q < NOWN; ++q)
#pragma unroll
            for (int jp = 0; jp < 2; ++jp)
#pragma unroll
                for (int u = 0; u < NU; ++u) {
                    const int r = q * WV + d;
                    const f32x4 v = {acc[jp][4 * u][r], acc[jp][4 * u + 1][r], acc[jp][4 * u + 2][r], acc[jp][4 * u + 3][r]};
                    red[((((dst * (WV - 1) + (d - 1)) * NOWN + q) * 2 + jp) * NU + u) * 64 + lane] = v;
                }
    }
}

template <int NB, int WV>
__device__ __forceinline__ void exchange_read(const f32x4 (&acc)[2][NB], const f32x4 *red, int wave, int lane,
                                              float (&sum)[4 / WV][2][NB])
{
    constexpr int NU = NB / 4, NOWN = 4 / WV;
    f32x4 part[WV - 1][NOWN][2][NU];    // all reads in flight before the first add
#pragma unroll
    for (int d = 1; d < WV; ++d)
#pragma unroll
        for (int q = 0; q < NOWN; ++q)
#pragma unroll
            for (int jp = 0; jp < 2; ++jp)
#pragma unroll
                for (int u = 0; u < NU; ++u)
                    part[d - 1][q][jp][u] = red[((((wave * (WV - 1) + (d - 1)) * NOWN + q) * 2 + jp) * NU + u) * 64 + lane];
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int q = 0; q < NOWN; ++q)
#pragma unroll
        for (int jp = 0; jp < 2; ++jp)
#pragma unroll
            for (int u = 0; u < NU; ++u) {
                const int r = q * WV;
                f32x4 t = {acc[jp][4 * u][r], acc[jp][4 * u + 1][r], acc[jp][4 * u + 2][r], acc[jp][4 * u + 3][r]};
#pragma unroll
                for (int d = 1; d < WV; ++d) t += part[d - 1][q][jp][u];   // fixed order: own part, then the others
                sum[q][jp][4 * u] = t.x; sum[q][jp][4 * u + 1] = t.y; sum[q][jp][4 * u + 2] = t.z; sum[q][jp][4 * u + 3] = t.w;
            }
}

// With two waves per tile the running state of the fused kernel lives in LDS (32 values per lane would not fit
// the register file next to the accumulators and the three B buffers); with four waves it stays in registers (16
// values per lane; the 16 KB would push the workgroup past half of the 160 KB of a compute unit).
template <int WV> constexpr bool state_in_lds() { return WV == 2; }

template <int NB, int WV> constexpr int exchange_bytes() { return WV * (WV - 1) * (4 / WV) * 2 * (NB / 4) * 64 * 16; }

template <int NB, int KS, int WV, bool FUSED> constexpr int lds_bytes()
{
    return exchange_bytes<NB, WV>()                               // token-split exchange
           + WV * 32 * KS * 64                                    // x rows, one area per wave
           + WV * 32 * KS * 4                                     // per-token weights
           + (FUSED && state_in_lds<WV>() ? 32 * NB * 16 * 4 : 0);   // running state of the tile
}

// NB = dstate / 16 (4 or 8); WV = waves per workgroup = token split (2 or 4); KS = 32-token steps per wave per
// chunk (chunk_size = 32 * KS * WV); ALL32 = initial states, states, out are all fp32 (or absent): element-type
// branches fold away.
template <int NB, int KS, int WV, bool HAS_SEQ, bool FUSED, bool ALL32>
__global__ void __launch_bounds__(64 * WV, 2) mfma_kernel(const Params p)
{
    constexpr int NBD = NB / 2;         // dwords of B per lane per row
    constexpr int NU = NB / 4;          // 128-bit units per state row per lane
    constexpr int QW = 32 * KS;         // tokens per wave per chunk
    constexpr int NOWN = 4 / WV;        // accumulator components (MFMA row groups) a wave owns after the reduction
    constexpr int TPL = QW > 64 ? QW / 64 : 1;      // tokens per lane when the wave's weights are computed
    extern __shared__ __attribute__((aligned(16))) char lds_raw[];
    char *xst_all = lds_raw;                                          // x rows: the first 8 or 16 KB
    float *wbuf = (float *)(xst_all + WV * QW * 64);
    f32x4 *red = (f32x4 *)(xst_all + WV * QW * 68);
    constexpr bool ST_LDS = FUSED && state_in_lds<WV>();

    const int tid = threadIdx.x, lane = tid & 63, i16 = lane & 15, kg = lane >> 4;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // running state in LDS: [wave][owned component q][jp][unit] of 64 lanes x 16 bytes, lane-private
    f32x4 *stl = (f32x4 *)((char *)red + exchange_bytes<NB, WV>()) + wave * NOWN * 2 * NU * 64 + lane;

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

    // x and B are read with raw buffer loads: a scalar resource descriptor per chunk (base = first token of the
    // chunk for this batch/head or group, extent = the tokens that exist), a loop-invariant 32-bit per-lane byte
    // offset and a scalar row offset.  No vector address arithmetic in the main loop, and rows past the end of a
    // ragged last chunk read as zero instead of being fetched.  Prefetches are issued unconditionally -- a
    // branch around a load makes the compiler wait for *all* loads before the next use -- so a chunk past the
    // end of this workgroup's range gets an empty extent instead: every lane is out of range, nothing is fetched.
    const char *xrow = (const char *)p.x + 2 * (b * p.sx_b + h * p.sx_h);
    const char *Brow = (const char *)p.B + 2 * (b * p.sB_b + g * p.sB_g);
    const int64_t xrb = 2 * p.sx_l, Brb = 2 * p.sB_l;            // row pitch in bytes
    auto chunk_rsrc = [&](const char *base, int64_t pitch, int c) {
        int64_t extent = (int64_t)(L - c * Q) * pitch;           // bytes from the chunk's first token to the end
        extent = extent > 0x7fffffffLL ? 0x7fffffffLL : extent;
        const int cc = c < c_end ? c : c_begin;                  // keep the base inside the tensor
        return __builtin_amdgcn_make_buffer_rsrc((void *)(base + (int64_t)cc * Q * pitch), 0,
                                                 c < c_end ? (int)extent : 0, 0x00020000);
    };

    // B: lane (i16, kg) reads NB consecutive columns of the 8 tokens 8kg..8kg+7 of a step
    const int Blane = (int)((wave * QW + 8 * kg) * Brb) + 2 * NB * i16;
    auto load_B_row = [&](int gstep, int j, uint32_t (&bo)[NBD]) {      // gstep = (c - c_begin) * KS + s
        const int c = c_begin + gstep / KS, s = gstep % KS;
        const auto rs = chunk_rsrc(Brow, Brb, c);
        if constexpr (NBD == 4) {
            const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(rs, Blane, (int)((32 * s + j) * Brb), 0);
            bo[0] = v.x; bo[1] = v.y; bo[2] = v.z; bo[3] = v.w;
        } else {
            const u32x2 v = __builtin_amdgcn_raw_buffer_load_b64(rs, Blane, (int)((32 * s + j) * Brb), 0);
            bo[0] = v.x; bo[1] = v.y;
        }
    };
    auto load_B = [&](int gstep, uint32_t (&bo)[8][NBD]) {
#pragma unroll
        for (int j = 0; j < 8; ++j) load_B_row(gstep, j, bo[j]);
    };
    // x goes from global memory straight into a wave-private LDS area (buffer load with LDS destination:
    // lane l deposits its 16 bytes at byte 16*l of a 1 KB block).  Two instructions cover the 32 token rows of a
    // step; 4 lanes fetch one 64-byte row of the slice.  Which row a lane fetches is chosen so that the operand
    // reads below are free of bank conflicts: instruction i puts token 8*kg + 4*i + m of the step at row slot
    // 4*m + kg, so the four kg groups of a read hit four different 64-byte bank groups.
    // MFMA row i of this wave is headdim row pair rot(i) = WV*(i/WV) + (i%WV + wave)%WV (see exchange_write).
    char *xst = xst_all + wave * QW * 64;
    const int xlane = (int)((wave * QW + 8 * ((lane >> 2) & 3) + (lane >> 4)) * xrb) + 2 * p0 + 16 * (lane & 3);
    auto load_x = [&](int c, int s, int i) {     // tokens 8*kg + 4*i + (0..3) of step s of chunk c
        const auto rs = chunk_rsrc(xrow, xrb, c);
#if defined(__HIP_DEVICE_COMPILE__)      // the LDS address space does not exist in the host pass
        typedef __attribute__((address_space(3))) void *lds_ptr;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lds_ptr)(xst + (2 * s + i) * 1024), 16, xlane,
                                                 (int)((32 * s + 4 * i) * xrb), 0, 0);
#else
        (void)rs; (void)s; (void)i; (void)xlane;
#endif
    };
    const int rot = (i16 & ~(WV - 1)) | ((i16 + wave) & (WV - 1));
    const int xst_rd = 64 * kg + 4 * rot;         // + 1024 * (2*s + j/4) + 256 * (j%4) for token j of step s

    // Per-chunk scalars and per-token decay inputs, fetched one chunk ahead of their use.
    // Lane l looks after tokens TPL*l .. TPL*l + TPL-1 of the wave's share (lanes repeat when the share is < 64).
    struct Meta { float dtv[TPL], cs[TPL], last; int32_t id[TPL], id_last; };
    const int ktok = wave * QW + ((lane * TPL) & (QW - 1));
    auto load_meta = [&](int c) {
        Meta m;
#pragma unroll
        for (int t = 0; t < TPL; ++t) {
            m.dtv[t] = dtb[c * p.sdt_c + (ktok + t) * p.sdt_k];
            m.cs[t] = dab[c * p.sda_c + (ktok + t) * p.sda_k];
            m.id[t] = 0;
        }
        m.last = dab[c * p.sda_c + (int64_t)(Q - 1) * p.sda_k];
        m.id_last = 0;
        if (HAS_SEQ) {
#pragma unroll
            for (int t = 0; t < TPL; ++t) m.id[t] = sqb[(int64_t)min(c * Q + ktok + t, L - 1) * p.ssq_l];
            m.id_last = sqb[(int64_t)(min((c + 1) * Q, L) - 1) * p.ssq_l];
        }
        return m;
    };

    uint32_t bX[8][NBD], bY[8][NBD], bZ[8][NBD];
    Meta mcur = load_meta(c_begin), mnext = mcur;
    // Rows past the end of the sequence are not fetched and may leave their LDS slots untouched; their weight
    // is zero, so the slots only have to hold finite numbers.
#pragma unroll
    for (int i = 0; i < 2 * KS; ++i) *(u32x4 *)(xst + i * 1024 + 16 * lane) = (u32x4){0u, 0u, 0u, 0u};
    __builtin_amdgcn_s_waitcnt(0xc07f);          // lgkmcnt(0): the zeros are in place before any row lands
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int s = 0; s < KS; ++s) { load_x(c_begin, s, 0); load_x(c_begin, s, 1); }
    __builtin_amdgcn_sched_barrier(0);           // the 16 B row loads below stay behind the x requests
    load_B(0, bX);
    load_B(1, bY);
    __builtin_amdgcn_s_waitcnt((16 & 15) | (7 << 4) | (15 << 8) | ((16 >> 4) << 14));   // vmcnt(16): x rows are in

    // Owner rows of this lane after the token reduction: owned component q covers headdim rows prow + 2*WV*q + jp.
    // Element offsets inside one (headdim x dstate) slice.
    const int prow = p0 + 2 * (4 * kg + wave);
    const int ncol = NB * i16;
    const int vo_out = prow * (int)p.so_p + ncol, vo_st = prow * (int)p.sst_p + ncol, vo_fin = prow * (int)p.sf_p + ncol;
    const int64_t slice_out = (int64_t)(p.headdim - 1) * p.so_p + p.dstate;
    const int64_t slice_st = (int64_t)(p.headdim - 1) * p.sst_p + p.dstate;
    const int64_t slice_fin = (int64_t)(p.headdim - 1) * p.sf_p + p.dstate;
    auto store_tile_row = [&](__amdgpu_buffer_rsrc_t rs, int dt, int voff, int soff, const float (&v)[NB]) {
#pragma unroll
        for (int u = 0; u < NU; ++u) {
            const float q[4] = {v[4 * u], v[4 * u + 1], v[4 * u + 2], v[4 * u + 3]};
            store_row<4>(rs, dt, voff, soff + 4 * u, q);
        }
    };

    float st[ST_LDS ? 1 : NOWN][2][NB];
    if (ST_LDS) {
        // out[:, 0] = initial state (kernels/ssd_state_passing.py:66), and the state's home in LDS
        const auto rs0 = slice_rsrc(p.out, esize_of(dt_out), b * p.so_b + c_begin * p.so_c + h * p.so_h, slice_out);
#pragma unroll
        for (int q = 0; q < NOWN; ++q)
#pragma unroll
            for (int jp = 0; jp < 2; ++jp)
#pragma unroll
                for (int u = 0; u < NU; ++u) {
                    float v[4] = {0.f, 0.f, 0.f, 0.f};
                    if (p.init) {
                        const int64_t off = b * p.sin_b + h * p.sin_h + (int64_t)(prow + 2 * WV * q + jp) * p.sin_p + ncol + 4 * u;
#pragma unroll
                        for (int j = 0; j < 4; ++j) v[j] = load_as_f32(p.init, off + j, dt_init);
                    }
                    stl[((q * 2 + jp) * NU + u) * 64] = (f32x4){v[0], v[1], v[2], v[3]};
                    store_row<4>(rs0, dt_out, vo_out, (2 * WV * q + jp) * (int)p.so_p + 4 * u, v);
                }
    } else if (FUSED) {
#pragma unroll
        for (int q = 0; q < NOWN; ++q)
#pragma unroll
        for (int jp = 0; jp < 2; ++jp) {
            if (p.init) {
                const int64_t off = b * p.sin_b + h * p.sin_h + (int64_t)(prow + 2 * WV * q + jp) * p.sin_p + ncol;
                if (dt_init == DT_F32) {
#pragma unroll
                    for (int u = 0; u < NU; ++u) {
                        const f32x4 v = *(const f32x4 *)((const float *)p.init + off + 4 * u);
                        st[q][jp][4 * u] = v.x; st[q][jp][4 * u + 1] = v.y; st[q][jp][4 * u + 2] = v.z; st[q][jp][4 * u + 3] = v.w;
                    }
                } else {
#pragma unroll
                    for (int j = 0; j < NB; ++j) st[q][jp][j] = load_as_f32(p.init, off + j, dt_init);
                }
            } else {
#pragma unroll
                for (int j = 0; j < NB; ++j) st[q][jp][j] = 0.f;
            }
        }
    }
    int32_t prev_id = 0;
    int gstep = 0;

    // One 32-token step of this wave of chunk c: bc holds the step's raw B rows, bn receives those of two steps
    // ahead.  All memory instructions of the step -- the B rows for step + 2, the x rows of the same step of the
    // next chunk, the state entering this chunk (out[:, c], kernels/ssd_state_passing.py:66-84) and the
    // next chunk's decay inputs -- are spread over the MFMA loop, one or two per four MFMAs: a burst of them
    // would stall the wave on the memory pipeline's issue queue.
    auto step = [&](int c, int s, f32x4 (&acc)[2][NB], uint32_t (&bc)[8][NBD], uint32_t (&bn)[8][NBD]) {
        // The x rows of this step were requested one chunk ago, as the first two vector-memory operations of
        // the same step (or in the prologue, before 16 B rows).  Memory operations complete in order, so the rows
        // are in LDS once no more than the operations issued after them are outstanding: at least the B rows of
        // the rest of that step and 8 B rows + 2 x requests for every other step of the chunk.  The compiler does
        // not track this dependence; the wait is explicit.
        constexpr int kAfterX = (8 - 2 * (8 / NB)) + (KS - 1) * 10;
        __builtin_amdgcn_s_waitcnt((kAfterX & 15) | (7 << 4) | (15 << 8) | ((kAfterX >> 4) << 14));
        uint32_t xr[8];
#pragma unroll
        for (int j = 0; j < 8; ++j)
            xr[j] = *(const uint32_t *)(xst + xst_rd + 1024 * (2 * s + (j >> 2)) + 256 * (j & 3));
        const f32x4 wlo = *(const f32x4 *)&wbuf[wave * QW + 32 * s + 8 * kg];
        const f32x4 whi = *(const f32x4 *)&wbuf[wave * QW + 32 * s + 8 * kg + 4];
        const float wv[8] = {wlo.x, wlo.y, wlo.z, wlo.w, whi.x, whi.y, whi.z, whi.w};

        // x * w in fp32, split into bf16 hi + bf16 lo, packed along the token axis
        uint32_t ahi[2][4], alo[2][4];
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
            for (int jp = 0; jp < 2; ++jp) {
                const uint32_t r0 = xr[2 * q], r1_ = xr[2 * q + 1];
                const float v0 = __builtin_bit_cast(float, jp ? (r0 & 0xffff0000u) : (r0 << 16)) * wv[2 * q];
                const float v1 = __builtin_bit_cast(float, jp ? (r1_ & 0xffff0000u) : (r1_ << 16)) * wv[2 * q + 1];
                const uint32_t hp = pack_bf16(v0, v1);
                const float h0 = __builtin_bit_cast(float, hp << 16);
                const float h1 = __builtin_bit_cast(float, hp & 0xffff0000u);
                ahi[jp][q] = hp;
                alo[jp][q] = pack_bf16(v0 - h0, v1 - h1);
            }
        bf16x8 Ahi[2], Alo[2];
#pragma unroll
        for (int jp = 0; jp < 2; ++jp) {
            Ahi[jp] = __builtin_bit_cast(bf16x8, (u32x4){ahi[jp][0], ahi[jp][1], ahi[jp][2], ahi[jp][3]});
            Alo[jp] = __builtin_bit_cast(bf16x8, (u32x4){alo[jp][0], alo[jp][1], alo[jp][2], alo[jp][3]});
        }
        // Everything that reads this step's x rows is complete above this line; the requests that overwrite
        // them with the next chunk's rows are issued below it.
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int jn = 0; jn < NB; ++jn) {
            const uint32_t sel = (jn & 1) ? 0x07060302u : 0x05040100u;
            u32x4 f;
            f.x = __builtin_amdgcn_perm(bc[1][jn >> 1], bc[0][jn >> 1], sel);
            f.y = __builtin_amdgcn_perm(bc[3][jn >> 1], bc[2][jn >> 1], sel);
            f.z = __builtin_amdgcn_perm(bc[5][jn >> 1], bc[4][jn >> 1], sel);
            f.w = __builtin_amdgcn_perm(bc[7][jn >> 1], bc[6][jn >> 1], sel);
            const bf16x8 Bf = __builtin_bit_cast(bf16x8, f);
#pragma unroll
            for (int jp = 0; jp < 2; ++jp) {
                acc[jp][jn] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(Ahi[jp], Bf, acc[jp][jn], 0, 0, 0);
                acc[jp][jn] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(Alo[jp], Bf, acc[jp][jn], 0, 0, 0);
            }
#pragma unroll
            for (int j = jn * 8 / NB; j < (jn + 1) * 8 / NB; ++j) load_B_row(gstep + 2, j, bn[j]);
            if (jn < 2) load_x(c + 1, s, jn);
            if (FUSED && !ST_LDS && s == 0 && jn < NOWN * 2 * NU) {      // NOWN * 2 * NU <= NB stores, one per iteration
                const int q = jn / (2 * NU), jp = (jn / NU) % 2, u = jn % NU;
                const float v[4] = {st[q][jp][4 * u], st[q][jp][4 * u + 1], st[q][jp][4 * u + 2], st[q][jp][4 * u + 3]};
                store_row<4>(slice_rsrc(p.out, esize_of(dt_out), b * p.so_b + c * p.so_c + h * p.so_h, slice_out), dt_out,
                             vo_out, (2 * WV * q + jp) * (int)p.so_p + 4 * u, v);
            }
            if (s == 0 && jn == NB - 1) mnext = load_meta(min(c + 1, c_end - 1));
            __builtin_amdgcn_sched_barrier(0);
        }
        ++gstep;
    };

    // One chunk.  b0 (and b1 when KS == 2) hold the raw B rows of its steps; three buffers rotate so that every
    // step can prefetch two steps ahead.
    auto chunk = [&](int c, uint32_t (&b0)[8][NBD], uint32_t (&b1)[8][NBD], uint32_t (&b2)[8][NBD]) {
        // ---- per-token weights of this wave's token quarter (kernels/ssd_chunk_state.py:134-156)
#pragma unroll
        for (int t = 0; t < TPL; ++t) {
            float e = mcur.last - mcur.cs[t];
            if (p.clamp) e = fminf(e, 0.f);
            float wv = __expf(e) * mcur.dtv[t];
            if (c * Q + ktok + t >= L) wv = 0.f;
            if (HAS_SEQ && mcur.id[t] != mcur.id_last) wv = 0.f;
            wbuf[ktok + t] = wv;
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront", "local");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront", "local");

        f32x4 acc[2][NB];
#pragma unroll
        for (int jp = 0; jp < 2; ++jp)
#pragma unroll
            for (int jn = 0; jn < NB; ++jn) acc[jp][jn] = (f32x4){0.f, 0.f, 0.f, 0.f};

        step(c, 0, acc, b0, b2);
        if constexpr (KS >= 2) step(c, 1, acc, b1, b0);
        if constexpr (KS == 4) {
            step(c, 2, acc, b2, b1);
            step(c, 3, acc, b0, b2);
        }

        // ---- sum the token shares of the WV waves
        lds_barrier();                      // previous chunk's exchange reads are done
        exchange_write<NB, WV>(acc, red, wave, lane);
        lds_barrier();
        float sum[NOWN][2][NB];
        exchange_read<NB, WV>(acc, red, wave, lane, sum);

        // ---- per-chunk states (side output) and the recurrence (kernels/ssd_state_passing.py:69-84)
        if (p.states) {
            const auto rs = slice_rsrc(p.states, esize_of(dt_states), b * p.sst_b + c * p.sst_c + h * p.sst_h, slice_st);
#pragma unroll
            for (int q = 0; q < NOWN; ++q)
#pragma unroll
                for (int jp = 0; jp < 2; ++jp)
                    store_tile_row(rs, dt_states, vo_st, (2 * WV * q + jp) * (int)p.sst_p, sum[q][jp]);
        }
        if (FUSED) {
            float sc = __expf(mcur.last);
            if (HAS_SEQ) {
                if (mcur.id_last != prev_id) sc = 0.f;
                prev_id = mcur.id_last;
            }
            if constexpr (ST_LDS) {
                // state <- sc * state + sum, back to LDS and out to out[:, c + 1] (or final_states after the last chunk)
                const bool last = c == p.C - 1;
                const auto rs = last ? slice_rsrc(p.fin, 4, b * p.sf_b + h * p.sf_h, slice_fin)
                                     : slice_rsrc(p.out, esize_of(dt_out), b * p.so_b + (c + 1) * p.so_c + h * p.so_h, slice_out);
                const int dt_dst = last ? (int)DT_F32 : dt_out;
                const int vo = last ? vo_fin : vo_out, pitch = last ? (int)p.sf_p : (int)p.so_p;
#pragma unroll
                for (int q = 0; q < NOWN; ++q)
#pragma unroll
                    for (int jp = 0; jp < 2; ++jp)
#pragma unroll
                        for (int u = 0; u < NU; ++u) {
                            const f32x4 o = stl[((q * 2 + jp) * NU + u) * 64];
                            const float v[4] = {sc * o.x + sum[q][jp][4 * u], sc * o.y + sum[q][jp][4 * u + 1],
                                                sc * o.z + sum[q][jp][4 * u + 2], sc * o.w + sum[q][jp][4 * u + 3]};
                            stl[((q * 2 + jp) * NU + u) * 64] = (f32x4){v[0], v[1], v[2], v[3]};
                            store_row<4>(rs, dt_dst, vo, (2 * WV * q + jp) * pitch + 4 * u, v);
                        }
            } else {
#pragma unroll
                for (int q = 0; q < NOWN; ++q)
#pragma unroll
                    for (int jp = 0; jp < 2; ++jp)
#pragma unroll
                        for (int j = 0; j < NB; ++j) st[q][jp][j] = sc * st[q][jp][j] + sum[q][jp][j];
            }
        }
        mcur = mnext;
    };

    int c = c_begin;
    if constexpr (KS == 2) {             // two steps rotate the three buffers by two; one or four steps by one
        for (;;) {
            chunk(c, bX, bY, bZ); if (++c >= c_end) break;
            chunk(c, bZ, bX, bY); if (++c >= c_end) break;
            chunk(c, bY, bZ, bX); if (++c >= c_end) break;
        }
    } else {
        for (;;) {
            chunk(c, bX, bY, bZ); if (++c >= c_end) break;
            chunk(c, bY, bZ, bX); if (++c >= c_end) break;
            chunk(c, bZ, bX, bY); if (++c >= c_end) break;
        }
    }
    if (FUSED && !ST_LDS) {
#pragma unroll
        for (int q = 0; q < NOWN; ++q)
#pragma unroll
            for (int jp = 0; jp < 2; ++jp)
                store_tile_row(slice_rsrc(p.fin, 4, b * p.sf_b + h * p.sf_h, slice_fin), DT_F32, vo_fin,
                               (2 * WV * q + jp) * (int)p.sf_p, st[q][jp]);
    }
}

static bool aligned(const void *ptr, size_t a) { return ((uintptr_t)ptr % a) == 0; }

bool mfma_supported(const Params &p)
{
    if (p.dt_in != DT_BF16) return false;
    if (p.headdim % 32 != 0) return false;
    if (p.dstate != 64 && p.dstate != 128) return false;
    if (p.Q != 128 && p.Q != 256) return false;
    const int nb = p.dstate / 16;                       // bf16 of B per lane per row
    if (!aligned(p.x, 4) || (p.sx_b | p.sx_l | p.sx_h) % 2) return false;
    if (!aligned(p.B, 4) || (p.sB_b | p.sB_l | p.sB_g) % 2) return false;
    (void)nb;
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

template <int NB, int KS, int WV, bool SEQ, bool FUSED>
static hipError_t launch_one(const Params &p, dim3 grid, hipStream_t s)
{
    const bool all32 = (!p.out || p.dt_out == DT_F32) && (!p.states || p.dt_states == DT_F32) &&
                       (!p.init || p.dt_init == DT_F32);
    constexpr int lds = lds_bytes<NB, KS, WV, FUSED>();
    // more than 64 KB of LDS per workgroup has to be requested explicitly, once per kernel
    static std::atomic<uint64_t> configured[2];
    {
        const hipError_t e = all32 ? ensure_dynamic_lds((const void *)mfma_kernel<NB, KS, WV, SEQ, FUSED, true>, lds, configured[1])
                                   : ensure_dynamic_lds((const void *)mfma_kernel<NB, KS, WV, SEQ, FUSED, false>, lds, configured[0]);
        if (e != hipSuccess) return e;
    }
    if (all32) hipLaunchKernelGGL((mfma_kernel<NB, KS, WV, SEQ, FUSED, true>), grid, dim3(64 * WV), lds, s, p);
    else hipLaunchKernelGGL((mfma_kernel<NB, KS, WV, SEQ, FUSED, false>), grid, dim3(64 * WV), lds, s, p);
    return hipGetLastError();
}

template <int NB, int KS, int WV>
static hipError_t launch_nb_ks(const Params &p, bool fused, hipStream_t s)
{
    const int per_xcd = (p.n_items + 7) / 8;
    const bool seq = p.seq != nullptr;
    dim3 grid(per_xcd * 8);
    if (fused) return seq ? launch_one<NB, KS, WV, true, true>(p, grid, s) : launch_one<NB, KS, WV, false, true>(p, grid, s);
    return seq ? launch_one<NB, KS, WV, true, false>(p, grid, s) : launch_one<NB, KS, WV, false, false>(p, grid, s);
}

static std::atomic<int> g_force_split{0};       // 0 = choose from the problem size; 2 or 4 = forced (process-wide hook)
int set_token_split(int wv) { return g_force_split.exchange(wv); }

hipError_t launch_mfma(const Params &p_in, bool fused, hipStream_t s)
{
    Params p = p_in;
    const int n_pt = p.headdim / 32;
    p.n_items = fused ? p.batch * p.nheads * n_pt : p.batch * p.C * p.nheads * n_pt;
    if (p.n_items <= 0) return hipSuccess;
    // Token split.  The kernels are bound by instruction issue, and two waves per state tile need 17 % fewer
    // vector instructions per tile than four (half the reduction traffic): measured 11-18 % faster for the
    // unfused launch, whose (batch, chunk, head, slice) items are plentiful.  The fused launch walks the chunks of
    // a tile serially with the running state in registers; there four waves win (2-wave workgroups spill and a
    // tile's chunk takes twice as long), 285 vs 361 us at b=4 L=8192 H=80.
    int wv = (!fused && p.n_items > 2 * (p.n_cu > 0 ? p.n_cu : 256)) ? 2 : 4;     // more than two tiles per compute unit
    const int forced = g_force_split.load(std::memory_order_relaxed);
    if (forced == 2 || forced == 4) wv = forced;
    const int nb = p.dstate / 16, q128 = p.Q / 128;     // chunk 128 or 256
    if (wv == 4) {
        if (nb == 8 && q128 == 2) return launch_nb_ks<8, 2, 4>(p, fused, s);
        if (nb == 8 && q128 == 1) return launch_nb_ks<8, 1, 4>(p, fused, s);
        if (nb == 4 && q128 == 2) return launch_nb_ks<4, 2, 4>(p, fused, s);
        return launch_nb_ks<4, 1, 4>(p, fused, s);
    }
    if (nb == 8 && q128 == 2) return launch_nb_ks<8, 4, 2>(p, fused, s);
    if (nb == 8 && q128 == 1) return launch_nb_ks<8, 2, 2>(p, fused, s);
    if (nb == 4 && q128 == 2) return launch_nb_ks<4, 4, 2>(p, fused, s);
    return launch_nb_ks<4, 2, 2>(p, fused, s);
}

}  // namespace ssd
