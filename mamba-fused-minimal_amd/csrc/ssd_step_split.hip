// Fused chunk-state + state-passing kernel, step split: three state tiles per workgroup, every wave working on all
// three (gfx950; dstate 128, chunk 256, bf16 x / B, fp32 states).
//
// A workgroup is four waves and three (32 headdim rows) x (128 dstate columns) tiles of one (batch, group).  Of the
// eight 32-token steps of a chunk, wave w takes steps 2w and 2w + 1 -- for all three tiles.  What that buys over one
// tile per wave:
//   * one transposed B operand (ds_read_b64_tr_b16 pair) feeds twelve MFMAs instead of four, so the bf16 hi/lo split
//     of the next step's x * w (three tiles' worth) fits into the issue slots the MFMAs leave free;
//   * a step's B tile is used by one wave only: B, like x, sits in rings private to a wave and the steps need no
//     barrier;
//   * four waves share three tiles: 192 instead of 256 MFMAs per wave and chunk, and the fourth SIMD of the compute
//     unit works.
// The price: a wave's accumulators hold partial sums (its 64 tokens) of all three tiles.  Wave w owns the running
// state of dstate columns 32w .. 32w + 31 of every tile; at the end of a chunk the partial sums of the other columns
// go to their owners through LDS (three rounds, wave w -> wave w + r + 1), into ring slots that are free at that
// moment.  The accumulators are indexed by the column block relative to the owned ones, it' = (it - 2w) mod 8, so
// that every wave runs the same code: it' = 0, 1 are owned.
// Per-chunk recurrence as in kernels/ssd_state_passing.py:69-84 on the contraction of
// kernels/ssd_chunk_state.py:134-173.
#include "ssd_params.h"

#include <utility>

namespace ssd {

namespace ss {

template <int... I, class F>
__device__ __forceinline__ void static_for_impl(std::integer_sequence<int, I...>, F &&f) { (f(std::integral_constant<int, I>{}), ...); }
template <int N, class F>
__device__ __forceinline__ void static_for(F &&f) { static_for_impl(std::make_integer_sequence<int, N>{}, f); }

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

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void *base, int64_t bytes)
{
    return __builtin_amdgcn_make_buffer_rsrc((void *)base, 0, (int)(bytes > 0x7fffffffLL ? 0x7fffffffLL : bytes),
                                             0x00020000);
}

// s_waitcnt immediate that only waits for the vector-memory counter to drop to n (gfx9 field layout)
constexpr int vmcnt_imm(int n) { return (n & 15) | (7 << 4) | (15 << 8) | ((n >> 4) << 14); }

constexpr int NT = 8, SPC = 8, Q = 256, T = 3;
constexpr int kBslot = NT * 1024;                 // a step's B tile: 32 tokens x 128 columns bf16
constexpr int kXslot = T * 2048;                  // a step's x rows of the three tiles
constexpr int kBring = 2 * kBslot, kXring = 3 * kXslot, kWbuf = 2 * T * 64 * 4;
constexpr int kWaveLds = kBring + kXring + kWbuf; // 36352
constexpr int kLds = 4 * kWaveLds;                // 145408
constexpr int kStoresPerBoundary = T * 4;         // owned blocks of 1 KB

struct Frag { uint32_t hi[2][4], lo[2][4]; };

template <bool HAS_SEQ>
__global__ void __launch_bounds__(256, 1) step_split_kernel(const Params p)
{
    extern __shared__ __attribute__((aligned(16))) char lds[];
    const int lane = threadIdx.x & 63, i16 = lane & 15, kg = lane >> 4;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    char *mine = lds + wave * kWaveLds;
    char *bring = mine;                    // 2 slots x 8 blocks of 1 KB (16 tokens x 32 columns each)
    char *xring = mine + kBring;           // 3 slots x 3 tiles x (32 tokens x 64 bytes)
    char *wbuf = xring + kXring;           // 2 chunk parities x 3 tiles x this wave's 64 token weights

    // ---- workgroup -> three tiles of one (batch, group); consecutive workgroups sit on one XCD
    const int n_wg = p.n_items;
    const int per_xcd = (n_wg + 7) >> 3;
    const int wg = (int)(blockIdx.x & 7) * per_xcd + (int)(blockIdx.x >> 3);
    if (wg >= n_wg) return;                                              // whole workgroup
    const int n_pt = p.headdim >> 5, hpg = p.nheads / p.ngroups, tpg = hpg * n_pt, wpg = (tpg + T - 1) / T;
    const int bg = wg / wpg, b = bg / p.ngroups, g = bg % p.ngroups;
    int th[T], tp0[T];
    bool live[T];
#pragma unroll
    for (int t = 0; t < T; ++t) {
        const int j = T * (wg % wpg) + t, jc = min(j, tpg - 1);         // a short last workgroup repeats its last tile
        live[t] = j < tpg;
        th[t] = g * hpg + jc / n_pt;
        tp0[t] = 32 * (jc % n_pt);
    }
    const int C = p.C, L = p.seqlen;
    const int tok_w = 64 * wave;           // this wave's first token inside a chunk

    const char *Brow = (const char *)p.B + 2 * (b * p.sB_b + g * p.sB_g);
    const char *xrow[T];
#pragma unroll
    for (int t = 0; t < T; ++t) xrow[t] = (const char *)p.x + 2 * (b * p.sx_b + th[t] * p.sx_h + tp0[t]);
    const int64_t xrb = 2 * p.sx_l, Brb = 2 * p.sB_l;            // row pitch in bytes
    auto chunk_rsrc = [&](const char *base, int64_t pitch, int c) {
        const int cc = c < C ? c : 0;
        return make_rsrc(base + (int64_t)cc * Q * pitch, c < C ? (int64_t)(L - c * Q) * pitch : 0);
    };
    const int32_t *sqb = HAS_SEQ ? p.seq + b * p.ssq_b : nullptr;

    // ---- requests.  Layouts inside a slot are those of the four-tile kernel: a B tile as 8 blocks of 1 KB, block
    // (token half th, column pair) = 16 tokens x 32 columns row-major, the two 32-byte halves of rows 8..15 swapped;
    // an x tile as two 1 KB blocks, request i fetching tokens 8 kg' + 4 i + m into row slot 4 m + kg'.
    const int Blane = (int)((lane >> 2) * Brb) + 16 * ((lane & 3) ^ ((lane >> 5) << 1));
    auto load_B = [&](__amdgpu_buffer_rsrc_t rs, int slot, int sl) {     // the 8 blocks of step sl of the chunk behind rs
#if defined(__HIP_DEVICE_COMPILE__)
        typedef __attribute__((address_space(3))) void *lds_ptr;
#pragma unroll
        for (int bi = 0; bi < NT; ++bi) {
            const int hf = bi / (NT / 2), pair = bi % (NT / 2);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lds_ptr)(bring + slot * kBslot + bi * 1024), 16, Blane,
                                                     (int)((tok_w + 32 * sl + 16 * hf) * Brb) + 64 * pair, 0, 0);
        }
#else
        (void)rs; (void)slot; (void)sl; (void)Blane;
#endif
    };
    const int xlane = (int)((8 * ((lane >> 2) & 3) + (lane >> 4)) * xrb) + 16 * (lane & 3);
    auto load_x = [&](const __amdgpu_buffer_rsrc_t (&rs)[T], int xs, int sl) {   // 6 requests: three tiles of step sl
#if defined(__HIP_DEVICE_COMPILE__)
        typedef __attribute__((address_space(3))) void *lds_ptr;
#pragma unroll
        for (int t = 0; t < T; ++t)
#pragma unroll
            for (int i = 0; i < 2; ++i)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rs[t], (lds_ptr)(xring + xs * kXslot + t * 2048 + i * 1024), 16, xlane,
                                                         (int)((tok_w + 32 * sl + 4 * i) * xrb), 0, 0);
#else
        (void)rs; (void)xs; (void)sl; (void)xlane;
#endif
    };
    constexpr int kLoadsX = 2 * T, kLoadsB = NT, kTouch = 2;
    // x comes from HBM and the rings are too small to request it more than two steps ahead, so the rows of step + 4
    // are touched one dword each two steps before they are requested: the request then finds them in L2.  The
    // loaded value is never used; the register stays allocated to these loads for the whole kernel (a load that
    // returns late must not find it reassigned).
    uint32_t touched = 0;
    auto touch_x = [&](int c, int sl) {          // step sl of chunk c: lanes 0-31 / 32-63 = tokens of tiles 0 / 1, then tile 2
        const int64_t tok = (int64_t)min(c * Q + tok_w + 32 * sl + (lane & 31), L - 1);
        const char *a01 = (lane < 32 ? xrow[0] : xrow[1]) + tok * xrb;
        const char *a2 = xrow[2] + tok * xrb;
#if defined(__HIP_DEVICE_COMPILE__)
        asm volatile("global_load_dword %0, %1, off\n\tglobal_load_dword %0, %2, off" : "+v"(touched) : "v"(a01), "v"(a2) : "memory");
#else
        (void)a01; (void)a2;
#endif
    };

    // transposing reads of the B tile: address of (column block it' relative to the owned ones, tokens 8 kg ..):
    // the block pair index is ((it' >> 1) + wave) & 3, the 32-byte half it' & 1 (swapped for odd kg)
    uint32_t Bt_addr[NT];
    {
        const uint32_t off = (kg >> 1) * (NT / 2) * 1024 + (8 * (kg & 1) + (i16 >> 2)) * 64 + (kg & 1) * 32 + (i16 & 3) * 8;
        uint32_t ring = 0;
#if defined(__HIP_DEVICE_COMPILE__)
        ring = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char *)bring;
#endif
#pragma unroll
        for (int it = 0; it < NT; ++it) Bt_addr[it] = ring + (off ^ ((it & 1) ? 32u : 0u)) + (((it >> 1) + wave) & 3) * 1024;
    }
    auto read_Bt = [&](auto slotc, uint32_t addr, u32x2 &lo, u32x2 &hi) {
        constexpr int off = decltype(slotc)::value * kBslot;
#if defined(__HIP_DEVICE_COMPILE__)
        asm volatile("ds_read_b64_tr_b16 %0, %2 offset:%3\n\tds_read_b64_tr_b16 %1, %2 offset:%4"
                     : "=&v"(lo), "=&v"(hi) : "v"(addr), "n"(off), "n"(off + 256) : "memory");
#else
        lo = hi = (u32x2){0u, 0u}; (void)addr; (void)off;
#endif
    };
    auto wait_Bt = [&](auto nc, u32x2 &lo, u32x2 &hi) {     // at most nc LDS operations issued behind the pair
#if defined(__HIP_DEVICE_COMPILE__)
        asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(lo), "+v"(hi) : "n"(decltype(nc)::value) : "memory");
#else
        (void)lo; (void)hi;
#endif
    };
    const int xst_rd = 64 * kg + 4 * i16;     // + 1024 * (j/4) + 256 * (j%4) for token 8kg + j of a step

    // ---- per-token weights of this wave's 64 tokens, per tile (kernels/ssd_chunk_state.py:134-156)
    struct Meta { float dtv[T], cs[T], last[T]; int32_t id, id_last; };
    auto load_meta = [&](int c) {
        Meta m;
        const int cc = c < C ? c : C - 1;
#pragma unroll
        for (int t = 0; t < T; ++t) {
            const float *dtp = p.dt + b * p.sdt_b + th[t] * p.sdt_h + cc * p.sdt_c;
            const float *dap = p.dacs + b * p.sda_b + th[t] * p.sda_h + cc * p.sda_c;
            m.dtv[t] = dtp[tok_w + lane];
            m.cs[t] = dap[tok_w + lane];
            m.last[t] = dap[Q - 1];
        }
        m.id = 0; m.id_last = 0;
        if (HAS_SEQ) {
            m.id = sqb[(int64_t)min(cc * Q + tok_w + lane, L - 1) * p.ssq_l];
            m.id_last = sqb[(int64_t)(min((cc + 1) * Q, L) - 1) * p.ssq_l];
        }
        return m;
    };
    auto put_weights = [&](int c, int par, const Meta &m) {
#pragma unroll
        for (int t = 0; t < T; ++t) {
            float e = m.last[t] - m.cs[t];
            if (p.clamp) e = fminf(e, 0.f);
            float w = __expf(e) * m.dtv[t];
            if (c * Q + tok_w + lane >= L) w = 0.f;
            if (HAS_SEQ && m.id != m.id_last) w = 0.f;
            *(float *)(wbuf + ((par * T + t) * 64 + lane) * 4) = w;
        }
    };
    // operands of (x slot xs, tile t, step sl of the chunk with weight parity par): tokens 8kg .. 8kg+7
    auto read_operands = [&](int xs, int t, int par, int sl, uint32_t (&xr)[8], float (&wv)[8]) {
#pragma unroll
        for (int j = 0; j < 8; ++j)
            xr[j] = *(const uint32_t *)(xring + xs * kXslot + t * 2048 + xst_rd + 1024 * (j >> 2) + 256 * (j & 3));
        const f32x4 wlo = *(const f32x4 *)(wbuf + ((par * T + t) * 64 + 32 * sl + 8 * kg) * 4);
        const f32x4 whi = *(const f32x4 *)(wbuf + ((par * T + t) * 64 + 32 * sl + 8 * kg + 4) * 4);
        wv[0] = wlo.x; wv[1] = wlo.y; wv[2] = wlo.z; wv[3] = wlo.w;
        wv[4] = whi.x; wv[5] = whi.y; wv[6] = whi.z; wv[7] = whi.w;
    };
    // tokens (2q, 2q+1) of headdim row 2*i16 + jp: x * w in fp32, split into bf16 hi + bf16 lo
    auto frag_piece = [&](int q, int jp, const uint32_t (&xr)[8], const float (&wv)[8], Frag &f) {
        const uint32_t r0 = xr[2 * q], r1_ = xr[2 * q + 1];
        const float x0 = __builtin_bit_cast(float, jp ? (r0 & 0xffff0000u) : (r0 << 16));
        const float x1 = __builtin_bit_cast(float, jp ? (r1_ & 0xffff0000u) : (r1_ << 16));
        uint32_t hp = pack_bf16(x0 * wv[2 * q], x1 * wv[2 * q + 1]);
        asm volatile("" : "+v"(hp));
        const float h0 = __builtin_bit_cast(float, hp << 16);
        const float h1 = __builtin_bit_cast(float, hp & 0xffff0000u);
        f.hi[jp][q] = hp;
        f.lo[jp][q] = pack_bf16(__builtin_fmaf(x0, wv[2 * q], -h0), __builtin_fmaf(x1, wv[2 * q + 1], -h1));
    };

    // ---- state.  acc[t][it'][jp][r]: dstate column 16 * ((it' + 2 wave) % 8) + 4 kg + r of headdim row 2 i16 + jp of
    // tile t; it' < 2: the running state, otherwise this wave's partial sum of the current chunk
    f32x4 acc[T][NT][2];
    const int col0 = 32 * wave;            // first owned column
    // owned blocks -> memory, through 1 KB of LDS each so that four adjacent lanes write 64 contiguous bytes (the
    // accumulators hold a block as lane%16 = row; see the four-tile kernel).  `stage` is a free ring slot.
    auto store_owned = [&](char *stage, float *dst, const int64_t (&base)[T], int64_t slice, int pitch) {
        const int voff = 2 * (lane >> 2) * pitch + 4 * (lane & 3);
        f32x4 *wr = (f32x4 *)(stage + i16 * 64 + ((kg ^ (i16 >> 2)) << 4));
        const f32x4 *rd = (const f32x4 *)(stage + (lane >> 2) * 64 + (((lane & 3) ^ (lane >> 4)) << 4));
        constexpr int kLag = 4, NB = T * 4;
        f32x4 v[NB];
#pragma unroll
        for (int k = 0; k < NB + kLag; ++k) {
            if (k < NB) {
                *(f32x4 *)((char *)wr + (k & 3) * 1024) = acc[k >> 2][(k >> 1) & 1][k & 1];
                v[k] = *(const f32x4 *)((const char *)rd + (k & 3) * 1024);
            }
            if (k >= kLag) {
                const int j = k - kLag, t = j >> 2, q = (j >> 1) & 1, jp = j & 1;
                const auto rs = make_rsrc(dst + base[t], live[t] ? slice * 4 : 0);
                const u32x4 d = __builtin_bit_cast(u32x4, v[j]);
                __builtin_amdgcn_raw_buffer_store_b128(d, rs, 4 * voff, 4 * (jp * pitch + col0 + 16 * q), 0);
                asm volatile("s_nop 3" ::"v"(d) : "memory");
            }
        }
    };
    int64_t obase[T], fbase[T];
#pragma unroll
    for (int t = 0; t < T; ++t) {
        obase[t] = b * p.so_b + th[t] * p.so_h + (int64_t)tp0[t] * p.so_p;
        fbase[t] = b * p.sf_b + th[t] * p.sf_h + (int64_t)tp0[t] * p.sf_p;
    }
    const int64_t slice_o = (int64_t)31 * p.so_p + p.dstate, slice_f = (int64_t)31 * p.sf_p + p.dstate;

#pragma unroll
    for (int t = 0; t < T; ++t)
#pragma unroll
        for (int q = 0; q < 2; ++q)
#pragma unroll
            for (int jp = 0; jp < 2; ++jp) {
                acc[t][q][jp] = (f32x4){0.f, 0.f, 0.f, 0.f};
                if (p.init)
                    acc[t][q][jp] = *(const f32x4 *)((const float *)p.init + b * p.sin_b + th[t] * p.sin_h +
                                                     (int64_t)(tp0[t] + 2 * i16 + jp) * p.sin_p + col0 + 16 * q + 4 * kg);
            }

    // ---- prologue: the rings hold finite numbers wherever no row lands (rows past the end of the sequence)
#pragma unroll
    for (int i = 0; i < (kBring + kXring) / 1024; ++i) *(u32x4 *)(mine + i * 1024 + 16 * lane) = (u32x4){0u, 0u, 0u, 0u};
    __builtin_amdgcn_s_waitcnt(0xc07f);          // lgkmcnt(0): the zeros are in place before any row lands
    Meta mcur = load_meta(0);
    __amdgpu_buffer_rsrc_t rsx0[T], rsx1[T];
#pragma unroll
    for (int t = 0; t < T; ++t) { rsx0[t] = chunk_rsrc(xrow[t], xrb, 0); rsx1[t] = chunk_rsrc(xrow[t], xrb, 1); }
    __amdgpu_buffer_rsrc_t rsB0 = chunk_rsrc(Brow, Brb, 0), rsB1 = chunk_rsrc(Brow, Brb, 1);
    // the request order every step keeps: x two steps ahead, then B one step ahead
    load_x(rsx0, 0, 0);
    load_B(rsB0, 0, 0);
    load_x(rsx0, 1, 1);
    touch_x(1, 0);
    touch_x(1, 1);
    __builtin_amdgcn_sched_barrier(0);
    put_weights(0, 0, mcur);
    Meta mnext = load_meta(1);
    Frag fA[T], fB[T];
    {
        __builtin_amdgcn_s_waitcnt(vmcnt_imm(kLoadsB + kLoadsX + 2 * kTouch));   // x of step 0 has landed (what follows it
                                                                             // above; the loads of mnext only make this wait longer)
        asm volatile("" ::: "memory");
#pragma unroll
        for (int t = 0; t < T; ++t) {
            uint32_t xr[8]; float wv[8];
            read_operands(0, t, 0, 0, xr, wv);
#pragma unroll
            for (int q = 0; q < 4; ++q) { frag_piece(q, 0, xr, wv, fA[t]); frag_piece(q, 1, xr, wv, fA[t]); }
        }
    }
    int32_t prev_id = 0;
    int xs = 0;                             // x slot of the current step (step counter mod 3)
    // out[:, 0] = the initial state (owned columns); B slot 1, not requested into yet, is the staging area
    store_owned(bring + kBslot, (float *)p.out, obase, slice_o, (int)p.so_p);
    __builtin_amdgcn_s_waitcnt(0xc07f);     // the staging reads have returned before rows land there
    __builtin_amdgcn_s_barrier();           // every wave has zeroed its rings before anyone's exchange touches them

    // One step: sl = 0 / 1 (compile time) of chunk c; par = weight parity of the chunk.
    // fc = this step's x operands, fn receives the next step's.
    auto step = [&](int c, auto slc, int par, Frag (&fc)[T], Frag (&fn)[T]) {
        constexpr int sl = decltype(slc)::value;
        const int xs_n1 = xs == 2 ? 0 : xs + 1, xs_n2 = xs == 0 ? 2 : xs - 1;      // slots of step + 1, step + 2
        // requests, the most urgent first: B of step + 1, x of step + 2 (the same step of the next chunk), and the
        // touches for step + 4
        if constexpr (sl == 0) load_B(rsB0, 1, 1);
        else load_B(rsB1, 0, 0);
        load_x(rsx1, xs_n2, sl);
        touch_x(c + 2, sl);
        if constexpr (sl == 0) {
            // chunk boundary (out[:, c] left at the end of the previous chunk): s <- exp(dA_chunk) s
            float sc[T];
#pragma unroll
            for (int t = 0; t < T; ++t) sc[t] = __expf(mcur.last[t]);
            if (HAS_SEQ) {
                if (mcur.id_last != prev_id)
#pragma unroll
                    for (int t = 0; t < T; ++t) sc[t] = 0.f;
                prev_id = mcur.id_last;
            }
#pragma unroll
            for (int t = 0; t < T; ++t)
#pragma unroll
                for (int q = 0; q < 2; ++q)
#pragma unroll
                    for (int jp = 0; jp < 2; ++jp) acc[t][q][jp] *= sc[t];
        }
        // The rows this step reads -- its B tile and, for the next step's operands, x of step + 1 -- were requested
        // at the start of the previous step, x last.  Behind them came that step's touches, the state stores if a
        // chunk ended in between, and the requests above.
        __builtin_amdgcn_s_waitcnt(vmcnt_imm(kTouch + (sl == 0 ? kStoresPerBoundary : 0) + kLoadsB + kLoadsX + kTouch));
        asm volatile("" ::: "memory");
        if constexpr (sl == 1) put_weights(c + 1, par ^ 1, mnext);

        bf16x8 h0[T], h1[T], l0[T], l1[T];
#pragma unroll
        for (int t = 0; t < T; ++t) {
            h0[t] = __builtin_bit_cast(bf16x8, (u32x4){fc[t].hi[0][0], fc[t].hi[0][1], fc[t].hi[0][2], fc[t].hi[0][3]});
            h1[t] = __builtin_bit_cast(bf16x8, (u32x4){fc[t].hi[1][0], fc[t].hi[1][1], fc[t].hi[1][2], fc[t].hi[1][3]});
            l0[t] = __builtin_bit_cast(bf16x8, (u32x4){fc[t].lo[0][0], fc[t].lo[0][1], fc[t].lo[0][2], fc[t].lo[0][3]});
            l1[t] = __builtin_bit_cast(bf16x8, (u32x4){fc[t].lo[1][0], fc[t].lo[1][1], fc[t].lo[1][2], fc[t].lo[1][3]});
        }
        // next step's operands are prepared tile by tile inside the MFMA loop: its x rows landed with this step's
        // (requested before them), its weights are in place (same chunk, or written above)
        const int par_n = sl == 0 ? par : par ^ 1;
        uint32_t xr[8]; float wv[8];
        u32x2 blo[2], bhi[2];
        __builtin_amdgcn_sched_barrier(0);
        read_Bt(std::integral_constant<int, sl>{}, Bt_addr[0], blo[0], bhi[0]);
        static_for<NT>([&](auto itc) {
            constexpr int it = decltype(itc)::value;
            // operand reads of the next step's tile it / 2 (tiles 0..2 in iterations 0, 2, 4), issued before the
            // wait so that the count below covers them
            if constexpr (it % 2 == 0 && it / 2 < T) read_operands(xs_n1, it / 2, par_n, sl ^ 1, xr, wv);
            if constexpr (it + 1 < NT) read_Bt(std::integral_constant<int, sl>{}, Bt_addr[it + 1], blo[(it + 1) & 1], bhi[(it + 1) & 1]);
            // LDS operations complete in order: behind the pair of this iteration came the operand reads above (10,
            // in the even iterations that have them) and the next pair (2)
            constexpr int behind = ((it % 2 == 0 && it / 2 < T) ? 10 : 0) + (it + 1 < NT ? 2 : 0);
            wait_Bt(std::integral_constant<int, behind>{}, blo[it & 1], bhi[it & 1]);
            const bf16x8 Bt = __builtin_bit_cast(bf16x8, (u32x4){blo[it & 1].x, blo[it & 1].y, bhi[it & 1].x, bhi[it & 1].y});
            constexpr bool fresh = it >= 2 && sl == 0;      // first contribution to a partial sum of this chunk
#pragma unroll
            for (int t = 0; t < T; ++t) {
                const f32x4 z = {0.f, 0.f, 0.f, 0.f};
                acc[t][it][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(Bt, h0[t], fresh ? z : acc[t][it][0], 0, 0, 0);
                acc[t][it][1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(Bt, h1[t], fresh ? z : acc[t][it][1], 0, 0, 0);
                acc[t][it][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(Bt, l0[t], acc[t][it][0], 0, 0, 0);
                acc[t][it][1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(Bt, l1[t], acc[t][it][1], 0, 0, 0);
            }
            // the operands read in iteration it (even) are split in iterations it and it + 1
            if constexpr (it / 2 < T) {
                constexpr int t = it / 2, half = it % 2;
#pragma unroll
                for (int e = 4 * half; e < 4 * half + 4; ++e) frag_piece(e >> 1, e & 1, xr, wv, fn[t]);
            }
            __builtin_amdgcn_sched_barrier(0);
        });
        xs = xs_n1;
    };

    for (int c = 0; c < C; ++c) {
        const int par = c & 1;
        step(c, std::integral_constant<int, 0>{}, par, fA, fB);
        step(c, std::integral_constant<int, 1>{}, par, fB, fA);
        // ---- the partial sums go to their owners.  Inbox of a wave: its B slot 1 (the step just finished) and the x
        // slot of that step -- `xs` already points one further, so that slot is xs - 1.
        const int xfree = xs == 0 ? 2 : xs - 1;
        __builtin_amdgcn_s_waitcnt(0xc07f);
        __builtin_amdgcn_s_barrier();           // every wave is through with the slots that now serve as inboxes
        static_for<3>([&](auto rc) {
            constexpr int r = decltype(rc)::value;
            const int d = (wave + r + 1) & 3;
            char *inbox_b = lds + d * kWaveLds + kBslot + 16 * lane;
            char *inbox_x = lds + d * kWaveLds + kBring + xfree * kXslot + 16 * lane;
#pragma unroll
            for (int k = 0; k < T * 4; ++k) {
                const int t = k >> 2, q = (k >> 1) & 1, jp = k & 1;
                char *dst = k < 8 ? inbox_b + k * 1024 : inbox_x + (k - 8) * 1024;
                *(f32x4 *)dst = acc[t][2 * (r + 1) + q][jp];
            }
            __builtin_amdgcn_s_waitcnt(0xc07f);
            __builtin_amdgcn_s_barrier();       // the partial sums of this round are in their inboxes
            const char *my_b = mine + kBslot + 16 * lane, *my_x = mine + kBring + xfree * kXslot + 16 * lane;
#pragma unroll
            for (int k = 0; k < T * 4; ++k) {
                const int t = k >> 2, q = (k >> 1) & 1, jp = k & 1;
                acc[t][q][jp] += *(const f32x4 *)(k < 8 ? my_b + k * 1024 : my_x + (k - 8) * 1024);
            }
            if constexpr (r < 2) {
                __builtin_amdgcn_s_waitcnt(0xc07f);
                __builtin_amdgcn_s_barrier();   // read before the next round overwrites
            }
        });
        // the owned columns now hold the state entering chunk c + 1: out[:, c + 1], or the final state.  B slot 1 --
        // the inbox, read by now (LDS operations complete in order) -- is the staging area until the next step
        // requests rows into it.
        if (c + 1 < C) store_owned(bring + kBslot, (float *)p.out + (int64_t)(c + 1) * p.so_c, obase, slice_o, (int)p.so_p);
        else store_owned(bring + kBslot, p.fin, fbase, slice_f, (int)p.sf_p);
        __builtin_amdgcn_s_waitcnt(0xc07f);     // inbox and staging reads have returned before rows land there
        mcur = mnext;
        mnext = load_meta(c + 2);              // used one and a half steps from here
#pragma unroll
        for (int t = 0; t < T; ++t) { rsx0[t] = rsx1[t]; rsx1[t] = chunk_rsrc(xrow[t], xrb, c + 2); }
        rsB0 = rsB1;
        rsB1 = chunk_rsrc(Brow, Brb, c + 2);
    }
#if defined(__HIP_DEVICE_COMPILE__)
    asm volatile("s_waitcnt vmcnt(0)" : "+v"(touched));      // the last touches have returned before the register is given up
#endif
}

static bool aligned(const void *ptr, size_t a) { return ((uintptr_t)ptr % a) == 0; }

}  // namespace ss

bool step_split_supported(const Params &p)
{
    using ss::aligned;
    if (p.states || !p.out || !p.fin) return false;
    if (p.dt_in != DT_BF16 || p.dt_out != DT_F32 || (p.init && p.dt_init != DT_F32)) return false;
    if (p.headdim % 32 != 0 || p.dstate != 128 || p.Q != 256) return false;
    if (!aligned(p.x, 16) || (p.sx_b | p.sx_l | p.sx_h) % 8) return false;
    if (!aligned(p.B, 16) || (p.sB_b | p.sB_l | p.sB_g) % 8) return false;
    if ((int64_t)p.Q * 2 * p.sx_l >= (1LL << 31) || (int64_t)p.Q * 2 * p.sB_l >= (1LL << 31)) return false;
    if (p.sdt_k != 1 || p.sda_k != 1) return false;
    if (!aligned(p.out, 16) || (p.so_b | p.so_c | p.so_h | p.so_p) % 4) return false;
    if (!aligned(p.fin, 16) || (p.sf_b | p.sf_h | p.sf_p) % 4) return false;
    if (p.init && (!aligned(p.init, 16) || (p.sin_b | p.sin_h | p.sin_p) % 4)) return false;
    if ((int64_t)p.headdim * p.so_p >= (1LL << 28) || (int64_t)p.headdim * p.sf_p >= (1LL << 28)) return false;
    return true;
}

hipError_t launch_step_split(const Params &p_in, hipStream_t s)
{
    Params p = p_in;
    const int tpg = (p.nheads / p.ngroups) * (p.headdim / 32);
    p.n_items = p.batch * p.ngroups * ((tpg + ss::T - 1) / ss::T);        // workgroups
    if (p.n_items <= 0) return hipSuccess;
    static bool configured = false;
    if (!configured) {
        hipError_t e = hipFuncSetAttribute((const void *)ss::step_split_kernel<false>, hipFuncAttributeMaxDynamicSharedMemorySize, ss::kLds);
        if (e == hipSuccess)
            e = hipFuncSetAttribute((const void *)ss::step_split_kernel<true>, hipFuncAttributeMaxDynamicSharedMemorySize, ss::kLds);
        if (e != hipSuccess) return e;
        configured = true;
    }
    const dim3 grid(((p.n_items + 7) / 8) * 8);
    if (p.seq) hipLaunchKernelGGL(ss::step_split_kernel<true>, grid, dim3(256), ss::kLds, s, p);
    else hipLaunchKernelGGL(ss::step_split_kernel<false>, grid, dim3(256), ss::kLds, s, p);
    return hipGetLastError();
}

}  // namespace ssd
