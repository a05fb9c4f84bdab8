// Fused chunk-state + state-passing kernel: four state tiles per workgroup, B shared through LDS (gfx950).
//
// A workgroup is four waves; each wave owns the (32 headdim rows) x (all dstate columns) tile of one
// (batch, head, row slice) and walks the whole sequence, the four tiles sharing one (batch, group) and therefore
// the same B rows.  The running state lives in the MFMA accumulators: at a chunk boundary a wave stores them as
// out[:, c] (the state entering chunk c), multiplies them by exp(dA_chunk) -- or by zero where seq_idx changes --
// and the chunk's 32-token steps accumulate sum_k B_k (x*w)_k on top: s <- exp(dA_chunk) * s + states_c
// (kernels/ssd_state_passing.py:69-84 applied to the contraction of kernels/ssd_chunk_state.py:134-173).  There is
// no token split, no LDS reduction and the per-chunk `states` tensor never exists, so callers that ask for it get
// the token-split kernel instead.
//
// Data movement per 32-token step:
//   * B: the step's 32 x dstate tile is fetched ONCE per workgroup, straight into a ring in LDS (buffer loads with
//     LDS destination, each wave a quarter of the tile), three steps ahead.  The MFMA computes the state
//     transposed, D[n][p] = sum_k B[k][n] * xw[k][p], so B is the A operand: lane (i, kg) needs the 8 tokens
//     8kg..8kg+7 of column 16*it + i.  ds_read_b64_tr_b16 delivers exactly that from the row-major tile: within a
//     16-lane group, lane i receives 16-bit element i%4 of the 8-byte words addressed by lanes i/4, i/4+4, i/4+8,
//     i/4+12; with lane s addressing (token 4*half + s/4, columns 4*(s%4)..+3) lane i ends up with four consecutive
//     tokens of column i.  No v_perm, no B registers, a quarter of the vector-memory instructions.
//   * x: each wave fetches its own rows into a private four-slot LDS ring, three steps ahead, reads them back as
//     (token, row pair) dwords, scales by the per-token weight in fp32 and splits into bf16 hi + bf16 lo (two MFMAs
//     keep ~16 mantissa bits of x*w); the operands of step g+1 are prepared while the MFMAs of step g run.
//   * out: accumulator register r of tile (it, jp) is dstate column 16*it + 4*kg + r of headdim row 2*j + jp, so
//     the four registers of a tile are one 16-byte store and the state never moves between registers.
// One s_barrier per step orders the shared ring: a wave passes it after its own part of the step's B tile has
// landed and after it has finished reading the previous step's tile.
#include "ssd_params.h"
#include "ssd_tile.h"      // schedule:: the compile-time model of the step loop's memory queue

#include <utility>

namespace ssd {

namespace quad {

using namespace tile;      // register types, static_for, pack_bf16, make_rsrc, vmcnt_imm, Frag (ssd_tile.h)

typedef __attribute__((ext_vector_type(4))) short s16x4;

__device__ __forceinline__ int esize_of(int dt) { return dt == DT_F32 ? 4 : 2; }

// Four consecutive state values of one row -> fp32 / bf16 / f16 destination.  The data registers of a wide store
// are read out over several cycles after issue; wait states that depend on them keep a following writer of the
// same registers (here the decay multiplication of the accumulators) away.
__device__ __forceinline__ void store4(__amdgpu_buffer_rsrc_t rs, int dt, int voff, int soff, f32x4 v)
{
    if (dt == DT_F32) {
        const u32x4 q = __builtin_bit_cast(u32x4, v);
        __builtin_amdgcn_raw_buffer_store_b128(q, rs, 4 * voff, 4 * soff, 0);
        asm volatile("s_nop 3" ::"v"(q) : "memory");
    } else if (dt == DT_BF16) {
        const u32x2 q = {pack_bf16(v.x, v.y), pack_bf16(v.z, v.w)};
        __builtin_amdgcn_raw_buffer_store_b64(q, rs, 2 * voff, 2 * soff, 0);
        asm volatile("s_nop 3" ::"v"(q) : "memory");
    } else {
        typedef __attribute__((ext_vector_type(2))) _Float16 h2;
        const h2 a = {(_Float16)v.x, (_Float16)v.y}, c = {(_Float16)v.z, (_Float16)v.w};
        const u32x2 q = {__builtin_bit_cast(uint32_t, a), __builtin_bit_cast(uint32_t, c)};
        __builtin_amdgcn_raw_buffer_store_b64(q, rs, 2 * voff, 2 * soff, 0);
        asm volatile("s_nop 3" ::"v"(q) : "memory");
    }
}

// Steps of B and x kept in LDS (requested ring - 1 steps ahead, into the next chunk at most).  A ring of 8 was
// measured too (chunk 256 only): same time, so the requests are not what the kernel waits for.
constexpr int kRingSteps = 4;
template <int SPC> constexpr int ring_of() { return kRingSteps <= SPC ? kRingSteps : 4; }

// x ring + two weight slots: a chunk's weights are written half a chunk ahead, while the current chunk's are in use
template <int NT, int SPC> constexpr int wave_lds() { return ring_of<SPC>() * 2048 + 2 * 32 * SPC * 4; }
constexpr int kStage = 2048;        // per wave: two 16 x 16 fp32 blocks of the state on their way to memory
template <int NT, int SPC> constexpr int lds_bytes() { return ring_of<SPC>() * NT * 1024 + 4 * (wave_lds<NT, SPC>() + kStage); }

// NT = dstate / 16 (4 or 8); SPC = 32-token steps per chunk (chunk_size / 32: 4 or 8);
// F32IO = out and initial states are fp32 (or the latter absent): element-type branches fold away.
// CO = chunk states only (kernels/ssd_chunk_state.py:202-232): a workgroup walks p.n_seg-th of the chunks, the
// accumulators restart from zero at every chunk boundary and what they held goes to states[:, c - 1]; nothing is
// carried from chunk to chunk, so the segments of a sequence are independent workgroups.
template <int NT, int SPC, bool HAS_SEQ, bool F32IO, bool CO>
__global__ void __launch_bounds__(256, 2) quad_kernel(const Params p)
{
    constexpr int Q = 32 * SPC;
    constexpr int kRing = ring_of<SPC>(), kDist = kRing - 1;
    constexpr int TPL = Q / 64;         // tokens per lane when the chunk's weights are computed (2 or 4)
    constexpr int NTW = NT / 4;         // B tile blocks (32 tokens x 16 columns, 1 KB) a wave fetches per step
    extern __shared__ __attribute__((aligned(16))) char lds[];
    const int lane = threadIdx.x & 63, i16 = lane & 15, kg = lane >> 4;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    char *bring = lds;                                                   // kRing x NT blocks of 1 KB, shared
    char *xring = lds + kRing * NT * 1024 + wave * wave_lds<NT, SPC>();  // kRing slots x (32 tokens x 64 bytes)
    char *wbuf = xring + kRing * 2048;                                   // 2 slots x Q weights
    char *stage = lds + kRing * NT * 1024 + 4 * wave_lds<NT, SPC>() + wave * kStage;

    // Work item -> (batch, head, row slice); the four items of a workgroup share batch and group (checked on the
    // host).  Consecutive workgroups sit on the same XCD (workgroups are dealt round-robin over the p.n_xcd XCDs), so
    // a batch's B is fetched from HBM by one or two L2 slices only.
    const int n_wg = p.n_items >> 2, n_seg = CO ? p.n_seg : 1;
    const int per_xcd = (n_wg * n_seg + p.n_xcd - 1) / p.n_xcd;          // workgroups per XCD
    const int vwg = (int)(blockIdx.x % p.n_xcd) * per_xcd + (int)(blockIdx.x / p.n_xcd);
    if (vwg >= n_wg * n_seg) return;                                     // whole workgroup: no barrier is skipped
    int wg = vwg, c0 = 0, c1 = p.C;
    if (CO) {
        // (batch, segment) pairs one after the other: the workgroups running side by side on an XCD read the
        // same B rows
        const int wpb = n_wg / p.batch, bs = vwg / wpb, cps = (p.C + n_seg - 1) / n_seg;
        wg = (bs / n_seg) * wpb + vwg % wpb;
        c0 = (bs % n_seg) * cps;
        c1 = min(p.C, c0 + cps);
        if (c0 >= c1) return;
    }
    const int item = 4 * wg + wave;
    const int n_pt = p.headdim >> 5;
    const int pt = item % n_pt;
    const int r1 = item / n_pt;
    const int h = r1 % p.nheads;
    const int b = r1 / p.nheads;
    const int C = c1, L = p.seqlen;      // chunks at and beyond c1 are not this workgroup's: never requested
    const int g = h / (p.nheads / p.ngroups);
    const int p0 = pt * 32;
    const int dt_out = F32IO ? (int)DT_F32 : (CO ? p.dt_states : p.dt_out), dt_init = F32IO ? (int)DT_F32 : p.dt_init;

    const char *xrow = (const char *)p.x + 2 * (b * p.sx_b + h * p.sx_h);
    const char *Brow = (const char *)p.B + 2 * (b * p.sB_b + g * p.sB_g);
    const int64_t xrb = 2 * p.sx_l, Brb = 2 * p.sB_l;            // row pitch in bytes
    // descriptor of chunk c: base = its first token, extent = the tokens that exist (none past the last chunk)
    auto chunk_rsrc = [&](const char *base, int64_t pitch, int c) {
        const int cc = c < C ? c : 0;
        return make_rsrc(base + (int64_t)cc * Q * pitch, c < C ? (int64_t)(L - c * Q) * pitch : 0);
    };
    const float *dtb = p.dt + b * p.sdt_b + h * p.sdt_h;
    const float *dab = p.dacs + b * p.sda_b + h * p.sda_h;
    const int32_t *sqb = HAS_SEQ ? p.seq + b * p.ssq_b : nullptr;

    // ---- request helpers -------------------------------------------------------------------------------------
    // A step's B tile (32 tokens x dstate) sits in LDS as NT blocks of 1 KB, block (th, pair) = 16 tokens (token
    // half th) x 32 columns (column pair `pair`), row-major: one request fetches a block, lane l the 16 bytes
    // (token l/4, piece l%4) -- four adjacent lanes read 64 contiguous bytes, which the memory pipeline merges into
    // one request (every lane in another row would cost four times the cycles there) -- and deposits them at byte
    // 16*l.  For the tokens 8..15 of a block the two 32-byte halves are swapped (piece ^ 2), see the reads below.
    const int Blane = (int)((lane >> 2) * Brb) + 16 * ((lane & 3) ^ ((lane >> 5) << 1));
    auto load_B = [&](__amdgpu_buffer_rsrc_t rs, int s, int bi) {       // block bi of step s of the chunk behind rs
#if defined(__HIP_DEVICE_COMPILE__)      // the LDS address space does not exist in the host pass
        typedef __attribute__((address_space(3))) void *lds_ptr;
        const int th = bi / (NT / 2), pair = bi % (NT / 2);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lds_ptr)(bring + ((s % kRing) * NT + bi) * 1024), 16, Blane,
                                                 (int)((32 * s + 16 * th) * Brb) + 64 * pair, 0, 0);
#else
        (void)rs; (void)s; (void)bi; (void)Blane;
#endif
    };
    // The transposing read for (16 columns `it`, tokens 8kg + 4*half .. +3): lane (i16, kg) addresses the 8 bytes
    // of token 8kg + 4*half + i16/4, columns 4*(i16%4)..+3 of that column block and receives column i16 of those
    // four tokens.  Token 8kg + 4*half + j is row 8*(kg%2) + 4*half + j of block (kg/2, it/2), and the column block
    // is the 32-byte half it%2 of the row -- swapped for kg odd, so that the lane groups kg and kg + 1, 512 bytes
    // apart, touch different banks.  Btr[it%2] holds the lane's part of the address.
    // The reads are written as inline assembly with explicit s_waitcnt: given the intrinsic, the compiler orders
    // every such read behind ALL outstanding loads that write LDS (s_waitcnt vmcnt(0)), which would serialise the
    // three-steps-ahead requests with their use.
    uint32_t Btr[2];
    Btr[0] = (kg >> 1) * (NT / 2) * 1024 + (8 * (kg & 1) + (i16 >> 2)) * 64 + (kg & 1) * 32 + (i16 & 3) * 8;   // + 256 * half
    Btr[1] = Btr[0] ^ 32;
#if defined(__HIP_DEVICE_COMPILE__)
    Btr[0] += (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char *)bring;
    Btr[1] += (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char *)bring;
#endif
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Wunused-lambda-capture"   // the host pass sees no use of Btr
    const uint32_t Btr0 = Btr[0], Btr1 = Btr[1];
    auto read_Bt = [&, Btr0, Btr1](auto slotc, auto itc, u32x2 &lo, u32x2 &hi) {    // ring slot, column block
        constexpr int it = decltype(itc)::value;
        constexpr int off = (decltype(slotc)::value * NT + (it >> 1)) * 1024;
#if defined(__HIP_DEVICE_COMPILE__)
        asm volatile("ds_read_b64_tr_b16 %0, %2 offset:%3\n\tds_read_b64_tr_b16 %1, %2 offset:%4"
                     : "=&v"(lo), "=&v"(hi) : "v"((it & 1) ? Btr1 : Btr0), "n"(off), "n"(off + 256) : "memory");
#else
        lo = hi = (u32x2){0u, 0u}; (void)Btr0; (void)Btr1; (void)off;
#endif
    };
#pragma clang diagnostic pop
    // The results of a read_Bt become valid here.  LDS operations complete in order, so the pair has arrived once
    // no more LDS operations are outstanding than were issued after it: nc = that number, at least.
    auto wait_Bt = [&](auto nc, u32x2 &lo, u32x2 &hi) {
#if defined(__HIP_DEVICE_COMPILE__)
        asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(lo), "+v"(hi) : "n"(decltype(nc)::value) : "memory");
#else
        (void)lo; (void)hi;
#endif
    };
    // x: two requests cover the 32 token rows of a step, 4 lanes per 64-byte row of the slice; lane l deposits
    // its 16 bytes at byte 16*l of a 1 KB block.  Request i fetches tokens 8*kg' + 4*i + m into row slot
    // 4*m + kg' (kg' = (l/4)%4, m = l/16), so the four kg groups of an operand read below hit different banks.
    const int xlane = (int)((8 * ((lane >> 2) & 3) + (lane >> 4)) * xrb) + 2 * p0 + 16 * (lane & 3);
    auto load_x = [&](__amdgpu_buffer_rsrc_t rs, int s, int i) {
#if defined(__HIP_DEVICE_COMPILE__)
        typedef __attribute__((address_space(3))) void *lds_ptr;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lds_ptr)(xring + (s % kRing) * 2048 + i * 1024), 16, xlane,
                                                 (int)((32 * s + 4 * i) * xrb), 0, 0);
#else
        (void)rs; (void)s; (void)i; (void)xlane;
#endif
    };
    const int xst_rd = 64 * kg + 4 * i16;     // + 2048 * slot + 1024 * (j/4) + 256 * (j%4) for token 8kg + j

    // decay inputs of a chunk: TPL consecutive tokens per lane, plus the chunk-level scalars
    struct Meta { float dtv[TPL], cs[TPL], last; int32_t id[TPL], id_last; };
    auto load_meta = [&](int c) {
        Meta m;
        const int cc = c < C ? c : C - 1;
        const float *dtp = dtb + cc * p.sdt_c + TPL * lane;
        const float *dap = dab + cc * p.sda_c + TPL * lane;
        if constexpr (TPL == 4) {
            const f32x4 a = *(const f32x4 *)dtp, d = *(const f32x4 *)dap;
            m.dtv[0] = a.x; m.dtv[1] = a.y; m.dtv[2] = a.z; m.dtv[3] = a.w;
            m.cs[0] = d.x; m.cs[1] = d.y; m.cs[2] = d.z; m.cs[3] = d.w;
        } else {
            const f32x2 a = *(const f32x2 *)dtp, d = *(const f32x2 *)dap;
            m.dtv[0] = a.x; m.dtv[1] = a.y; m.cs[0] = d.x; m.cs[1] = d.y;
        }
        m.last = dab[cc * p.sda_c + (Q - 1)];
        m.id_last = 0;
#pragma unroll
        for (int t = 0; t < TPL; ++t) m.id[t] = 0;
        if (HAS_SEQ) {
#pragma unroll
            for (int t = 0; t < TPL; ++t) m.id[t] = sqb[(int64_t)min(cc * Q + TPL * lane + t, L - 1) * p.ssq_l];
            m.id_last = sqb[(int64_t)(min((cc + 1) * Q, L) - 1) * p.ssq_l];
        }
        return m;
    };
    // per-token weights of chunk c (kernels/ssd_chunk_state.py:134-156) -> weight slot ws
    auto put_weights = [&](int c, int ws, const Meta &m) {
        float w[TPL];
#pragma unroll
        for (int t = 0; t < TPL; ++t) {
            float e = m.last - m.cs[t];
            if (p.clamp) e = fminf(e, 0.f);
            w[t] = __expf(e) * m.dtv[t];
            if (c * Q + TPL * lane + t >= L) w[t] = 0.f;
            if (HAS_SEQ && m.id[t] != m.id_last) w[t] = 0.f;
        }
        if constexpr (TPL == 4) *(f32x4 *)(wbuf + ws * Q * 4 + 16 * lane) = (f32x4){w[0], w[1], w[2], w[3]};
        else *(f32x2 *)(wbuf + ws * Q * 4 + 8 * lane) = (f32x2){w[0], w[1]};
    };

    // ---- operand helpers -------------------------------------------------------------------------------------
    // x dwords (token, headdim row pair i16) and weights of the 8 tokens 8kg..8kg+7 of step s
    auto read_operands = [&](int s, int ws, uint32_t (&xr)[8], float (&wv)[8]) {
#pragma unroll
        for (int j = 0; j < 8; ++j)
            xr[j] = *(const uint32_t *)(xring + (s % kRing) * 2048 + xst_rd + 1024 * (j >> 2) + 256 * (j & 3));
        const f32x4 wlo = *(const f32x4 *)(wbuf + ws * Q * 4 + 4 * (32 * s + 8 * kg));
        const f32x4 whi = *(const f32x4 *)(wbuf + ws * Q * 4 + 4 * (32 * s + 8 * kg + 4));
        wv[0] = wlo.x; wv[1] = wlo.y; wv[2] = wlo.z; wv[3] = wlo.w;
        wv[4] = whi.x; wv[5] = whi.y; wv[6] = whi.z; wv[7] = whi.w;
    };
    // tokens (2q, 2q+1) of headdim row 2*i16 + jp: x * w in fp32, split into bf16 hi + bf16 lo
    auto frag_piece = [&](int q, int jp, const uint32_t (&xr)[8], const float (&wv)[8], Frag &f) {
        const uint32_t r0 = xr[2 * q], r1_ = xr[2 * q + 1];
        const float x0 = __builtin_bit_cast(float, jp ? (r0 & 0xffff0000u) : (r0 << 16));
        const float x1 = __builtin_bit_cast(float, jp ? (r1_ & 0xffff0000u) : (r1_ << 16));
        uint32_t hp = pack_bf16(x0 * wv[2 * q], x1 * wv[2 * q + 1]);
        asm volatile("" : "+v"(hp));      // keeps the compiler from converting the product a second time to get h0
        const float h0 = __builtin_bit_cast(float, hp << 16);
        const float h1 = __builtin_bit_cast(float, hp & 0xffff0000u);
        f.hi[jp][q] = hp;
        // the residual of the exact product, as a fused multiply-add everywhere: left to the compiler, some copies
        // of this code would subtract from the rounded product instead and the bits would depend on the copy
        f.lo[jp][q] = pack_bf16(__builtin_fmaf(x0, wv[2 * q], -h0), __builtin_fmaf(x1, wv[2 * q + 1], -h1));
    };

    // ---- state ---------------------------------------------------------------------------------------------
    // acc[it][jp][r]: dstate column 16*it + 4*kg + r of headdim row p0 + 2*i16 + jp
    f32x4 acc[NT][2];
    const int64_t slice_out = (int64_t)(p.headdim - 1) * (CO ? p.sst_p : p.so_p) + p.dstate;
    const int64_t slice_fin = (int64_t)(p.headdim - 1) * p.sf_p + p.dstate;
    auto store_state = [&](__amdgpu_buffer_rsrc_t rs, int dt, int row_pitch) {
        // The accumulators hold a 16 x 16 block as (lane%16 = row, lane/16 = group of four columns): neighbouring
        // lanes sit in different rows, 512 bytes apart, and the memory pipeline, which merges only what adjacent
        // lanes address, would take every lane's 16 bytes as a request of its own (measured: 64 cycles of the
        // compute unit's store path per instruction instead of 16).  So each block passes through 1 KB of LDS and
        // comes back as (lane/4 = row, lane%4 = group): four adjacent lanes then write 64 contiguous bytes.  The
        // column group is XORed with row/4 in LDS, which keeps both the 16-byte writes and reads off shared banks.
        const int voff = (p0 + 2 * (lane >> 2)) * row_pitch + 4 * (lane & 3);
        f32x4 *wr = (f32x4 *)(stage + i16 * 64 + ((kg ^ (i16 >> 2)) << 4));
        const f32x4 *rd = (const f32x4 *)(stage + (lane >> 2) * 64 + (((lane & 3) ^ (lane >> 4)) << 4));
        if (dt != DT_F32) {
            // 16-bit destination: the two blocks (it, jp = 0 / 1) -- the same 16 columns of adjacent rows -- go
            // through LDS together and come back as (lane/4 = row pair, (lane/2)%2 = jp, lane%2 = 8 columns), so
            // that every lane stores 16 bytes: half the store instructions of the 32-bit case
            const int i = lane >> 2, jq = (lane >> 1) & 1, half = lane & 1;
            const int voff2 = (p0 + 2 * i + jq) * row_pitch + 8 * half;
            const char *rd2 = stage + jq * 1024 + i * 64;
            char *wr1 = stage + 1024 + i16 * 64 + ((kg ^ (i16 >> 2) ^ 1) << 4);
            const int sw = (i >> 2) ^ jq;       // block 1 is shifted by one column group: the two blocks of a read
                                                // instruction then sit on different banks
            // (the pair it + 1 is written and read back -- LDS operations of a wave execute in order -- before the
            // pair it is converted and stored, so that its reads have returned by then)
            f32x4 a[NT], d[NT];
#pragma unroll
            for (int k = 0; k <= NT; ++k) {
                if (k < NT) {
                    *wr = acc[k][0];
                    *(f32x4 *)((char *)wr1) = acc[k][1];
                    a[k] = *(const f32x4 *)(rd2 + (((2 * half) ^ sw) << 4));
                    d[k] = *(const f32x4 *)(rd2 + (((2 * half + 1) ^ sw) << 4));
                }
                if (k >= 1) {
                    const int it = k - 1;
                    const f32x4 u = a[it], w = d[it];
                    u32x4 q;
                    if (dt == DT_BF16) {
                        q = (u32x4){pack_bf16(u.x, u.y), pack_bf16(u.z, u.w), pack_bf16(w.x, w.y), pack_bf16(w.z, w.w)};
                    } else {
                        typedef __attribute__((ext_vector_type(2))) _Float16 h2;
                        const h2 e0 = {(_Float16)u.x, (_Float16)u.y}, e1 = {(_Float16)u.z, (_Float16)u.w};
                        const h2 e2 = {(_Float16)w.x, (_Float16)w.y}, e3 = {(_Float16)w.z, (_Float16)w.w};
                        q = (u32x4){__builtin_bit_cast(uint32_t, e0), __builtin_bit_cast(uint32_t, e1),
                                    __builtin_bit_cast(uint32_t, e2), __builtin_bit_cast(uint32_t, e3)};
                    }
                    __builtin_amdgcn_raw_buffer_store_b128(q, rs, 2 * voff2, 2 * (16 * it), 0);
                    asm volatile("s_nop 3" ::"v"(q) : "memory");
                }
            }
            return;
        }
        // LDS operations of one wave execute in order, so block k + 1 may be written right behind the read of
        // block k; the store of a block follows kLag blocks later, when its read has long returned
        constexpr int kLag = 4;
        f32x4 v[2 * NT];
#pragma unroll
        for (int k = 0; k < 2 * NT + kLag; ++k) {
            if (k < 2 * NT) {
                *wr = acc[k >> 1][k & 1];
                v[k] = *rd;
            }
            if (k >= kLag) {
                const int j = k - kLag;
                store4(rs, dt, voff, (j & 1) * row_pitch + 16 * (j >> 1), v[j]);
            }
        }
    };
#pragma unroll
    for (int it = 0; it < NT; ++it)
#pragma unroll
        for (int jp = 0; jp < 2; ++jp) {
            acc[it][jp] = (f32x4){0.f, 0.f, 0.f, 0.f};
            if (!CO && p.init) {
                const int64_t off = b * p.sin_b + h * p.sin_h + (int64_t)(p0 + 2 * i16 + jp) * p.sin_p + 16 * it + 4 * kg;
                if (dt_init == DT_F32) {
                    acc[it][jp] = *(const f32x4 *)((const float *)p.init + off);
                } else {
                    const uint16_t *src = (const uint16_t *)p.init + off;
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        acc[it][jp][r] = dt_init == DT_BF16 ? bf16_bits_to_f32(src[r])
                                                            : (float)__builtin_bit_cast(_Float16, src[r]);
                }
            }
        }

    // ---- prologue: rows past the end of the sequence are not fetched and leave their LDS slots untouched; their
    // weight is zero, so the slots only have to hold finite numbers.
#pragma unroll
    for (int i = 0; i < 2 * kRing; ++i) *(u32x4 *)(xring + i * 1024 + 16 * lane) = (u32x4){0u, 0u, 0u, 0u};
#pragma unroll
    for (int i = 0; i < kRing * NTW; ++i)
        *(u32x4 *)(bring + (i * 4 + wave) * 1024 + 16 * lane) = (u32x4){0u, 0u, 0u, 0u};
    __builtin_amdgcn_s_waitcnt(0xc07f);          // lgkmcnt(0): the zeros are in place before any row lands
    __builtin_amdgcn_s_barrier();
    Meta mcur = load_meta(c0);
    __amdgpu_buffer_rsrc_t rsx0 = chunk_rsrc(xrow, xrb, c0), rsx1 = chunk_rsrc(xrow, xrb, c0 + 1);
    __amdgpu_buffer_rsrc_t rsB0 = chunk_rsrc(Brow, Brb, c0), rsB1 = chunk_rsrc(Brow, Brb, c0 + 1);
    // requests of the steps 0..kDist-1, in the order (x, x, B...) that every later step keeps
#pragma unroll
    for (int s = 0; s < kDist; ++s) {
        load_x(rsx0, s, 0); load_x(rsx0, s, 1);
#pragma unroll
        for (int k = 0; k < NTW; ++k) load_B(rsB0, s, wave * NTW + k);
        __builtin_amdgcn_sched_barrier(0);
    }
    put_weights(c0, 0, mcur);
    Frag fA, fB;
    // B operands (transposed blocks) travel kAhead iterations ahead of the MFMAs that use them, across the step
    // boundaries of a chunk: block t of the stream of (step, tile) pairs sits in slot t % 4.  An LDS read takes longer
    // than the four MFMAs of one iteration, so a single block in flight would leave the matrix pipe waiting every
    // iteration.  These are asynchronous results of inline assembly, which the compiler takes for complete: a value it
    // has to carry around the chunk loop, or past its end, it may copy or overwrite before the data is there.  So none
    // is in flight at the end of a chunk: the first blocks of a chunk are read at its top (the build checks the
    // generated code for such copies, isa_check.py).
    constexpr int kAhead = 3;
    static_assert(NT % 4 == 0 && kAhead < 4 && kAhead <= NT, "slot of a block = its tile index % 4");
    // vector-memory operations of one store_state, at least (a 16-bit `out` takes NT stores, a 32-bit one 2 NT; the
    // waits below may count fewer operations than were issued, never more)
    constexpr int kStores = F32IO ? 2 * NT : NT;
    // the loop's vector-memory queue, replayed at compile time: 2 x requests and NT / 4 B requests per step, the state
    // stores at the first step of every chunk
    constexpr tile::schedule::Loop kLoop{2, NT / 4, kStores, SPC, kDist, kRing};
    static_assert(tile::schedule::slots_ok(kLoop), "ring slots are reused too early");
    static_assert(tile::schedule::wait_prologue(kLoop) == (kDist - 1) * (2 + NTW), "prologue wait");
    u32x2 blo[4], bhi[4];
    {
        // everything up to this wave's B blocks of step 0 has landed: the requests of two steps were issued later
        __builtin_amdgcn_s_waitcnt(vmcnt_imm((kDist - 1) * (2 + NTW)));
        __builtin_amdgcn_s_barrier();   // ... and every other wave's blocks of step 0
        asm volatile("" ::: "memory");
        uint32_t xr[8]; float wv[8];
        read_operands(0, 0, xr, wv);
#pragma unroll
        for (int q = 0; q < 4; ++q) { frag_piece(q, 0, xr, wv, fA); frag_piece(q, 1, xr, wv, fA); }
        __builtin_amdgcn_sched_barrier(0);
    }
    int32_t prev_id = 0;
    Meta mnext = mcur;

    // One 32-token step s of chunk c (weight slot ws): fc = x operands of this step, fn receives those of step + 1.
    // Vector-memory requests of a step, in program order: [the state stores, step 0 only], the two x requests of
    // step + 3 (iteration 0), this wave's B requests of step + 3 (after the barrier in iteration NT - kAhead).
    // Memory operations complete in order and the compiler does not track loads that write LDS, so the waits for
    // them are explicit: "no more outstanding than were issued after the one needed".
    auto step = [&](int c, auto sc, int ws, Frag &fc, Frag &fn) {
        constexpr int s = decltype(sc)::value;
        // x rows of step + 1 (this wave's own, requested two steps ago): behind them came the B requests of that
        // step and all requests of the steps s + 2 - kDist .. s - 1 (with the state stores, if step 0 is among them)
        constexpr bool st_top = s >= 1 && s <= kDist - 2;         // step 0 among them
        static_assert(tile::schedule::wait_x(kLoop, s) == NTW + (kDist - 2) * (2 + NTW) + (st_top ? kStores : 0),
                      "wait for the x rows of step + 1");
        __builtin_amdgcn_s_waitcnt(vmcnt_imm(NTW + (kDist - 2) * (2 + NTW) + (st_top ? kStores : 0)));
        asm volatile("" ::: "memory");
        uint32_t xr[8]; float wv[8];
        if (s + 1 < SPC) read_operands(s + 1, ws, xr, wv);
        else read_operands(0, ws ^ 1, xr, wv);

        if (CO && s == 0) {
            // chunk boundary: states[:, c - 1] = what the previous chunk summed up, then start again from zero.  The
            // first chunk of the segment has nothing to hand over: its stores go through a descriptor of extent
            // zero, which drops them -- the waits count a boundary's stores whether or not they reach memory.
            const int cp = c > c0 ? c - 1 : c0;
            store_state(make_rsrc((char *)p.states + (b * p.sst_b + cp * p.sst_c + h * p.sst_h) * esize_of(dt_out),
                                  c > c0 ? slice_out * esize_of(dt_out) : 0), dt_out, (int)p.sst_p);
#pragma unroll
            for (int it = 0; it < NT; ++it)
#pragma unroll
                for (int jp = 0; jp < 2; ++jp) acc[it][jp] = (f32x4){0.f, 0.f, 0.f, 0.f};
        }
        if (!CO && s == 0) {
            // chunk boundary: out[:, c] = state entering the chunk, then s <- exp(dA_chunk) * s
            store_state(make_rsrc((char *)p.out + (b * p.so_b + c * p.so_c + h * p.so_h) * esize_of(dt_out),
                                  slice_out * esize_of(dt_out)), dt_out, (int)p.so_p);
            float sc = __expf(mcur.last);
            if (HAS_SEQ) {
                if (mcur.id_last != prev_id) sc = 0.f;
                prev_id = mcur.id_last;
            }
#pragma unroll
            for (int it = 0; it < NT; ++it)
#pragma unroll
                for (int jp = 0; jp < 2; ++jp) acc[it][jp] *= sc;
        }
        // requests of this step: x rows and this wave's B blocks of step + 3 (this chunk or the next)
        const auto rsB = s + kDist < SPC ? rsB0 : rsB1;
        const auto rsx = s + kDist < SPC ? rsx0 : rsx1;
        const int s3 = (s + kDist) % SPC;
        const bf16x8 h0 = __builtin_bit_cast(bf16x8, (u32x4){fc.hi[0][0], fc.hi[0][1], fc.hi[0][2], fc.hi[0][3]});
        const bf16x8 h1 = __builtin_bit_cast(bf16x8, (u32x4){fc.hi[1][0], fc.hi[1][1], fc.hi[1][2], fc.hi[1][3]});
        const bf16x8 l0 = __builtin_bit_cast(bf16x8, (u32x4){fc.lo[0][0], fc.lo[0][1], fc.lo[0][2], fc.lo[0][3]});
        const bf16x8 l1 = __builtin_bit_cast(bf16x8, (u32x4){fc.lo[1][0], fc.lo[1][1], fc.lo[1][2], fc.lo[1][3]});
        __builtin_amdgcn_sched_barrier(0);   // stores and operand reads above, the requests of this step below
        static_for<NT>([&](auto itc) {
            constexpr int it = decltype(itc)::value;
            // the blocks read behind this one (two reads each) may still be in flight: kAhead - 1 of them, fewer at the
            // end of a chunk's last step, where the next chunk's first blocks are not read yet
            constexpr int behind = s + 1 < SPC || NT - 1 - it > kAhead - 1 ? kAhead - 1 : NT - 1 - it;
            wait_Bt(std::integral_constant<int, 2 * behind>{}, blo[it % 4], bhi[it % 4]);
            const bf16x8 Bt = __builtin_bit_cast(bf16x8, (u32x4){blo[it % 4].x, blo[it % 4].y, bhi[it % 4].x, bhi[it % 4].y});
            if constexpr (it == NT - kAhead) {
                // The next read is the first of step + 1's tile: this wave's blocks of it (requested three steps
                // ago) have landed once only the requests of step - 1 and the x requests of this step (with the
                // stores, if either was step 0) are outstanding; the barrier publishes every wave's blocks.  It
                // also tells that all waves are through with the tile of step - 1, whose ring slot the B requests
                // below overwrite.
                constexpr bool st_mid = s < kDist - 1;       // step 0 among the steps s + 2 - kDist .. s
                static_assert(tile::schedule::wait_b(kLoop, s) == (kDist - 2) * (2 + NTW) + 2 + (st_mid ? kStores : 0),
                              "wait for the B blocks of step + 1");
                __builtin_amdgcn_s_waitcnt(vmcnt_imm((kDist - 2) * (2 + NTW) + 2 + (st_mid ? kStores : 0)));
                __builtin_amdgcn_s_barrier();
                asm volatile("" ::: "memory");
            }
            {
                constexpr int tn = it + kAhead;     // block kAhead iterations on: this step's tile or the next one's
                if constexpr (tn < NT || s + 1 < SPC)       // (the next chunk's first blocks: at its top)
                    read_Bt(std::integral_constant<int, (tn < NT ? s : s + 1) % kRing>{}, std::integral_constant<int, tn % NT>{},
                            blo[tn % 4], bhi[tn % 4]);
            }
            acc[it][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(Bt, h0, acc[it][0], 0, 0, 0);
            acc[it][1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(Bt, h1, acc[it][1], 0, 0, 0);
            acc[it][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(Bt, l0, acc[it][0], 0, 0, 0);
            acc[it][1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(Bt, l1, acc[it][1], 0, 0, 0);
            // next step's x operands, one or two eighths per iteration
#pragma unroll
            for (int e = it * 8 / NT; e < (it + 1) * 8 / NT; ++e) frag_piece(e >> 1, e & 1, xr, wv, fn);
            if (it == 0) { load_x(rsx, s3, 0); load_x(rsx, s3, 1); }
            if (it >= NT - kAhead && it < NT - kAhead + NTW) load_B(rsB, s3, wave * NTW + (it - (NT - kAhead)));
            if (s == 1 && it == NT - 1) mnext = load_meta(c + 1);
            __builtin_amdgcn_sched_barrier(0);
        });
        if (s == SPC / 2) put_weights(c + 1, ws ^ 1, mnext);
    };

    for (int c = c0; c < C; ++c) {
        const int ws = (c - c0) & 1;
        // the first blocks of step 0, whose tile every wave has published (prologue, or the barrier of the last step)
        __builtin_amdgcn_sched_barrier(0);
        static_for<kAhead>([&](auto ic) {
            constexpr int i = decltype(ic)::value;
            read_Bt(std::integral_constant<int, 0>{}, ic, blo[i], bhi[i]);
        });
        __builtin_amdgcn_sched_barrier(0);
        step(c, std::integral_constant<int, 0>{}, ws, fA, fB);
        step(c, std::integral_constant<int, 1>{}, ws, fB, fA);
        step(c, std::integral_constant<int, 2>{}, ws, fA, fB);
        step(c, std::integral_constant<int, 3>{}, ws, fB, fA);
        if constexpr (SPC == 8) {
            step(c, std::integral_constant<int, 4>{}, ws, fA, fB);
            step(c, std::integral_constant<int, 5>{}, ws, fB, fA);
            step(c, std::integral_constant<int, 6>{}, ws, fA, fB);
            step(c, std::integral_constant<int, 7>{}, ws, fB, fA);
        }
        mcur = mnext;
        rsx0 = rsx1; rsB0 = rsB1;
        rsx1 = chunk_rsrc(xrow, xrb, c + 2);
        rsB1 = chunk_rsrc(Brow, Brb, c + 2);
    }
    if (CO)
        store_state(make_rsrc((char *)p.states + (b * p.sst_b + (C - 1) * p.sst_c + h * p.sst_h) * esize_of(dt_out),
                              slice_out * esize_of(dt_out)), dt_out, (int)p.sst_p);
    else
        store_state(make_rsrc(p.fin + b * p.sf_b + h * p.sf_h, slice_fin * 4), DT_F32, (int)p.sf_p);
}

static bool aligned(const void *ptr, size_t a) { return ((uintptr_t)ptr % a) == 0; }

// what both uses of the kernel ask of the inputs
static bool inputs_ok(const Params &p)
{
    if (p.dt_in != DT_BF16) return false;
    if (p.headdim % 32 != 0) return false;
    if (p.dstate != 64 && p.dstate != 128) return false;
    if (p.Q != 128 && p.Q != 256) return false;
    if (((p.nheads / p.ngroups) * (p.headdim / 32)) % 4 != 0) return false;      // 4 tiles of one (batch, group)
    if (!aligned(p.x, 16) || (p.sx_b | p.sx_l | p.sx_h) % 8) return false;
    if (!aligned(p.B, 16) || (p.sB_b | p.sB_l | p.sB_g) % 8) return false;
    if ((int64_t)p.Q * 2 * p.sx_l >= (1LL << 31) || (int64_t)p.Q * 2 * p.sB_l >= (1LL << 31)) return false;
    if (p.sdt_k != 1 || p.sda_k != 1) return false;
    if (!aligned(p.dt, 16) || (p.sdt_b | p.sdt_h | p.sdt_c) % 4) return false;
    if (!aligned(p.dacs, 16) || (p.sda_b | p.sda_h | p.sda_c) % 4) return false;
    return true;
}

// rows of 16-byte pieces: fp32 rows start on multiples of 4 elements, 16-bit rows on multiples of 8
static bool rows_ok(const void *ptr, int dt, int64_t strides_or, int64_t row_stride, int headdim)
{
    return aligned(ptr, 16) && strides_or % (dt == DT_F32 ? 4 : 8) == 0 && (int64_t)headdim * row_stride < (1LL << 28);
}

}  // namespace quad

// The four-tiles-per-workgroup kernel serves the fused call without a `states` output, for bf16 x / B with 16-byte
// aligned rows, unit-stride dt / dA_cumsum rows, and head counts that put four tiles of one group in a workgroup.
bool quad_supported(const Params &p)
{
    using namespace quad;
    if (p.states || !p.out || !p.fin) return false;
    if (!inputs_ok(p)) return false;
    if (!rows_ok(p.out, p.dt_out, p.so_b | p.so_c | p.so_h | p.so_p, p.so_p, p.headdim)) return false;
    if (!rows_ok(p.fin, DT_F32, p.sf_b | p.sf_h | p.sf_p, p.sf_p, p.headdim)) return false;
    if (p.init && !rows_ok(p.init, p.dt_init, p.sin_b | p.sin_h | p.sin_p, p.sin_p, p.headdim)) return false;
    return true;
}

bool quad_inputs_supported(const Params &p) { return quad::inputs_ok(p); }

// ... and the chunk-state call (`states` only), under the same conditions.
bool quad_chunk_state_supported(const Params &p)
{
    using namespace quad;
    if (!p.states || p.out || p.fin) return false;
    if (!inputs_ok(p)) return false;
    return rows_ok(p.states, p.dt_states, p.sst_b | p.sst_c | p.sst_h | p.sst_p, p.sst_p, p.headdim);
}

template <int NT, int SPC, bool SEQ, bool F32IO, bool CO>
static hipError_t launch_quad_k(const Params &p, dim3 grid, hipStream_t s)
{
    constexpr int lds = quad::lds_bytes<NT, SPC>();
    static std::atomic<uint64_t> configured{0};
    const hipError_t e = ensure_dynamic_lds((const void *)quad::quad_kernel<NT, SPC, SEQ, F32IO, CO>, lds, configured);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL((quad::quad_kernel<NT, SPC, SEQ, F32IO, CO>), grid, dim3(256), lds, s, p);
    return hipGetLastError();
}

template <int NT, int SPC, bool CO>
static hipError_t launch_quad_t(const Params &p, hipStream_t s)
{
    dim3 grid((((p.n_items >> 2) * (CO ? p.n_seg : 1) + p.n_xcd - 1) / p.n_xcd) * p.n_xcd);
    const bool f32io = CO ? p.dt_states == DT_F32 : p.dt_out == DT_F32 && (!p.init || p.dt_init == DT_F32);
    if (p.seq) return f32io ? launch_quad_k<NT, SPC, true, true, CO>(p, grid, s) : launch_quad_k<NT, SPC, true, false, CO>(p, grid, s);
    return f32io ? launch_quad_k<NT, SPC, false, true, CO>(p, grid, s) : launch_quad_k<NT, SPC, false, false, CO>(p, grid, s);
}

template <bool CO>
static hipError_t launch_quad_c(const Params &p, hipStream_t s)
{
    const int nt = p.dstate / 16, spc = p.Q / 32;
    if (nt == 8 && spc == 8) return launch_quad_t<8, 8, CO>(p, s);
    if (nt == 8 && spc == 4) return launch_quad_t<8, 4, CO>(p, s);
    if (nt == 4 && spc == 8) return launch_quad_t<4, 8, CO>(p, s);
    return launch_quad_t<4, 4, CO>(p, s);
}

hipError_t launch_quad(const Params &p_in, hipStream_t s)
{
    Params p = p_in;
    p.n_items = p.batch * p.nheads * (p.headdim / 32);
    if (p.n_items <= 0) return hipSuccess;
    if (p.n_cu <= 0) p.n_cu = 256;
    p.n_xcd = p.n_cu >= 32 ? p.n_cu / 32 : 1;       // an XCD is 32 compute units on this part
    return launch_quad_c<false>(p, s);
}

// 0 = choose; otherwise the chunks a workgroup walks in the chunk-state launch (process-wide tuning hook, atomic)
static std::atomic<int> g_segment_chunks{0};
int set_quad_segment_chunks(int n) { return g_segment_chunks.exchange(n); }

hipError_t launch_quad_chunk_state(const Params &p_in, hipStream_t s)
{
    Params p = p_in;
    p.n_items = p.batch * p.nheads * (p.headdim / 32);
    if (p.n_items <= 0 || p.C <= 0) return hipSuccess;
    if (p.n_cu <= 0) p.n_cu = 256;
    p.n_xcd = p.n_cu >= 32 ? p.n_cu / 32 : 1;
    // Chunks per workgroup.  Measured times follow  (workgroups per compute unit, rounded up) x (chunks per
    // workgroup + 0.4): a workgroup's first requests have nothing to hide behind, which costs about 0.4 of a chunk,
    // and the compute unit with the most workgroups finishes last (b=4 L=8192 H=80: 190 / 162 / 160 / 177 / 219 us
    // for 1 / 2 / 4 / 8 / 32 chunks per workgroup).
    int cps = g_segment_chunks.load(std::memory_order_relaxed);
    if (cps <= 0) {
        double best = 0;
        for (int k = 1; k <= p.C; ++k) {
            const int nseg = (p.C + k - 1) / k;
            const int per_cu = ((p.n_items >> 2) * nseg + p.n_cu - 1) / p.n_cu;
            const double t = per_cu * (k + 0.4);
            if (cps <= 0 || t < best) { best = t; cps = k; }
        }
    }
    if (cps > p.C) cps = p.C;
    p.n_seg = (p.C + cps - 1) / cps;
    return launch_quad_c<true>(p, s);
}

}  // namespace ssd
