// The consumer of the passed states: the state-dependent half of the chunk scan,
//   y[b, cQ+m, h, p] = scale_m * sum_n C[b, cQ+m, g, n] * prev_states[b, c, h, p, n],
//   scale_m = exp(dA_cumsum[b, h, c, m]) * [seq_idx[b, cQ+m] == seq_idx[b, cQ-1]]   (the latter 0 for the first chunk)
// (kernels/ssd_chunk_scan.py:94-117).  The reference rounds the states to the element type of C before its dot;
// here an fp32 state enters the bf16 MFMAs as bf16 hi + bf16 lo, so the result follows the fp32 mathematics.
//
// One workgroup (four waves) takes one (batch, chunk, head, block of 64 or 32 headdim rows):
//   * the state block (rows x dstate fp32) is fetched once into LDS by buffer loads with LDS destination; every
//     wave converts it into its A operands (lane (i, kg): 8 consecutive dstate values of row 16j + i) and keeps them
//     in registers for the whole chunk;
//   * each wave owns a quarter of the chunk's tokens and walks it in blocks of 16 tokens: the C rows of a block
//     arrive in a private double-buffered LDS area (again loaded straight into LDS, one block ahead), are read
//     back as B operands (lane (i, kg): 8 consecutive dstate values of token i), and 2 * PB * NK MFMAs produce
//     D[p][token];
//   * accumulator register r of row block j is headdim row 16j + 4kg + r of token i: the four registers are 16
//     contiguous bytes of y, but adjacent lanes are different tokens.  The memory pipeline merges only what adjacent
//     lanes address, so the block passes through LDS and leaves as (lane / pieces = token, lane % pieces = 16-byte
//     piece): whole token rows per store.
// LDS tiles are row-major with the 16-byte piece index XORed with the row number: the loads with LDS destination
// fix where a lane's 16 bytes land (consecutive lanes, consecutive pieces), so the swizzle is applied on the
// global side, and the operand reads (16 lanes = 16 rows, same piece) then touch 16 different bank groups.
#include "ssd_tile.h"

namespace ssd {

namespace scan {

using namespace tile;      // register types, pack_bf16, make_rsrc, vmcnt_imm (ssd_tile.h)

// 16 bytes per lane from a buffer straight into LDS: lane l lands at byte 16 * l behind `dst`
__device__ __forceinline__ void load_to_lds(__amdgpu_buffer_rsrc_t rs, char *dst, int voff, int soff)
{
#if defined(__HIP_DEVICE_COMPILE__)      // the LDS address space does not exist in the host pass
    typedef __attribute__((address_space(3))) void *lds_ptr;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lds_ptr)dst, 16, voff, soff, 0, 0);
#else
    (void)rs; (void)dst; (void)voff; (void)soff;
#endif
}

// Four consecutive values of one y row (element offsets voff per lane + soff uniform) in y's element type,
// optionally added to what is there.  PLAIN: fp32, overwrite.  The data registers of a wide store are read out over
// several cycles after issue; the wait states that depend on them keep a following writer of the same registers away.
template <bool PLAIN>
__device__ __forceinline__ void store_y(__amdgpu_buffer_rsrc_t rsO, int dt_out, int accumulate, int voff, int soff, f32x4 v)
{
    if (PLAIN || dt_out == DT_F32) {
        if (!PLAIN && accumulate) {
            const u32x4 o = __builtin_amdgcn_raw_buffer_load_b128(rsO, 4 * voff, 4 * soff, 0);
            v += __builtin_bit_cast(f32x4, o);
        }
        const u32x4 q = __builtin_bit_cast(u32x4, v);
        __builtin_amdgcn_raw_buffer_store_b128(q, rsO, 4 * voff, 4 * soff, 0);
        asm volatile("s_nop 3" ::"v"(q) : "memory");
    } else {
        const bool bf = dt_out == DT_BF16;
        if (accumulate) {
            const u32x2 o = __builtin_amdgcn_raw_buffer_load_b64(rsO, 2 * voff, 2 * soff, 0);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const uint32_t w = (e & 1) ? (o[e >> 1] >> 16) : (o[e >> 1] & 0xffffu);
                v[e] += bf ? bf16_bits_to_f32(w) : (float)__builtin_bit_cast(_Float16, (uint16_t)w);
            }
        }
        u32x2 q;
        if (bf) {
            q = (u32x2){pack_bf16(v.x, v.y), pack_bf16(v.z, v.w)};
        } else {
            typedef __attribute__((ext_vector_type(2))) _Float16 h2;
            const h2 a = {(_Float16)v.x, (_Float16)v.y}, d = {(_Float16)v.z, (_Float16)v.w};
            q = (u32x2){__builtin_bit_cast(uint32_t, a), __builtin_bit_cast(uint32_t, d)};
        }
        __builtin_amdgcn_raw_buffer_store_b64(q, rsO, 2 * voff, 2 * soff, 0);
        asm volatile("s_nop 3" ::"v"(q) : "memory");
    }
}

// Eight consecutive values of one y row as 16-bit elements: one 16-byte store (and load, when accumulating).
__device__ __forceinline__ void store_y8(__amdgpu_buffer_rsrc_t rsO, int dt_out, int accumulate, int voff, int soff, f32x4 a, f32x4 d)
{
    const bool bf = dt_out == DT_BF16;
    float v[8] = {a.x, a.y, a.z, a.w, d.x, d.y, d.z, d.w};
    if (accumulate) {
        const u32x4 o = __builtin_amdgcn_raw_buffer_load_b128(rsO, 2 * voff, 2 * soff, 0);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const uint32_t w = (e & 1) ? (o[e >> 1] >> 16) : (o[e >> 1] & 0xffffu);
            v[e] += bf ? bf16_bits_to_f32(w) : (float)__builtin_bit_cast(_Float16, (uint16_t)w);
        }
    }
    u32x4 q;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        if (bf) {
            q[e] = pack_bf16(v[2 * e], v[2 * e + 1]);
        } else {
            typedef __attribute__((ext_vector_type(2))) _Float16 h2;
            const h2 t = {(_Float16)v[2 * e], (_Float16)v[2 * e + 1]};
            q[e] = __builtin_bit_cast(uint32_t, t);
        }
    }
    __builtin_amdgcn_raw_buffer_store_b128(q, rsO, 2 * voff, 2 * soff, 0);
    asm volatile("s_nop 3" ::"v"(q) : "memory");
}

template <int NK, int PB, bool S16 = false> constexpr int state_lds() { return PB * 16 * NK * 32 * (S16 ? 2 : 4); }   // rows x dstate
template <int NK, int PB> constexpr int wave_lds() { return 2 * 16 * NK * 32 * 2 + 16 * PB * 16 * 4; }   // 2 C blocks + y block
template <int NK, int PB, bool S16 = false> constexpr int lds_bytes() { return state_lds<NK, PB, S16>() + 4 * wave_lds<NK, PB>(); }

// NK = dstate / 32 (2 or 4); PB = headdim rows of the item / 16 (2 or 4); MB = 16-token blocks per wave = Q / 64;
// PLAIN = y is fp32 and overwritten (the element-type and accumulate branches fold away);
// S16 = the states are bf16 (what the reference hands its scan, kernels/ssd_chunk_scan.py:108): a row of the state is
// an MFMA operand as it lies in memory -- half the bytes, no hi + lo split, half the MFMAs.
template <int NK, int PB, int MB, bool PLAIN, bool S16>
__global__ void __launch_bounds__(256, 2) scan_states_kernel(const ScanParams p)
{
    constexpr int N = 32 * NK;
    constexpr int SE = S16 ? 2 : 4;     // bytes per state element
    constexpr int PRS = N * SE / 16;    // 16-byte pieces per state row
    constexpr int SWZ = PRS < 16 ? PRS - 1 : 15;     // row bits XORed into the piece index of a state row in LDS
    constexpr int PRC = N / 8;          // 16-byte pieces per C row (bf16)
    constexpr int OP = PB * 4;          // 16-byte pieces per y row of the item (fp32)
    constexpr int SI = PB * 16 * PRS / 64 / 4;   // state load instructions per wave
    constexpr int CI = 16 * PRC / 64;            // load instructions per C block
    extern __shared__ __attribute__((aligned(16))) char lds[];
    const int lane = threadIdx.x & 63, i16 = lane & 15, kg = lane >> 4;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    char *sld = lds;
    char *cbuf = lds + state_lds<NK, PB, S16>() + wave * wave_lds<NK, PB>();
    char *obuf = cbuf + 2 * 16 * N * 2;

    // item -> (batch, chunk, head, row block): row blocks and heads vary fastest, so the workgroups in flight share
    // the C rows of few (batch, chunk) pairs
    const int n_pt = p.headdim / (16 * PB);
    int item = blockIdx.x;
    const int pt = item % n_pt; item /= n_pt;
    const int h = item % p.nheads; item /= p.nheads;
    const int c = item % p.C;
    const int b = item / p.C;
    const int g = h / (p.nheads / p.ngroups);
    const int p0 = pt * 16 * PB;

    // per-token scale of every block of this wave (kernels/ssd_chunk_scan.py:86-88, 101-104), before any request
    // that the explicit waits below count
    float sc[MB];
    {
        const float *da = p.dacs + b * p.sda_b + h * p.sda_h + c * p.sda_c;
        int32_t prev = 0;
        if (p.seq && c >= 1) prev = p.seq[b * p.ssq_b + (int64_t)(c * p.Q - 1) * p.ssq_l];
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
            const int k = wave * 16 * MB + 16 * mb + i16;
            float s = __expf(da[(int64_t)k * p.sda_k]);
            if (p.seq) {
                const int l = c * p.Q + k;
                const int32_t id = l < p.seqlen ? p.seq[b * p.ssq_b + (int64_t)l * p.ssq_l] : -1;
                if (id != prev) s = 0.f;
            }
            sc[mb] = s;
        }
    }

    // ---- requests: the state block (all waves together), then this wave's first two C blocks
    const int64_t s_pitch = p.sst_p * SE;           // bytes
    const auto rsS = make_rsrc((const char *)p.states + SE * (b * p.sst_b + c * p.sst_c + h * p.sst_h + (int64_t)p0 * p.sst_p),
                               (int64_t)(16 * PB - 1) * s_pitch + N * SE);
#pragma unroll
    for (int i = 0; i < SI; ++i) {
        const int ins = wave * SI + i;                                  // covers LDS pieces 64 * ins .. + 63
        const int row = ins * (64 / PRS) + lane / PRS;
        const int q = (lane % PRS) ^ (row & SWZ);
        load_to_lds(rsS, sld + ins * 1024, row * (int)s_pitch + q * 16, 0);
    }
    const int64_t c_pitch = p.sC_l * 2;
    // descriptors start at the chunk's first token (byte offsets inside one are 32-bit: the limit is then a chunk's
    // extent, not the sequence's) and end with the sequence
    const int chunk_tokens = min(p.Q, p.seqlen - c * p.Q), wtok0 = wave * 16 * MB;
    const auto rsC = make_rsrc((const char *)p.Cm + 2 * (b * p.sC_b + g * p.sC_g) + (int64_t)c * p.Q * c_pitch,
                               (int64_t)(chunk_tokens - 1) * c_pitch + N * 2);
    // token (within the block) and global piece of this lane for load instruction i of a C block
    auto load_C = [&](int mb, int buf) {
#pragma unroll
        for (int i = 0; i < CI; ++i) {
            const int t = i * (64 / PRC) + lane / PRC;
            const int q = (lane % PRC) ^ (t & (PRC - 1));
            load_to_lds(rsC, cbuf + buf * 16 * N * 2 + i * 1024, t * (int)c_pitch + q * 16,
                        (wtok0 + 16 * mb) * (int)c_pitch);
        }
    };
    load_C(0, 0);
    if (MB > 1) load_C(1, 1);
    __builtin_amdgcn_sched_barrier(0);

    // ---- the state block as A operands: hi + lo bf16 of row 16j + i16, dstate 32ks + 8kg .. + 7
    // The compiler does not track loads that write LDS: wait until only the C requests are outstanding, then the
    // barrier publishes every wave's part.
    __builtin_amdgcn_s_waitcnt(vmcnt_imm(MB > 1 ? 2 * CI : CI));
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    u32x4 shi[PB][NK], slo[PB][NK];
#pragma unroll
    for (int j = 0; j < PB; ++j)
#pragma unroll
        for (int ks = 0; ks < NK; ++ks) {
            if constexpr (S16) {
                shi[j][ks] = *(const u32x4 *)(sld + (16 * j + i16) * (N * 2) + (((4 * ks + kg) ^ (i16 & SWZ)) << 4));
                slo[j][ks] = (u32x4){0u, 0u, 0u, 0u};
                continue;
            }
            const int q0 = 8 * ks + 2 * kg;
            const char *rowp = sld + (16 * j + i16) * (N * 4);
            const f32x4 a = *(const f32x4 *)(rowp + ((q0 ^ i16) << 4));
            const f32x4 d = *(const f32x4 *)(rowp + (((q0 + 1) ^ i16) << 4));
            const float v[8] = {a.x, a.y, a.z, a.w, d.x, d.y, d.z, d.w};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const uint32_t hp = pack_bf16(v[2 * e], v[2 * e + 1]);
                const float h0 = __builtin_bit_cast(float, hp << 16);
                const float h1 = __builtin_bit_cast(float, hp & 0xffff0000u);
                shi[j][ks][e] = hp;
                slo[j][ks][e] = pack_bf16(v[2 * e] - h0, v[2 * e + 1] - h1);
            }
        }

    const int64_t o_pitch = p.so_l;                 // elements
    const int esz = p.dt_out == DT_F32 ? 4 : 2;
    const auto rsO = make_rsrc((char *)p.out + esz * (b * p.so_b + h * p.so_h + p0 + (int64_t)c * p.Q * o_pitch),
                               ((int64_t)(chunk_tokens - 1) * o_pitch + 16 * PB) * esz);

    // ---- 16-token blocks.  Vector-memory operations of this wave from here on, in program order per block:
    // the C requests of block mb + 2, then the block's PB stores (preceded by PB loads when accumulating; the
    // waits below do not count those, which only makes them wait longer).
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        // C block mb has landed once no more operations are outstanding than were issued behind its requests
        // (a 16-bit y leaves as PB / 2 stores of 16 bytes; counting fewer operations than were issued is safe)
        constexpr int kNext = CI, kSt = PLAIN ? PB : PB / 2;
        const int behind = mb == 0 ? (MB > 1 ? kNext : 0)
                         : mb == 1 ? (MB > 2 ? kNext : 0) + kSt
                                   : kSt + (mb + 1 < MB ? kNext : 0) + kSt;
        // (the switch keeps the immediate a constant after unrolling)
        if (behind == 0) __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
        else if (behind == kNext) __builtin_amdgcn_s_waitcnt(vmcnt_imm(kNext));
        else if (behind == kSt) __builtin_amdgcn_s_waitcnt(vmcnt_imm(kSt));
        else if (behind == kNext + kSt) __builtin_amdgcn_s_waitcnt(vmcnt_imm(kNext + kSt));
        else if (behind == 2 * kSt) __builtin_amdgcn_s_waitcnt(vmcnt_imm(2 * kSt));
        else __builtin_amdgcn_s_waitcnt(vmcnt_imm(kNext + 2 * kSt));
        asm volatile("" ::: "memory");

        const char *cb = cbuf + (mb & 1) * 16 * N * 2 + i16 * (PRC * 16);
        bf16x8 cf[NK];
#pragma unroll
        for (int ks = 0; ks < NK; ++ks)
            cf[ks] = __builtin_bit_cast(bf16x8, *(const u32x4 *)(cb + ((((4 * ks + kg) ^ i16) & (PRC - 1)) << 4)));

        f32x4 acc[PB];
#pragma unroll
        for (int j = 0; j < PB; ++j) acc[j] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < NK; ++ks)
#pragma unroll
            for (int j = 0; j < PB; ++j)
                acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, shi[j][ks]), cf[ks], acc[j], 0, 0, 0);
        if constexpr (!S16) {
#pragma unroll
            for (int ks = 0; ks < NK; ++ks)
#pragma unroll
                for (int j = 0; j < PB; ++j)
                    acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, slo[j][ks]), cf[ks], acc[j], 0, 0, 0);
        }

        // the C operands are in registers (the MFMAs above read them): the buffer can take block mb + 2
        __builtin_amdgcn_sched_barrier(0);
        if (mb + 2 < MB) load_C(mb + 2, mb & 1);
        __builtin_amdgcn_sched_barrier(0);

        // y block through LDS: written as (token i16, piece 4j + kg), read as (token lane / OP, piece lane % OP)
#pragma unroll
        for (int j = 0; j < PB; ++j)
            *(f32x4 *)(obuf + i16 * (OP * 16) + ((((4 * j + kg) ^ i16) & (OP - 1)) << 4)) = acc[j] * sc[mb];
        if (!PLAIN && p.dt_out != DT_F32) {
            // 16-bit y: a lane takes two adjacent pieces of a token row, eight values, and stores 16 bytes
            constexpr int OP2 = OP / 2;
            f32x4 ya[PB / 2], yd[PB / 2];
#pragma unroll
            for (int r = 0; r < PB / 2; ++r) {
                const int t = r * (64 / OP2) + lane / OP2, pp = lane % OP2;
                ya[r] = *(const f32x4 *)(obuf + t * (OP * 16) + ((((2 * pp) ^ t) & (OP - 1)) << 4));
                yd[r] = *(const f32x4 *)(obuf + t * (OP * 16) + ((((2 * pp + 1) ^ t) & (OP - 1)) << 4));
            }
#pragma unroll
            for (int r = 0; r < PB / 2; ++r) {
                const int t = r * (64 / OP2) + lane / OP2, pp = lane % OP2;
                store_y8(rsO, p.dt_out, p.accumulate, t * (int)o_pitch + 8 * pp, (wtok0 + 16 * mb) * (int)o_pitch, ya[r], yd[r]);
            }
            continue;
        }
        f32x4 yv[PB];
#pragma unroll
        for (int r = 0; r < PB; ++r) {
            const int t = r * (64 / OP) + lane / OP;
            yv[r] = *(const f32x4 *)(obuf + t * (OP * 16) + ((((lane % OP) ^ t) & (OP - 1)) << 4));
        }
#pragma unroll
        for (int r = 0; r < PB; ++r) {
            const int t = r * (64 / OP) + lane / OP;
            const int piece = lane % OP;
            f32x4 v = yv[r];
            const int voff = t * (int)o_pitch + 4 * piece;              // elements, from the block's first token
            const int soff = (wtok0 + 16 * mb) * (int)o_pitch;
            store_y<PLAIN>(rsO, p.dt_out, p.accumulate, voff, soff, v);
        }
    }
}

// Second decomposition, for headdim % 64 == 0 and contiguous dA_cumsum rows: one workgroup takes one (batch, chunk),
// a block of 64 headdim rows and a run of `hb` heads of one group.  The chunk's C rows are fetched once into LDS
// and serve every head of the run; the state block of head i + 1 is requested (into the other half of a double
// buffer) before the work on head i starts, so its latency hides behind 128 MFMAs per wave.  Wave w owns the 16
// rows p0 + 16w .. + 15 of the block for ALL tokens of the chunk: the state is converted to bf16 hi + lo once per
// head and wave (not once per wave as above would need for whole rows), and a wave's results are 64 contiguous bytes
// per token, passed through 1 KB of LDS so that four adjacent lanes write them.
template <int NK, int MBT> constexpr int heads_lds()       // C tile + 2 state blocks + 2 dA_cumsum rows + 4 y blocks
{
    return 16 * MBT * NK * 64 + 2 * 64 * NK * 128 + 2 * 1024 + 4 * 1024;     // chunk_size <= 256: a row fits 1 KB
}

// NK = dstate / 32; MBT = chunk_size / 16
template <int NK, int MBT, bool PLAIN>
__global__ void __launch_bounds__(256, 1) scan_states_heads_kernel(const ScanParams p, int hb)
{
    constexpr int N = 32 * NK, Q = 16 * MBT;
    constexpr int PRS = N / 4, PRC = N / 8;
    constexpr int SI = 64 * PRS / 64 / 4;        // state load instructions per wave and head
    constexpr int CI = Q * PRC / 64 / 4;         // C load instructions per wave
    static_assert(Q * 4 <= 1024, "one request fetches a dA_cumsum row");
    extern __shared__ __attribute__((aligned(16))) char lds[];
    const int lane = threadIdx.x & 63, i16 = lane & 15, kg = lane >> 4;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    char *cld = lds;                                      // [Q tokens][N bf16], pieces swizzled
    char *sld = cld + Q * N * 2;                          // 2 x [64 rows][N fp32], pieces swizzled
    char *dld = sld + 2 * 64 * N * 4;                     // 2 x 1 KB: [Q] fp32 (a request always deposits 1 KB)
    char *obuf = dld + 2 * 1024 + wave * 1024;            // [16 tokens][64 bytes], pieces swizzled

    const int n_pt = p.headdim >> 6;
    const int runs = p.nheads / hb;
    int item = blockIdx.x;
    const int pt = item % n_pt; item /= n_pt;
    const int run = item % runs; item /= runs;
    const int c = item % p.C;
    const int b = item / p.C;
    const int h0 = run * hb;
    const int g = h0 / (p.nheads / p.ngroups);
    const int p0 = pt * 64;

    // tokens of this chunk whose sequence differs from the one the chunk's incoming state belongs to: bit mb of
    // `dead` = token 16 mb + i16 (kernels/ssd_chunk_scan.py:86-88, 101-104)
    uint32_t dead = 0;
    if (p.seq) {
        const int32_t prev = c >= 1 ? p.seq[b * p.ssq_b + (int64_t)(c * Q - 1) * p.ssq_l] : 0;
#pragma unroll
        for (int mb = 0; mb < MBT; ++mb) {
            const int l = c * Q + 16 * mb + i16;
            const int32_t id = l < p.seqlen ? p.seq[b * p.ssq_b + (int64_t)l * p.ssq_l] : -1;
            dead |= (id != prev ? 1u : 0u) << mb;
        }
    }

    // ---- requests.  State block and dA_cumsum row of head i -> buffer i % 2.
    const int64_t s_pitch = p.sst_p * 4;
    auto request_head = [&](int i) {
        const int h = h0 + i;
        const auto rsS = make_rsrc((const char *)p.states + 4 * (b * p.sst_b + c * p.sst_c + h * p.sst_h + (int64_t)p0 * p.sst_p),
                                   (int64_t)63 * s_pitch + N * 4);
#pragma unroll
        for (int k = 0; k < SI; ++k) {
            const int ins = wave * SI + k;
            const int row = ins * (64 / PRS) + lane / PRS;
            const int q = (lane % PRS) ^ (row & 15);
            load_to_lds(rsS, sld + (i & 1) * 64 * N * 4 + ins * 1024, row * (int)s_pitch + q * 16, 0);
        }
        if (wave == 0) {
            const auto rsD = make_rsrc(p.dacs + b * p.sda_b + h * p.sda_h + c * p.sda_c, Q * 4);
            load_to_lds(rsD, dld + (i & 1) * 1024, 16 * lane, 0);      // lanes past the row are out of range: zeros
        }
    };
    {
        const int64_t c_pitch = p.sC_l * 2;
        const auto rsC = make_rsrc((const char *)p.Cm + 2 * (b * p.sC_b + g * p.sC_g) + (int64_t)c * Q * c_pitch,
                                   (int64_t)(min(Q, p.seqlen - c * Q) - 1) * c_pitch + N * 2);
#pragma unroll
        for (int k = 0; k < CI; ++k) {
            const int ins = wave * CI + k;
            const int t = ins * (64 / PRC) + lane / PRC;                // token within the chunk
            const int q = (lane % PRC) ^ (t & (PRC - 1));
            load_to_lds(rsC, cld + ins * 1024, t * (int)c_pitch + q * 16, 0);
        }
    }
    request_head(0);
    __builtin_amdgcn_sched_barrier(0);

    const int64_t o_pitch = p.so_l;
    const int esz = p.dt_out == DT_F32 ? 4 : 2;
    const int voff = (lane >> 2) * (int)o_pitch + 4 * (lane & 3);       // after the pass through LDS: token lane / 4
    char *owr = obuf + i16 * 64 + ((kg ^ (i16 >> 2)) << 4);
    const char *ord = obuf + (lane >> 2) * 64 + (((lane & 3) ^ (lane >> 4)) << 4);

    for (int i = 0; i < hb; ++i) {
        // Everything requested for head i (and, the first time, the C tile) has landed: behind those requests this
        // wave only issued the stores of head i - 1.  The compiler does not track loads that write LDS, so the wait
        // is explicit; the barrier publishes the other waves' parts and tells that every wave is done with head
        // i - 1, whose buffers the requests for head i + 1 overwrite.
        if (i == 0) __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
        else __builtin_amdgcn_s_waitcnt(vmcnt_imm(MBT));
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        if (i + 1 < hb) request_head(i + 1);
        __builtin_amdgcn_sched_barrier(0);

        const int h = h0 + i;
        // this wave's 16 state rows as A operands: hi + lo bf16 of row 16 wave + i16, dstate 32 ks + 8 kg .. + 7
        u32x4 shi[NK], slo[NK];
        const char *rowp = sld + (i & 1) * 64 * N * 4 + (16 * wave + i16) * (N * 4);
#pragma unroll
        for (int ks = 0; ks < NK; ++ks) {
            const int q0 = 8 * ks + 2 * kg;
            const f32x4 a = *(const f32x4 *)(rowp + ((q0 ^ i16) << 4));
            const f32x4 d = *(const f32x4 *)(rowp + (((q0 + 1) ^ i16) << 4));
            const float v[8] = {a.x, a.y, a.z, a.w, d.x, d.y, d.z, d.w};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                uint32_t hp = pack_bf16(v[2 * e], v[2 * e + 1]);
                asm volatile("" : "+v"(hp));
                const float f0 = __builtin_bit_cast(float, hp << 16);
                const float f1 = __builtin_bit_cast(float, hp & 0xffff0000u);
                shi[ks][e] = hp;
                slo[ks][e] = pack_bf16(v[2 * e] - f0, v[2 * e + 1] - f1);
            }
        }
        const auto rsO = make_rsrc((char *)p.out + esz * (b * p.so_b + h * p.so_h + p0 + 16 * wave + (int64_t)c * Q * o_pitch),
                                   ((int64_t)(min(Q, p.seqlen - c * Q) - 1) * o_pitch + 16) * esz);
        const float *dal = (const float *)(dld + (i & 1) * 1024);

        // Software pipeline over the 16-token blocks: the C operands of block mb + 1 are read before the MFMAs of
        // block mb, and a block's result is written to LDS, read back (issued at once: LDS operations of a wave
        // execute in order) and stored only after the MFMAs of the next block, so that no LDS latency is waited for.
        auto read_C = [&](int mb, bf16x8 (&cf)[NK]) {
            const char *cb = cld + (16 * mb + i16) * (PRC * 16);
#pragma unroll
            for (int ks = 0; ks < NK; ++ks)
                cf[ks] = __builtin_bit_cast(bf16x8, *(const u32x4 *)(cb + ((((4 * ks + kg) ^ i16) & (PRC - 1)) << 4)));
        };
        bf16x8 cfn[NK];
        read_C(0, cfn);
        f32x4 vprev = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int mb = 0; mb < MBT; ++mb) {
            bf16x8 cf[NK];
#pragma unroll
            for (int ks = 0; ks < NK; ++ks) cf[ks] = cfn[ks];
            if (mb + 1 < MBT) read_C(mb + 1, cfn);
            float sc = __expf(dal[16 * mb + i16]);
            if ((dead >> mb) & 1) sc = 0.f;
            // two independent accumulation chains (hi and lo halves of the state)
            f32x4 ah = {0.f, 0.f, 0.f, 0.f}, al = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < NK; ++ks) {
                ah = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, shi[ks]), cf[ks], ah, 0, 0, 0);
                al = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, slo[ks]), cf[ks], al, 0, 0, 0);
            }
            if (mb > 0) store_y<PLAIN>(rsO, p.dt_out, p.accumulate, voff, (16 * (mb - 1)) * (int)o_pitch, vprev);
            // acc[r] = y[token 16 mb + i16][row 4 kg + r]: through LDS to (token lane / 4, 16-byte piece lane % 4)
            *(f32x4 *)owr = (ah + al) * sc;
            vprev = *(const f32x4 *)ord;
        }
        store_y<PLAIN>(rsO, p.dt_out, p.accumulate, voff, (16 * (MBT - 1)) * (int)o_pitch, vprev);
    }
}

// Any element types, any dstate / headdim / chunk size: one thread per output element.
__global__ void __launch_bounds__(256) scan_states_generic_kernel(const ScanParams p)
{
    const int64_t total = (int64_t)p.batch * p.seqlen * p.nheads * p.headdim;
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * blockDim.x) {
        const int pp = (int)(idx % p.headdim);
        int64_t r = idx / p.headdim;
        const int h = (int)(r % p.nheads); r /= p.nheads;
        const int l = (int)(r % p.seqlen);
        const int b = (int)(r / p.seqlen);
        const int c = l / p.Q, k = l - c * p.Q;
        const int g = h / (p.nheads / p.ngroups);
        float s = __expf(p.dacs[b * p.sda_b + h * p.sda_h + c * p.sda_c + (int64_t)k * p.sda_k]);
        if (p.seq) {
            const int32_t prev = c >= 1 ? p.seq[b * p.ssq_b + (int64_t)(c * p.Q - 1) * p.ssq_l] : 0;
            if (p.seq[b * p.ssq_b + (int64_t)l * p.ssq_l] != prev) s = 0.f;
        }
        const int64_t co = b * p.sC_b + (int64_t)l * p.sC_l + g * p.sC_g;
        const int64_t so = b * p.sst_b + c * p.sst_c + h * p.sst_h + (int64_t)pp * p.sst_p;
        float acc = 0.f;
        for (int n = 0; n < p.dstate; ++n)
            acc += load_as_f32(p.Cm, co + n, p.dt_C) * load_as_f32(p.states, so + n, p.dt_states);
        const int64_t oo = b * p.so_b + (int64_t)l * p.so_l + h * p.so_h + pp;
        float y = acc * s;
        if (p.accumulate) y += load_as_f32(p.out, oo, p.dt_out);
        store_from_f32(p.out, oo, p.dt_out, y);
    }
}

static bool aligned(const void *ptr, size_t a) { return ((uintptr_t)ptr % a) == 0; }

}  // namespace scan

// The MFMA kernel serves bf16 C and fp32 states with 16-byte aligned rows, dstate 64 / 128, chunk sizes 64 / 128 / 256
// and headdim a multiple of 32.
bool scan_states_mfma_supported(const ScanParams &p)
{
    using scan::aligned;
    if (p.dt_C != DT_BF16 || (p.dt_states != DT_F32 && p.dt_states != DT_BF16)) return false;
    if (p.dstate != 64 && p.dstate != 128) return false;
    if (p.Q != 64 && p.Q != 128 && p.Q != 256) return false;
    if (p.headdim % 32 != 0) return false;
    if (!aligned(p.Cm, 16) || !aligned(p.states, 16) || !aligned(p.out, 16)) return false;
    if ((p.sC_b | p.sC_l | p.sC_g) % 8 != 0) return false;
    if ((p.sst_b | p.sst_c | p.sst_h | p.sst_p) % (p.dt_states == DT_F32 ? 4 : 8) != 0) return false;
    const int per16 = p.dt_out == DT_F32 ? 4 : 8;
    if ((p.so_b | p.so_l | p.so_h) % per16 != 0) return false;
    // byte offsets inside one descriptor are 32-bit; the descriptors of C and y cover one chunk
    if ((int64_t)p.Q * p.sC_l * 2 >= 0x7fffffffLL || (int64_t)p.Q * p.so_l * (p.dt_out == DT_F32 ? 4 : 2) >= 0x7fffffffLL) return false;
    if ((int64_t)p.headdim * p.sst_p * 4 >= 0x7fffffffLL) return false;
    return (int64_t)p.batch * p.C * p.nheads * (p.headdim / 32) < 0x7fffffffLL;
}

template <int NK, int PB, int MB, bool PLAIN, bool S16 = false>
static hipError_t launch_scan_k(const ScanParams &p, hipStream_t s)
{
    constexpr int lds = scan::lds_bytes<NK, PB, S16>();
    static std::atomic<uint64_t> configured{0};
    const hipError_t e = ensure_dynamic_lds((const void *)scan::scan_states_kernel<NK, PB, MB, PLAIN, S16>, lds, configured);
    if (e != hipSuccess) return e;
    const int64_t items = (int64_t)p.batch * p.C * p.nheads * (p.headdim / (16 * PB));
    hipLaunchKernelGGL((scan::scan_states_kernel<NK, PB, MB, PLAIN, S16>), dim3((unsigned)items), dim3(256), lds, s, p);
    return hipGetLastError();
}

template <int NK, int PB>
static hipError_t launch_scan_q(const ScanParams &p, hipStream_t s)
{
    const bool plain = p.dt_out == DT_F32 && !p.accumulate;
    if (p.dt_states == DT_BF16) {
        switch (p.Q) {
        case 64: return plain ? launch_scan_k<NK, PB, 1, true, true>(p, s) : launch_scan_k<NK, PB, 1, false, true>(p, s);
        case 128: return plain ? launch_scan_k<NK, PB, 2, true, true>(p, s) : launch_scan_k<NK, PB, 2, false, true>(p, s);
        default: return plain ? launch_scan_k<NK, PB, 4, true, true>(p, s) : launch_scan_k<NK, PB, 4, false, true>(p, s);
        }
    }
    switch (p.Q) {
    case 64: return plain ? launch_scan_k<NK, PB, 1, true>(p, s) : launch_scan_k<NK, PB, 1, false>(p, s);
    case 128: return plain ? launch_scan_k<NK, PB, 2, true>(p, s) : launch_scan_k<NK, PB, 2, false>(p, s);
    default: return plain ? launch_scan_k<NK, PB, 4, true>(p, s) : launch_scan_k<NK, PB, 4, false>(p, s);
    }
}

template <int NK, int MBT, bool PLAIN>
static hipError_t launch_heads_k(const ScanParams &p, int hb, hipStream_t s)
{
    constexpr int lds = scan::heads_lds<NK, MBT>();
    static std::atomic<uint64_t> configured{0};
    const hipError_t e = ensure_dynamic_lds((const void *)scan::scan_states_heads_kernel<NK, MBT, PLAIN>, lds, configured);
    if (e != hipSuccess) return e;
    const int64_t items = (int64_t)p.batch * p.C * (p.nheads / hb) * (p.headdim / 64);
    hipLaunchKernelGGL((scan::scan_states_heads_kernel<NK, MBT, PLAIN>), dim3((unsigned)items), dim3(256), lds, s, p, hb);
    return hipGetLastError();
}

template <int NK, int MBT>
static hipError_t launch_heads_q(const ScanParams &p, int hb, hipStream_t s)
{
    return p.dt_out == DT_F32 && !p.accumulate ? launch_heads_k<NK, MBT, true>(p, hb, s) : launch_heads_k<NK, MBT, false>(p, hb, s);
}

// 0 = choose, 1 = one workgroup per head, 2 = runs of heads (process-wide tuning hook, atomic)
static std::atomic<int> g_scan_kernel_hook{0};

int set_scan_kernel(int k)
{
    return g_scan_kernel_hook.exchange(k);
}

hipError_t launch_scan_states(const ScanParams &p, hipStream_t s)
{
    if ((int64_t)p.batch * p.seqlen * p.nheads * p.headdim == 0) return hipSuccess;
    const int g_scan_kernel = g_scan_kernel_hook.load(std::memory_order_relaxed);
    if (scan_states_mfma_supported(p) && p.dt_states == DT_F32 && g_scan_kernel != 1 && p.headdim % 64 == 0 && p.sda_k == 1 &&
        ((uintptr_t)p.dacs % 16) == 0 && (p.sda_b | p.sda_h | p.sda_c) % 4 == 0) {
        // runs of heads: the longest divisor of the heads per group up to 10 (enough workgroups to fill the chip
        // matter more than the last bit of C reuse)
        const int per_group = p.nheads / p.ngroups;
        int hb = 1;
        for (int d = 2; d <= 10; ++d)
            if (per_group % d == 0) hb = d;
        const bool small = (int64_t)p.batch * p.C * (p.nheads / hb) * (p.headdim / 64) < 512;
        // measured at the Mamba2-2.7B layer shape: 229 us against 257 us for fp32 y written plainly; with bf16 y or
        // accumulation the one-workgroup-per-head kernel is the faster one (196 / 419 us against 208 / 576 us)
        const bool plain = p.dt_out == DT_F32 && !p.accumulate;
        if (g_scan_kernel == 2 || (!small && plain)) {
            if (p.dstate == 128) {
                switch (p.Q) {
                case 64: return launch_heads_q<4, 4>(p, hb, s);
                case 128: return launch_heads_q<4, 8>(p, hb, s);
                default: return launch_heads_q<4, 16>(p, hb, s);
                }
            }
            switch (p.Q) {
            case 64: return launch_heads_q<2, 4>(p, hb, s);
            case 128: return launch_heads_q<2, 8>(p, hb, s);
            default: return launch_heads_q<2, 16>(p, hb, s);
            }
        }
    }
    if (scan_states_mfma_supported(p)) {
        const bool wide = p.headdim % 64 == 0;
        if (p.dstate == 128) return wide ? launch_scan_q<4, 4>(p, s) : launch_scan_q<4, 2>(p, s);
        return wide ? launch_scan_q<2, 4>(p, s) : launch_scan_q<2, 2>(p, s);
    }
    const int64_t total = (int64_t)p.batch * p.seqlen * p.nheads * p.headdim;
    const int64_t blocks = (total + 255) / 256;
    hipLaunchKernelGGL(scan::scan_states_generic_kernel, dim3((unsigned)(blocks > 65536 ? 65536 : blocks)), dim3(256), 0, s, p);
    return hipGetLastError();
}

}  // namespace ssd
