// Fused chunk-state + state-passing kernel whose work is handed out by tickets and ordered by a flag chain (gfx950).
//
// Why: a compute unit's vector-memory pipe takes loads and stores one after the other (moving this path's bytes
// alone, with no arithmetic, takes 163 us on the 160 compute units that b=4 L=8192 H=80 fills when every state tile
// stays on one compute unit for the whole sequence), so every compute unit has to carry its share of the traffic
// whatever the number of tiles.  That means cutting a sequence's chunks loose from each other:
//
// A work item is R consecutive chunks of one unit, a unit being four state tiles -- (batch, head, 32 headdim rows) x
// all of dstate, one per wave -- that share (batch, group) and therefore B.  Persistent workgroups, one per compute
// unit, draw items from a ticket counter in chunk-major order (ticket t -> chunks R (t / units) ..., unit t % units),
// so an item only ever depends on an item with a smaller ticket:
//   1. each chunk state S_c = sum_k B_k (x w)_k (kernels/ssd_chunk_state.py:134-173) is accumulated from zero in the
//      MFMA accumulators, independent of every other chunk, and parked in registers (R tiles of 64 per lane);
//   2. the wave then waits for the flag of (tile, first chunk), which says that out[:, c0] -- the state entering the
//      item -- is complete, reads it back, runs s_{c+1} = exp(dA_c) [same sequence] s_c + S_c
//      (kernels/ssd_state_passing.py:69-84) over its R chunks in registers, stores the last state first, raises the
//      flag of (tile, c0 + R) once that store is acknowledged, and stores the other R - 1 states after that.  Chunk 0
//      starts from initial_states (or zero) and also writes out[:, 0]; an item whose first decay is zero (a sequence
//      boundary) neither waits nor reads.
// A link of the chain costs a few memory round trips (8 us measured under load); with R chunks per item there are
// C / R links per sequence, consecutive items of a unit start R times further apart than with single chunks, and
// only every R-th passed state is read back.
// This chain replaces the reference's global barrier between its two phases (kernels/fused_globalbar.py:130-137)
// and its per-(batch, head) completion counters with a throttle semaphore (kernels/fused_concurrent.py:81-84, 141,
// 205-208).  It cannot deadlock and assumes nothing about which workgroups are resident: tickets are only drawn by
// running workgroups, a workgroup finishes its items in ticket order, and the unfinished item with the smallest
// ticket never waits for an unfinished one.  The wait is bounded all the same: after p.spin_limit polls a wave sets
// the error word of the workspace, goes on with whatever out[:, c0] holds and still raises its flag, so that every
// workgroup drains and the host can report the failure.
//
// Data movement inside a chunk is that of the four-tiles-per-workgroup kernel (ssd_quad.hip): B once per workgroup
// through a four-step LDS ring read back with transposing loads, x rows through a per-wave ring, bf16 hi + lo
// operands, all requests three steps ahead -- across chunk and item boundaries: the ticket of the next item is known
// while an item runs, so the first steps of the next chunk are always on their way when the current one ends.
#pragma once
#include "ssd_tile.h"
#include "ssd_cost.h"

namespace ssd {

namespace chain {

using namespace tile;

// steps of B and x kept in LDS (requested ring - 1 steps ahead): 8 where a chunk has 8 steps -- one workgroup per
// compute unit leaves the room, and the burst of state stores that ends an item drains behind requests that far
// ahead -- else 4
template <int SPC> constexpr int ring_of() { return SPC >= 8 ? 8 : 4; }
// B rows are read by every head of a group and come from L2 after the first reader: three steps ahead cover that
// latency, and the four-step ring leaves LDS to others
constexpr int kRingB = 4, kDistB = kRingB - 1;
// per wave: x ring + two weight slots (the next item's weights are written while the current item's are in use)
template <int SPC> constexpr int wave_lds() { return ring_of<SPC>() * 2048 + 2 * 32 * SPC * 4; }
constexpr int kStage = 1024;        // per wave: a 16 x 16 fp32 block of the state on its way to or from memory
constexpr int kTicketBytes = 64;
// With the scan's state half in the chain step (SCAN): a ring of C tiles (32 tokens x dstate bf16 each, laid out like a
// B tile), shared by the four waves, requested kDistC tiles ahead
constexpr int kRingC = 6, kDistC = kRingC - 1;
template <int NT, int SPC, bool SCAN = false> constexpr int lds_bytes()
{
    return kRingB * NT * 1024 + 4 * (wave_lds<SPC>() + kStage) + (SCAN ? kRingC * NT * 1024 : 0) + kTicketBytes;
}

// How the passed states cross between compute units.  The L2 caches, one per XCD (32 compute units), are not
// coherent with each other, and a device-scope release / acquire pair writes back and invalidates a whole L2
// (measured: 1.2 ms per launch at b=4 L=8192 H=80 -- unusable).  Two ways remain, chosen per launch:
//  * LOCAL: every unit belongs to one XCD.  Each XCD has its own ticket counter over its own units, a workgroup reads
//    the id of the XCD it runs on from the hardware and draws from that counter, so producer and consumer of a passed
//    state always share an L2: plain stores (written through the per-CU cache into L2), the flag raised once they
//    have been acknowledged, flag polls that miss the per-CU cache (sc1), and plain read-back loads -- a compute unit
//    reads each out[:, c] once, so its own cache cannot hold an older copy.  A link of the chain costs L2 latencies.
//  * GLOBAL (few units, or units that do not spread evenly over the XCDs): one counter; the state stores, the
//    read-back loads and the flags carry the device-scope cache policy (sc1: written through to memory, read around
//    the L2), nothing is flushed.  A link costs memory latencies (about 9 us measured).
constexpr int kAuxDevice = 16;      // sc1
constexpr int kMaxXcd = kChainMaxXcd;

// workspace layout: ssd_params.h
constexpr int kWsHeaderInts = kChainWsHeaderInts, kWsOwner = kChainWsOwnerWord;

// NT = dstate / 16 (4 or 8); SPC = 32-token steps per chunk (4 or 8); R = chunks per work item (1, 2 or 4).
// initial_states and final_states are fp32; out is fp32 (OUTM == 0), bf16 (1) or not wanted at all (2).  With bf16
// passed states the state that
// crosses from one item to the next must not be the rounded one -- the reference carries it in fp32 registers over
// the whole sequence (kernels/ssd_state_passing.py:61-84) --, so an item's last state goes to memory twice: rounded
// into out, and in fp32 into a slot of the workspace (p.carry: one 32 x dstate slot per tile and item), which is what
// the next item reads back.  Per launch that is 1 / R of an fp32 `out` written and read on top of the bf16 one.
// Without `out` those slots are all that is written of the passed states.
// SCAN: the chain step also consumes the passed states -- the state-dependent half of the chunk scan,
//   y[b, cQ + m, h, p] (+)= exp(dA_cumsum[b, h, c, m]) [seq_idx[cQ + m] == seq_idx[cQ - 1]] sum_n C[b, cQ + m, g, n] out[b, c, h, p, n]
// (kernels/ssd_chunk_scan.py:94-117) -- while a wave holds the state entering each of its item's chunks in registers.
template <int NT, int SPC, int R, bool HAS_SEQ, bool LOCAL, int OUTM, bool SCAN>
__global__ void __launch_bounds__(256, 1) chain_kernel(const Params p)
{
    constexpr bool OUT16 = OUTM == 1, NO_OUT = OUTM == 2, CARRY = OUTM != 0;
    static_assert(!SCAN || OUTM != 1, "the scan variant stores fp32 passed states or none");
    constexpr int Q = 32 * SPC;
    constexpr int kRing = ring_of<SPC>(), kDist = kRing - 1;
    static_assert(kDist < SPC, "the requests of a step reach into the next chunk at most");
    // the step loop's vector-memory queue, replayed at compile time (ssd_tile.h): 2 x requests and NT / 4 B requests
    // per step, no stores inside the loop
    constexpr schedule::Loop kLoop{2, NT / 4, 0, SPC, kDist, kRing, kDistB};
    static_assert(schedule::slots_ok(kLoop), "ring slots are reused too early");
    constexpr int TPL = Q / 64;         // tokens per lane when an item's weights are computed (2 or 4)
    constexpr int NTW = NT / 4;         // B tile blocks (32 tokens x 16 columns, 1 KB) a wave fetches per step
    extern __shared__ __attribute__((aligned(16))) char lds[];
    const int lane = threadIdx.x & 63, i16 = lane & 15, kg = lane >> 4;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    char *bring = lds;                                                   // kRingB x NT blocks of 1 KB, shared
    char *xring = lds + kRingB * NT * 1024 + wave * wave_lds<SPC>();     // kRing slots x (32 tokens x 64 bytes)
    char *wbuf = xring + kRing * 2048;                                   // 2 slots x Q weights
    char *stage = lds + kRingB * NT * 1024 + 4 * wave_lds<SPC>() + wave * kStage;
    char *cring = lds + kRingB * NT * 1024 + 4 * (wave_lds<SPC>() + kStage);      // kRingC x NT blocks of 1 KB, shared (SCAN)
#if defined(__HIP_DEVICE_COMPILE__)      // typed as LDS: a volatile access through a generic pointer would go the flat way
    typedef __attribute__((address_space(3))) volatile int lds_int;
    lds_int *tq = (lds_int *)(__attribute__((address_space(3))) char *)(lds + lds_bytes<NT, SPC, SCAN>() - kTicketBytes);
#else
    volatile int *tq = (volatile int *)(lds + lds_bytes<NT, SPC, SCAN>() - kTicketBytes);
#endif

    constexpr int kAux = LOCAL ? 0 : kAuxDevice;
    // this workgroup's share of the units: all of them, or those of the XCD it runs on (contiguous ranges)
    int xcd_hw = 0, slot = 0, unit0 = 0, n_units = p.n_items >> 2;
    if (LOCAL) {
#if defined(__HIP_DEVICE_COMPILE__)
        xcd_hw = __builtin_amdgcn_s_getreg((3 << 11) | 20) & 15;       // XCC_ID, bits 3:0
#endif
        slot = xcd_hw % p.n_xcd;
        const int base = n_units / p.n_xcd, rem = n_units % p.n_xcd;
        unit0 = slot * base + min(slot, rem);
        n_units = base + (slot < rem ? 1 : 0);
    }
    const int n_super = (p.C + R - 1) / R;      // items per unit
    const int total = n_units * n_super;
    const int n_pt = p.headdim >> 5;
    const int L = p.seqlen, C = p.C;
    const int64_t xrb = 2 * p.sx_l, Brb = 2 * p.sB_l;            // row pitch in bytes
    const int epoch = p.epoch, bank = epoch & 1;
    int *const ws_ticket = p.ws + kChainWsBankStride * bank + slot, *const ws_err = p.ws + kChainWsErrWord + bank;
    int *const ws_flags = p.ws + kWsHeaderInts;

    // ---- work items ------------------------------------------------------------------------------------------
    // A workgroup walks a stream of chunks: the R chunks of its current item, then those of the next.  `Item` is one
    // chunk of that stream as wave `wave` sees it.
    struct Item {
        int valid, c, r, b, h, tile, p0;           // r: position of the chunk in its work item
        __amdgpu_buffer_rsrc_t rsx, rsB;
        const char *xb, *Bb, *Cb;                  // chunk 0 of the tile's x rows and of its group's B (and, SCAN, C) rows
        const float *dtp, *dap;
        const int32_t *sqb;
    };
    // chunk r of the item behind ticket t (a ticket past the end, or a chunk past the sequence, gives an invalid
    // chunk whose requests fetch nothing)
    auto decode = [&](int t, int r) {
        Item I;
        // a ticket is an index into this slot's items; anything else (past the end, or a negative value that no
        // counter hands out) gives the invalid chunk and never reaches the address arithmetic below
        const bool in_range = (unsigned)t < (unsigned)total;
        const int tv = in_range ? t : 0;
        const int k = tv / n_units;
        I.c = k * R + r;
        I.r = r;
        I.valid = in_range && I.c < C;
        if (!I.valid) I.c = 0;
        I.tile = 4 * (unit0 + tv - k * n_units) + wave;
        const int r1 = I.tile / n_pt;
        I.p0 = 32 * (I.tile - r1 * n_pt);
        I.b = r1 / p.nheads;
        I.h = r1 - I.b * p.nheads;
        const int g = I.h / (p.nheads / p.ngroups);
        // descriptor of the chunk: base = its first token, extent = the tokens that exist
        I.xb = (const char *)p.x + 2 * (I.b * p.sx_b + I.h * p.sx_h);
        I.Bb = (const char *)p.B + 2 * (I.b * p.sB_b + g * p.sB_g);
        I.Cb = SCAN ? (const char *)p.Cm + 2 * (I.b * p.sC_b + g * p.sC_g) : nullptr;
        I.rsx = make_rsrc(I.xb + (int64_t)I.c * Q * xrb, I.valid ? (int64_t)(L - I.c * Q) * xrb : 0);
        I.rsB = make_rsrc(I.Bb + (int64_t)I.c * Q * Brb, I.valid ? (int64_t)(L - I.c * Q) * Brb : 0);
        I.dtp = p.dt + I.b * p.sdt_b + I.h * p.sdt_h + (int64_t)I.c * p.sdt_c;
        I.dap = p.dacs + I.b * p.sda_b + I.h * p.sda_h + (int64_t)I.c * p.sda_c;
        I.sqb = HAS_SEQ ? p.seq + I.b * p.ssq_b : nullptr;
        return I;
    };
    // the chunk after I in the stream: the item's next chunk, or the first chunk of the item behind ticket t_next
    auto successor = [&](const Item &I, int t_cur, int t_next) {
        if (I.r + 1 < R && I.c + 1 < C) {
            Item J = I;             // same tile, one chunk on
            (void)t_cur;
            J.c = I.c + 1;
            J.r = I.r + 1;
            J.rsx = make_rsrc(I.xb + (int64_t)J.c * Q * xrb, (int64_t)(L - J.c * Q) * xrb);
            J.rsB = make_rsrc(I.Bb + (int64_t)J.c * Q * Brb, (int64_t)(L - J.c * Q) * Brb);
            J.dtp = I.dtp + p.sdt_c;
            J.dap = I.dap + p.sda_c;
            return J;
        }
        return decode(t_next, 0);
    };

    // ---- request helpers (layouts as in ssd_quad.hip) ---------------------------------------------------------
    // A step's B tile (32 tokens x dstate) sits in LDS as NT blocks of 1 KB, block (th, pair) = 16 tokens (token
    // half th) x 32 columns (column pair `pair`), row-major: one request fetches a block, lane l the 16 bytes
    // (token l/4, piece l%4) and deposits them at byte 16*l.  For the tokens 8..15 of a block the two 32-byte halves
    // are swapped (piece ^ 2), which keeps the transposing reads below off shared banks.
    const int Blane = (int)((lane >> 2) * Brb) + 16 * ((lane & 3) ^ ((lane >> 5) << 1));
    auto load_B = [&](__amdgpu_buffer_rsrc_t rs, int s, int bi) {       // block bi of step s of the chunk behind rs
#if defined(__HIP_DEVICE_COMPILE__)      // the LDS address space does not exist in the host pass
        typedef __attribute__((address_space(3))) void *lds_ptr;
        const int th = bi / (NT / 2), pair = bi % (NT / 2);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lds_ptr)(bring + ((s % kRingB) * NT + bi) * 1024), 16, Blane,
                                                 (int)((32 * s + 16 * th) * Brb) + 64 * pair, 0, 0);
#else
        (void)rs; (void)s; (void)bi; (void)Blane;
#endif
    };
    // The transposing read for (16 columns `it`, tokens 8kg + 4*half .. +3): lane (i16, kg) addresses the 8 bytes of
    // token 8kg + 4*half + i16/4, columns 4*(i16%4)..+3 of that column block and receives column i16 of those four
    // tokens.  Inline assembly with explicit s_waitcnt: given the intrinsic, the compiler would order every such
    // read behind ALL outstanding loads that write LDS.
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
    // The results of a read_Bt become valid here: LDS operations complete in order, so the pair has arrived once no
    // more LDS operations are outstanding than were issued after it (nc = that number, at least).
    auto wait_Bt = [&](auto nc, u32x2 &lo, u32x2 &hi) {
#if defined(__HIP_DEVICE_COMPILE__)
        asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(lo), "+v"(hi) : "n"(decltype(nc)::value) : "memory");
#else
        (void)lo; (void)hi;
#endif
    };
    // x: two requests cover the 32 token rows of a step, 4 lanes per 64-byte row of the slice; lane l deposits its
    // 16 bytes at byte 16*l of a 1 KB block.  Request i fetches tokens 8*kg' + 4*i + m into row slot 4*m + kg'
    // (kg' = (l/4)%4, m = l/16), so the four kg groups of an operand read below hit different banks.
    const int xlane0 = (int)((8 * ((lane >> 2) & 3) + (lane >> 4)) * xrb) + 16 * (lane & 3);
    auto load_x = [&](__amdgpu_buffer_rsrc_t rs, int p0, int s, int i) {
#if defined(__HIP_DEVICE_COMPILE__)
        typedef __attribute__((address_space(3))) void *lds_ptr;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lds_ptr)(xring + (s % kRing) * 2048 + i * 1024), 16, xlane0 + 2 * p0,
                                                 (int)((32 * s + 4 * i) * xrb), 0, 0);
#else
        (void)rs; (void)p0; (void)s; (void)i; (void)xlane0;
#endif
    };
    const int xst_rd = 64 * kg + 4 * i16;     // + 2048 * slot + 1024 * (j/4) + 256 * (j%4) for token 8kg + j

    // decay inputs of an item's chunk: TPL consecutive tokens per lane, plus the chunk-level scalars
    struct Meta { float dtv[TPL], cs[TPL], last; int32_t id[TPL], id_last, id_prev; };
    auto load_meta = [&](const Item &I) {
        Meta m;
        const float *dtp = I.dtp + TPL * lane;
        const float *dap = I.dap + TPL * lane;
        if constexpr (TPL == 4) {
            const f32x4 a = *(const f32x4 *)dtp, d = *(const f32x4 *)dap;
            m.dtv[0] = a.x; m.dtv[1] = a.y; m.dtv[2] = a.z; m.dtv[3] = a.w;
            m.cs[0] = d.x; m.cs[1] = d.y; m.cs[2] = d.z; m.cs[3] = d.w;
        } else {
            const f32x2 a = *(const f32x2 *)dtp, d = *(const f32x2 *)dap;
            m.dtv[0] = a.x; m.dtv[1] = a.y; m.cs[0] = d.x; m.cs[1] = d.y;
        }
        m.last = I.dap[Q - 1];
        m.id_last = m.id_prev = 0;
#pragma unroll
        for (int t = 0; t < TPL; ++t) m.id[t] = 0;
        if (HAS_SEQ) {
            // a lane's TPL ids with one load where they are contiguous, aligned and inside the sequence
            const int32_t *ip = I.sqb + (int64_t)(I.c * Q + TPL * lane) * p.ssq_l;
            if (p.ssq_l == 1 && (I.c + 1) * Q <= L && ((uintptr_t)(I.sqb + I.c * Q) & 15) == 0) {
                if constexpr (TPL == 4) {
                    typedef __attribute__((ext_vector_type(4))) int32_t i32x4;
                    const i32x4 q = *(const i32x4 *)ip;
                    m.id[0] = q.x; m.id[1] = q.y; m.id[2] = q.z; m.id[3] = q.w;
                } else {
                    typedef __attribute__((ext_vector_type(2))) int32_t i32x2;
                    const i32x2 q = *(const i32x2 *)ip;
                    m.id[0] = q.x; m.id[1] = q.y;
                }
            } else {
#pragma unroll
                for (int t = 0; t < TPL; ++t) m.id[t] = I.sqb[(int64_t)min(I.c * Q + TPL * lane + t, L - 1) * p.ssq_l];
            }
            m.id_last = I.sqb[(int64_t)(min((I.c + 1) * Q, L) - 1) * p.ssq_l];
            // id of the previous chunk's last token; the recurrence starts from id 0 (kernels/ssd_state_passing.py:68)
            if (I.c > 0) m.id_prev = I.sqb[(int64_t)(I.c * Q - 1) * p.ssq_l];
        }
        return m;
    };
    // per-token weights of a chunk (kernels/ssd_chunk_state.py:134-156) -> weight slot ws
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
    // Inside the step loop the same reads are inline assembly with a wait of their own, like the B operands below: the
    // compiler counts LDS operations it has not issued itself as absent, so a wait that it puts in front of the first
    // use of a read of its own would also wait for every transposing read issued behind that read -- each step would
    // start by draining the reads that are meant to run ahead of its matrix instructions.  Six instructions: four pairs
    // of x dwords 256 bytes apart, two quads of weights.
    struct Ops { u32x2 x[4]; f32x4 w[2]; };
    constexpr int kOpReads = 6;
    uint32_t xop_base = (uint32_t)xst_rd, wop_base = (uint32_t)(32 * kg);
#if defined(__HIP_DEVICE_COMPILE__)
    xop_base += (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char *)xring;
    wop_base += (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char *)wbuf;
#endif
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Wunused-lambda-capture"
    auto read_ops = [&, xop_base, wop_base](auto sc, int ws, Ops &o) {      // step sc of the chunk whose weights are in slot ws
        constexpr int s = decltype(sc)::value;
        constexpr int xo = (s % kRing) * 8, wo = 128 * s;                   // in units of 256 bytes; in bytes
        const uint32_t wb = wop_base + (uint32_t)(ws * Q * 4);
#if defined(__HIP_DEVICE_COMPILE__)
        asm volatile("ds_read2st64_b32 %0, %6 offset0:%8 offset1:%9\n\t"
                     "ds_read2st64_b32 %1, %6 offset0:%10 offset1:%11\n\t"
                     "ds_read2st64_b32 %2, %6 offset0:%12 offset1:%13\n\t"
                     "ds_read2st64_b32 %3, %6 offset0:%14 offset1:%15\n\t"
                     "ds_read_b128 %4, %7 offset:%16\n\t"
                     "ds_read_b128 %5, %7 offset:%17"
                     : "=&v"(o.x[0]), "=&v"(o.x[1]), "=&v"(o.x[2]), "=&v"(o.x[3]), "=&v"(o.w[0]), "=&v"(o.w[1])
                     : "v"(xop_base), "v"(wb), "n"(xo), "n"(xo + 1), "n"(xo + 2), "n"(xo + 3), "n"(xo + 4), "n"(xo + 5),
                       "n"(xo + 6), "n"(xo + 7), "n"(wo), "n"(wo + 16)
                     : "memory");
#else
        for (int i = 0; i < 4; ++i) o.x[i] = (u32x2){0u, 0u};
        o.w[0] = o.w[1] = (f32x4){0.f, 0.f, 0.f, 0.f};
        (void)wb; (void)xo; (void)wo;
#endif
    };
#pragma clang diagnostic pop
    // ... valid once no more LDS operations are outstanding than were issued behind them (nc)
    auto wait_ops = [&](auto nc, Ops &o) {
#if defined(__HIP_DEVICE_COMPILE__)
        asm volatile("s_waitcnt lgkmcnt(%6) ; operands"
                     : "+v"(o.x[0]), "+v"(o.x[1]), "+v"(o.x[2]), "+v"(o.x[3]), "+v"(o.w[0]), "+v"(o.w[1])
                     : "n"(decltype(nc)::value) : "memory");
#else
        (void)o;
#endif
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
        // the residual of the exact product, as a fused multiply-add everywhere
        f.lo[jp][q] = pack_bf16(__builtin_fmaf(x0, wv[2 * q], -h0), __builtin_fmaf(x1, wv[2 * q + 1], -h1));
    };

    // acc[it][jp][r]: dstate column 16*it + 4*kg + r of headdim row p0 + 2*i16 + jp
    f32x4 acc[NT][2];

    // ---- chunk states parked in registers, and the chain step of an item --------------------------------------
    // The accumulators hold a 16 x 16 block as (lane%16 = row, lane/16 = group of four columns); each block passes
    // through 1 KB of LDS and comes back as (lane/4 = row, lane%4 = group), so that four adjacent lanes read and
    // write 64 contiguous bytes of a state row (the memory pipeline merges only what adjacent lanes address).  The
    // column group is XORed with row/4 in LDS, which keeps both the 16-byte writes and reads off shared banks.  A
    // chunk state is parked in that layout: held[r][j] = block j of chunk r of the item, scale[r] its decay.
    f32x4 held[R][2 * NT];
    float scale[R];
    auto park_into = [&](f32x4 (&dst)[2 * NT]) {
        f32x4 *wr = (f32x4 *)(stage + i16 * 64 + ((kg ^ (i16 >> 2)) << 4));
        const f32x4 *rd = (const f32x4 *)(stage + (lane >> 2) * 64 + (((lane & 3) ^ (lane >> 4)) << 4));
        // LDS operations of one wave execute in order, so block k + 1 may be written right behind the read of block k
#pragma unroll
        for (int k = 0; k < 2 * NT; ++k) {
            *wr = acc[k >> 1][k & 1];
            dst[k] = *rd;
        }
    };
    // The state entering an item, fetched early.  The last of an item's R parking places is free until its last chunk
    // ends; where the predecessor's flag is already up when that chunk starts -- the rule once every compute unit
    // has its rhythm: the predecessor finished most of an item ago --, the state is read into that place while the
    // chunk's steps run (early_fetch, called from the steps) and enters the recurrence here, before the place is
    // taken.  The chain step then neither polls nor waits for a read.  Not where the scan's state half needs that state
    // once more, nor for single-chunk items.
    constexpr bool EARLY = !SCAN && R > 1;
    bool early_have = false;          // held[R - 1] holds the state entering the current item
    int early_flag = 0;
    auto park = [&](const Item &I, const Meta &m) {
        float sc = __expf(m.last);
        if (HAS_SEQ && m.id_last != m.id_prev) sc = 0.f;
        sc = __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, sc)));
        if constexpr (EARLY) {
            if (I.r == R - 1 && early_have) {
                const float s0 = scale[0];
#pragma unroll
                for (int k = 0; k < 2 * NT; ++k) {
                    const f32x4 pv = held[R - 1][k];
                    held[0][k] = (f32x4){__builtin_fmaf(pv.x, s0, held[0][k].x), __builtin_fmaf(pv.y, s0, held[0][k].y),
                                         __builtin_fmaf(pv.z, s0, held[0][k].z), __builtin_fmaf(pv.w, s0, held[0][k].w)};
                }
            }
        }
        static_for<R>([&](auto rc) {
            constexpr int r = decltype(rc)::value;
            if (I.r == r) { park_into(held[r]); scale[r] = sc; }
        });
    };
    // A flag poll must not be served by the per-CU cache: a device-scope load (sc1) misses there (sc0 does not:
    // measured) and is answered by the L2, where a LOCAL producer's plain store has put the flag, or by memory, where
    // a GLOBAL producer's device-scope store has.
    auto load_flag = [&](const int *f) { return __hip_atomic_load(f, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); };
    auto raise_flag = [&](int *f) {
        if (lane == 0) {
            if (LOCAL) *(volatile int *)f = epoch;
            else __hip_atomic_store(f, epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    };
    // where the state entering the item that starts at chunk c0 > 0 of I's tile lies: out[:, c0], or the fp32 slot of
    // the workspace (a slot holds the tile's 32 rows only)
    constexpr int kCarrySlotBytes = 32 * NT * 16 * 4;
    auto entering_state = [&](const Item &I, int c0, int &pitch, int &row0) {
        pitch = CARRY ? NT * 16 : (int)p.so_p;
        row0 = CARRY ? 0 : I.p0;
        if (CARRY) return make_rsrc((const char *)p.carry + ((int64_t)I.tile * n_super + c0 / R) * kCarrySlotBytes, kCarrySlotBytes);
        return make_rsrc((const float *)p.out + I.b * p.so_b + I.h * p.so_h + (int64_t)c0 * p.so_c,
                         ((int64_t)(p.headdim - 1) * p.so_p + p.dstate) * 4);
    };
    // Steps 0 and 2 of an item's last chunk (I.r == R - 1: the item has all its R chunks, and scale[0] is known): look
    // at the predecessor's flag, and two steps later -- the answer has arrived behind the requests of those steps --
    // ask for the state if it is up.
    auto early_fetch = [&](const Item &I, int s) {
        if constexpr (EARLY) {
            const int c0 = I.c - I.r;
            const bool wanted = I.r == R - 1 && c0 > 0 && scale[0] != 0.f;
            if (s == 0) {
                early_have = false;
                if (wanted) early_flag = load_flag(ws_flags + (int64_t)I.tile * C + c0);
            } else if (wanted && __builtin_amdgcn_readfirstlane(early_flag) == epoch) {
                int pitch, row0;
                const __amdgpu_buffer_rsrc_t rs = entering_state(I, c0, pitch, row0);
                const int row = row0 + 2 * (lane >> 2), col = 4 * (lane & 3);
#pragma unroll
                for (int k = 0; k < 2 * NT; ++k)
                    held[R - 1][k] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(
                                                                   rs, 4 * (row * pitch + col), 4 * ((k & 1) * pitch + 16 * (k >> 1)), kAux));
                early_have = true;
            }
        }
    };
    // I: the last chunk of the item (chunks I.c - I.r .. I.c)
    auto chain_step = [&](const Item &I, int ws_free) {
        const int c0 = I.c - I.r, n = I.r + 1;
        const bool use_prev = (c0 > 0 || p.init != nullptr) && scale[0] != 0.f;
        const int64_t slice_out = (int64_t)(p.headdim - 1) * p.so_p + p.dstate;
        const int64_t slice_fin = (int64_t)(p.headdim - 1) * p.sf_p + p.dstate;
        const int64_t slice_in = (int64_t)(p.headdim - 1) * p.sin_p + p.dstate;
        using out_t = std::conditional_t<OUT16, uint16_t, float>;
        constexpr int kOutBytes = sizeof(out_t);
        const out_t *outb = (const out_t *)p.out + I.b * p.so_b + I.h * p.so_h;
        // the fp32 slot of (tile, item g) holds the state entering that item's first chunk g * R
        constexpr int kSlotBytes = 32 * NT * 16 * 4;
        auto carry_slot = [&](int c) { return make_rsrc((const char *)p.carry + ((int64_t)I.tile * n_super + c / R) * kSlotBytes, kSlotBytes); };
        const __amdgpu_buffer_rsrc_t rs_prev =
            c0 > 0 ? (CARRY ? carry_slot(c0) : make_rsrc(outb + (int64_t)c0 * p.so_c, slice_out * 4))
                   : make_rsrc((const float *)p.init + I.b * p.sin_b + I.h * p.sin_h, p.init ? slice_in * 4 : 0);
        const int pitch_prev = c0 > 0 ? (CARRY ? NT * 16 : (int)p.so_p) : (int)p.sin_p;
        const int row = I.p0 + 2 * (lane >> 2), col = 4 * (lane & 3);
        const int row_prev = CARRY && c0 > 0 ? 2 * (lane >> 2) : row;      // a slot holds the tile's 32 rows only
        int *const flag = ws_flags + (int64_t)I.tile * C;
        // chunk j of the item ends in out[:, c0 + j + 1], the sequence's last chunk in final_states
        auto store_chunk = [&](int j, const f32x4 (&v)[2 * NT], int aux) {
            const bool fin = c0 + j + 1 == C;
            if (NO_OUT && !fin) return;
            const __amdgpu_buffer_rsrc_t rs = fin ? make_rsrc(p.fin + I.b * p.sf_b + I.h * p.sf_h, slice_fin * 4)
                                                  : make_rsrc(outb + (int64_t)(c0 + j + 1) * p.so_c, slice_out * kOutBytes);
            const int pitch = fin ? (int)p.sf_p : (int)p.so_p;
            if (OUT16 && !fin) {
                // nobody reads these back inside the launch: plain stores whatever the mode
#pragma unroll
                for (int k = 0; k < 2 * NT; ++k) store4_bf16(rs, row * pitch + col, (k & 1) * pitch + 16 * (k >> 1), v[k]);
            } else {
#pragma unroll
                for (int k = 0; k < 2 * NT; ++k) store4_f32(rs, row * pitch + col, (k & 1) * pitch + 16 * (k >> 1), v[k], aux);
            }
        };
        // the item's last state in fp32, for the item behind it (where `out` is not an fp32 tensor to read it back from)
        auto store_carry = [&](int c_next, const f32x4 (&v)[2 * NT]) {
            const __amdgpu_buffer_rsrc_t rs = carry_slot(c_next);
#pragma unroll
            for (int k = 0; k < 2 * NT; ++k)
                store4_f32(rs, 2 * (lane >> 2) * (NT * 16) + col, (k & 1) * (NT * 16) + 16 * (k >> 1), v[k], kAux);
        };

        // held[j] <- exp(dA_j) [same sequence] held[j - 1] + held[j] for the chunks jb < j < je
        auto carry_on = [&](int jb, int je) {
            static_for<R>([&](auto jc) {
                constexpr int j = decltype(jc)::value;
                if (j > jb && j < je) {
                    const float sc = scale[j];
#pragma unroll
                    for (int k = 0; k < 2 * NT; ++k) {
                        const f32x4 pv = held[j > 0 ? j - 1 : 0][k];
                        held[j][k] = (f32x4){__builtin_fmaf(pv.x, sc, held[j][k].x), __builtin_fmaf(pv.y, sc, held[j][k].y),
                                             __builtin_fmaf(pv.z, sc, held[j][k].z), __builtin_fmaf(pv.w, sc, held[j][k].w)};
                    }
                }
            });
        };
        // the state the next item waits for: stored, acknowledged (by the L2 both sides share, or by memory), flagged.
        // (Letting the next chunk's first wait for its own x rows stand in for the wait here -- memory operations
        // complete in order -- saves it but raises the flag later: no gain at b=4 L=8192 H=80, and slower where the
        // chain sets the pace: 1.19 ms instead of 1.10 ms at L=131072 H=128.)
        auto hand_on = [&]() {
            static_for<R>([&](auto jc) {
                constexpr int j = decltype(jc)::value;
                if (j == n - 1) {
                    if (CARRY && c0 + n < C) store_carry(c0 + n, held[j]);
                    store_chunk(j, held[j], kAux);
                }
            });
            if (c0 + n < C) {
                asm volatile("" ::: "memory");
                __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
                asm volatile("" ::: "memory");
                raise_flag(flag + c0 + n);
            }
        };
        // A sequence that starts at chunk jz > 0 of the item (decay zero) cuts the item in two: the states from jz on do
        // not depend on the state entering the item, so they are finished and handed on before this wave waits for
        // its own predecessor -- with packed sequences the chain then is as long as a sequence, not as the batch row.
        int jz = 0;
        if (HAS_SEQ) {
            static_for<R>([&](auto jc) {
                constexpr int j = decltype(jc)::value;
                if (j >= 1 && j < n && scale[j] == 0.f) jz = j;
            });
        }
        // SCAN: y of the item's first chunk needs the state entering the item whatever the decay says -- the tokens in
        // front of a sequence start inside that chunk still belong to the old sequence --, so an item whose first decay
        // is zero waits for its predecessor as well, after it has handed on everything (nothing it passes on depends
        // on that state).
        const bool cut0 = SCAN && c0 > 0 && !use_prev && jz == 0;
        const int head = jz > 0 ? jz : (cut0 ? 0 : n);           // chunks [0, head) depend on the state entering the item

        // SCAN: what the y loop below needs from memory and does not depend on the chain is asked for now: the first
        // tiles of C, and the chunks' dA_cumsum rows (and sequence ids), TPL tokens per lane
        const int64_t Crb = 2 * p.sC_l;
        const int Clane = (int)((lane >> 2) * Crb) + 16 * ((lane & 3) ^ (lane >> 4));
        const int n_tiles = n * SPC;
        // tile t of the item = step t % SPC of chunk c0 + t / SPC; a wave fetches NTW of its NT blocks (16 tokens x 32
        // columns, 1 KB: lane l the 16 bytes (token l/4, piece (l%4) ^ (l/16)), so that the operand reads of 16 tokens
        // at one piece fall on 16 different bank groups); tiles past the item's end: requests that fetch nothing
        // The request cursor: the next tile to ask for, its chunk's descriptor pieces and its ring slot.
        int rq_t = 0, rq_st = 0, rq_slot = 0;
        const char *rq_base = I.Cb + (int64_t)c0 * Q * Crb;       // first row of the chunk
        int64_t rq_bytes = (int64_t)(L - c0 * Q) * Crb;           // rows of the sequence from there on
        auto load_C = [&]() {
#if defined(__HIP_DEVICE_COMPILE__)
            typedef __attribute__((address_space(3))) void *lds_ptr;
            const __amdgpu_buffer_rsrc_t rs = make_rsrc(rq_base, rq_t < n_tiles ? rq_bytes : 0);
            char *dst = cring + rq_slot * NT * 1024;
#pragma unroll
            for (int k = 0; k < NTW; ++k) {
                const int bi = wave * NTW + k, th = bi / (NT / 2), pair = bi % (NT / 2);
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lds_ptr)(dst + bi * 1024), 16, Clane, (int)((32 * rq_st + 16 * th) * Crb) + 64 * pair, 0, 0);
            }
            ++rq_t;
            rq_slot = rq_slot + 1 == kRingC ? 0 : rq_slot + 1;
            if (++rq_st == SPC) { rq_st = 0; rq_base += (int64_t)Q * Crb; rq_bytes -= (int64_t)Q * Crb; }
#else
            (void)Clane; (void)n_tiles; (void)rq_t; (void)rq_st; (void)rq_slot; (void)rq_base; (void)rq_bytes;
#endif
        };
        float ycs[R][TPL];
        int32_t yid[R][TPL], yprev[R];
        if constexpr (SCAN) {
#pragma unroll 1
            for (int t = 0; t < kDistC; ++t) load_C();
            static_for<R>([&](auto jc) {
                constexpr int j = decltype(jc)::value;
                if (j < n) {
                    const float *dap = I.dap + (int64_t)(j - I.r) * p.sda_c + TPL * lane;
                    if constexpr (TPL == 4) {
                        const f32x4 d = *(const f32x4 *)dap;
                        ycs[j][0] = d.x; ycs[j][1] = d.y; ycs[j][2] = d.z; ycs[j][3] = d.w;
                    } else {
                        const f32x2 d = *(const f32x2 *)dap;
                        ycs[j][0] = d.x; ycs[j][1] = d.y;
                    }
                    if (HAS_SEQ) {
                        const int c = c0 + j;
#pragma unroll
                        for (int t = 0; t < TPL; ++t) yid[j][t] = I.sqb[(int64_t)min(c * Q + TPL * lane + t, L - 1) * p.ssq_l];
                        // the scan compares with the last token in front of the chunk; 0 in front of the first chunk
                        yprev[j] = c > 0 ? I.sqb[(int64_t)(c * Q - 1) * p.ssq_l] : 0;
                    }
                }
            });
        }

        if (jz > 0) {
            carry_on(jz, n);
            hand_on();
        } else if (cut0) {
            carry_on(0, n);
            hand_on();
        }

        const bool early = EARLY && early_have && n == R && c0 > 0;     // the entering state is in held[0] already
        if (!early && (SCAN ? c0 > 0 : (use_prev && c0 > 0))) {
            // out[:, c0] of this tile is complete once its flag is up
            int polls = 0;
            while (load_flag(flag + c0) != epoch) {
                __builtin_amdgcn_s_sleep(1);
                if (++polls >= p.spin_limit) {
                    if (lane == 0) __hip_atomic_fetch_or(ws_err, kChainErrTimeout, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    break;
                }
            }
            asm volatile("" ::: "memory");
        }
        f32x4 s[2 * NT];       // the state entering the item
        if (!early && (use_prev || c0 == 0 || SCAN)) {
            // chunk 0 copies initial_states to out[:, 0] even if a sequence boundary wipes them out at once
            const bool read = use_prev || p.init != nullptr || (SCAN && c0 > 0);
#pragma unroll
            for (int k = 0; k < 2 * NT; ++k) {
                s[k] = (f32x4){0.f, 0.f, 0.f, 0.f};
                if (read)
                    s[k] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(
                                                         rs_prev, 4 * (row_prev * pitch_prev + col),
                                                         4 * ((k & 1) * pitch_prev + 16 * (k >> 1)), kAux));
            }
            if (use_prev) {
                // the recurrence enters the item: held[0] becomes the state after chunk c0
                const float sc = scale[0];
#pragma unroll
                for (int k = 0; k < 2 * NT; ++k)
                    held[0][k] = (f32x4){__builtin_fmaf(s[k].x, sc, held[0][k].x), __builtin_fmaf(s[k].y, sc, held[0][k].y),
                                         __builtin_fmaf(s[k].z, sc, held[0][k].z), __builtin_fmaf(s[k].w, sc, held[0][k].w)};
            }
            if (c0 == 0 && !NO_OUT) {
#pragma unroll
                for (int k = 0; k < 2 * NT; ++k) {
                    if (OUT16) store4_bf16(make_rsrc(outb, slice_out * 2), row * (int)p.so_p + col, (k & 1) * (int)p.so_p + 16 * (k >> 1), s[k]);
                    else store4_f32(make_rsrc(outb, slice_out * 4), row * (int)p.so_p + col, (k & 1) * (int)p.so_p + 16 * (k >> 1), s[k], 0);
                }
            }
        }
        // ... and runs through its chunks, in place: held[j] becomes the state after chunk c0 + j (an item that starts
        // a sequence starts from its first chunk state)
        carry_on(0, head);
        if (jz == 0 && !cut0) hand_on();
        // the states inside the item, which nobody waits for.  (Spreading these stores over the steps of the next item
        // was measured: 250 us instead of 215 at b=4 L=8192 H=80; the non-temporal hint on these stores: 220
        // instead of 213.)
        static_for<R>([&](auto jc) {
            constexpr int j = decltype(jc)::value;
            if (j < n - 1) store_chunk(j, held[j], 0);
        });

        if constexpr (SCAN) {
            // ---- the scan's state half: y of chunk c0 + j from E_j, the state entering it (s for j = 0, held[j - 1] after)
            // E_j as MFMA A operands, bf16 hi + lo (the reference rounds the state to C's element type,
            // kernels/ssd_chunk_scan.py:106-110; hi + lo follows the fp32 mathematics): a 16 x 16 block goes through
            // LDS back into the accumulator layout (lane%16 = row, lane/16 = group of four columns), the inverse of
            // park_into, and the blocks 2u and 2u + 1 of a row parity jp form the 32-deep slab u, lane group kg holding
            // the columns 32u + 4kg .. + 3 and 32u + 16 + 4kg .. + 3 -- the C operand below is read in the same order.
            u32x4 shi[2][NT / 2], slo[2][NT / 2];
            auto to_operands = [&](const f32x4 (&E)[2 * NT]) {
                f32x4 *wr = (f32x4 *)(stage + (lane >> 2) * 64 + (((lane & 3) ^ (lane >> 4)) << 4));
                const f32x4 *rd = (const f32x4 *)(stage + i16 * 64 + ((kg ^ (i16 >> 2)) << 4));
#pragma unroll
                for (int u = 0; u < NT / 2; ++u) {
                    f32x4 A[4];          // blocks 4u .. 4u + 3 = (it, jp) = (2u, 0), (2u, 1), (2u + 1, 0), (2u + 1, 1)
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        *wr = E[4 * u + k];
                        A[k] = *rd;
                    }
#pragma unroll
                    for (int jp = 0; jp < 2; ++jp) {
                        const float v[8] = {A[jp].x, A[jp].y, A[jp].z, A[jp].w, A[2 + jp].x, A[2 + jp].y, A[2 + jp].z, A[2 + jp].w};
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const uint32_t hp = pack_bf16(v[2 * e], v[2 * e + 1]);
                            const float h0 = __builtin_bit_cast(float, hp << 16);
                            const float h1 = __builtin_bit_cast(float, hp & 0xffff0000u);
                            shi[jp][u][e] = hp;
                            slo[jp][u][e] = pack_bf16(v[2 * e] - h0, v[2 * e + 1] - h1);
                        }
                    }
                }
            };
            const int esz = p.dt_y == DT_F32 ? 4 : 2;
            const int64_t yrb = p.sy_l * esz;            // bytes between tokens
            const char *yb = (const char *)p.y + esz * (I.b * p.sy_b + I.h * p.sy_h + I.p0);
            // memory operations of a tile besides its C requests: bf16 y, 16 tokens x 64 bytes per store, one per
            // 16-token block (two with fp32 y), as many loads in front when adding to what y holds
            const int mode = (p.dt_y == DT_F32 ? 1 : 0) + (p.y_accumulate ? 2 : 0);
            // every request has landed and every wave is through with the ring slots of the item before
            asm volatile("" ::: "memory");
            __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
            int slot = 0;                                        // ring slot of the tile consumed next
            // C operands (lane (token i16, kg): columns 32u + 4kg .. + 3 and 32u + 16 + 4kg .. + 3 of slab u) and per-token
            // scales of the two 16-token blocks of a tile
            struct TileOps { bf16x8 cop[2][NT / 2]; float sc[2]; };
            // A tile has landed once no more operations are outstanding than were issued behind its requests (those of
            // the kDistC - 1 tiles after it and the loads and stores of kDistC tiles); the barrier publishes every
            // wave's blocks and says that all waves are through with the tile before, whose slot the next request
            // overwrites.  Then the tile's operands are read.
            auto open_tile = [&](int st, TileOps &o) {
                constexpr int kReq = (kDistC - 1) * NTW;
                if (mode == 0) __builtin_amdgcn_s_waitcnt(vmcnt_imm(kReq + kDistC * 2));
                else if (mode == 1 || mode == 2) __builtin_amdgcn_s_waitcnt(vmcnt_imm(kReq + kDistC * 4));
                else __builtin_amdgcn_s_waitcnt(vmcnt_imm(kReq + kDistC * 8));
                __builtin_amdgcn_s_barrier();
                asm volatile("" ::: "memory");
                load_C();
                const char *tile_c = cring + slot * NT * 1024;
                slot = slot + 1 == kRingC ? 0 : slot + 1;
#pragma unroll
                for (int tb = 0; tb < 2; ++tb) {
#pragma unroll
                    for (int u = 0; u < NT / 2; ++u) {
                        const char *blk = tile_c + (tb * (NT / 2) + u) * 1024 + 64 * i16 + 8 * (kg & 1);
                        const u32x2 c0v = *(const u32x2 *)(blk + 16 * ((kg >> 1) ^ (i16 >> 2)));
                        const u32x2 c1v = *(const u32x2 *)(blk + 16 * ((2 + (kg >> 1)) ^ (i16 >> 2)));
                        o.cop[tb][u] = __builtin_bit_cast(bf16x8, (u32x4){c0v.x, c0v.y, c1v.x, c1v.y});
                    }
                    o.sc[tb] = *(const float *)(wbuf + ws_free * Q * 4 + 4 * (32 * st + 16 * tb + i16));
                }
            };
            // the tile's two blocks: 2 x NT matrix instructions each, then the results scaled, turned into rows through
            // LDS and stored
            auto finish_tile = [&](int st, const TileOps &o, __amdgpu_buffer_rsrc_t rsy) {
                f32x4 Dv[2][2];
#pragma unroll
                for (int tb = 0; tb < 2; ++tb) {
                    f32x4 D0 = {0.f, 0.f, 0.f, 0.f}, D1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int u = 0; u < NT / 2; ++u) {
                        D0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, shi[0][u]), o.cop[tb][u], D0, 0, 0, 0);
                        D1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, shi[1][u]), o.cop[tb][u], D1, 0, 0, 0);
                        D0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, slo[0][u]), o.cop[tb][u], D0, 0, 0, 0);
                        D1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, slo[1][u]), o.cop[tb][u], D1, 0, 0, 0);
                    }
                    Dv[tb][0] = D0; Dv[tb][1] = D1;
                }
#pragma unroll
                for (int tb = 0; tb < 2; ++tb) {
                    const f32x4 D0 = Dv[tb][0], D1 = Dv[tb][1];
                    // lane (token i16, kg): D0[r] / D1[r] = headdim rows p0 + 8kg + 2r / + 2r + 1 -- eight consecutive
                    // values of the token's y row; through LDS they become (lane/4 = token, lane%4 = piece), so that
                    // four adjacent lanes address 64 (fp32: 2 x 64) contiguous bytes
                    const float sc = o.sc[tb];
                    const float v[8] = {D0.x * sc, D1.x * sc, D0.y * sc, D1.y * sc, D0.z * sc, D1.z * sc, D0.w * sc, D1.w * sc};
                    char *wr = stage + i16 * 64 + ((kg ^ (i16 >> 2)) << 4);
                    const char *rd = stage + (lane >> 2) * 64 + (((lane & 3) ^ (lane >> 4)) << 4);
                    const int tok = 32 * st + 16 * tb;           // first token of the block
                    if (mode == 0) {
                        *(u32x4 *)wr = (u32x4){pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3]), pack_bf16(v[4], v[5]), pack_bf16(v[6], v[7])};
                        const u32x4 q = *(const u32x4 *)rd;
                        __builtin_amdgcn_raw_buffer_store_b128(q, rsy, (int)((lane >> 2) * yrb) + 16 * (lane & 3), (int)(tok * yrb), 0);
                        asm volatile("s_nop 3" ::"v"(q) : "memory");
                    } else {
                        // fp32 in flight: two passes of four values each
                        *(f32x4 *)wr = (f32x4){v[0], v[1], v[2], v[3]};
                        f32x4 a = *(const f32x4 *)rd;
                        *(f32x4 *)wr = (f32x4){v[4], v[5], v[6], v[7]};
                        f32x4 d = *(const f32x4 *)rd;
                        if (p.dt_y == DT_F32) {
                            const int voff = (int)((lane >> 2) * yrb) + 32 * (lane & 3);
                            if (p.y_accumulate) {
                                a += __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rsy, voff, (int)(tok * yrb), 0));
                                d += __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rsy, voff, (int)(tok * yrb) + 16, 0));
                            }
                            const u32x4 qa = __builtin_bit_cast(u32x4, a), qd = __builtin_bit_cast(u32x4, d);
                            __builtin_amdgcn_raw_buffer_store_b128(qa, rsy, voff, (int)(tok * yrb), 0);
                            __builtin_amdgcn_raw_buffer_store_b128(qd, rsy, voff, (int)(tok * yrb) + 16, 0);
                            asm volatile("s_nop 3" ::"v"(qa), "v"(qd) : "memory");
                        } else {
                            const int voff = (int)((lane >> 2) * yrb) + 16 * (lane & 3);
                            const u32x4 o_ = __builtin_amdgcn_raw_buffer_load_b128(rsy, voff, (int)(tok * yrb), 0);
                            const float f[8] = {a.x, a.y, a.z, a.w, d.x, d.y, d.z, d.w};
                            u32x4 q;
#pragma unroll
                            for (int e = 0; e < 4; ++e)
                                q[e] = pack_bf16(f[2 * e] + bf16_bits_to_f32(o_[e] & 0xffffu), f[2 * e + 1] + bf16_bits_to_f32(o_[e] >> 16));
                            __builtin_amdgcn_raw_buffer_store_b128(q, rsy, voff, (int)(tok * yrb), 0);
                            asm volatile("s_nop 3" ::"v"(q) : "memory");
                        }
                    }
                }
            };
#pragma unroll 1
            for (int j = 0; j < n; ++j) {
                static_for<R>([&](auto jc) {
                    constexpr int jj = decltype(jc)::value;
                    if (j == jj) {
                        if constexpr (jj == 0) to_operands(s);
                        else to_operands(held[jj - 1]);
                        // per-token scale of the chunk -> the free weight slot (kernels/ssd_chunk_scan.py:86-88, 101-104)
                        float w[TPL];
#pragma unroll
                        for (int q = 0; q < TPL; ++q) {
                            w[q] = __expf(ycs[jj][q]);
                            if (HAS_SEQ && yid[jj][q] != yprev[jj]) w[q] = 0.f;
                        }
                        if constexpr (TPL == 4) *(f32x4 *)(wbuf + ws_free * Q * 4 + 16 * lane) = (f32x4){w[0], w[1], w[2], w[3]};
                        else *(f32x2 *)(wbuf + ws_free * Q * 4 + 8 * lane) = (f32x2){w[0], w[1]};
                    }
                });
                const int c = c0 + j;
                const int rows = min(Q, L - c * Q);
                const __amdgpu_buffer_rsrc_t rsy = make_rsrc(yb + (int64_t)c * Q * yrb, (int64_t)(rows - 1) * yrb + 32 * esz);
                // Two tiles per trip: the operands of a tile are read in front of the matrix instructions of the tile
                // before it, so that their way from LDS (and the wait and the barrier in front of it) runs beside those
                // instructions.  A chunk's first tile has nothing in front of it: the conversion above.
                TileOps oa, ob;
                open_tile(0, oa);
#pragma unroll 1
                for (int st = 0; st < SPC; st += 2) {
                    open_tile(st + 1, ob);
                    finish_tile(st, oa, rsy);
                    if (st + 2 < SPC) open_tile(st + 2, oa);
                    finish_tile(st + 1, ob, rsy);
                }
            }
        }
    };

    // ---- tickets ---------------------------------------------------------------------------------------------
    // Tickets are worked on in the order they are drawn only if every workgroup draws one per item: two tickets drawn
    // together at the start would put the second a whole item later than its neighbours' first ones, and the items
    // that depend on it (same unit, next chunks: a smaller ticket distance than there are workgroups when units are
    // few) would all be waiting by then.  So a workgroup starts with one ticket; the second is drawn while the first
    // chunk of the first item runs and the third while its second chunk runs (below), after that one per item.  Only
    // a first item of a single chunk needs its successor from its first steps on and draws it here.
    if (threadIdx.x == 0) {
        const int t = __hip_atomic_fetch_add(ws_ticket, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const int c_first = ((unsigned)t < (unsigned)total ? t / n_units : 0) * R;
        const bool single = !(R > 1 && c_first + 1 < C);
        tq[0] = t;
        tq[1] = single ? __hip_atomic_fetch_add(ws_ticket, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : -1;
        if (t == 0) {
            // One thread per slot and launch (all of them write the same values, so that the launch does not depend
            // on a particular slot being served).  First: is the workspace what the epoch promises?  The launch
            // before must have been epoch - 1 (a clearing leaves 0), and the flags this launch looks at must lie
            // inside what the last clearing covered -- beyond it the memory holds anything, possibly this epoch.
            const int before = __hip_atomic_load(p.ws + kChainWsEpochWord, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            const int cleared = __hip_atomic_load(p.ws + kChainWsClearedWord, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if ((before != epoch - 1 && before != epoch) || (int64_t)cleared < kWsHeaderInts + (int64_t)p.n_items * p.C)
                __hip_atomic_fetch_or(ws_err, kChainErrWorkspace, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            // What the next launch on this workspace (epoch + 1, the other parity) must find at zero -- nothing of
            // it is touched by this launch --, and how many items each slot of this launch has to hand out.
            int *const other = p.ws + kChainWsBankStride * (bank ^ 1);
            for (int i = 0; i < kChainWsBankStride; ++i) __hip_atomic_store(other + i, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(p.ws + kChainWsErrWord + (bank ^ 1), 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(p.ws + kChainWsEpochWord, epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            int *const totals = p.ws + kChainWsBankStride * bank + kChainWsTotalOffset;
            const int all_units = p.n_items >> 2, slots = LOCAL ? p.n_xcd : 1;
            for (int i = 0; i < kMaxXcd; ++i) {
                const int u = i < slots ? all_units / slots + (i < all_units % slots ? 1 : 0) : 0;
                __hip_atomic_store(totals + i, u * n_super, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
    }
    // rows past the end of the sequence are not fetched and leave their LDS slots untouched; their weight is zero,
    // so the slots only have to hold finite numbers
#pragma unroll
    for (int i = 0; i < 2 * kRing; ++i) *(u32x4 *)(xring + i * 1024 + 16 * lane) = (u32x4){0u, 0u, 0u, 0u};
#pragma unroll
    for (int i = 0; i < kRingB * NTW; ++i)
        *(u32x4 *)(bring + (i * 4 + wave) * 1024 + 16 * lane) = (u32x4){0u, 0u, 0u, 0u};
    __builtin_amdgcn_s_waitcnt(0xc07f);          // lgkmcnt(0): the zeros are in place before any row lands
    __builtin_amdgcn_s_barrier();
    // the tickets of the current and of the next item; the one after that is drawn while the current item runs
    int t_cur = __builtin_amdgcn_readfirstlane(tq[0]), t_nxt = __builtin_amdgcn_readfirstlane(tq[1]);
    bool second_late = t_nxt < 0;                // the second ticket is still to be drawn (first item only)
    if (second_late) t_nxt = total;              // no item; not looked at before the ticket is there
    Item cur = decode(t_cur, 0);
    Item nxt = successor(cur, t_cur, t_nxt);
    if (!cur.valid) {                            // whole workgroup: no barrier is skipped
        // Nothing to do -- or ticket counters that an earlier launch of the same parity left behind (an epoch that does
        // not follow the one before): then nobody draws ticket 0, and this is where the broken promise shows.
        if (threadIdx.x == 0) {
            const int before = __hip_atomic_load(p.ws + kChainWsEpochWord, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (before != epoch - 1 && before != epoch)
                __hip_atomic_fetch_or(ws_err, kChainErrWorkspace, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        return;
    }

    Meta mcur = load_meta(cur);
    // requests of the steps 0..kDist-1 (B: 0..kDistB-1), in the order (x, x, B...) that every later step keeps
#pragma unroll
    for (int s = 0; s < kDist; ++s) {
        load_x(cur.rsx, cur.p0, s, 0); load_x(cur.rsx, cur.p0, s, 1);
        // (beyond the B distance: requests with an empty descriptor, which fetch nothing -- they keep the number of
        // operations per step, which the waits below count, the same from the first step on.  What such a request
        // deposits is zeros, so it is aimed at the one ring slot no real request has been made for yet.)
#pragma unroll
        for (int k = 0; k < NTW; ++k) load_B(s < kDistB ? cur.rsB : make_rsrc(nullptr, 0), s < kDistB ? s : kDistB, wave * NTW + k);
        __builtin_amdgcn_sched_barrier(0);
    }
    put_weights(cur.c, 0, mcur);
    Frag fA, fB;
    // B operands (transposed blocks) travel kAhead iterations ahead of the MFMAs that use them, across the step
    // boundaries of a chunk: block t of the stream of (step, tile) pairs sits in slot t % 4.  They are asynchronous
    // results of inline assembly, which the compiler takes for complete: where it has to keep such a value for long, or
    // carry it around the chunk loop, it may copy it to another register right behind the read, before the data is
    // there.  So none is in flight at the end of a chunk: the first blocks of a chunk are read at its top.
    constexpr int kAhead = 3;
    static_assert(NT % 4 == 0 && kAhead < 4 && kAhead <= NT, "slot of a block = its tile index % 4");
    static_assert(SPC % kRing == 0 && SPC % kRingB == 0, "ring slots repeat from item to item");
    u32x2 blo[4], bhi[4];
    {
        // everything up to this wave's B blocks of step 0 has landed: the requests of the other steps were issued later
        static_assert(schedule::wait_prologue(kLoop) == (kDist - 1) * (2 + NTW), "prologue wait");
        __builtin_amdgcn_s_waitcnt(vmcnt_imm(schedule::wait_prologue(kLoop)));
        __builtin_amdgcn_s_barrier();   // ... and every other wave's blocks of step 0
        asm volatile("" ::: "memory");
        uint32_t xr[8]; float wv[8];
        read_operands(0, 0, xr, wv);
#pragma unroll
        for (int q = 0; q < 4; ++q) { frag_piece(q, 0, xr, wv, fA); frag_piece(q, 1, xr, wv, fA); }
        __builtin_amdgcn_sched_barrier(0);
    }
    Meta mnext = mcur;
    int t_new = 0;          // the ticket drawn during this item (wave 0, lane 0)
    // One 32-token step s of the current item (weight slot ws): fc = x operands of this step, fn receives those of
    // the step after it (the next item's first step after the last one).  Vector-memory requests of a step, in
    // program order: the two x requests of step + 3 (iteration 0), this wave's B requests of step + 3 (after the
    // barrier in iteration NT - kAhead); steps past the item's last belong to the next item.  Memory operations
    // complete in order and the compiler does not track loads that write LDS, so the waits for them are explicit:
    // "no more outstanding than were issued after the one needed".  Operations the counts leave out (the ticket
    // draw, the next item's decay inputs) only make a wait longer than needed, never shorter; the chain step
    // between two items ends with every operation complete.
    auto step = [&](auto sc, int ws, Frag &fc, Frag &fn) {
        constexpr int s = decltype(sc)::value;
        // x rows of step + 1 (this wave's own, requested two steps ago): behind them came the B requests of that
        // step and all requests of the steps s + 2 - kDist .. s - 1
        static_assert(schedule::wait_x(kLoop, s) == NTW + (kDist - 2) * (2 + NTW), "wait for the x rows of step + 1");
        __builtin_amdgcn_s_waitcnt(vmcnt_imm(NTW + (kDist - 2) * (2 + NTW)));
        asm volatile("" ::: "memory");
        uint32_t xr[8]; float wv[8];
        Ops ops;
        if constexpr (s + 1 < SPC) read_ops(std::integral_constant<int, s + 1>{}, ws, ops);
        else read_ops(std::integral_constant<int, 0>{}, ws ^ 1, ops);
        if (s == 0 && (cur.r == 0 || (second_late && cur.r == 1)) && threadIdx.x == 0)
            t_new = __hip_atomic_fetch_add(ws_ticket, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (s == 0 || s == 2) early_fetch(cur, s);
        // published by this step's barrier: the ticket after next, or (first item) the next one and then that
        if (s == SPC - 2 && (cur.r == 0 || (second_late && cur.r == 1)) && threadIdx.x == 0)
            tq[second_late && cur.r == 0 ? 1 : 2] = t_new;
        // requests of this step: x rows of step + kDist and this wave's B blocks of step + kDistB (this item or the next)
        const auto rsB = s + kDistB < SPC ? cur.rsB : nxt.rsB;
        const auto rsx = s + kDist < SPC ? cur.rsx : nxt.rsx;
        const int xp0 = s + kDist < SPC ? cur.p0 : nxt.p0;
        const int s3 = (s + kDist) % SPC, s3b = (s + kDistB) % SPC;
        const bf16x8 h0 = __builtin_bit_cast(bf16x8, (u32x4){fc.hi[0][0], fc.hi[0][1], fc.hi[0][2], fc.hi[0][3]});
        const bf16x8 h1 = __builtin_bit_cast(bf16x8, (u32x4){fc.hi[1][0], fc.hi[1][1], fc.hi[1][2], fc.hi[1][3]});
        const bf16x8 l0 = __builtin_bit_cast(bf16x8, (u32x4){fc.lo[0][0], fc.lo[0][1], fc.lo[0][2], fc.lo[0][3]});
        const bf16x8 l1 = __builtin_bit_cast(bf16x8, (u32x4){fc.lo[1][0], fc.lo[1][1], fc.lo[1][2], fc.lo[1][3]});
        __builtin_amdgcn_sched_barrier(0);   // operand reads above, the requests of this step below
        static_for<NT>([&](auto itc) {
            constexpr int it = decltype(itc)::value;
            // the blocks read behind this one (two reads each) may still be in flight: kAhead - 1 of them, fewer at the
            // end of a chunk's last step, where the next chunk's first blocks are not read yet
            constexpr int behind = s + 1 < SPC || NT - 1 - it > kAhead - 1 ? kAhead - 1 : NT - 1 - it;
            // (the step's operand reads stand behind the first kAhead blocks of its tile and are waited for in iteration 1)
            wait_Bt(std::integral_constant<int, 2 * behind + (it <= 1 ? kOpReads : 0)>{}, blo[it % 4], bhi[it % 4]);
            const bf16x8 Bt = __builtin_bit_cast(bf16x8, (u32x4){blo[it % 4].x, blo[it % 4].y, bhi[it % 4].x, bhi[it % 4].y});
            if constexpr (it == NT - kAhead) {
                // The next read is the first of step + 1's tile: this wave's blocks of it (requested three steps
                // ago) have landed once only the requests of step - 1 and the x requests of this step are
                // outstanding; the barrier publishes every wave's blocks.  It also tells that all waves are through
                // with the tile of step - 1, whose ring slot the B requests below overwrite.
                static_assert(schedule::wait_b(kLoop, s) == (kDistB - 2) * (2 + NTW) + 2, "wait for the B blocks of step + 1");
                __builtin_amdgcn_s_waitcnt(vmcnt_imm(schedule::wait_b(kLoop, s)));
                __builtin_amdgcn_s_barrier();
                asm volatile("" ::: "memory");
            }
            {
                constexpr int tn = it + kAhead;     // block kAhead iterations on: this step's tile or the next one's
                if constexpr (tn < NT || s + 1 < SPC)       // (the next chunk's first blocks: at its top)
                    read_Bt(std::integral_constant<int, (tn < NT ? s : s + 1) % kRingB>{}, std::integral_constant<int, tn % NT>{},
                            blo[tn % 4], bhi[tn % 4]);
            }
            // a chunk's first step starts its sums: the accumulators are not cleared, the MFMA takes zero instead
            constexpr f32x4 zero = {0.f, 0.f, 0.f, 0.f};
            acc[it][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(Bt, h0, s == 0 ? zero : acc[it][0], 0, 0, 0);
            acc[it][1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(Bt, h1, s == 0 ? zero : acc[it][1], 0, 0, 0);
            acc[it][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(Bt, l0, acc[it][0], 0, 0, 0);
            acc[it][1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(Bt, l1, acc[it][1], 0, 0, 0);
            // next step's x operands, spread over the iterations after the first (their LDS reads, issued at the top
            // of the step, get the first iteration to arrive: behind them came the blocks read in iterations 0 and 1)
            if constexpr (it == 1) {
                constexpr int after = ((kAhead < NT || s + 1 < SPC) ? 2 : 0) + ((1 + kAhead < NT || s + 1 < SPC) ? 2 : 0);
                wait_ops(std::integral_constant<int, after>{}, ops);
#pragma unroll
                for (int j = 0; j < 8; ++j) xr[j] = ops.x[j >> 1][j & 1];
#pragma unroll
                for (int j = 0; j < 8; ++j) wv[j] = ops.w[j >> 2][j & 3];
            }
            {
                constexpr int e0 = it == 0 ? 0 : (it - 1) * 8 / (NT - 1), e1 = it == 0 ? 0 : it * 8 / (NT - 1);
#pragma unroll
                for (int e = e0; e < e1; ++e) frag_piece(e >> 1, e & 1, xr, wv, fn);
            }
            if (it == 0) { load_x(rsx, xp0, s3, 0); load_x(rsx, xp0, s3, 1); }
            if (it >= NT - kAhead && it < NT - kAhead + NTW) load_B(rsB, s3b, wave * NTW + (it - (NT - kAhead)));
            if (s == 1 && it == NT - 1 && nxt.valid) mnext = load_meta(nxt);
            __builtin_amdgcn_sched_barrier(0);
        });
        if (s == SPC / 2) put_weights(nxt.c, ws ^ 1, mnext);
    };

    for (int n = 0; cur.valid; ++n) {
        const int ws = n & 1;
        // the first blocks of step 0, whose tile every wave has published (prologue, or the barrier of the last step)
        __builtin_amdgcn_sched_barrier(0);
        static_for<kAhead>([&](auto ic) {
            constexpr int i = decltype(ic)::value;
            read_Bt(std::integral_constant<int, 0>{}, ic, blo[i], bhi[i]);
        });
        __builtin_amdgcn_sched_barrier(0);
        step(std::integral_constant<int, 0>{}, ws, fA, fB);
        step(std::integral_constant<int, 1>{}, ws, fB, fA);
        step(std::integral_constant<int, 2>{}, ws, fA, fB);
        step(std::integral_constant<int, 3>{}, ws, fB, fA);
        if constexpr (SPC == 8) {
            step(std::integral_constant<int, 4>{}, ws, fA, fB);
            step(std::integral_constant<int, 5>{}, ws, fB, fA);
            step(std::integral_constant<int, 6>{}, ws, fA, fB);
            step(std::integral_constant<int, 7>{}, ws, fB, fA);
        }
        park(cur, mcur);
        if (second_late && cur.r == 0) t_nxt = __builtin_amdgcn_readfirstlane(tq[1]);     // drawn during this chunk
        if (!(cur.r + 1 < R && cur.c + 1 < C)) {
            // the item's last chunk: the chain step, then the tickets move up
            chain_step(cur, ws);
            t_cur = t_nxt;
            t_nxt = __builtin_amdgcn_readfirstlane(tq[2]);
            second_late = false;
        }
        mcur = mnext;
        cur = nxt;
        nxt = successor(cur, t_cur, t_nxt);
    }
    if (LOCAL && threadIdx.x == 0) {
        // every workgroup that drew from a slot's counter must sit on the same XCD; anything else (hardware ids that
        // do not spread over p.n_xcd slots) would break the L2 argument above, and is reported instead of ignored
        const int seen = __hip_atomic_fetch_max(p.ws + kWsOwner + slot, xcd_hw + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (seen != 0 && seen != xcd_hw + 1) __hip_atomic_fetch_or(ws_err, kChainErrXcd, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

template <int NT, int SPC, int R, bool SEQ, bool LOCAL, int OUTM, bool SCAN>
static hipError_t launch_kernel(const Params &p, int n_wg, hipStream_t s)
{
    constexpr int lds = lds_bytes<NT, SPC, SCAN>();
    static_assert(lds <= 160 * 1024, "LDS of a compute unit");
    static std::atomic<uint64_t> configured{0};
    const hipError_t e = ensure_dynamic_lds((const void *)chain_kernel<NT, SPC, R, SEQ, LOCAL, OUTM, SCAN>, lds, configured);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL((chain_kernel<NT, SPC, R, SEQ, LOCAL, OUTM, SCAN>), dim3(n_wg), dim3(256), lds, s, p);
    return hipGetLastError();
}

}  // namespace chain

}  // namespace ssd
