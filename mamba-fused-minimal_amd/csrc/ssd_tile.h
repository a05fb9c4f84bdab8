// Building blocks shared by the kernels that keep a (32 headdim rows) x (all dstate columns) state tile per wave
// (gfx950): register types, bf16 packing, buffer descriptors, explicit wait-count immediates, and the 16-byte
// state store with its data hazard guard.
#pragma once
#include "ssd_params.h"

#include <utility>

namespace ssd {
namespace tile {

// compile-time loop: f(std::integral_constant<int, 0>{}), ..., f(std::integral_constant<int, N - 1>{})
template <int... I, class F>
__device__ __forceinline__ void static_for_impl(std::integer_sequence<int, I...>, F &&f) { (f(std::integral_constant<int, I>{}), ...); }
template <int N, class F>
__device__ __forceinline__ void static_for(F &&f) { static_for_impl(std::make_integer_sequence<int, N>{}, f); }

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi)
{
    bf16x2 v = {(__bf16)lo, (__bf16)hi};
    return __builtin_bit_cast(uint32_t, v);
}

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void *base, int64_t bytes)
{
    return __builtin_amdgcn_make_buffer_rsrc((void *)base, 0, (int)(bytes > 0x7fffffffLL ? 0x7fffffffLL : (bytes < 0 ? 0 : bytes)),
                                             0x00020000);
}

// s_waitcnt immediate that only waits for the vector-memory counter to drop to n (gfx9 field layout)
constexpr int vmcnt_imm(int n) { return (n & 15) | (7 << 4) | (15 << 8) | ((n >> 4) << 14); }

// Four consecutive fp32 state values of one row.  The data registers of a wide store are read out over several
// cycles after issue; wait states that depend on them keep a following writer of the same registers away.
// aux: cache policy bits of the store (0 = default; 1 = sc0, 2 = nt, 16 = sc1).
__device__ __forceinline__ void store4_f32(__amdgpu_buffer_rsrc_t rs, int voff, int soff, f32x4 v, int aux = 0)
{
    const u32x4 q = __builtin_bit_cast(u32x4, v);
    if (aux == 17) __builtin_amdgcn_raw_buffer_store_b128(q, rs, 4 * voff, 4 * soff, 17);
    else if (aux == 16) __builtin_amdgcn_raw_buffer_store_b128(q, rs, 4 * voff, 4 * soff, 16);
    else if (aux == 1) __builtin_amdgcn_raw_buffer_store_b128(q, rs, 4 * voff, 4 * soff, 1);
    else __builtin_amdgcn_raw_buffer_store_b128(q, rs, 4 * voff, 4 * soff, 0);
    asm volatile("s_nop 3" ::"v"(q) : "memory");
}

// The same four values rounded to bf16 (nearest even): 8 bytes, default cache policy.
__device__ __forceinline__ void store4_bf16(__amdgpu_buffer_rsrc_t rs, int voff, int soff, f32x4 v)
{
    const u32x2 q = {pack_bf16(v.x, v.y), pack_bf16(v.z, v.w)};
    __builtin_amdgcn_raw_buffer_store_b64(q, rs, 2 * voff, 2 * soff, 0);
    asm volatile("s_nop 3" ::"v"(q) : "memory");
}


// Compile-time model of the vector-memory queue of the step loops that stream x and B through LDS rings
// (ssd_quad.hip, ssd_chain.hip).  Per 32-token step t these kernels issue, in this program order,
//     [st state stores]     top of the step, only where t is the first step of a chunk and the kernel stores there
//     xr requests           the x rows of step t + dist                     (MFMA iteration 0)
//     -- wait W2, s_barrier --                                              (MFMA iteration NT - kAhead)
//     bw requests           this wave's B blocks of step t + dist
// after a prologue that issues (xr, bw) for the steps 0 .. dist - 1, and they wait
//     W0, end of the prologue:   this wave's B blocks of step 0 have landed
//     W1, top of step t (before its stores):   the x rows of step t + 1 have landed
//     W2, iteration NT - kAhead of step t:     this wave's B blocks of step t + 1 have landed.
// Memory operations complete in the order they were issued, so "X has landed" is "at most n operations are
// outstanding" with n = the number issued after X.  replay() walks the program order and counts that number for every
// wait; the kernels static_assert their s_waitcnt immediates against it (operations the model leaves out -- decay
// inputs, tickets, a chain step -- are issued after X or complete before it, and only make a wait longer).
namespace schedule {

// st: stores at a chunk's first step (0 = none); dist_b: the B requests' own distance where it is shorter than that
// of the x requests (B rows come from L2 after their first reader, x rows from memory), -1 = the same
struct Loop { int xr, bw, st, spc, dist, ring; int dist_b = -1; };
constexpr int b_dist(Loop k) { return k.dist_b < 0 ? k.dist : k.dist_b; }
constexpr int kSteps = 48;                           // steps replayed: several chunks past the prologue
struct Waits { int w0; int w1[kSteps]; int w2[kSteps]; };

constexpr Waits replay(Loop k)
{
    Waits r{};
    int last_x[kSteps + 16] = {}, last_b[kSteps + 16] = {};
    int n = 0;      // operations issued so far
    for (int t = 0; t < k.dist; ++t) {
        n += k.xr; last_x[t] = n - 1;
        n += k.bw;          // beyond the B distance these are requests that fetch nothing: every step issues the same number
        if (t < b_dist(k)) last_b[t] = n - 1;
    }
    r.w0 = n - 1 - last_b[0];
    for (int t = 0; t < kSteps; ++t) {
        r.w1[t] = n - 1 - last_x[t + 1];
        if (k.st > 0 && t % k.spc == 0) n += k.st;
        n += k.xr; last_x[t + k.dist] = n - 1;
        r.w2[t] = n - 1 - last_b[t + 1];
        n += k.bw; last_b[t + b_dist(k)] = n - 1;
    }
    return r;
}
// the largest count that is safe for step s of every chunk (the fewest operations behind the one needed)
constexpr int wait_x(Loop k, int s)
{
    const Waits r = replay(k);
    int m = r.w1[s];
    for (int t = s; t < kSteps; t += k.spc) m = r.w1[t] < m ? r.w1[t] : m;
    return m;
}
constexpr int wait_b(Loop k, int s)
{
    const Waits r = replay(k);
    int m = r.w2[s];
    for (int t = s; t < kSteps; t += k.spc) m = r.w2[t] < m ? r.w2[t] : m;
    return m;
}
constexpr int wait_prologue(Loop k) { return replay(k).w0; }
// Ring slots.  The request for step t + dist, issued in step t, overwrites the slot of step t + dist - ring.  x: a
// wave reads the rows of step u at the top of step u - 1, so u = t + dist - ring must satisfy u - 1 < t.  B: every
// wave has consumed the tile of step u by the end of step u, and the requests of step t follow that step's barrier,
// so u < t.  Both hold with a ring one longer than the distance; requests must not reach past the next chunk, and
// the slot of a step must not depend on the chunk.
// (A B ring shorter than the x ring: one longer than the B distance, by the same argument.)
constexpr bool slots_ok(Loop k)
{
    return k.ring == k.dist + 1 && k.dist < k.spc && k.spc % k.ring == 0 && k.spc <= kSteps / 3 && b_dist(k) <= k.dist &&
           b_dist(k) >= 1 && k.spc % (b_dist(k) + 1) == 0;
}

}  // namespace schedule

// bf16 hi / lo halves of the scaled x operand of one 32-token step: [row parity][token pair]
struct Frag { uint32_t hi[2][4], lo[2][4]; };

}  // namespace tile
}  // namespace ssd
