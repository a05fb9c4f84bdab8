// Stand-alone inter-chunk recurrence  s = exp(dA_c) * s + states_c  (exclusive scan written to `out`,
// inclusive last value to `final`).  Pure streaming: each lane owns VEC consecutive state elements of one
// (batch, head) and walks the chunks serially; the loads of states_c do not depend on the running state,
// so four chunks are kept in flight per lane to cover HBM latency.
//
// Reference semantics: kernels/ssd_state_passing.py:27-84.
#include "ssd_params.h"

namespace ssd {

typedef __attribute__((ext_vector_type(4))) float f32x4;

template <int VEC> struct Vals { float v[VEC]; };

template <int VEC>
__device__ __forceinline__ Vals<VEC> load_vals(const void *base, int64_t off, int dt)
{
    Vals<VEC> r;
    if (VEC == 4 && dt == DT_F32) {
        f32x4 q = *(const f32x4 *)((const float *)base + off);
        r.v[0] = q.x; r.v[1] = q.y; r.v[2] = q.z; r.v[3] = q.w;
    } else {
#pragma unroll
        for (int j = 0; j < VEC; ++j) r.v[j] = load_as_f32(base, off + j, dt);
    }
    return r;
}

template <int VEC>
__device__ __forceinline__ void store_vals(void *base, int64_t off, int dt, const Vals<VEC> &r)
{
    if (VEC == 4 && dt == DT_F32) {
        f32x4 q = {r.v[0], r.v[1], r.v[2], r.v[3]};
        *(f32x4 *)((float *)base + off) = q;
    } else {
#pragma unroll
        for (int j = 0; j < VEC; ++j) store_from_f32(base, off + j, dt, r.v[j]);
    }
}

// D = chunks in flight per lane
template <int VEC, int D>
__global__ void __launch_bounds__(256) state_passing_kernel(const PassParams p)
{
    const int d0 = (blockIdx.x * 256 + threadIdx.x) * VEC;
    const int h = blockIdx.y, b = blockIdx.z;
    if (d0 >= p.dim) return;
    const int64_t st_base = b * p.sst_b + h * p.sst_h + d0;
    const int64_t out_base = b * p.so_b + h * p.so_h + d0;
    const float *da = p.da + b * p.sda_b + h * p.sda_h;
    const int32_t *sq = p.seq ? p.seq + b * p.ssq_b : nullptr;

    Vals<VEC> s;
    if (p.init) s = load_vals<VEC>(p.init, b * p.sin_b + h * p.sin_h + d0, p.dt_init);
    else {
#pragma unroll
        for (int j = 0; j < VEC; ++j) s.v[j] = 0.f;
    }
    // `out` may be the buffer `states` lives in (slot c holds the chunk state of chunk c and receives the state that
    // enters chunk c): a lane only ever touches its own elements, reads slot c before it writes it, and memory
    // operations of one lane on one address keep their program order -- hence the first loads before the first store
    // the chunk's decay and the id of its last token travel with its state: requested D chunks ahead as well
    auto last_id = [&](int c) { return sq ? sq[(int64_t)(min((c + 1) * p.Q, p.seqlen) - 1) * p.ssq_l] : 0; };
    Vals<VEC> nxt[D];
    float dan[D];
    int32_t idn[D];
#pragma unroll
    for (int i = 0; i < D; ++i)
        if (i < p.C) {
            nxt[i] = load_vals<VEC>(p.states, st_base + i * p.sst_c, p.dt_states);
            dan[i] = da[i * p.sda_c];
            idn[i] = last_id(i);
        }
    store_vals<VEC>(p.out, out_base, p.dt_out, s);
    int32_t prev = 0;
    for (int c0 = 0; c0 < p.C; c0 += D) {
#pragma unroll
        for (int i = 0; i < D; ++i) {
            const int c = c0 + i;
            if (c < p.C) {
                const Vals<VEC> cur = nxt[i];
                float sc = __expf(dan[i]);
                const int32_t id = idn[i];
                if (c + D < p.C) {
                    nxt[i] = load_vals<VEC>(p.states, st_base + (int64_t)(c + D) * p.sst_c, p.dt_states);
                    dan[i] = da[(c + D) * p.sda_c];
                    idn[i] = last_id(c + D);
                }
                if (sq) {
                    if (id != prev) sc = 0.f;
                    prev = id;
                }
#pragma unroll
                for (int j = 0; j < VEC; ++j) s.v[j] = sc * s.v[j] + cur.v[j];
                if (c < p.C - 1) store_vals<VEC>(p.out, out_base + (int64_t)(c + 1) * p.so_c, p.dt_out, s);
                else store_vals<VEC>(p.fin, b * p.sf_b + h * p.sf_h + d0, DT_F32, s);
            }
        }
    }
}

hipError_t launch_state_passing(const PassParams &p, hipStream_t s)
{
    if (p.batch <= 0 || p.nheads <= 0 || p.dim <= 0 || p.C <= 0) return hipSuccess;
    auto al = [](const void *q, size_t a) { return q == nullptr || ((uintptr_t)q % a) == 0; };
    const bool vec = p.dim % 4 == 0 && al(p.states, 16) && al(p.out, 16) && al(p.fin, 16) && al(p.init, 16) &&
                     (p.sst_b | p.sst_c | p.sst_h | p.so_b | p.so_c | p.so_h | p.sf_b | p.sf_h | p.sin_b | p.sin_h) % 4 == 0;
    if (vec) {
        dim3 grid((p.dim / 4 + 255) / 256, p.nheads, p.batch), block(256);
        // four chunks in flight per lane cover HBM latency when at least four workgroups sit on every compute unit;
        // smaller launches keep eight in flight (b=1 H=80, 128 chunks: 170 -> 164 us)
        if ((int64_t)grid.x * grid.y * grid.z < 1024) hipLaunchKernelGGL((state_passing_kernel<4, 8>), grid, block, 0, s, p);
        else hipLaunchKernelGGL((state_passing_kernel<4, 4>), grid, block, 0, s, p);
    } else {
        dim3 grid((p.dim + 255) / 256, p.nheads, p.batch), block(256);
        hipLaunchKernelGGL((state_passing_kernel<1, 4>), grid, block, 0, s, p);
    }
    return hipGetLastError();
}

}  // namespace ssd
