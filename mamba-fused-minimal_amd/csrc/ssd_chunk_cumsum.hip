// dt preparation and per-chunk cumulative sum of dt * A: the producer of the (batch, nheads, nchunks, chunk_size)
// fp32 tensors `dt` and `dA_cumsum` that the chunk-state / state-passing kernels consume.
//
// Reference semantics (kernels/ssd_chunk_state.py:33-79):
//   d = float(dt[b, l, h]) (+ dt_bias[h]); softplus(d) where d <= 20; clamp to [dt_min, dt_max];
//   tokens past the end of the sequence get d = 0;  dt_out[b, h, c, k] = d;  dA_cumsum[b, h, c, k] = sum_{j<=k} d_j * A[h].
//
// HBM-bound streaming work with a transpose in the middle: dt arrives token-major (heads contiguous), the outputs
// are head-major (the chunk's tokens contiguous).  A workgroup takes one (batch, chunk) and a tile of 32 heads:
// reads are 32 consecutive heads per token, the tile is transposed through LDS, and each wave then owns whole head
// rows: a lane holds EPL consecutive tokens, sums them serially, the 64 lane totals are scanned with DPP-free
// shuffles, and both outputs leave as contiguous rows.
#include "ssd_params.h"

namespace ssd {

namespace {

constexpr int kHeadTile = 32;
constexpr int kMaxQ = 1024;

__device__ __forceinline__ float wave_inclusive_scan(float v, int lane)
{
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const float o = __shfl_up(v, d, 64);
        if (lane >= d) v += o;
    }
    return v;
}

__global__ void __launch_bounds__(256) chunk_cumsum_kernel(const CumsumParams p)
{
    extern __shared__ float tile[];                 // [kHeadTile][Q + 1]
    const int Q = p.Q, pitch = Q + 1;
    const int b = blockIdx.z, c = blockIdx.y, h0 = blockIdx.x * kHeadTile;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int lim = min(Q, p.seqlen - c * Q);

    // ---- load + bias + softplus + clamp, token-major: thread (token = tid / 32 + 8 i, head = tid % 32)
    const int hh = tid & (kHeadTile - 1);
    const int h = h0 + hh;
    const bool hv = h < p.nheads;
    const float bias = (hv && p.dt_bias) ? load_as_f32(p.dt_bias, (int64_t)h * p.sbias, p.dt_bias_type) : 0.f;
    for (int k = tid / kHeadTile; k < Q; k += 256 / kHeadTile) {
        float d = 0.f;
        if (hv && k < lim) {
            d = load_as_f32(p.dt, b * p.sdt_b + (int64_t)(c * Q + k) * p.sdt_l + (int64_t)h * p.sdt_h, p.dt_type) + bias;
            if (p.softplus && d <= 20.f) d = log1pf(expf(d));
            d = fminf(fmaxf(d, p.dt_min), p.dt_max);
        }
        tile[hh * pitch + k] = d;
    }
    __syncthreads();

    // ---- per head row: scan and store
    const int epl = (Q + 63) >> 6;                  // tokens per lane
    for (int r = wave; r < kHeadTile; r += 4) {
        const int hr = h0 + r;
        if (hr >= p.nheads) break;                  // wave-uniform
        const float a = load_as_f32(p.A, (int64_t)hr * p.sA, p.A_type);
        const float *row = tile + r * pitch;
        float v[kMaxQ / 64];
        float run = 0.f;
#pragma unroll
        for (int e = 0; e < kMaxQ / 64; ++e) {
            const int k = lane * epl + e;
            const float d = (e < epl && k < Q) ? row[k] : 0.f;
            run += d * a;
            v[e] = run;
        }
        const float before = wave_inclusive_scan(run, lane) - run;     // total of the lanes to the left
        float *dt_out = p.dt_out + b * p.so_b + (int64_t)hr * p.so_h + (int64_t)c * p.so_c;
        float *da_out = p.dacs + b * p.sa_b + (int64_t)hr * p.sa_h + (int64_t)c * p.sa_c;
#pragma unroll
        for (int e = 0; e < kMaxQ / 64; ++e) {
            const int k = lane * epl + e;
            if (e < epl && k < Q) {
                dt_out[(int64_t)k * p.so_k] = row[k];
                da_out[(int64_t)k * p.sa_k] = v[e] + before;
            }
        }
    }
}

}  // namespace

hipError_t launch_chunk_cumsum(const CumsumParams &p, hipStream_t s)
{
    dim3 grid((p.nheads + kHeadTile - 1) / kHeadTile, p.C, p.batch);
    const size_t lds = (size_t)kHeadTile * (p.Q + 1) * sizeof(float);
    static bool big_lds = false;        // more than 64 KB of LDS has to be requested explicitly, once
    if (lds > 65536 && !big_lds) {
        hipError_t e = hipFuncSetAttribute((const void *)chunk_cumsum_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                           kHeadTile * (kMaxQ + 1) * (int)sizeof(float));
        if (e != hipSuccess) return e;
        big_lds = true;
    }
    hipLaunchKernelGGL(chunk_cumsum_kernel, grid, dim3(256), lds, s, p);
    return hipGetLastError();
}

bool chunk_cumsum_supported(const CumsumParams &p) { return p.Q >= 1 && p.Q <= kMaxQ && p.C <= 65535 && p.batch <= 65535; }

}  // namespace ssd
