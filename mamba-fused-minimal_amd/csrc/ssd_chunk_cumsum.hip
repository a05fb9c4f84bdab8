// dt preparation and per-chunk cumulative sum of dt * A: the producer of the (batch, nheads, nchunks, chunk_size)
// fp32 tensors `dt` and `dA_cumsum` that the chunk-state / state-passing kernels consume.
//
// Reference semantics (kernels/ssd_chunk_state.py:33-79):
//   d = float(dt[b, l, h]) (+ dt_bias[h]); softplus(d) where d <= 20; clamp to [dt_min, dt_max];
//   tokens past the end of the sequence get d = 0;  dt_out[b, h, c, k] = d;  dA_cumsum[b, h, c, k] = sum_{j<=k} d_j * A[h].
//
// HBM-bound streaming work with a transpose in the middle: dt arrives token-major (heads contiguous), the outputs
// are head-major (the chunk's tokens contiguous).  A workgroup takes one (batch, chunk) and a tile of 32 heads -- 16
// where a lane can fetch four consecutive heads with one load (unit head stride, aligned rows, nheads % 4 == 0):
// an eighth of the load instructions, and 80 heads make five full tiles instead of two and a half --, the tile is
// transposed through LDS, and each wave then owns whole head rows: a lane holds EPL consecutive tokens, sums them serially, the 64 lane totals are scanned with
// data-parallel-primitive moves, and both outputs leave as contiguous rows.
#include "ssd_params.h"

namespace ssd {

namespace {

constexpr int kMaxQ = 1024;

// EPL = tokens per lane in the scan = ceil(chunk_size / 64); VEC = outputs have unit stride along the chunk and
// 16-byte aligned rows, so a lane's EPL = 4 results leave as one 16-byte store
// kHeadTile = heads per workgroup; VLOAD = a lane loads four consecutive heads of a token at once (kHeadTile 16)
template <int EPL, bool VEC, int kHeadTile, bool VLOAD>
__global__ void __launch_bounds__(256) chunk_cumsum_kernel(const CumsumParams p)
{
    extern __shared__ __attribute__((aligned(16))) float tile[];     // [kHeadTile][Q + 4]: rows stay 16-byte aligned
    const int Q = p.Q, pitch = Q + 4;
    const int b = blockIdx.z, c = blockIdx.y, h0 = blockIdx.x * kHeadTile;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int lim = min(Q, p.seqlen - c * Q);
    if (p.clear) {
        // on the way: the workspace of the chain kernel that this launch is in front of
        const int n_wg = gridDim.x * gridDim.y * gridDim.z, wg = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);
        for (int i = wg * 256 + tid; i < p.n_clear; i += n_wg * 256) p.clear[i] = chain_workspace_clear(i, p.n_clear);
    }

    auto activate = [&](float d) {
        if (p.softplus && d <= 20.f) {
            // log1p(t) = log(u) * t / (u - 1) with u = fl(1 + t): the quotient compensates the rounding of u,
            // so the hardware exp / log instructions suffice (a libm log1pf made this kernel ALU-bound)
            const float t = __expf(d), u = 1.f + t;
            d = u == 1.f ? t : __logf(u) * __fdividef(t, u - 1.f);
        }
        return fminf(fmaxf(d, p.dt_min), p.dt_max);
    };
    if constexpr (VLOAD) {
        // ---- thread (token = tid / 4 + 64 i, heads 4 (tid % 4) .. + 3): 8 or 16 bytes per load
        const int hq = 4 * (tid & 3), h = h0 + hq;
        const bool hv = h < p.nheads;                                   // nheads % 4 == 0: all four or none
        float bias[4] = {0.f, 0.f, 0.f, 0.f};
        if (hv && p.dt_bias)
#pragma unroll
            for (int j = 0; j < 4; ++j) bias[j] = load_as_f32(p.dt_bias, (int64_t)(h + j) * p.sbias, p.dt_bias_type);
        constexpr int NIT = EPL;                    // token rows per thread: chunk_size <= 64 * EPL
        const int64_t esz = p.dt_type == DT_F32 ? 4 : 2;
        const char *src = (const char *)p.dt + (b * p.sdt_b + (int64_t)(c * Q + tid / 4) * p.sdt_l + h) * esz;
        const int64_t step = 64 * p.sdt_l * esz;
        float d[NIT][4];
#pragma unroll
        for (int i = 0; i < NIT; ++i) {
            const int k = tid / 4 + 64 * i;
#pragma unroll
            for (int j = 0; j < 4; ++j) d[i][j] = 0.f;
            if (hv && k < lim) {
                if (p.dt_type == DT_F32) {
                    typedef __attribute__((ext_vector_type(4))) float f32x4;
                    const f32x4 q = *(const f32x4 *)(src + i * step);
                    d[i][0] = q.x; d[i][1] = q.y; d[i][2] = q.z; d[i][3] = q.w;
                } else {
                    typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;
                    const u32x2 q = *(const u32x2 *)(src + i * step);
                    const uint32_t w[2] = {q.x, q.y};
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const uint32_t bits = (w[j >> 1] >> (16 * (j & 1))) & 0xffffu;
                        d[i][j] = p.dt_type == DT_BF16 ? bf16_bits_to_f32(bits) : (float)__builtin_bit_cast(_Float16, (uint16_t)bits);
                    }
                }
            }
        }
#pragma unroll
        for (int i = 0; i < NIT; ++i) {
            const int k = tid / 4 + 64 * i;
            if (k < Q) {
#pragma unroll
                for (int j = 0; j < 4; ++j) tile[(hq + j) * pitch + k] = (hv && k < lim) ? activate(d[i][j] + bias[j]) : 0.f;
            }
        }
    } else {
    // ---- load + bias + softplus + clamp, token-major: thread (token = tid / 32 + 8 i, head = tid % 32)
    const int hh = tid & (kHeadTile - 1);
    const int h = h0 + hh;
    const bool hv = h < p.nheads;
    const float bias = (hv && p.dt_bias) ? load_as_f32(p.dt_bias, (int64_t)h * p.sbias, p.dt_bias_type) : 0.f;
    // all of a thread's loads (up to 32 at a time) are issued before the first is used: the kernel is otherwise a
    // chain of memory latencies
    constexpr int NIT = 8 * EPL;                    // token rows per thread: chunk_size <= 64 * EPL
    const char *dt_base = (const char *)p.dt;
    const int64_t esz = p.dt_type == DT_F32 ? 4 : 2;
    const int64_t off0 = (b * p.sdt_b + (int64_t)(c * Q + tid / kHeadTile) * p.sdt_l + (int64_t)h * p.sdt_h) * esz;
    const int64_t step = 8 * p.sdt_l * esz;
#pragma unroll 32
    for (int i = 0; i < NIT; ++i) {
        const int k = tid / kHeadTile + 8 * i;
        if (k >= Q) break;
        float d = 0.f;
        if (hv && k < lim) {
            d = activate(load_as_f32(dt_base + off0 + i * step, 0, p.dt_type) + bias);
        }
        tile[hh * pitch + k] = d;
    }
    }
    __syncthreads();

    // ---- per head row: scan and store.  A wave owns rows wave, wave + 4, ...; NR of them are processed together
    // so that the cross-lane steps of their scans overlap instead of queueing behind one another.
    constexpr int NR = EPL <= 4 ? kHeadTile / 4 : 2;
    typedef __attribute__((ext_vector_type(4))) float f32x4;
    for (int r0 = wave; r0 < kHeadTile; r0 += 4 * NR) {
        float dv[NR][EPL], v[NR][EPL], run[NR], tot[NR];
#pragma unroll
        for (int i = 0; i < NR; ++i) {
            const int r = r0 + 4 * i, hr = h0 + r;
            const bool valid = r < kHeadTile && hr < p.nheads;           // wave-uniform
            const float a = valid ? load_as_f32(p.A, (int64_t)hr * p.sA, p.A_type) : 0.f;
            const float *row = tile + (valid ? r : 0) * pitch;
            if constexpr (VEC && EPL == 4) {
                const f32x4 q = 4 * lane < Q ? *(const f32x4 *)(row + 4 * lane) : (f32x4){0.f, 0.f, 0.f, 0.f};
                dv[i][0] = q.x; dv[i][1] = q.y; dv[i][2] = q.z; dv[i][3] = q.w;
            } else {
#pragma unroll
                for (int e = 0; e < EPL; ++e) {
                    const int k = lane * EPL + e;
                    dv[i][e] = k < Q ? row[k] : 0.f;
                }
            }
            run[i] = 0.f;
#pragma unroll
            for (int e = 0; e < EPL; ++e) {
                run[i] += dv[i][e] * a;
                v[i][e] = run[i];
            }
            tot[i] = run[i];
        }
#pragma unroll
        for (int i = 0; i < NR; ++i) tot[i] = wave_inclusive_sum(tot[i]);
#pragma unroll
        for (int i = 0; i < NR; ++i) {
            const int r = r0 + 4 * i, hr = h0 + r;
            if (r >= kHeadTile || hr >= p.nheads) continue;               // wave-uniform
            const float before = tot[i] - run[i];                         // total of the lanes to the left
            float *dt_out = p.dt_out + b * p.so_b + (int64_t)hr * p.so_h + (int64_t)c * p.so_c;
            float *da_out = p.dacs + b * p.sa_b + (int64_t)hr * p.sa_h + (int64_t)c * p.sa_c;
            if constexpr (VEC && EPL == 4) {
                if (4 * lane < Q) {         // chunk_size is a multiple of 4 here
                    *(f32x4 *)(dt_out + 4 * lane) = (f32x4){dv[i][0], dv[i][1], dv[i][2], dv[i][3]};
                    *(f32x4 *)(da_out + 4 * lane) =
                        (f32x4){v[i][0] + before, v[i][1] + before, v[i][2] + before, v[i][3] + before};
                }
            } else {
#pragma unroll
                for (int e = 0; e < EPL; ++e) {
                    const int k = lane * EPL + e;
                    if (k < Q) {
                        dt_out[(int64_t)k * p.so_k] = dv[i][e];
                        da_out[(int64_t)k * p.sa_k] = v[i][e] + before;
                    }
                }
            }
        }
    }
}

}  // namespace

template <int EPL, bool VEC, int HT = 32, bool VLOAD = false>
static hipError_t launch_t(const CumsumParams &p, hipStream_t s)
{
    const dim3 grid((p.nheads + HT - 1) / HT, p.C, p.batch);
    const size_t lds = (size_t)HT * (p.Q + 4) * sizeof(float);
    // more than 64 KB of LDS has to be asked for, once per kernel and device
    static std::atomic<uint64_t> configured{0};
    const hipError_t e = ensure_dynamic_lds((const void *)chunk_cumsum_kernel<EPL, VEC, HT, VLOAD>,
                                            lds > 65536 ? HT * (kMaxQ + 4) * (int)sizeof(float) : 0, configured);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL((chunk_cumsum_kernel<EPL, VEC, HT, VLOAD>), grid, dim3(256), lds, s, p);
    return hipGetLastError();
}

hipError_t launch_chunk_cumsum(const CumsumParams &p, hipStream_t s)
{
    const int epl = (p.Q + 63) / 64;
    const bool vec = p.Q % 4 == 0 && p.so_k == 1 && p.sa_k == 1 && ((uintptr_t)p.dt_out | (uintptr_t)p.dacs) % 16 == 0 &&
                     (p.so_b | p.so_h | p.so_c | p.sa_b | p.sa_h | p.sa_c) % 4 == 0;
    // four heads per load: unit head stride, every token row and the base on a multiple of four elements
    const int64_t esz = p.dt_type == DT_F32 ? 4 : 2;
    const bool vload = p.sdt_h == 1 && p.nheads % 4 == 0 && (p.sdt_l | p.sdt_b) % 4 == 0 && (uintptr_t)p.dt % (4 * esz) == 0;
    if (epl == 1) return launch_t<1, false>(p, s);
    if (epl == 2) return vload ? launch_t<2, false, 16, true>(p, s) : launch_t<2, false>(p, s);
    if (epl <= 4) {
        if (vec && epl == 4) return vload ? launch_t<4, true, 16, true>(p, s) : launch_t<4, true>(p, s);
        return launch_t<4, false>(p, s);
    }
    if (epl <= 8) return launch_t<8, false>(p, s);
    return launch_t<16, false>(p, s);
}

bool chunk_cumsum_supported(const CumsumParams &p) { return p.Q >= 1 && p.Q <= kMaxQ && p.C <= 65535 && p.batch <= 65535; }

}  // namespace ssd
