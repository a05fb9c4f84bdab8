/*
 * ssd_gfx950.h -- C ABI of libssd_gfx950.so: the Mamba2 SSD chunk-state + state-passing path for
 * AMD MI355X (gfx950), written as hand-coded HIP kernels.
 *
 * Every entry point
 *   - takes device pointers, element strides and sizes only (no C++ or framework types);
 *   - enqueues its kernels on the given hipStream_t (passed as void*; NULL = the default stream) and
 *     returns without synchronising;
 *   - returns 0 on success, a negative ssd_status for rejected arguments, or a positive hipError_t
 *     reported by the launch; it never throws and never prints.
 * Tensors are described by ssd_tensor: a data pointer, an element type and per-dimension strides counted
 * in elements, so views (for example x and B carved out of a packed projection, or the stride-Q view
 * dA_cumsum[..., -1]) are passed without copies.  The innermost stride of x, B, states, out,
 * initial_states and final_states must be 1.
 *
 * Threads: an entry point may be called from any host thread; a call holds no state of its own beyond its
 * arguments.  What the library keeps per process is atomic: a cache of device properties, a per-device record of
 * which kernels have been given their LDS size, and the three ssd_set_* hooks below, which are process-wide test and
 * tuning knobs (a value set in one thread changes the kernel choice of later calls in every thread, never their
 * results beyond rounding).  Calls that overlap in time must not share a workspace (ssd_fused_opts) or the static
 * scratch (ssd_fused_chunk_state_passing_fwd_static).
 *
 * Replaces, in the reference repository (RishiAstra/mamba-fused-minimal):
 *   ssd_chunk_state_fwd                -> kernels/ssd_chunk_state.py:202-232 (_chunk_state_fwd) and the
 *                                         Triton kernel it launches, kernels/ssd_chunk_state.py:97-173
 *   ssd_state_passing_fwd              -> kernels/ssd_state_passing.py:87-115 (_state_passing_fwd) and
 *                                         kernels/ssd_state_passing.py:27-84
 *   ssd_fused_chunk_state_passing_fwd  -> kernels/fused_globalbar.py:201-266 and
 *                                         kernels/fused_concurrent.py:255-331 (the two fused wrappers used by
 *                                         main.py:85 and main.py:100) and their kernels
 */
#ifndef SSD_GFX950_H
#define SSD_GFX950_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SSD_ABI_VERSION 1

typedef enum ssd_dtype {
    SSD_F32 = 0,
    SSD_BF16 = 1,
    SSD_F16 = 2
} ssd_dtype;

typedef enum ssd_status {
    SSD_OK = 0,
    SSD_ERR_NULL = -1,        /* a required pointer is NULL */
    SSD_ERR_SHAPE = -2,       /* sizes inconsistent (nheads % ngroups, nchunks != ceil(seqlen/chunk), <= 0 ...) */
    SSD_ERR_DTYPE = -3,       /* element type not supported for this argument */
    SSD_ERR_STRIDE = -4,      /* innermost stride != 1 where the kernels need it */
    SSD_ERR_DEVICE = -5,      /* current device is not gfx950, or no device */
    SSD_ERR_SCRATCH = -6,     /* a kernel was asked for that needs a workspace, and none (or too small a one) was given */
    /* reported by ssd_fused_workspace_status about the last launch of the ticket / flag-chain kernel (outputs unusable): */
    SSD_ERR_CHAIN_TIMEOUT = -7,    /* a bounded flag wait ran out */
    SSD_ERR_CHAIN_XCD = -8,        /* workgroups of two XCDs drew from one per-XCD ticket counter */
    SSD_ERR_CHAIN_INCOMPLETE = -9, /* a ticket counter that owns work items was never served: their outputs were not written */
    SSD_ERR_CHAIN_WORKSPACE = -10  /* the workspace was not what ssd_fused_opts.epoch promised */
} ssd_status;

/* A strided device tensor.  stride[i] is in elements; unused trailing entries are ignored. */
typedef struct ssd_tensor {
    void *data;
    int32_t dtype;            /* ssd_dtype */
    int32_t reserved;
    int64_t stride[5];
} ssd_tensor;

/* Problem sizes.  nchunks must equal ceil(seqlen / chunk_size). */
typedef struct ssd_dims {
    int32_t batch, seqlen, nheads, headdim, dstate, ngroups, chunk_size, nchunks;
} ssd_dims;

/* ABI version of the loaded library (== SSD_ABI_VERSION it was built with). */
int ssd_version(void);

/* Static text for a status / hipError_t returned by the calls below. */
const char *ssd_status_string(int status);

/*
 * Chunk state (reference: kernels/ssd_chunk_state.py:202-232 / :97-173):
 *   states[b,c,h,p,n] = sum_{k < lim} x[b,cQ+k,h,p] * B[b,cQ+k,h/(H/G),n] * w_k,
 *   w_k = exp(min(dA_cumsum[b,h,c,Q-1] - dA_cumsum[b,h,c,k], 0)) * dt[b,h,c,k] * [seq_idx[b,cQ+k] == seq_idx[b,cQ+lim-1]],
 *   lim = min(Q, seqlen - cQ).
 * x (b,L,H,P) and B (b,L,G,N): bf16, f16 or f32, same type.  dt, dA_cumsum (b,H,C,Q): f32.
 * seq_idx (b,L) int32, data == NULL when absent.  states (b,C,H,P,N): f32, bf16 or f16.
 * clamp != 0 keeps the min(.,0) above (the unfused reference kernel); 0 drops it (the fused reference kernels).
 */
int ssd_chunk_state_fwd(const ssd_tensor *x, const ssd_tensor *B, const ssd_tensor *dt,
                        const ssd_tensor *dA_cumsum, const ssd_tensor *seq_idx, const ssd_tensor *states,
                        const ssd_dims *dims, int clamp, void *stream);

/*
 * State passing (reference: kernels/ssd_state_passing.py:87-115 / :27-84), on a flattened state axis:
 *   s = initial_states or 0;  out[:,0] = s;
 *   for c: s = exp(dA_chunk[b,h,c]) * [id(c) == id(c-1)] * s + states[b,c,h];  out[:,c+1] = s (c < C-1) else final = s
 *   id(c) = seq_idx[b, min((c+1)Q, seqlen) - 1], id(-1) = 0.
 * states (b,C,H,dim): f32/bf16/f16.  dA_chunk (b,H,C) f32, any strides.  initial_states (b,H,dim) nullable.
 * out (b,C,H,dim): f32/bf16/f16.  final_states (b,H,dim): f32.  seqlen and chunk_size are only read when
 * seq_idx is given.
 */
int ssd_state_passing_fwd(const ssd_tensor *states, const ssd_tensor *dA_chunk, const ssd_tensor *initial_states,
                          const ssd_tensor *seq_idx, const ssd_tensor *out, const ssd_tensor *final_states,
                          int32_t batch, int32_t nchunks, int32_t nheads, int32_t dim,
                          int32_t seqlen, int32_t chunk_size, void *stream);

/*
 * Fused chunk state + state passing in one launch (reference: kernels/fused_globalbar.py:201-266,
 * kernels/fused_concurrent.py:255-331).  Arguments as in the two calls above, except that
 * initial_states is (b,H,P,N), out is (b,C,H,P,N), final_states is (b,H,P,N) f32, and the chunk-end decay
 * is read from dA_cumsum[..., Q-1].  states->data == NULL (or states == NULL) means "do not materialise the
 * per-chunk states"; otherwise they are written as a side effect exactly as ssd_chunk_state_fwd would.
 * With few state tiles (batch * nheads * headdim / 32 below 512) and many chunks the call runs as a chunk-state launch
 * that keeps every compute unit busy plus a streaming recurrence; that needs a place for the chunk states: a fp32
 * `out` serves as one (the recurrence then works in place), and so does a fp32 `states` buffer.  With a 16-bit `out`
 * and no `states` such a problem stays on the kernel with one workgroup per tile, which is slower (the library never
 * allocates): a caller in that position gains by passing `states`.  Arguments that only the plain FMA kernel takes
 * (fp32 or fp16 x / B, sizes off the MFMA tiling) run as the same two launches from two chunks upwards, given a fp32
 * `out` or a fp32 `states`.
 */
int ssd_fused_chunk_state_passing_fwd(const ssd_tensor *x, const ssd_tensor *B, const ssd_tensor *dt,
                                      const ssd_tensor *dA_cumsum, const ssd_tensor *seq_idx,
                                      const ssd_tensor *initial_states, const ssd_tensor *states,
                                      const ssd_tensor *out, const ssd_tensor *final_states,
                                      const ssd_dims *dims, int clamp, void *stream);

/*
 * The fused call with a caller-provided workspace, which opens the kernel that spreads ONE sequence's chunks over
 * all compute units.  The reference does the same job with scratch tensors it allocates per call: two ticket
 * counters and a global barrier (kernels/fused_globalbar.py:130-137, 237-238), or per-(batch, head) completion
 * counters plus a throttle semaphore (kernels/fused_concurrent.py:81-84, 141, 205-208, 296-298).  Here work items
 * (four state tiles sharing B x up to four consecutive chunks) are drawn from a ticket counter in chunk-major order;
 * an item accumulates its chunk states from zero, then waits for the flag of the state entering its first chunk,
 * reads that state back from `out`, runs s <- exp(dA_chunk) [same sequence] s + chunk state over its chunks, stores
 * the last state first and raises the next flag once that store is acknowledged.  An item only waits for an item with
 * a smaller ticket and tickets are drawn by running workgroups only, so the chain makes progress whatever workgroups
 * are resident.  The wait is bounded nevertheless (spin_limit polls): a wave that gives up sets the error word of the
 * workspace and still raises its own flag, so the launch always drains; ssd_fused_workspace_status reports it.
 *
 * workspace: device memory, 4-byte aligned, at least ssd_fused_workspace_bytes(dims) -- with bf16 `out`: 16-byte
 * aligned and at least ssd_fused_workspace_bytes_for(dims, SSD_BF16, chunks_per_item), see below --; the call clears what it uses
 * (a small fill launch, no memset node), so the memory may hold anything and may be reused by later calls on the
 * same stream (a caller that keeps a workspace to itself can save the fill launch: `epoch` below).  Two calls whose kernels may overlap (different streams) need workspaces of their own.
 * kernel: SSD_KERNEL_AUTO lets the library choose between this kernel and those of ssd_fused_chunk_state_passing_fwd
 * (which it runs when the shape, element types, a `states` output or too small a workspace rule the chain kernel out:
 * it needs bf16 x / B, fp32 initial / final states, fp32 or bf16 out, no `states`, dstate 64 or 128, chunk 128 or
 * 256); SSD_KERNEL_CHAIN insists on it
 * and returns SSD_ERR_SCRATCH where it cannot run; SSD_KERNEL_CHAIN_LOCAL / _GLOBAL also fix how passed states cross
 * between compute units, which the library otherwise chooses from the number of units per XCD (LOCAL: one ticket
 * counter per XCD over that XCD's share of the units, states exchanged through its L2; GLOBAL: one counter, states
 * exchanged through memory with device-scope accesses).  The results do not depend on the choice beyond rounding.
 * opts == NULL behaves as ssd_fused_chunk_state_passing_fwd.
 */
typedef struct ssd_fused_opts {
    void *workspace;
    uint64_t workspace_bytes;
    int32_t spin_limit;       /* flag polls before a wave gives up; 0 = default (about 4 million) */
    int32_t kernel;           /* SSD_KERNEL_AUTO, or one of the SSD_KERNEL_CHAIN values to insist on that kernel */
    int32_t chunks_per_item;  /* chain kernel: consecutive chunks per work item, 1, 2 or 4; 0 = choose */
    int32_t epoch;            /* chain kernel: 0 = the workspace may hold anything, the call clears it with a small fill
                                 launch (default).  n > 0 = a promise that saves that launch: the call before this one on
                                 this workspace (same stream, or ordered before it) was made with epoch n - 1, or with
                                 epoch 0 if n == 2, no other use of the memory came in between, and this call has no more
                                 (state tile, chunk) pairs -- batch * nheads * headdim / 32 * nchunks -- than the epoch-0
                                 call that cleared the workspace last (the flags behind those it cleared hold
                                 anything).  Flags carry the epoch and the ticket counters exist once per parity, so the
                                 kernel leaves what the next epoch needs at zero by itself.  Only calls that ran the chain
                                 kernel count (see used_workspace).  Start again from 0 before n would overflow, and
                                 whenever a call needs more pairs than the last clearing covered.  A broken promise is
                                 detected by the kernel where it can be (wrong epoch before, flags outside the cleared
                                 part) and reported as SSD_ERR_CHAIN_WORKSPACE by ssd_fused_workspace_status. */
    int32_t *used_workspace;  /* host memory or NULL: set to 1 if the call ran the chain kernel -- and so used the
                                 workspace and its epoch --, to 0 if another kernel family served it */
} ssd_fused_opts;

enum { SSD_KERNEL_AUTO = 0, SSD_KERNEL_CHAIN = 1, SSD_KERNEL_CHAIN_LOCAL = 2, SSD_KERNEL_CHAIN_GLOBAL = 3 };

uint64_t ssd_fused_workspace_bytes(const ssd_dims *dims);
/*
 * The same for a given element type of `out`.  The reference's state passing keeps the running state in fp32
 * registers over the whole sequence whatever `out` is stored as (kernels/ssd_state_passing.py:61-84); the chain
 * kernel hands it from work item to work item through memory, so with bf16 `out` every item's last state is also
 * written in fp32 to the workspace, where the next item reads it: 32 x dstate x 4 bytes per (state tile, item)
 * behind the flags, i.e. 1 / chunks_per_item of an fp32 `out`.  chunks_per_item: the value the call will be given in
 * ssd_fused_opts (0 = the library's choice for these sizes on the current device; with bf16 `out` items of one chunk
 * are not offered).  Returns 0 where the chain kernel does not take that type (fp16 `out`, chunks_per_item == 1 with
 * bf16): such calls run on the other kernels and need no workspace.  SSD_F32: ssd_fused_workspace_bytes(dims).
 */
uint64_t ssd_fused_workspace_bytes_for(const ssd_dims *dims, int out_dtype, int chunks_per_item);

int ssd_fused_chunk_state_passing_fwd_ws(const ssd_tensor *x, const ssd_tensor *B, const ssd_tensor *dt,
                                         const ssd_tensor *dA_cumsum, const ssd_tensor *seq_idx,
                                         const ssd_tensor *initial_states, const ssd_tensor *states,
                                         const ssd_tensor *out, const ssd_tensor *final_states,
                                         const ssd_dims *dims, int clamp, const ssd_fused_opts *opts, void *stream);

/*
 * Waits for `stream` and reads what the last launch of the chain kernel left in the header of a workspace used by
 * ssd_fused_chunk_state_passing_fwd_ws: SSD_OK, or -- the outputs are then unusable --
 *   SSD_ERR_CHAIN_WORKSPACE   the workspace was not what the call's epoch promised (another epoch before it, or more
 *                             (state tile, chunk) pairs than the last clearing covered);
 *   SSD_ERR_CHAIN_XCD         workgroups that report different XCDs drew from one per-XCD ticket counter (the LOCAL
 *                             variant's assumption about the device does not hold);
 *   SSD_ERR_CHAIN_INCOMPLETE  a ticket counter handed out fewer work items than it owns (LOCAL: an XCD that owns
 *                             state tiles received no workgroup), so part of the outputs was never written;
 *   SSD_ERR_CHAIN_TIMEOUT     a wave gave up waiting for the state entering its work item.
 * Read it before the next launch on the same workspace, which starts the record afresh.  A call that ran another
 * kernel family (SSD_KERNEL_AUTO: see ssd_query_fused_plan) leaves the workspace alone; memory the chain kernel has
 * never cleared reports SSD_OK.  No counterpart in the reference, whose spin loops are unbounded and whose failure mode
 * is a hang (kernels/fused_concurrent.py:11, 300).
 * ssd_fused_workspace_status_of decodes a host copy of the first SSD_WORKSPACE_HEADER_INTS ints of a workspace the
 * same way, for a caller that brings the header back with a copy of its own (no synchronisation here, no device
 * needed).
 */
#define SSD_WORKSPACE_HEADER_INTS 128
int ssd_fused_workspace_status(const void *workspace, void *stream);
int ssd_fused_workspace_status_of(const int32_t *header);

/*
 * ssd_fused_chunk_state_passing_fwd_ws without a workspace argument and without any allocation.  It has no
 * counterpart in the reference; it is for callers that cannot allocate device memory or have it allocated on their
 * behalf: code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  The ticket counters and
 * flags live in a fixed 1 MiB array inside the library's own code object (one copy per GPU, held until the process
 * ends); the call clears what it uses with a small fill launch and runs the chain kernel, whatever the problem size
 * (the kernel choice of the other entry points is not made here: SSD_ERR_SHAPE for arguments that kernel does not
 * cover -- it needs bf16 x / B, fp32 out / initial / final states (bf16 out needs room the array does not have),
 * dstate 64 or 128, chunk 128 or 256 --,
 * SSD_ERR_SCRATCH when batch * nheads * (headdim / 32) * nchunks + 128 ints do not fit the array, i.e. above 262 016
 * (state tile, chunk) pairs).  Every call on a GPU shares that GPU's array: two calls whose kernels may overlap
 * (different streams, different host threads) race on it and must be serialised by the caller.
 * ssd_fused_static_status is ssd_fused_workspace_status for that array.
 */
int ssd_fused_chunk_state_passing_fwd_static(const ssd_tensor *x, const ssd_tensor *B, const ssd_tensor *dt,
                                             const ssd_tensor *dA_cumsum, const ssd_tensor *seq_idx,
                                             const ssd_tensor *initial_states, const ssd_tensor *out,
                                             const ssd_tensor *final_states, const ssd_dims *dims, int clamp,
                                             void *stream);
int ssd_fused_static_status(void *stream);

/*
 * Which kernel family the three calls above would pick for these arguments: 1 = bf16 MFMA path,
 * 0 = generic FMA path (other element types or shapes the MFMA tiling does not cover), negative = rejected.
 * Pure host logic; launches nothing.
 */
int ssd_query_path(const ssd_tensor *x, const ssd_tensor *B, const ssd_dims *dims);

/*
 * Which kernel family a fused call on plain tensors of these sizes would run, and why: the library ranks its fused
 * kernels by an estimate of their duration (a fit to measured times, per compute unit) and this call returns the
 * ranking.  Assumed: bf16 x / B, fp32 dt / dA_cumsum / out / final_states, contiguous, no `states` output -- the
 * arguments every family covers.  has_workspace != 0 asks about ssd_fused_chunk_state_passing_fwd_ws with a
 * workspace of ssd_fused_workspace_bytes(dims) and SSD_KERNEL_AUTO, 0 about ssd_fused_chunk_state_passing_fwd.
 * compute_units: of the device the call would run on; 0 = 256 (MI355X).  Pure host logic: touches no device and
 * launches nothing, so it also answers on a machine without a GPU.  No counterpart in the reference, whose two fused
 * wrappers each have one kernel (kernels/fused_globalbar.py:201-266, kernels/fused_concurrent.py:255-331).
 * estimate_us[f] is 0 for a family that does not apply to the sizes.
 */
enum { SSD_FAMILY_GENERIC = 0, SSD_FAMILY_TOKEN_SPLIT = 1, SSD_FAMILY_FOUR_TILE = 2, SSD_FAMILY_PAIR = 3,
       SSD_FAMILY_CHAIN = 4, SSD_FAMILY_COUNT = 5 };

typedef struct ssd_fused_plan {
    int32_t family;                         /* SSD_FAMILY_* the call would run */
    int32_t chunks_per_item;                /* of the chain kernel when that is the family, else 0 */
    float estimate_us[SSD_FAMILY_COUNT];    /* the model's estimate per family (chain: at its best chunks per item) */
} ssd_fused_plan;

int ssd_query_fused_plan(const ssd_dims *dims, int has_workspace, int compute_units, ssd_fused_plan *plan);

/*
 * dt preparation and per-chunk cumulative sum, the producer of `dt` and `dA_cumsum` for the three calls above.
 * Replaces _chunk_cumsum_fwd / _chunk_cumsum_fwd_kernel (kernels/ssd_chunk_state.py:176-199, 33-79):
 *   d = float(dt[b,l,h]) (+ dt_bias[h]); d = log1p(exp(d)) where dt_softplus and d <= 20; d = clamp(d, dt_min, dt_max);
 *   d = 0 for tokens past seqlen;  dt_out[b,h,c,k] = d;  dA_cumsum[b,h,c,k] = sum_{j<=k} d_j * A[h].
 * dt: (batch, seqlen, nheads) f32/bf16/f16, any strides; A, dt_bias (nullable): (nheads), f32/bf16/f16;
 * dt_out, dA_cumsum: (batch, nheads, nchunks, chunk_size) fp32, any strides.  chunk_size <= 1024.
 */
int ssd_chunk_cumsum_fwd(const ssd_tensor *dt, const ssd_tensor *A, const ssd_tensor *dt_bias, const ssd_tensor *dt_out,
                         const ssd_tensor *dA_cumsum, int32_t batch, int32_t seqlen, int32_t nheads, int32_t chunk_size,
                         int dt_softplus, float dt_min, float dt_max, void *stream);

/*
 * dt preparation + chunk state + state passing in one call: ssd_chunk_cumsum_fwd followed by
 * ssd_fused_chunk_state_passing_fwd (reference: kernels/ssd_chunk_state.py:176-199 followed by
 * kernels/fused_globalbar.py:201-266 / kernels/fused_concurrent.py:255-331, as main.py:78-100 calls them).
 * dt_raw: (batch, seqlen, nheads) f32/bf16/f16; A, dt_bias (nullable): (nheads).  dt_out and dA_cumsum
 * (batch, nheads, nchunks, chunk_size) fp32 are OUTPUTS here (the stages after the path read them); the other
 * arguments are those of ssd_fused_chunk_state_passing_fwd without `states`.  Two launches on `stream`; dt_out and
 * dA_cumsum are exactly what ssd_chunk_cumsum_fwd writes.
 */
int ssd_fused_cumsum_chunk_state_passing_fwd(const ssd_tensor *x, const ssd_tensor *B, const ssd_tensor *dt_raw,
                                             const ssd_tensor *A, const ssd_tensor *dt_bias, const ssd_tensor *seq_idx,
                                             const ssd_tensor *initial_states, const ssd_tensor *dt_out,
                                             const ssd_tensor *dA_cumsum, const ssd_tensor *out,
                                             const ssd_tensor *final_states, const ssd_dims *dims, int dt_softplus,
                                             float dt_min, float dt_max, int clamp, void *stream);

/*
 * The same with a workspace (ssd_fused_opts as in ssd_fused_chunk_state_passing_fwd_ws), which opens the ticket /
 * flag-chain kernel to this call as well.  Still two launches: where that kernel runs, the producer's launch clears
 * its workspace on the way, so the fill launch of ssd_fused_chunk_state_passing_fwd_ws is not needed.  Without a
 * usable workspace it behaves as ssd_fused_cumsum_chunk_state_passing_fwd.  No counterpart in the reference beyond
 * the two calls it composes (kernels/ssd_chunk_state.py:176-199, kernels/fused_concurrent.py:255-331).
 */
int ssd_fused_cumsum_chunk_state_passing_fwd_ws(const ssd_tensor *x, const ssd_tensor *B, const ssd_tensor *dt_raw,
                                                const ssd_tensor *A, const ssd_tensor *dt_bias, const ssd_tensor *seq_idx,
                                                const ssd_tensor *initial_states, const ssd_tensor *dt_out,
                                                const ssd_tensor *dA_cumsum, const ssd_tensor *out,
                                                const ssd_tensor *final_states, const ssd_dims *dims, int dt_softplus,
                                                float dt_min, float dt_max, int clamp, const ssd_fused_opts *opts,
                                                void *stream);

/*
 * The consumer of the passed states: the state-dependent half of the chunk scan.  Replaces that part of
 * _chunk_scan_fwd_kernel (kernels/ssd_chunk_scan.py:94-117; wrapper _chunk_scan_fwd, :172-224):
 *   y[b,cQ+m,h,p] = scale_m * sum_n C[b,cQ+m,h/(H/G),n] * prev_states[b,c,h,p,n],
 *   scale_m = exp(dA_cumsum[b,h,c,m]) * [seq_idx[b,cQ+m] == seq_idx[b,cQ-1]]  (the latter taken as 0 when c == 0).
 * C: (batch, seqlen, ngroups, dstate); prev_states: (batch, nchunks, nheads, headdim, dstate), the `out` of the
 * state passing / fused calls above; dA_cumsum as above; seq_idx nullable; y: (batch, seqlen, nheads, headdim),
 * f32/bf16/f16.  Innermost strides of C, prev_states and y must be 1.  accumulate != 0 adds to what y holds (the
 * intra-chunk half of the scan computed elsewhere) instead of overwriting it.  bf16 C with fp32 or bf16 states,
 * dstate 64/128, chunk size 64/128/256 and headdim % 32 == 0 run on the matrix cores: a fp32 state enters as bf16
 * hi + lo (the reference rounds the state to C's element type), a bf16 state as it is; everything else on a plain
 * FMA kernel (one thread per output element, orders of magnitude slower).  Size limits of the matrix-core kernels: one
 * chunk of C rows and one chunk of y rows (chunk_size * row pitch in bytes) must stay below 2 GiB; the sequence length
 * itself is not limited by them.
 */
int ssd_chunk_scan_states_fwd(const ssd_tensor *C, const ssd_tensor *prev_states, const ssd_tensor *dA_cumsum,
                              const ssd_tensor *seq_idx, const ssd_tensor *y, const ssd_dims *dims, int accumulate,
                              void *stream);

/*
 * Chunk state + state passing + the consumer above in ONE launch: the ticket / flag-chain kernel multiplies the state
 * entering each chunk by that chunk's C rows in its chain step, while the state sits in registers, so the passed
 * states need not reach memory at all.  Replaces kernels/fused_concurrent.py:255-331 (or fused_globalbar.py:201-266)
 * followed by the state-dependent half of kernels/ssd_chunk_scan.py:94-117, as main.py:85-86 and :100-101 call them.
 *   y[b,cQ+m,h,p] (+)= exp(dA_cumsum[b,h,c,m]) * [seq_idx[b,cQ+m] == seq_idx[b,cQ-1]] * sum_n C[b,cQ+m,g,n] * out[b,c,h,p,n]
 * with out[:, c] the state entering chunk c exactly as ssd_fused_chunk_state_passing_fwd defines it -- in fp32, split
 * into bf16 hi + lo for the matrix cores (the reference rounds it to C's element type, kernels/ssd_chunk_scan.py:106-110).
 * Arguments of ssd_fused_chunk_state_passing_fwd_ws without `states`, plus C (batch, seqlen, ngroups, dstate; the
 * element type of x) and y (batch, seqlen, nheads, headdim; fp32 or bf16, innermost stride 1); accumulate != 0 adds to
 * what y holds.  `out` MAY BE ABSENT (out == NULL or out->data == NULL): then the only trace of the passed states is
 * one 32 x dstate fp32 slot per (state tile, work item) in the workspace, and final_states.  opts: as in
 * ssd_fused_chunk_state_passing_fwd_ws; the workspace must hold ssd_fused_scan_workspace_bytes(dims, with_out,
 * opts->chunks_per_item) bytes, 16-byte aligned (with_out: `out` is given, fp32; work items are two chunks long
 * whatever chunks_per_item says -- what the register file holds next to the operands of the second product).
 * The one-launch kernel takes what the chain kernel takes (bf16 x / B / C, fp32 out if any, dstate 64 or 128, chunk 128
 * or 256, four state tiles per (batch, group), 16-byte aligned rows) and needs the workspace; with SSD_KERNEL_AUTO it
 * serves the calls WITHOUT `out` -- with `out` it saves no traffic and is slower than the two calls, so it runs there
 * only where opts->kernel insists.  Any other call WITH `out` runs as ssd_fused_chunk_state_passing_fwd[_ws] followed by
 * ssd_chunk_scan_states_fwd (the epoch of opts counts for the first of them; *opts->used_workspace says whether the
 * chain kernel ran); without `out` and without that kernel there is no place for the passed states: SSD_ERR_SCRATCH
 * (the library never allocates).
 */
uint64_t ssd_fused_scan_workspace_bytes(const ssd_dims *dims, int with_out, int chunks_per_item);
int ssd_fused_chunk_state_passing_scan_fwd(const ssd_tensor *x, const ssd_tensor *B, const ssd_tensor *C, const ssd_tensor *dt,
                                           const ssd_tensor *dA_cumsum, const ssd_tensor *seq_idx,
                                           const ssd_tensor *initial_states, const ssd_tensor *out,
                                           const ssd_tensor *final_states, const ssd_tensor *y, const ssd_dims *dims,
                                           int clamp, int accumulate, const ssd_fused_opts *opts, void *stream);

/*
 * Tuning / test hook with no counterpart in the reference: which matrix-core kernel serves ssd_chunk_scan_states_fwd
 * where both apply.  0 = let the library choose (the default); 1 = one workgroup per (batch, chunk, head);
 * 2 = one workgroup per run of heads, with the chunk's C rows kept in LDS across the run (needs headdim % 64 == 0
 * and contiguous dA_cumsum rows; other calls are served as with 0).  Returns the previous setting, or SSD_ERR_SHAPE.
 */
int ssd_set_scan_kernel(int kernel);

/*
 * Tuning / test hook with no counterpart in the reference: which bf16 MFMA kernel family serves the calls above.
 * 0 = let the library choose from the problem size (the default); 2 or 4 = the token-split kernels with that many
 * waves per state tile; 1 = one wave per state tile (the kernel with four tiles per workgroup) wherever that
 * kernel applies.  While the setting is not 0 the library does not pick the ticket / flag-chain kernel by itself either
 * (ssd_fused_chunk_state_passing_fwd_ws).  A process-wide hook for tests and tuning: it is atomic, so changing it while
 * another thread launches is safe, but that thread's choice of kernel is then either the old or the new one.  The
 * setting holds for every later call of this process.  Returns the previous setting, or
 * SSD_ERR_SHAPE for a value other than 0, 1, 2, 4.  Results agree between the settings to rounding (the tokens are summed in
 * another order), not bit for bit.
 */
int ssd_set_token_split(int waves);

/*
 * Measurement hook with no counterpart in the reference: the memory traffic of the fused call on these tensors with
 * all arithmetic, all dependencies between chunks and all waiting on other workgroups removed -- every x row read
 * once, every B row once per four state tiles, one 32 x dstate fp32 tile written per (state tile, chunk), by one
 * persistent workgroup per compute unit with the fused kernels' request and store patterns.  Its duration is the floor
 * the memory system of the device sets for the path's access pattern (bench.py reports it as roofline.mover_us next to
 * the fused call's time).  dt, dA_cumsum and final_states are only checked, not moved (6 % of the path's bytes).
 * `out` IS OVERWRITTEN (with zeros).  Arguments the ticket / flag-chain kernel does not cover (it needs bf16 x / B,
 * fp32 out, dstate 64 or 128, chunk 128 or 256, four state tiles per (batch, group)): SSD_ERR_SHAPE.
 */
int ssd_measure_traffic_floor(const ssd_tensor *x, const ssd_tensor *B, const ssd_tensor *dt, const ssd_tensor *dA_cumsum,
                              const ssd_tensor *out, const ssd_tensor *final_states, const ssd_dims *dims, void *stream);
/*
 * The same with one side of the traffic left out (no counterpart in the reference either): part 0 = loads and stores
 * (ssd_measure_traffic_floor), 1 = the loads only (`out` is left alone), 2 = the stores only.  What the three durations
 * say together is how reads and writes share the device's memory system (bench.py: roofline.mover_loads_us,
 * roofline.mover_stores_us).  Other values of part: SSD_ERR_SHAPE.
 */
int ssd_measure_traffic_floor_part(const ssd_tensor *x, const ssd_tensor *B, const ssd_tensor *dt,
                                   const ssd_tensor *dA_cumsum, const ssd_tensor *out, const ssd_tensor *final_states,
                                   const ssd_dims *dims, int part, void *stream);

/*
 * Test hook with no counterpart in the reference: the number of XCDs (L2 caches) the LOCAL variant of the ticket /
 * flag-chain kernel deals its units to; 0 = compute units / 32 (the default; 8 on MI355X), at most 16.  A wrong count
 * is what the kernel's own checks exist for (SSD_ERR_CHAIN_XCD, SSD_ERR_CHAIN_INCOMPLETE) and how the tests provoke
 * them.  Process-wide and atomic like the hooks below.  Returns the previous setting, or SSD_ERR_SHAPE.
 */
int ssd_set_chain_xcds(int xcds);

/*
 * Tuning / test hook with no counterpart in the reference: how many consecutive chunks a workgroup of the
 * four-tiles-per-workgroup kernel walks when that kernel serves ssd_chunk_state_fwd (chunk states are independent of
 * each other, so a sequence is cut into segments that run as separate workgroups).  0 = let the library choose from
 * the problem size (the default); values above the number of chunks mean one segment.  The results do not depend on
 * the setting, bit for bit.  Returns the previous setting, or SSD_ERR_SHAPE for a negative value.
 */
int ssd_set_segment_chunks(int chunks);

#ifdef __cplusplus
}
#endif
#endif /* SSD_GFX950_H */
