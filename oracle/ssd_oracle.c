/*
 * Plain-C CPU oracle for the Mamba2 SSD chunk-state + state-passing path.
 *
 * TEST INFRASTRUCTURE ONLY: built into oracle/libssd_oracle.so and loaded by the tests (and the smoke
 * check) as a second, loop-level restatement that pins the PyTorch oracle in oracle/ssd_oracle.py.
 * Nothing that ships links or loads it.
 *
 * Each function follows the reference lines cited above it.  All tensors are dense, row-major, with
 * the shapes given in the comments; x and B arrive already widened to float.
 *
 * Pin status: every function here is checked against closed forms and against the token-serial
 * recurrence (ssd_oracle_token_recurrence) in tests/test_oracle.py; none is "parity unpinned".
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define IDX4(a, b, c, d, B_, C_, D_) ((((size_t)(a) * (B_) + (b)) * (C_) + (c)) * (D_) + (d))

/* kernels/ssd_chunk_state.py:114-173 (unfused kernel; clamp != 0 keeps the min(.,0) of line 153,
 * clamp == 0 reproduces kernels/fused_globalbar.py:106).
 *   x (b,L,H,P)  B (b,L,G,N)  dt,dAcs (b,H,C,Q)  seq_idx (b,L) or NULL  ->  states (b,C,H,P,N)      */
int ssd_oracle_chunk_state(const float *x, const float *B, const float *dt, const float *dAcs,
                           const int32_t *seq_idx, float *states,
                           int b_, int L, int H, int P, int N, int G, int Q, int clamp)
{
    if (H % G) return -1;
    const int C = (L + Q - 1) / Q, ratio = H / G;
    double *acc = (double *)malloc(sizeof(double) * (size_t)P * N);
    if (!acc) return -2;
    for (int b = 0; b < b_; ++b)
    for (int c = 0; c < C; ++c)
    for (int h = 0; h < H; ++h) {
        const int g = h / ratio;                                   /* :121 */
        const int lim = (L - c * Q) < Q ? (L - c * Q) : Q;         /* :139 */
        const float *dt_c = dt + IDX4(b, h, c, 0, H, C, Q);
        const float *cs_c = dAcs + IDX4(b, h, c, 0, H, C, Q);
        const float last = cs_c[Q - 1];                            /* :134, index Q-1 */
        const int32_t id_last = seq_idx ? seq_idx[(size_t)b * L + c * Q + lim - 1] : 0;   /* :141 */
        memset(acc, 0, sizeof(double) * (size_t)P * N);
        for (int k = 0; k < lim; ++k) {
            const size_t t = (size_t)c * Q + k;
            float e = last - cs_c[k];
            if (clamp && e > 0.0f) e = 0.0f;                       /* :153 */
            float w = expf(e) * dt_c[k];
            if (seq_idx && seq_idx[(size_t)b * L + t] != id_last) w = 0.0f;   /* :156 */
            const float *xr = x + IDX4(b, t, h, 0, L, H, P);
            const float *Br = B + IDX4(b, t, g, 0, L, G, N);
            for (int p = 0; p < P; ++p) {
                const double xw = (double)xr[p] * (double)w;
                for (int n = 0; n < N; ++n) acc[(size_t)p * N + n] += xw * (double)Br[n];   /* :157-159 */
            }
        }
        float *dst = states + IDX4(b, c, h, 0, C, H, (size_t)P * N);
        for (size_t i = 0; i < (size_t)P * N; ++i) dst[i] = (float)acc[i];
    }
    free(acc);
    return 0;
}

/* kernels/ssd_state_passing.py:61-84.
 *   states (b,C,H,dim)  dA_chunk (b,H,C)  init (b,H,dim) or NULL  seq_idx (b,L) or NULL
 *   ->  out (b,C,H,dim)  final (b,H,dim)                                                            */
int ssd_oracle_state_passing(const float *states, const float *dA_chunk, const float *init,
                             const int32_t *seq_idx, float *out, float *final_states,
                             int b_, int C, int H, int dim, int L, int Q)
{
    float *s = (float *)malloc(sizeof(float) * (size_t)dim);
    if (!s) return -2;
    for (int b = 0; b < b_; ++b)
    for (int h = 0; h < H; ++h) {
        for (int i = 0; i < dim; ++i) s[i] = init ? init[((size_t)b * H + h) * dim + i] : 0.0f;   /* :61-65 */
        memcpy(out + IDX4(b, 0, h, 0, C, H, dim), s, sizeof(float) * dim);                        /* :66 */
        int32_t prev = 0;                                                                         /* :68 */
        for (int c = 0; c < C; ++c) {
            float scale = expf(dA_chunk[((size_t)b * H + h) * C + c]);                            /* :72 */
            if (seq_idx) {
                int end = (c + 1) * Q < L ? (c + 1) * Q : L;
                int32_t cur = seq_idx[(size_t)b * L + end - 1];                                   /* :74 */
                if (cur != prev) scale = 0.0f;                                                    /* :75 */
                prev = cur;
            }
            const float *nw = states + IDX4(b, c, h, 0, C, H, dim);
            for (int i = 0; i < dim; ++i) s[i] = scale * s[i] + nw[i];                            /* :77 */
            float *dst = (c < C - 1) ? out + IDX4(b, c + 1, h, 0, C, H, dim)
                                     : final_states + ((size_t)b * H + h) * dim;                  /* :78-81 */
            memcpy(dst, s, sizeof(float) * dim);
        }
    }
    free(s);
    return 0;
}

/* No counterpart in the reference: the chunk-free recurrence in double precision,
 *   h_t = [id_t == id_{t-1}] exp(dt_t A_h) h_{t-1} + dt_t x_t (outer) B_t,   h_{-1} = init, id_{-1} = 0,
 * snapshotted at chunk boundaries: out[:,c] = h_{cQ-1}, final = h_{L-1}.
 *   x (b,L,H,P)  B (b,L,G,N)  dt_tok (b,L,H)  A (H)  init (b,H,P,N) or NULL  seq_idx (b,L) or NULL
 *   ->  out (b,C,H,P,N) double,  final (b,H,P,N) double                                            */
int ssd_oracle_token_recurrence(const float *x, const float *B, const float *dt_tok, const float *A,
                                const float *init, const int32_t *seq_idx, double *out, double *final_states,
                                int b_, int L, int H, int P, int N, int G, int Q)
{
    if (H % G) return -1;
    const int C = (L + Q - 1) / Q, ratio = H / G;
    const size_t PN = (size_t)P * N;
    double *hst = (double *)malloc(sizeof(double) * PN);
    if (!hst) return -2;
    for (int b = 0; b < b_; ++b)
    for (int h = 0; h < H; ++h) {
        const int g = h / ratio;
        for (size_t i = 0; i < PN; ++i) hst[i] = init ? (double)init[((size_t)b * H + h) * PN + i] : 0.0;
        memcpy(out + IDX4(b, 0, h, 0, C, H, PN), hst, sizeof(double) * PN);
        int32_t prev = 0;
        for (int t = 0; t < L; ++t) {
            const double dtv = (double)dt_tok[((size_t)b * L + t) * H + h];
            double a = exp(dtv * (double)A[h]);
            if (seq_idx) {
                int32_t cur = seq_idx[(size_t)b * L + t];
                if (cur != prev) a = 0.0;
                prev = cur;
            }
            const float *xr = x + IDX4(b, t, h, 0, L, H, P);
            const float *Br = B + IDX4(b, t, g, 0, L, G, N);
            for (int p = 0; p < P; ++p) {
                const double xv = dtv * (double)xr[p];
                for (int n = 0; n < N; ++n) hst[(size_t)p * N + n] = a * hst[(size_t)p * N + n] + xv * (double)Br[n];
            }
            if ((t + 1) % Q == 0 && (t + 1) / Q < C)
                memcpy(out + IDX4(b, (t + 1) / Q, h, 0, C, H, PN), hst, sizeof(double) * PN);
        }
        memcpy(final_states + ((size_t)b * H + h) * PN, hst, sizeof(double) * PN);
    }
    free(hst);
    return 0;
}
