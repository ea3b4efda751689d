/*
 * cc1d_oracle.c — plain-C, double-precision restatement of the causal depthwise conv1d
 * operator family.  TEST INFRASTRUCTURE ONLY: nothing in the product links, loads or
 * calls this file; tests use it as an independent check of the PyTorch oracle and of the
 * GPU results.
 *
 * Scalar loops, no blocking, no vector tricks: every function states the arithmetic
 * once, element by element, and cites the reference lines it follows.  Tensors are
 * dense, logical (batch, dim, seqlen) order, float32 in (16-bit inputs are widened by
 * the caller, which is exact) and float64 out.
 */
#include <math.h>
#include <stdint.h>
#include <stddef.h>

static double act_silu(double z) { return z / (1.0 + exp(-z)); }

/* d silu / dz = s (1 + z (1 - s)), csrc/causal_conv1d_bwd.cu:168-170 */
static double act_silu_grad(double z) {
    const double s = 1.0 / (1.0 + exp(-z));
    return s * (1.0 + z * (1.0 - s));
}

/* xpad[b,c,p]: x for p >= 0, initial_states[b,c,p+W-1] for -(W-1) <= p < 0, else 0
 * (causal_conv1d_interface.py:158-160; csrc/causal_conv1d_fwd.cu:254-266). */
static double xpad_at(const float *x, const float *init, int D, int L, int W, int b, int c, int p) {
    if (p >= 0) return (double)x[((size_t)b * D + c) * L + p];
    if (init != NULL && p >= -(W - 1)) return (double)init[((size_t)b * D + c) * (W - 1) + (p + W - 1)];
    return 0.0;
}

static int seq_at(const int32_t *seq, int L, int b, int p) {
    return p >= 0 ? seq[(size_t)b * L + p] : -1;   /* csrc/causal_conv1d_fwd.cu:308 */
}

/* pre-activation z[b,c,t], with the seq_idx tap mask of csrc/causal_conv1d_fwd.cu:322-329 */
static double z_at(const float *x, const float *w, const float *bias, const int32_t *seq,
                   const float *init, int D, int L, int W, int b, int c, int t) {
    double z = bias != NULL ? (double)bias[c] : 0.0;
    for (int k = 0; k < W; ++k) {
        const int p = t - (W - 1 - k);
        if (seq != NULL && seq_at(seq, L, b, p) != seq_at(seq, L, b, t)) continue;
        z += (double)w[(size_t)c * W + k] * xpad_at(x, init, D, L, W, b, c, p);
    }
    return z;
}

/* Forward: out (B,D,L) and, if final_states != NULL, final_states (B,D,W-1) =
 * xpad[L-(W-1) .. L) (causal_conv1d_interface.py:162-165). */
void cc1d_oracle_fwd(const float *x, const float *w, const float *bias, const int32_t *seq,
                     const float *init, int B, int D, int L, int W, int silu, double *out,
                     double *final_states) {
    for (int b = 0; b < B; ++b)
        for (int c = 0; c < D; ++c) {
            for (int t = 0; t < L; ++t) {
                double v;
                if (seq != NULL && seq_at(seq, L, b, t) < 0) {
                    v = 0.0;                        /* csrc/causal_conv1d_fwd.cu:317-321 */
                } else {
                    v = z_at(x, w, bias, seq, init, D, L, W, b, c, t);
                    if (silu) v = act_silu(v);
                }
                out[((size_t)b * D + c) * L + t] = v;
            }
            if (final_states != NULL)
                for (int i = 0; i < W - 1; ++i)
                    final_states[((size_t)b * D + c) * (W - 1) + i] =
                        xpad_at(x, init, D, L, W, b, c, L - (W - 1) + i);
        }
}

/* g[b,c,t] = dout * act'(z); zero outside [0, L) and at padding positions. */
static double g_at(const float *x, const float *w, const float *bias, const float *dout,
                   const int32_t *seq, const float *init, int D, int L, int W, int silu, int b,
                   int c, int t) {
    if (t < 0 || t >= L) return 0.0;
    if (seq != NULL && seq_at(seq, L, b, t) < 0) return 0.0;
    double g = (double)dout[((size_t)b * D + c) * L + t];
    if (silu) g *= act_silu_grad(z_at(x, w, bias, seq, init, D, L, W, b, c, t));
    return g;
}

/* Backward in closed form (csrc/causal_conv1d_bwd.cu:458-561):
 *   dx[p]      = sum_k w[W-1-k] g[p+k]            (+ dfinal[p-(L-(W-1))] for p >= L-(W-1))
 *   dinit[i]   = the same at p = i-(W-1)          (+ dfinal[i-L] for i >= L)
 *   dw[c,k]   += sum_{b,t} g[t] xpad[t-(W-1-k)],   db[c] += sum_{b,t} g[t]
 * with taps masked by seq_idx equality.  dw (D,W) and db (D) are overwritten. */
void cc1d_oracle_bwd(const float *x, const float *w, const float *bias, const float *dout,
                     const int32_t *seq, const float *init, const float *dfinal, int B, int D,
                     int L, int W, int silu, double *dx, double *dw, double *db, double *dinit) {
    for (int c = 0; c < D; ++c) {
        for (int k = 0; k < W; ++k) dw[(size_t)c * W + k] = 0.0;
        if (db != NULL) db[c] = 0.0;
    }
    for (int b = 0; b < B; ++b)
        for (int c = 0; c < D; ++c) {
            for (int p = -(W - 1); p < L; ++p) {
                double acc = 0.0;
                for (int k = 0; k < W; ++k) {
                    const int t = p + k;
                    if (t < 0 || t >= L) continue;
                    if (seq != NULL && seq_at(seq, L, b, t) != seq_at(seq, L, b, p)) continue;
                    acc += (double)w[(size_t)c * W + (W - 1 - k)] *
                           g_at(x, w, bias, dout, seq, init, D, L, W, silu, b, c, t);
                }
                if (dfinal != NULL && p >= L - (W - 1))
                    acc += (double)dfinal[((size_t)b * D + c) * (W - 1) + (p - (L - (W - 1)))];
                if (p >= 0) dx[((size_t)b * D + c) * L + p] = acc;
                else if (dinit != NULL) dinit[((size_t)b * D + c) * (W - 1) + (p + W - 1)] = acc;
            }
            for (int t = 0; t < L; ++t) {
                const double g = g_at(x, w, bias, dout, seq, init, D, L, W, silu, b, c, t);
                if (db != NULL) db[c] += g;
                for (int k = 0; k < W; ++k) {
                    const int p = t - (W - 1 - k);
                    if (seq != NULL && seq_at(seq, L, b, p) != seq_at(seq, L, b, t)) continue;
                    dw[(size_t)c * W + k] += g * xpad_at(x, init, D, L, W, b, c, p);
                }
            }
        }
}

/* Decode step (csrc/causal_conv1d_update.cu:43-113).  state is (SB, D, S) float, updated
 * in place with exact copies; out (B, D, L) double.  cache == NULL: linear shift,
 * new_state = concat(state, x)[-S:] (causal_conv1d_interface.py:230-231).  Otherwise
 * circular: window read at (cs-(W-1)+i) mod S, x[i] written at (cs+i) mod S
 * (causal_conv1d_interface.py:233-238).  idx[b] < 0: zero output, state untouched. */
void cc1d_oracle_update(const float *x, float *state, const float *w, const float *bias,
                        const int32_t *cache, const int32_t *idx, int B, int D, int L, int W,
                        int S, int silu, double *out) {
    for (int b = 0; b < B; ++b) {
        const int sb = idx != NULL ? idx[b] : b;
        for (int c = 0; c < D; ++c) {
            double *o = out + ((size_t)b * D + c) * L;
            if (sb < 0) {
                for (int i = 0; i < L; ++i) o[i] = 0.0;
                continue;
            }
            float *st = state + ((size_t)sb * D + c) * S;
            const float *xr = x + ((size_t)b * D + c) * L;
            float win[8];                                /* W-1 history values + current */
            int cs = 0;
            if (cache != NULL) {
                cs = ((cache[b] % S) + S) % S;
                for (int i = 0; i < W - 1; ++i) win[i] = st[(((cs - (W - 1) + i) % S) + S) % S];
            } else {
                for (int i = 0; i < W - 1; ++i) win[i] = st[S - (W - 1) + i];
                /* shift by L: new[j] = concat(state, x)[L + j] */
                for (int j = 0; j < S; ++j) {
                    const int src = L + j;
                    st[j] = src < S ? st[src] : xr[src - S];
                }
            }
            for (int i = 0; i < L; ++i) {
                if (cache != NULL) st[(cs + i) % S] = xr[i];
                win[W - 1] = xr[i];
                double z = bias != NULL ? (double)bias[c] : 0.0;
                for (int k = 0; k < W; ++k) z += (double)w[(size_t)c * W + k] * (double)win[k];
                o[i] = silu ? act_silu(z) : z;
                for (int k = 0; k < W - 1; ++k) win[k] = win[k + 1];
            }
        }
    }
}

/* Varlen final-state gather (causal_conv1d_varlen.py:21-31, 79-85): states (batch, D, S). */
void cc1d_oracle_varlen_states(const float *x, const int64_t *cu, int batch, int D, int S,
                               float *states) {
    for (int b = 0; b < batch; ++b) {
        const int64_t end = cu[b + 1];
        int64_t start = cu[b];
        if (start < end - S) start = end - S;
        for (int c = 0; c < D; ++c)
            for (int s = 0; s < S; ++s) {
                const int64_t row = end - (S - s);
                states[((size_t)b * D + c) * S + s] = row >= start ? x[(size_t)row * D + c] : 0.0f;
            }
    }
}
