/*
 * CPU oracle for cosine linear attention -- TEST INFRASTRUCTURE ONLY.
 *
 * This file is a plain-C restatement of the reference algorithm and exists only as a
 * checker: tests, the smoke check and the benchmark's cpu_baseline leg may load it; the
 * shipped HIP path never does.  Everything is computed in double precision from inputs
 * that the caller has already rounded to the storage type under test.
 *
 * Layout: every tensor is contiguous (BH, N, D) -- batch and head are flattened because
 * each (batch, head) pair is an independent scan (Cuda_Kernel/combined_kernel_general.cu:266,
 * grid(N,H,D_value); index ((n*H+h)*S+s)*D+d at :136,:143).
 *
 * Each function cites the reference lines it follows.  How each one is pinned
 * (tests/test_oracle_pinning.py):
 *   cott_oracle_causal_loop      brute-force triple sum on tiny inputs; numpy cumsum form;
 *                                masked-quadratic form below; flip identity for `reversed`
 *   cott_oracle_causal_masked    independent algorithm for the same quantity
 *   cott_oracle_causal_bwd       torch.autograd on the cumsum closed form, fp64 gradcheck,
 *                                central finite differences, operand-permutation identities
 *   cott_oracle_noncausal(_bwd)  associativity (QK^T)V == Q(K^TV); autograd; finite differences
 *   cott_oracle_decode_step      N steps from a zero state reproduce the causal rows
 */
#include <stddef.h>
#include <stdlib.h>
#include <string.h>

/* Generic causal "cumsum and contract":
 *   out[s,j] = sum_i A[s,i] * sum_{s' <= s (>= s if reversed)} B[s',i] * C[s',j]
 * Recurrent form: the running state is updated with position s BEFORE the dot product, so the
 * diagonal s'=s is included (combined_kernel_general.cu:126-130 loop order and `reversed`
 * index, :143-144 state update, :148-149 contraction, :163-165 store;
 * GPT_Trainer/GPTCosAttention.py:262-267 is the same recurrence in PyTorch). */
void cott_oracle_causal_loop(const double *A, const double *B, const double *C, double *out,
                             long BH, long N, long Di, long Dj, int reversed)
{
#pragma omp parallel for schedule(dynamic)
    for (long bh = 0; bh < BH; ++bh) {
        double *state = (double *)calloc((size_t)(Di * Dj), sizeof(double));
        const double *a = A + bh * N * Di, *b = B + bh * N * Di, *c = C + bh * N * Dj;
        double *o = out + bh * N * Dj;
        for (long s_ = 0; s_ < N; ++s_) {
            long s = reversed ? N - s_ - 1 : s_;
            for (long i = 0; i < Di; ++i) {
                double bi = b[s * Di + i];
                for (long j = 0; j < Dj; ++j) state[i * Dj + j] += bi * c[s * Dj + j];
            }
            for (long j = 0; j < Dj; ++j) o[s * Dj + j] = 0.0;
            for (long i = 0; i < Di; ++i) {
                double ai = a[s * Di + i];
                for (long j = 0; j < Dj; ++j) o[s * Dj + j] += ai * state[i * Dj + j];
            }
        }
        free(state);
    }
}

/* Same quantity by the masked quadratic form ((A B^T) o tril) C  (triu if reversed):
 * Cuda_Kernel/speed_test.py:15-20 (`masked_fill(mask == 0, 0)` then matmul with V);
 * GPT_Trainer/GPTCosAttention.py:293-316.  O(N^2) -- small inputs only. */
void cott_oracle_causal_masked(const double *A, const double *B, const double *C, double *out,
                               long BH, long N, long Di, long Dj, int reversed)
{
#pragma omp parallel for schedule(dynamic)
    for (long bh = 0; bh < BH; ++bh) {
        const double *a = A + bh * N * Di, *b = B + bh * N * Di, *c = C + bh * N * Dj;
        double *o = out + bh * N * Dj;
        for (long s = 0; s < N; ++s) {
            for (long j = 0; j < Dj; ++j) o[s * Dj + j] = 0.0;
            long lo = reversed ? s : 0, hi = reversed ? N - 1 : s;
            for (long t = lo; t <= hi; ++t) {
                double p = 0.0;
                for (long i = 0; i < Di; ++i) p += a[s * Di + i] * b[t * Di + i];
                for (long j = 0; j < Dj; ++j) o[s * Dj + j] += p * c[t * Dj + j];
            }
        }
    }
}

/* Causal backward, closed forms of Cuda_Kernel/Custom_Kernel.py:
 *   :63  grad_Q = ((V[...,None] * K[...,None,:]).cumsum(2) * dO[...,None]).sum(-2)
 *   :68  grad_K = ((dO[...,None] * Q[...,None,:]).flip(2).cumsum(2).flip(2) * V[...,None]).sum(-2)
 *   :72  grad_V = (same suffix cumsum * K[...,None,:]).sum(-1)
 * The prefix cumsum is the running matrix P[dv][dk] = sum_{s'<=s} V[s',dv] K[s',dk]; the suffix
 * cumsum is R[dv][dk] = sum_{s'>=s} dO[s',dv] Q[s',dk] (shared by grad_K and grad_V, :78-88). */
void cott_oracle_causal_bwd(const double *Q, const double *K, const double *V, const double *dO,
                            double *dQ, double *dK, double *dV,
                            long BH, long N, long Dk, long Dv)
{
#pragma omp parallel for schedule(dynamic)
    for (long bh = 0; bh < BH; ++bh) {
        double *P = (double *)calloc((size_t)(Dv * Dk), sizeof(double));
        double *R = (double *)calloc((size_t)(Dv * Dk), sizeof(double));
        const double *q = Q + bh * N * Dk, *k = K + bh * N * Dk;
        const double *v = V + bh * N * Dv, *g = dO + bh * N * Dv;
        double *dq = dQ + bh * N * Dk, *dk = dK + bh * N * Dk, *dv = dV + bh * N * Dv;
        for (long s = 0; s < N; ++s) {
            for (long e = 0; e < Dv; ++e)
                for (long d = 0; d < Dk; ++d) P[e * Dk + d] += v[s * Dv + e] * k[s * Dk + d];
            for (long d = 0; d < Dk; ++d) {
                double acc = 0.0;
                for (long e = 0; e < Dv; ++e) acc += P[e * Dk + d] * g[s * Dv + e];
                dq[s * Dk + d] = acc;
            }
        }
        for (long s = N - 1; s >= 0; --s) {
            for (long e = 0; e < Dv; ++e)
                for (long d = 0; d < Dk; ++d) R[e * Dk + d] += g[s * Dv + e] * q[s * Dk + d];
            for (long d = 0; d < Dk; ++d) {
                double acc = 0.0;
                for (long e = 0; e < Dv; ++e) acc += R[e * Dk + d] * v[s * Dv + e];
                dk[s * Dk + d] = acc;
            }
            for (long e = 0; e < Dv; ++e) {
                double acc = 0.0;
                for (long d = 0; d < Dk; ++d) acc += R[e * Dk + d] * k[s * Dk + d];
                dv[s * Dv + e] = acc;
            }
        }
        free(P);
        free(R);
    }
}

/* Non-causal form O = A (B^T C): BERT_Trainer/BertCosAttention.py:249
 * einsum("nhsw,nhwe->nhse", Q, einsum("nhse,nhsw->nhew", K, V)). */
void cott_oracle_noncausal(const double *A, const double *B, const double *C, double *out,
                           long BH, long N, long Di, long Dj)
{
#pragma omp parallel for schedule(dynamic)
    for (long bh = 0; bh < BH; ++bh) {
        double *state = (double *)calloc((size_t)(Di * Dj), sizeof(double));
        const double *a = A + bh * N * Di, *b = B + bh * N * Di, *c = C + bh * N * Dj;
        double *o = out + bh * N * Dj;
        for (long s = 0; s < N; ++s)
            for (long i = 0; i < Di; ++i)
                for (long j = 0; j < Dj; ++j) state[i * Dj + j] += b[s * Di + i] * c[s * Dj + j];
        for (long s = 0; s < N; ++s)
            for (long j = 0; j < Dj; ++j) {
                double acc = 0.0;
                for (long i = 0; i < Di; ++i) acc += a[s * Di + i] * state[i * Dj + j];
                o[s * Dj + j] = acc;
            }
        free(state);
    }
}

/* Non-causal backward.  grad_Q = dO (V^T K) and grad_K = V (dO^T Q) follow
 * GPT_Trainer/GPTCosAttention.py:34-35.  Line :36 of that file writes grad_V as Q (dO^T K),
 * which is not the derivative of Q (K^T V); the derivative is K (Q^T dO) and that is what is
 * computed here (the reference's `Multiply` is unused -- its call is commented out at :283). */
void cott_oracle_noncausal_bwd(const double *Q, const double *K, const double *V, const double *dO,
                               double *dQ, double *dK, double *dV,
                               long BH, long N, long Dk, long Dv)
{
#pragma omp parallel for schedule(dynamic)
    for (long bh = 0; bh < BH; ++bh) {
        double *S = (double *)calloc((size_t)(Dk * Dv), sizeof(double)); /* K^T V  */
        double *T = (double *)calloc((size_t)(Dk * Dv), sizeof(double)); /* Q^T dO */
        const double *q = Q + bh * N * Dk, *k = K + bh * N * Dk;
        const double *v = V + bh * N * Dv, *g = dO + bh * N * Dv;
        double *dq = dQ + bh * N * Dk, *dk = dK + bh * N * Dk, *dv = dV + bh * N * Dv;
        for (long s = 0; s < N; ++s)
            for (long d = 0; d < Dk; ++d)
                for (long e = 0; e < Dv; ++e) {
                    S[d * Dv + e] += k[s * Dk + d] * v[s * Dv + e];
                    T[d * Dv + e] += q[s * Dk + d] * g[s * Dv + e];
                }
        for (long s = 0; s < N; ++s) {
            for (long d = 0; d < Dk; ++d) {
                double a1 = 0.0, a2 = 0.0;
                for (long e = 0; e < Dv; ++e) {
                    a1 += g[s * Dv + e] * S[d * Dv + e];
                    a2 += v[s * Dv + e] * T[d * Dv + e];
                }
                dq[s * Dk + d] = a1;
                dk[s * Dk + d] = a2;
            }
            for (long e = 0; e < Dv; ++e) {
                double a3 = 0.0;
                for (long d = 0; d < Dk; ++d) a3 += k[s * Dk + d] * T[d * Dv + e];
                dv[s * Dv + e] = a3;
            }
        }
        free(S);
        free(T);
    }
}

/* One recurrent decode step on a (BH, Dk, Dv) state:
 *   S[dk][dv] += k[dk] * v[dv] ;  o[dv] = sum_dk q[dk] * S[dk][dv]   (state updated first)
 * GPT_Trainer/GPTCosAttention.py:264 (update) and :267 (read).  The reference stores the state
 * transposed, (Dv, Dk) = v (x) k; the value of o is the same. */
void cott_oracle_decode_step(double *S, const double *q, const double *k, const double *v, double *o,
                             long BH, long Dk, long Dv)
{
#pragma omp parallel for
    for (long bh = 0; bh < BH; ++bh) {
        double *s = S + bh * Dk * Dv;
        const double *qq = q + bh * Dk, *kk = k + bh * Dk, *vv = v + bh * Dv;
        double *oo = o + bh * Dv;
        for (long e = 0; e < Dv; ++e) oo[e] = 0.0;
        for (long d = 0; d < Dk; ++d)
            for (long e = 0; e < Dv; ++e) {
                s[d * Dv + e] += kk[d] * vv[e];
                oo[e] += qq[d] * s[d * Dv + e];
            }
    }
}
