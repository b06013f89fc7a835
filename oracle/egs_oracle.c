/*
 * CPU oracle, C restatement (loop level) of the fused expert gather / scatter-with-linear
 * path.  TEST INFRASTRUCTURE ONLY: linked by tests/, the smoke check and the cpu_baseline
 * leg of bench.py; never by the shipped library.
 *
 * Formulas restated from the reference:
 *   gather   Y[b,e,k,j]  = sum_i X[b,Ind[b,e,k],i] * W[e,i,j]        egs/baselines.py:69-76, egs/triton_kernels.py:589
 *   scatter  out[b,t,i]  = sum_{e,k:Ind=t} sum_j Y[b,e,k,j]*W[e,j,i]  egs/baselines.py:174-184, egs/triton_kernels.py:618
 *   dW       dW[e,i,j]   = sum_{b,k} X[b,Ind[b,e,k],i] * G[b,e,k,j]   egs/baselines.py:146, egs/triton_kernels.py:283
 * The two weight layouts ([E,I,J] and [E,J,I]) mirror the stride swaps at
 * egs/triton_kernels.py:468, :504 and :521.
 *
 * Inputs are float32 (low-precision tensors are passed as their exact float32 values),
 * every accumulation is in double and results are returned as double.
 * Pinned by tests/test_oracle.py against the numpy oracle, the brute-force Python loops and
 * closed-form special cases; it has no data-dependent branches beyond the index lookup.
 */
#include <stdint.h>
#include <stddef.h>
#include <string.h>

#define W_EIJ 0
#define W_EJI 1

/* weight element for reduction index r (over I) and output column j */
static inline double w_at(const float *W, int layout, int I, int J, int e, int i, int j)
{
    return layout == W_EIJ ? (double)W[((size_t)e * I + i) * J + j]
                           : (double)W[((size_t)e * J + j) * I + i];
}

/* Y[b,e,k,j] = sum_i X[b,Ind[b,e,k],i] * Wl[e](i,j)   -- X is [B,T,I], Y is [B,E,K,J] */
int egs_oracle_gather(const float *X, const float *W, const int64_t *Ind, double *Y,
                      int B, int T, int E, int K, int I, int J, int w_layout)
{
    for (int b = 0; b < B; ++b)
        for (int e = 0; e < E; ++e)
            for (int k = 0; k < K; ++k) {
                int64_t t = Ind[((size_t)b * E + e) * K + k];
                double *y = Y + (((size_t)b * E + e) * K + k) * J;
                if (t < 0 || t >= T) return -1;
                const float *x = X + ((size_t)b * T + t) * I;
                for (int j = 0; j < J; ++j) {
                    double s = 0.0;
                    for (int i = 0; i < I; ++i) s += (double)x[i] * w_at(W, w_layout, I, J, e, i, j);
                    y[j] = s;
                }
            }
    return 0;
}

/* out[b,Ind[b,e,k],i] += sum_j Y[b,e,k,j] * Wl[e](i,j)   -- out is [B,T,I], zeroed here.
 * w_layout W_EJI is the scatter forward (W stored [E,J,I]); W_EIJ is the gather dX. */
int egs_oracle_scatter(const float *Y, const float *W, const int64_t *Ind, double *out,
                       int B, int T, int E, int K, int I, int J, int w_layout)
{
    memset(out, 0, sizeof(double) * (size_t)B * T * I);
    for (int b = 0; b < B; ++b)
        for (int e = 0; e < E; ++e)
            for (int k = 0; k < K; ++k) {
                int64_t t = Ind[((size_t)b * E + e) * K + k];
                const float *y = Y + (((size_t)b * E + e) * K + k) * J;
                if (t < 0 || t >= T) return -1;
                double *o = out + ((size_t)b * T + t) * I;
                for (int i = 0; i < I; ++i) {
                    double s = 0.0;
                    for (int j = 0; j < J; ++j) s += (double)y[j] * w_at(W, w_layout, I, J, e, i, j);
                    o[i] += s;
                }
            }
    return 0;
}

/* dW(e,i,j) = sum_{b,k} Xs[b,Ind[b,e,k],i] * Ys[b,e,k,j], stored [E,I,J] or [E,J,I] */
int egs_oracle_dw(const float *Xs, const float *Ys, const int64_t *Ind, double *dW,
                  int B, int T, int E, int K, int I, int J, int dw_layout)
{
    memset(dW, 0, sizeof(double) * (size_t)E * I * J);
    for (int b = 0; b < B; ++b)
        for (int e = 0; e < E; ++e)
            for (int k = 0; k < K; ++k) {
                int64_t t = Ind[((size_t)b * E + e) * K + k];
                if (t < 0 || t >= T) return -1;
                const float *x = Xs + ((size_t)b * T + t) * I;
                const float *y = Ys + (((size_t)b * E + e) * K + k) * J;
                for (int i = 0; i < I; ++i)
                    for (int j = 0; j < J; ++j) {
                        size_t at = dw_layout == W_EIJ ? ((size_t)e * I + i) * J + j
                                                       : ((size_t)e * J + j) * I + i;
                        dW[at] += (double)x[i] * (double)y[j];
                    }
            }
    return 0;
}
