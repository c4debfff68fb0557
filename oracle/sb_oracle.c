/*
 * CPU oracle, second restatement: brute-force float64 evaluation of the stick-breaking
 * PRODUCT formula with hand-derived gradients.  TEST INFRASTRUCTURE ONLY -- nothing in the
 * shipped package links or loads this; tests use it to pin oracle/sb_oracle.py (which
 * follows the reference's logsigmoid + cumulative-sum statement, sb_ref.py:8-25) against
 * an independent formulation:
 *
 *   beta_ij = sigmoid(s q_i.k_j)                       (sb_ref.py:12,17: logsigmoid(logits))
 *   A_ij    = beta_ij * prod_{j<k<i} (1 - beta_ik)     (sb_ref.py:19-24 in product form)
 *   o_i     = sum_j A_ij v_j,   rem_i = 1 - sum_j A_ij (sb_ref.py:25)
 *   keys j < i, or j <= i with attend_current          (sb_varlen/sb_varlen_fwd.py:48-51)
 *
 * Gradients are derived from the product form directly (not copied from the kernel's
 * algebra at sb_varlen_bwd.py:416-430, so that agreement is evidence):
 *   dL/dA_ij = dO_i.v_j - drem_i
 *   d log A_ij / d z_ik = [k == j](1 - beta_ik) - [j < k](beta_ik)      (k in the row's range)
 *   dz_ik = sum_j A_ij dL/dA_ij dlogA_ij/dz_ik
 * evaluated with explicit loops, O(T^3) -- small T only.
 *
 * Layout: one dense problem, q,k,v,do row-major [T][D] doubles; drem [T].
 */
#include <math.h>
#include <stdlib.h>
#include <string.h>

static double sigmoid(double z) { return z >= 0 ? 1.0 / (1.0 + exp(-z)) : exp(z) / (1.0 + exp(z)); }

/* last visible key of row i (inclusive), -1 if none */
static int last_key(int i, int attend_current) { return attend_current ? i : i - 1; }

void sb_oracle_forward(const double* q, const double* k, const double* v, int T, int D, double scale,
                       int attend_current, double* o, double* rem, double* A /* [T][T] or NULL */) {
    double* beta = (double*)malloc(sizeof(double) * (size_t)T);
    for (int i = 0; i < T; ++i) {
        int hi = last_key(i, attend_current);
        for (int j = 0; j <= hi; ++j) {
            double z = 0;
            for (int d = 0; d < D; ++d) z += q[i * D + d] * k[j * D + d];
            beta[j] = sigmoid(z * scale);
        }
        for (int d = 0; d < D; ++d) o[i * D + d] = 0;
        double total = 0;
        for (int j = 0; j < T; ++j) {
            double a = 0;
            if (j <= hi) {
                a = beta[j];
                for (int kk = j + 1; kk <= hi; ++kk) a *= (1.0 - beta[kk]);   /* explicit product */
            }
            if (A) A[(size_t)i * T + j] = a;
            total += a;
            for (int d = 0; d < D; ++d) o[i * D + d] += a * v[j * D + d];
        }
        rem[i] = 1.0 - total;
    }
    free(beta);
}

void sb_oracle_backward(const double* q, const double* k, const double* v, const double* dO,
                        const double* drem, int T, int D, double scale, int attend_current,
                        double* dq, double* dk, double* dv) {
    double* A = (double*)malloc(sizeof(double) * (size_t)T * T);
    double* o = (double*)malloc(sizeof(double) * (size_t)T * D);
    double* rem = (double*)malloc(sizeof(double) * (size_t)T);
    double* beta = (double*)malloc(sizeof(double) * (size_t)T);
    sb_oracle_forward(q, k, v, T, D, scale, attend_current, o, rem, A);
    memset(dq, 0, sizeof(double) * (size_t)T * D);
    memset(dk, 0, sizeof(double) * (size_t)T * D);
    memset(dv, 0, sizeof(double) * (size_t)T * D);
    for (int i = 0; i < T; ++i) {
        int hi = last_key(i, attend_current);
        for (int j = 0; j <= hi; ++j) {
            double z = 0;
            for (int d = 0; d < D; ++d) z += q[i * D + d] * k[j * D + d];
            beta[j] = sigmoid(z * scale);
        }
        for (int kk = 0; kk <= hi; ++kk) {
            double dz = 0;
            for (int j = 0; j <= kk; ++j) {       /* A_ij depends on z_ik only for j <= k */
                double dA = -drem[i];
                for (int d = 0; d < D; ++d) dA += dO[i * D + d] * v[j * D + d];
                double dlog = (j == kk) ? (1.0 - beta[kk]) : -beta[kk];
                dz += A[(size_t)i * T + j] * dA * dlog;
            }
            for (int d = 0; d < D; ++d) {
                dq[i * D + d] += scale * dz * k[kk * D + d];
                dk[kk * D + d] += scale * dz * q[i * D + d];
            }
        }
        for (int j = 0; j <= hi; ++j)
            for (int d = 0; d < D; ++d) dv[j * D + d] += A[(size_t)i * T + j] * dO[i * D + d];
    }
    free(A); free(o); free(rem); free(beta);
}
