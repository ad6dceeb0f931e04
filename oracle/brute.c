/* O(L^2) brute-force evaluation of bidirectional linear attention in double
 * precision.  Test infrastructure only: it shares no algebra with the
 * state-based formulas (no K^T V state is ever formed), so it pins them.
 *
 *   o_i = scale * sum_j (qn_i . kn_j) v_j / ( (1/L) sum_j (q_i . k_j) + eps )
 *
 * which is flash_bla/ops/linear_attn/naive.py:10-12 with the matrix products
 * re-associated as (Q K^T) V.  normalize=0 drops the denominator
 * (flash_bla/ops/simple_la/naive.py:17-18).  qn/kn are the numerator features
 * (q_rope/k_rope of naive.py:21-23); pass q/k themselves for the plain operator.
 * One call handles one (batch, head): arrays are [L, DK] and [L, DV] row-major.
 */
#include <stddef.h>

void brute_linear_attn(const double *q, const double *k, const double *qn, const double *kn,
                       const double *v, double *o, long L, long DK, long DV,
                       double scale, double eps, int normalize)
{
    for (long i = 0; i < L; ++i) {
        double den = 0.0;
        for (long c = 0; c < DV; ++c) o[i * DV + c] = 0.0;
        for (long j = 0; j < L; ++j) {
            double a_num = 0.0, a_den = 0.0;
            for (long d = 0; d < DK; ++d) {
                a_num += qn[i * DK + d] * kn[j * DK + d];
                a_den += q[i * DK + d] * k[j * DK + d];
            }
            den += a_den;
            for (long c = 0; c < DV; ++c) o[i * DV + c] += a_num * v[j * DV + c];
        }
        double z = normalize ? den / (double)L + eps : 1.0;
        for (long c = 0; c < DV; ++c) o[i * DV + c] = scale * o[i * DV + c] / z;
    }
}
