/* Per-token evaluation of piecewise (PISA) attention in double precision, one
 * head per call.  Test infrastructure only.  It walks the steps of the
 * reference's forward kernel one query token at a time, with the kernel's own
 * base-2 running-maximum bookkeeping, and shares no code and no matrix algebra
 * with oracle/piecewise.py (which evaluates the closed form densely in numpy):
 *
 *   chunk statistics   flash_bla/ops/piecewise_attn/kernel.py:105-118,176
 *                      kc_c = mean of the chunk's keys (divided by the chunk's
 *                      true length), vc_c = SUM of its values,
 *                      H = sum over all chunks of (K_c - kc_c)^T V_c
 *   phase 1 (exact)    kernel.py:214-236   selected chunks in index order, keys
 *                      past T masked, running maximum m, sum l, accumulator acc
 *   phase 2 (means)    kernel.py:238-276   every chunk that is not selected, as
 *                      ONE group (the kernel's GROUP_SIZE >= NT): with a single
 *                      group the kernel's running g (never rescaled between
 *                      groups, :263-276) is exactly what is computed here
 *   phase 3 (1st ord.) kernel.py:278-285   acc += (q H) * g * (1/T) * scale
 *   final              kernel.py:287-292   o = acc / (l + g)
 *
 * Arrays are row-major: q,k [T,K]; v,o [T,V]; indices [NT,NS] (key chunks
 * selected for the query chunk a token belongs to).  work: caller-provided
 * scratch of NT*K + NT*V + K*V doubles.
 */
#include <math.h>
#include <stddef.h>

static const double LOG2E = 1.44269504; /* the constant the kernel multiplies by (kernel.py:214) */

void pisa_tokens(const double *q, const double *k, const double *v, const long *indices,
                 double *o, double *work, long T, long K, long V, long BT, long NS, double scale)
{
    const long NT = (T + BT - 1) / BT;
    double *kc = work;               /* [NT,K] chunk mean keys   */
    double *vc = kc + NT * K;        /* [NT,V] chunk value sums  */
    double *H = vc + NT * V;         /* [K,V]                    */

    for (long a = 0; a < K * V; ++a) H[a] = 0.0;
    for (long c = 0; c < NT; ++c) {
        const long lo = c * BT, hi = (lo + BT < T) ? lo + BT : T;
        const double n = (double)(hi - lo);
        for (long d = 0; d < K; ++d) {
            double s = 0.0;
            for (long j = lo; j < hi; ++j) s += k[j * K + d];
            kc[c * K + d] = s / n;
        }
        for (long e = 0; e < V; ++e) {
            double s = 0.0;
            for (long j = lo; j < hi; ++j) s += v[j * V + e];
            vc[c * V + e] = s;
        }
        for (long j = lo; j < hi; ++j)
            for (long d = 0; d < K; ++d) {
                const double centred = k[j * K + d] - kc[c * K + d];
                for (long e = 0; e < V; ++e) H[d * V + e] += centred * v[j * V + e];
            }
    }

    const double sm_scale = scale * LOG2E;
    const long last_len = T - (NT - 1) * BT;

    for (long i = 0; i < T; ++i) {
        const double *qi = q + i * K;
        const long *sel = indices + (i / BT) * NS;
        double *acc = o + i * V;
        double m = -INFINITY, l = 0.0;
        for (long e = 0; e < V; ++e) acc[e] = 0.0;

        /* phase 1: one running-maximum update per selected chunk */
        for (long s = 0; s < NS; ++s) {
            const long lo = sel[s] * BT;
            double blockmax = -INFINITY;
            for (long j = lo; j < lo + BT && j < T; ++j) {
                double dot = 0.0;
                for (long d = 0; d < K; ++d) dot += qi[d] * k[j * K + d];
                if (dot * sm_scale > blockmax) blockmax = dot * sm_scale;
            }
            const double m_new = blockmax > m ? blockmax : m;
            const double alpha = (m == -INFINITY) ? 0.0 : exp2(m - m_new);
            l *= alpha;
            for (long e = 0; e < V; ++e) acc[e] *= alpha;
            for (long j = lo; j < lo + BT && j < T; ++j) {
                double dot = 0.0;
                for (long d = 0; d < K; ++d) dot += qi[d] * k[j * K + d];
                const double p = exp2(dot * sm_scale - m_new);
                l += p;
                for (long e = 0; e < V; ++e) acc[e] += p * v[j * V + e];
            }
            m = m_new;
        }

        /* phase 2: all unselected chunks as a single group */
        double groupmax = -INFINITY;
        for (long c = 0; c < NT; ++c) {
            int picked = 0;
            for (long s = 0; s < NS; ++s) picked |= (sel[s] == c);
            if (picked) continue;
            double dot = 0.0;
            for (long d = 0; d < K; ++d) dot += qi[d] * kc[c * K + d];
            if (dot * sm_scale > groupmax) groupmax = dot * sm_scale;
        }
        double g = 0.0;
        if (groupmax > -INFINITY) {
            const double m_new = groupmax > m ? groupmax : m;
            const double alpha = (m == -INFINITY) ? 0.0 : exp2(m - m_new);
            l *= alpha;
            for (long e = 0; e < V; ++e) acc[e] *= alpha;
            m = m_new;
            for (long c = 0; c < NT; ++c) {
                int picked = 0;
                for (long s = 0; s < NS; ++s) picked |= (sel[s] == c);
                if (picked) continue;
                double dot = 0.0;
                for (long d = 0; d < K; ++d) dot += qi[d] * kc[c * K + d];
                const double p = exp2(dot * sm_scale - m);
                for (long e = 0; e < V; ++e) acc[e] += p * vc[c * V + e];
                g += p * (double)(c == NT - 1 ? last_len : BT);
            }
        }

        /* phase 3: first-order correction through H, then the division */
        const double coeff = g * (1.0 / (double)T) * scale;
        for (long e = 0; e < V; ++e) {
            double r = 0.0;
            for (long d = 0; d < K; ++d) r += qi[d] * H[d * V + e];
            acc[e] += r * coeff;
        }
        l += g;
        for (long e = 0; e < V; ++e) acc[e] /= l;
    }
}
