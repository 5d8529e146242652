/*
 * CPU oracle, part 2: a plain-C restatement of the reference's TILED attention
 * algorithm (its three Triton kernels), as opposed to eager_ref.py which restates
 * the eager function those kernels replace.
 *
 * TEST INFRASTRUCTURE ONLY.  The shipped library never links or calls this file.
 *
 * What follows which reference lines (attention_kernel.py in the reference):
 *   oracle_attn_fwd        :11-100   online softmax whose running max starts at
 *                                    the sink logit (:53), 64-wide KV tiles over
 *                                    [lo,hi) (:60-65), additive -1e6 mask from the
 *                                    causal (:68) and too-old (:71) predicates,
 *                                    z = l + exp(sink-m), O = acc/z, M = m+log z
 *                                    (:93-98).  Output goes straight to the
 *                                    (B,S,H,D) layout the wrapper produces (:272).
 *   oracle_attn_bwd_delta  :102-120  D_i = sum_d dO_i,d * O_i,d.
 *   oracle_attn_bwd        :122-217  per q-tile: p = exp(s - M) (:199),
 *                                    dV += p^T dO (:201-204), dP = dO V^T (:206),
 *                                    dS = p (dP - D) (:207), dK += scale dS^T Q
 *                                    (:209-212), dQ = scale dS K (:214-217),
 *                                    dSinks_h += sum_i -exp(sink-M_i) D_i (:173-176).
 *   head mapping           :36,152   kv head = h / (H / G).
 *   absent sinks           :39-42    a NULL sinks pointer means logit 0.
 *
 * Differences from the reference, all deliberate and none changing the math:
 *   - arithmetic is carried in double (inputs/outputs are float) so this is a
 *     tighter ground truth than either fp32 eager or the kernels;
 *   - rows and keys are bounds-checked instead of zero-padding S to 64 (:233-239);
 *   - dK/dV are summed sequentially instead of by atomics (:204,212);
 *   - `seqlens` (right padding) is an addition: keys >= len are masked like
 *     too-old keys, and query rows >= len see no key at all.
 *   - start_q (:44-47) is taken by value as q_offset.
 *   - `doc_start` (packed rows) is an addition: keys before the first token of the
 *     query's own document are masked.
 *
 * Pinning: tests/test_oracle_tiled.py checks every function here against
 * eager_ref.py (itself pinned by golden vectors and closed forms).
 */
#include <limits.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>

#define TILE 64
#define MASK_ADD (-1.0e6)

static inline int imax(int a, int b) { return a > b ? a : b; }
static inline int imin(int a, int b) { return a < b ? a : b; }

/* 1 when key j is hidden from the query at absolute position pos; `first` is the
   first key of the query's own document (0 unless rows are packed). */
static inline int masked(int j, int pos, int window, int len, int first)
{
    if (j > pos) return 1;                          /* :68  */
    if (window > 0 && j < pos - window + 1) return 1; /* :71  */
    if (j >= len || pos >= len) return 1;           /* right padding */
    if (j < first) return 1;                        /* another document of a packed row */
    return 0;
}

int oracle_attn_fwd(const float *q, const float *k, const float *v, const float *sinks,
                    float *o, float *lse,
                    int B, int H, int G, int Sq, int Skv, int D,
                    float scale, int window, int q_offset, const int *seqlens, const int *doc_start)
{
    if (!q || !k || !v || !o || !lse || G <= 0 || H % G) return -1;
    const int r = H / G;
    #pragma omp parallel for collapse(2) schedule(dynamic)
    for (int b = 0; b < B; ++b)
    for (int h = 0; h < H; ++h) {
        const int len = seqlens ? seqlens[b] : INT_MAX;
        const int g = h / r;
        const double sink = sinks ? (double)sinks[h] : 0.0;
        const float *kb = k + ((size_t)b * G + g) * Skv * D;
        const float *vb = v + ((size_t)b * G + g) * Skv * D;
        double *acc = (double *)malloc(sizeof(double) * TILE * D);
        double m_i[TILE], l_i[TILE], s[TILE];
        for (int m0 = 0; m0 < Sq; m0 += TILE) {
            const int rows = imin(TILE, Sq - m0);
            for (int i = 0; i < rows; ++i) { m_i[i] = sink; l_i[i] = 0.0; }
            memset(acc, 0, sizeof(double) * TILE * D);
            int lo = 0, hi = imin(Skv, q_offset + m0 + TILE);
            if (window > 0) lo = imax(0, q_offset + m0 - window);
            for (int n0 = lo; n0 < hi; n0 += TILE) {
                const int cols = imin(TILE, Skv - n0);
                for (int i = 0; i < rows; ++i) {
                    const int pos = q_offset + m0 + i;
                    const int first = doc_start ? doc_start[(size_t)b * Sq + m0 + i] : 0;
                    const float *qi = q + (((size_t)b * H + h) * Sq + m0 + i) * D;
                    double mx = m_i[i];
                    for (int j = 0; j < cols; ++j) {
                        double dot = 0.0;
                        for (int d = 0; d < D; ++d) dot += (double)qi[d] * (double)kb[(size_t)(n0 + j) * D + d];
                        s[j] = dot * scale + (masked(n0 + j, pos, window, len, first) ? MASK_ADD : 0.0);
                        if (s[j] > mx) mx = s[j];
                    }
                    const double alpha = exp(m_i[i] - mx);
                    double lsum = 0.0;
                    for (int d = 0; d < D; ++d) acc[i * D + d] *= alpha;
                    for (int j = 0; j < cols; ++j) {
                        const double p = exp(s[j] - mx);
                        lsum += p;
                        const float *vj = vb + (size_t)(n0 + j) * D;
                        for (int d = 0; d < D; ++d) acc[i * D + d] += p * (double)vj[d];
                    }
                    l_i[i] = l_i[i] * alpha + lsum;
                    m_i[i] = mx;
                }
            }
            for (int i = 0; i < rows; ++i) {
                const double z = l_i[i] + exp(sink - m_i[i]);
                float *oi = o + (((size_t)b * Sq + m0 + i) * H + h) * D;
                for (int d = 0; d < D; ++d) oi[d] = (float)(acc[i * D + d] / z);
                lse[((size_t)b * H + h) * Sq + m0 + i] = (float)(m_i[i] + log(z));
            }
        }
        free(acc);
    }
    return 0;
}

int oracle_attn_bwd_delta(const float *o, const float *d_o, float *delta,
                          int B, int H, int Sq, int D)
{
    if (!o || !d_o || !delta) return -1;
    #pragma omp parallel for collapse(2)
    for (int b = 0; b < B; ++b)
    for (int h = 0; h < H; ++h)
        for (int i = 0; i < Sq; ++i) {
            const float *oi = o + (((size_t)b * Sq + i) * H + h) * D;
            const float *gi = d_o + (((size_t)b * Sq + i) * H + h) * D;
            double acc = 0.0;
            for (int d = 0; d < D; ++d) acc += (double)oi[d] * (double)gi[d];
            delta[((size_t)b * H + h) * Sq + i] = (float)acc;
        }
    return 0;
}

int oracle_attn_bwd(const float *q, const float *k, const float *v, const float *sinks,
                    const float *lse, const float *delta, const float *d_o,
                    float *dq, float *dk, float *dv, float *dsinks,
                    int B, int H, int G, int Sq, int Skv, int D,
                    float scale, int window, int q_offset, const int *seqlens, const int *doc_start)
{
    if (!q || !k || !v || !lse || !delta || !d_o || !dq || !dk || !dv || G <= 0 || H % G) return -1;
    const int r = H / G;
    const size_t kv_elems = (size_t)B * G * Skv * D;
    double *dk_acc = (double *)calloc(kv_elems, sizeof(double));
    double *dv_acc = (double *)calloc(kv_elems, sizeof(double));
    if (!dk_acc || !dv_acc) { free(dk_acc); free(dv_acc); return -2; }
    /* one (b, kv head) per thread so that the sequential dK/dV sums never race */
    #pragma omp parallel for collapse(2) schedule(dynamic)
    for (int b = 0; b < B; ++b)
    for (int g = 0; g < G; ++g) {
        const int len = seqlens ? seqlens[b] : INT_MAX;
        const float *kb = k + ((size_t)b * G + g) * Skv * D;
        const float *vb = v + ((size_t)b * G + g) * Skv * D;
        double *dkb = dk_acc + ((size_t)b * G + g) * Skv * D;
        double *dvb = dv_acc + ((size_t)b * G + g) * Skv * D;
        double *dqrow = (double *)malloc(sizeof(double) * D);
        for (int h = g * r; h < (g + 1) * r; ++h) {
            for (int m0 = 0; m0 < Sq; m0 += TILE) {
                const int rows = imin(TILE, Sq - m0);
                int lo = 0, hi = imin(Skv, q_offset + m0 + TILE);
                if (window > 0) lo = imax(0, q_offset + m0 - window);
                for (int i = 0; i < rows; ++i) {
                    const int pos = q_offset + m0 + i;
                    const int first = doc_start ? doc_start[(size_t)b * Sq + m0 + i] : 0;
                    const size_t row = ((size_t)b * H + h) * Sq + m0 + i;
                    const float *qi = q + row * D;
                    const float *gi = d_o + (((size_t)b * Sq + m0 + i) * H + h) * D;
                    const double Mi = lse[row], Di = delta[row];
                    for (int d = 0; d < D; ++d) dqrow[d] = 0.0;
                    for (int n0 = lo; n0 < hi; n0 += TILE) {
                        const int cols = imin(TILE, Skv - n0);
                        for (int j = 0; j < cols; ++j) {
                            const float *kj = kb + (size_t)(n0 + j) * D;
                            const float *vj = vb + (size_t)(n0 + j) * D;
                            double dot = 0.0, dp = 0.0;
                            for (int d = 0; d < D; ++d) {
                                dot += (double)qi[d] * (double)kj[d];
                                dp += (double)gi[d] * (double)vj[d];
                            }
                            const double sij = dot * scale + (masked(n0 + j, pos, window, len, first) ? MASK_ADD : 0.0);
                            const double p = exp(sij - Mi);       /* :199 */
                            const double ds = p * (dp - Di);       /* :207 */
                            double *dkj = dkb + (size_t)(n0 + j) * D;
                            double *dvj = dvb + (size_t)(n0 + j) * D;
                            for (int d = 0; d < D; ++d) {
                                dvj[d] += p * (double)gi[d];               /* :201 */
                                dkj[d] += ds * (double)qi[d] * scale;      /* :209-212 */
                                dqrow[d] += ds * (double)kj[d] * scale;    /* :214 */
                            }
                        }
                    }
                    float *dqi = dq + row * D;
                    for (int d = 0; d < D; ++d) dqi[d] = (float)dqrow[d];
                }
            }
        }
        free(dqrow);
    }
    /* dSinks_h = sum over b,i of -exp(sink_h - M_i) * D_i  (:173-176), summed
       serially here rather than by atomics. */
    if (dsinks) {
        for (int h = 0; h < H; ++h) {
            const double sink = sinks ? (double)sinks[h] : 0.0;
            double acc = 0.0;
            for (int b = 0; b < B; ++b)
                for (int i = 0; i < Sq; ++i) {
                    const size_t row = ((size_t)b * H + h) * Sq + i;
                    acc += -exp(sink - (double)lse[row]) * (double)delta[row];
                }
            dsinks[h] = (float)acc;
        }
    }
    for (size_t e = 0; e < kv_elems; ++e) { dk[e] = (float)dk_acc[e]; dv[e] = (float)dv_acc[e]; }
    free(dk_acc); free(dv_acc);
    return 0;
}
