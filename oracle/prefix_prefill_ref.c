/* CPU restatement of the reference's prefix-prefill programs, in plain C.
 * TEST INFRASTRUCTURE ONLY: built into oracle/_build/ and loaded by the tests to
 * cross-check the PyTorch-eager oracle with an independent loop structure.  The
 * shipped library never links or calls this file.
 *
 * It walks the work exactly the way one Triton program does
 *   lazy_attn/lazy/attention/old_ops/prefix_prefill.py:95-407   (pos_mode 0, 1)
 *   lazy_attn/lazy/attention/ops/prefix_prefill.py:95-592       (pos_mode 2 + vanilla)
 * i.e. for one (request, q-head, query row): page-by-page over the paged cache with
 * a running max / running sum (online softmax, old_ops:287-313), then the causal
 * pass over the new tokens in tiles of 64 (old_ops:326-396), then acc / l
 * (old_ops:398).  All arithmetic is double; inputs are float32 copies of the
 * operands with their real strides (in elements), so the 5-D cache index math
 * (old_ops:172-181,196-199) is restated here too.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>

typedef struct {
    const float *q, *k, *v;          /* [T,Hq,D], [T,Hkv,D], [T,Hkv,D] */
    float *o;                        /* [T,Hq,D] */
    const float *k_cache;            /* [NB,Hkv,D/x,BS,x] */
    const float *v_cache;            /* [NB,Hkv,D,BS] */
    const int32_t *b_loc;            /* [B,NBmax] */
    const int32_t *q_offset;         /* [B,NBmax], same strides as b_loc (ops:180-182) */
    const int32_t *q_mask;           /* [B,NBmax] */
    const int32_t *is_lazy;          /* [B] or NULL */
    const int64_t *b_start_loc;      /* [B+1] */
    const int64_t *b_seq_len;        /* [B] */
    const float *table;              /* [max_pos, rotary_dim] */
    int64_t sq[3], sk[3], sv[3], so[3];
    int64_t skc[5], svc[4], sbl[2];
    int32_t batch, hq, hkv, d, bs, x, rotary_dim;
    int32_t pos_mode;                /* 0 natural, 1 offset, 2 block-uniform */
    int32_t rotate_new_k;
    int32_t sliding_window;
    int32_t skip_decode;
    float sm_scale;
} ref_params;

static void rotate(const double *in, double *out, const float *row, int d)
{
    int half = d / 2;
    for (int i = 0; i < half; ++i) {
        double c = row[i], s = row[half + i];
        out[i] = in[i] * c - in[i + half] * s;          /* old_ops:256 */
        out[i + half] = in[i] * s + in[i + half] * c;   /* old_ops:257 */
    }
}

int ref_prefix_prefill(const ref_params *p)
{
    const int d = p->d, bs = p->bs, x = p->x;
    const int group = p->hq / p->hkv;
    double *kraw = (double *)malloc(sizeof(double) * d * 4);
    if (!kraw) return -1;
    double *krot = kraw + d, *vvec = kraw + 2 * d, *acc = kraw + 3 * d;

    for (int b = 0; b < p->batch; ++b) {
        int64_t qs = p->b_start_loc[b];
        int64_t q_len = p->b_start_loc[b + 1] - qs;                 /* old_ops:101-106 */
        int64_t ctx_len = p->b_seq_len[b] - q_len;
        if (q_len <= 0) continue;
        if (p->skip_decode && q_len == 1) continue;                 /* old_ops:109-110 */
        int lazy_b = p->is_lazy ? p->is_lazy[b] : 1;
        int vanilla = (p->pos_mode == 2 && !lazy_b);                /* ops:398 */
        for (int h = 0; h < p->hq; ++h) {
            int g = h / group;                                      /* old_ops:99 */
            for (int64_t t = 0; t < q_len; ++t) {
                const float *qrow = p->q + (qs + t) * p->sq[0] + h * p->sq[1];
                double m_i = -INFINITY, l_i = 1.0;                  /* old_ops:157-158 */
                for (int i = 0; i < d; ++i) acc[i] = 0.0;
                /* ---- context pages (old_ops:162-313) ---- */
                for (int64_t start_n = 0; start_n < ctx_len; start_n += bs) {
                    int64_t j = start_n / bs;
                    int64_t off = b * p->sbl[0] + j * p->sbl[1];
                    int32_t bn = p->b_loc[off];
                    int32_t qm = (!vanilla && p->q_mask) ? p->q_mask[off] : 0;
                    int64_t seq_bound = start_n + bs - qm;          /* old_ops:167 */
                    if (seq_bound > ctx_len) seq_bound = ctx_len;
                    int64_t pos_base = start_n;
                    if (p->pos_mode == 1) {
                        int32_t qo = p->q_offset[off];
                        if (qo != 0) pos_base = qo - 1;             /* old_ops:186-191 */
                    } else if (p->pos_mode == 2) {
                        int32_t qo = p->q_offset ? p->q_offset[off] : 0;
                        pos_base = qo != 0 ? qo - 1 : 0;            /* ops:183-185 */
                    }
                    /* tile max over the page's valid slots */
                    double s_tile[512];
                    double m_ij = m_i;
                    for (int o_ = 0; o_ < bs; ++o_) {
                        int64_t n = start_n + o_;
                        if (n >= seq_bound) { s_tile[o_] = -INFINITY; continue; }
                        for (int dd = 0; dd < d; ++dd)
                            kraw[dd] = p->k_cache[bn * p->skc[0] + g * p->skc[1] +
                                                  (dd / x) * p->skc[2] + o_ * p->skc[3] +
                                                  (dd % x) * p->skc[4]];
                        const double *kk = kraw;
                        if (!vanilla) {
                            int64_t pos = (p->pos_mode == 2) ? pos_base : pos_base + o_;
                            rotate(kraw, krot, p->table + pos * p->rotary_dim, d);
                            kk = krot;
                        }
                        double s = 0.0;
                        for (int dd = 0; dd < d; ++dd) s += (double)qrow[dd * p->sq[2]] * kk[dd];
                        s *= p->sm_scale;                           /* old_ops:269 */
                        if (p->sliding_window > 0 &&
                            (ctx_len + t) - n >= p->sliding_window) s = -10000.0;
                        s_tile[o_] = s;
                        if (s > m_ij) m_ij = s;
                    }
                    if (m_ij == -INFINITY) continue;  /* empty page before any key: skip */
                    double alpha = exp(m_i - m_ij);                 /* old_ops:290 */
                    double l_ij = 0.0;
                    for (int i = 0; i < d; ++i) acc[i] *= alpha;
                    for (int o_ = 0; o_ < bs; ++o_) {
                        if (s_tile[o_] == -INFINITY) continue;
                        double pr = exp(s_tile[o_] - m_ij);
                        l_ij += pr;
                        for (int dd = 0; dd < d; ++dd)
                            acc[dd] += pr * p->v_cache[bn * p->svc[0] + g * p->svc[1] +
                                                       dd * p->svc[2] + o_ * p->svc[3]];
                    }
                    l_i = l_i * alpha + l_ij;                       /* old_ops:312 */
                    m_i = m_ij;
                }
                /* ---- new tokens, tiles of 64, causal (old_ops:326-396) ---- */
                for (int64_t start_n = 0; start_n <= t; start_n += 64) {
                    double s_tile[64];
                    double m_ij = m_i;
                    for (int c = 0; c < 64; ++c) {
                        int64_t m = start_n + c;
                        if (m > t || m >= q_len) { s_tile[c] = -INFINITY; continue; }
                        const float *krow = p->k + (qs + m) * p->sk[0] + g * p->sk[1];
                        for (int dd = 0; dd < d; ++dd) kraw[dd] = krow[dd * p->sk[2]];
                        const double *kk = kraw;
                        if (p->rotate_new_k && !vanilla) {
                            rotate(kraw, krot, p->table + (ctx_len + m) * p->rotary_dim, d);
                            kk = krot;
                        }
                        double s = 0.0;
                        for (int dd = 0; dd < d; ++dd) s += (double)qrow[dd * p->sq[2]] * kk[dd];
                        s *= p->sm_scale;
                        if (p->sliding_window > 0 && t - m >= p->sliding_window) s = -10000.0;
                        s_tile[c] = s;
                        if (s > m_ij) m_ij = s;
                    }
                    double alpha = exp(m_i - m_ij);
                    double l_ij = 0.0;
                    for (int i = 0; i < d; ++i) acc[i] *= alpha;
                    for (int c = 0; c < 64; ++c) {
                        if (s_tile[c] == -INFINITY) continue;
                        int64_t m = start_n + c;
                        double pr = exp(s_tile[c] - m_ij);
                        l_ij += pr;
                        const float *vrow = p->v + (qs + m) * p->sv[0] + g * p->sv[1];
                        for (int dd = 0; dd < d; ++dd) acc[dd] += pr * vrow[dd * p->sv[2]];
                    }
                    l_i = l_i * alpha + l_ij;
                    m_i = m_ij;
                }
                /* the running sum starts at 1.0 with m=-inf, so the first alpha is 0 and
                 * the initial 1.0 vanishes (old_ops:158,290,312) */
                float *orow = p->o + (qs + t) * p->so[0] + h * p->so[1];
                for (int dd = 0; dd < d; ++dd) orow[dd * p->so[2]] = (float)(acc[dd] / l_i);
            }
        }
    }
    free(kraw);
    (void)vvec;
    return 0;
}
