/*
 * CPU oracle (TEST INFRASTRUCTURE, never shipped): plain-C fp32 restatement of the tiled
 * FlashBias recurrences of the reference's Triton kernels.
 *
 *   fbo_fwd    follows flash_bias/flash_bias_triton.py:128-355  (_fwd_kernel)
 *   fbo_delta  follows flash_bias/flash_bias_triton.py:358-400  (_bwd_preprocess_do_o_dot)
 *   fbo_bwd    follows flash_bias/flash_bias_triton.py:450-869  (_bwd_kernel_one_col_block,
 *              serial key-block loop of :1001-1049, i.e. the non-atomic variant)
 *
 * All tensors are fp32 with the last dimension contiguous; every other dimension is
 * addressed through explicit element strides (batch, head, sequence) exactly as the
 * reference passes them (:1163-1177).  Factor tensors may have stride 0 in batch / head
 * (broadcast, :1135-1136); gradients of broadcast factors are *summed* over the broadcast
 * dimensions (the autograd meaning), which the serial loop below gives for free because it
 * accumulates with "+=" into whatever the strides address.
 *
 * Pinned by: the eager oracle (oracle/eager.py) on the fp32 plumbing configuration and on
 * ragged / causal / masked shapes, see tests/test_oracle.py.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

typedef struct {
    float *p;
    int64_t sb, sh, ss; /* element strides: batch, head, sequence; last dim contiguous */
} fbo_t;

typedef struct {
    int32_t B, H, Lq, Lk, d, r;
    int32_t causal;
    int32_t mask_type; /* 0 none, 1 vector (.., 1, Lk), 2 matrix (.., Lq, Lk) */
    int32_t block_m, block_n;
    float scale;
    fbo_t q, k, v, qb, kb, o, dO, dq, dk, dv, dqb, dkb;
    fbo_t mask;  /* sb, sh, ss = strides of batch, head, query row */
    float *lse;   /* (B, H, Lq) */
    float *delta; /* (B, H, Lq) */
} fbo_params;

static inline float *row(const fbo_t *t, int b, int h, int s) {
    return t->p + b * t->sb + h * t->sh + s * t->ss;
}

static inline int imin(int a, int b) { return a < b ? a : b; }

/* scores of one (query tile, key tile): scale * q k^T + q_b k_b^T, then -inf for
 * out-of-range keys and causal-hidden pairs, then + mask  (:243-282, :637-664) */
static void tile_scores(const fbo_params *P, int b, int h, int m0, int mlen, int n0, int nlen,
                        float *s, int ld) {
    for (int i = 0; i < mlen; ++i) {
        const float *qi = row(&P->q, b, h, m0 + i);
        const float *qbi = P->r ? row(&P->qb, b, h, m0 + i) : 0;
        for (int j = 0; j < nlen; ++j) {
            const float *kj = row(&P->k, b, h, n0 + j);
            float acc = 0.f;
            for (int c = 0; c < P->d; ++c) acc += qi[c] * kj[c];
            acc *= P->scale;
            if (P->r) {
                const float *kbj = row(&P->kb, b, h, n0 + j);
                float bacc = 0.f;
                for (int c = 0; c < P->r; ++c) bacc += qbi[c] * kbj[c];
                acc += bacc;
            }
            if (P->causal && (m0 + i) < (n0 + j)) acc = -INFINITY;
            if (P->mask_type == 1)
                acc += (P->mask.p + b * P->mask.sb + h * P->mask.sh)[n0 + j];
            else if (P->mask_type == 2)
                acc += (P->mask.p + b * P->mask.sb + h * P->mask.sh + (int64_t)(m0 + i) * P->mask.ss)[n0 + j];
            s[i * ld + j] = acc;
        }
    }
}

int fbo_fwd(const fbo_params *P) {
    const int BM = P->block_m, BN = P->block_n, d = P->d;
    if (BM <= 0 || BN <= 0) return -1;
#pragma omp parallel for collapse(2) schedule(dynamic)
    for (int bh = 0; bh < P->B * P->H; ++bh) {
        for (int m0 = 0; m0 < P->Lq; m0 += BM) {
            const int b = bh / P->H, h = bh % P->H;
            const int mlen = imin(BM, P->Lq - m0);
            float *s = (float *)malloc(sizeof(float) * BM * BN);
            float *acc = (float *)calloc((size_t)BM * d, sizeof(float));
            float *m_i = (float *)malloc(sizeof(float) * BM);
            float *lse_i = (float *)malloc(sizeof(float) * BM);
            for (int i = 0; i < BM; ++i) m_i[i] = lse_i[i] = -INFINITY;
            /* :202  causal tiles stop at the diagonal */
            const int end_n = P->causal ? imin(m0 + BM, P->Lk) : P->Lk;
            for (int n0 = 0; n0 < end_n; n0 += BN) {
                const int nlen = imin(BN, P->Lk - n0);
                tile_scores(P, b, h, m0, mlen, n0, nlen, s, BN);
                for (int i = 0; i < mlen; ++i) {
                    float mx = lse_i[i]; /* :283/:286  m_ij = max(rowmax, lse_i) */
                    for (int j = 0; j < nlen; ++j) mx = fmaxf(mx, s[i * BN + j]);
                    float l = 0.f;
                    for (int j = 0; j < nlen; ++j) {
                        s[i * BN + j] = expf(s[i * BN + j] - mx);
                        l += s[i * BN + j];
                    }
                    const float alpha = expf(m_i[i] - mx); /* :291 */
                    for (int c = 0; c < d; ++c) acc[i * d + c] *= alpha;
                    for (int j = 0; j < nlen; ++j) {
                        const float p = s[i * BN + j];
                        const float *vj = row(&P->v, b, h, n0 + j);
                        for (int c = 0; c < d; ++c) acc[i * d + c] += p * vj[c];
                    }
                    m_i[i] = mx;                                       /* :321 */
                    lse_i[i] = mx + logf(expf(lse_i[i] - mx) + l);     /* :322-323 */
                }
            }
            for (int i = 0; i < mlen; ++i) {
                const float os = expf(m_i[i] - lse_i[i]); /* :325 */
                float *oi = row(&P->o, b, h, m0 + i);
                for (int c = 0; c < d; ++c) oi[c] = acc[i * d + c] * os;
                P->lse[(int64_t)bh * P->Lq + m0 + i] = lse_i[i];
            }
            free(s); free(acc); free(m_i); free(lse_i);
        }
    }
    return 0;
}

int fbo_delta(const fbo_params *P) {
    for (int bh = 0; bh < P->B * P->H; ++bh) {
        const int b = bh / P->H, h = bh % P->H;
        for (int i = 0; i < P->Lq; ++i) {
            const float *oi = row(&P->o, b, h, i), *doi = row(&P->dO, b, h, i);
            float acc = 0.f;
            for (int c = 0; c < P->d; ++c) acc += oi[c] * doi[c]; /* :398 */
            P->delta[(int64_t)bh * P->Lq + i] = acc;
        }
    }
    return 0;
}

/* Gradient buffers must be zero on entry: every output is accumulated with "+=" so that
 * stride-0 (broadcast) factor gradients come out summed. */
int fbo_bwd(const fbo_params *P) {
    const int BM = P->block_m, BN = P->block_n, d = P->d, r = P->r;
    if (BM <= 0 || BN <= 0) return -1;
    float *s = (float *)malloc(sizeof(float) * BM * BN);
    float *ds = (float *)malloc(sizeof(float) * BM * BN);
    for (int bh = 0; bh < P->B * P->H; ++bh) {
        const int b = bh / P->H, h = bh % P->H;
        const float *lse = P->lse + (int64_t)bh * P->Lq;
        const float *delta = P->delta + (int64_t)bh * P->Lq;
        for (int n0 = 0; n0 < P->Lk; n0 += BN) {
            const int nlen = imin(BN, P->Lk - n0);
            /* :498  first query tile that can see this key block */
            const int begin_m = P->causal ? (n0 / BM) * BM : 0;
            for (int m0 = begin_m; m0 < P->Lq; m0 += BM) {
                const int mlen = imin(BM, P->Lq - m0);
                tile_scores(P, b, h, m0, mlen, n0, nlen, s, BN);
                for (int i = 0; i < mlen; ++i) {
                    const float *doi = row(&P->dO, b, h, m0 + i);
                    for (int j = 0; j < nlen; ++j) {
                        const float p = expf(s[i * BN + j] - lse[m0 + i]); /* :670 */
                        const float *vj = row(&P->v, b, h, n0 + j);
                        float *dvj = row(&P->dv, b, h, n0 + j);
                        float dp = 0.f;
                        for (int c = 0; c < d; ++c) {
                            dvj[c] += p * doi[c]; /* :697 */
                            dp += doi[c] * vj[c]; /* :705 */
                        }
                        s[i * BN + j] = p;
                        ds[i * BN + j] = p * (dp - delta[m0 + i]); /* :714 */
                    }
                }
                for (int i = 0; i < mlen; ++i) {
                    const float *qi = row(&P->q, b, h, m0 + i);
                    float *dqi = row(&P->dq, b, h, m0 + i);
                    for (int j = 0; j < nlen; ++j) {
                        const float g = ds[i * BN + j];
                        const float *kj = row(&P->k, b, h, n0 + j);
                        float *dkj = row(&P->dk, b, h, n0 + j);
                        for (int c = 0; c < d; ++c) {
                            dkj[c] += g * qi[c] * P->scale; /* :717 */
                            dqi[c] += g * kj[c] * P->scale; /* :728 */
                        }
                        if (r) {
                            const float *qbi = row(&P->qb, b, h, m0 + i);
                            const float *kbj = row(&P->kb, b, h, n0 + j);
                            float *dqbi = row(&P->dqb, b, h, m0 + i);
                            float *dkbj = row(&P->dkb, b, h, n0 + j);
                            for (int c = 0; c < r; ++c) {
                                dkbj[c] += g * qbi[c]; /* :719 */
                                dqbi[c] += g * kbj[c]; /* :732 */
                            }
                        }
                    }
                }
            }
        }
    }
    free(s); free(ds);
    return 0;
}

int fbo_params_size(void) { return (int)sizeof(fbo_params); }
