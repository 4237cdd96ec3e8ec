/*
 * Sanitizer driver for the C oracle (TEST INFRASTRUCTURE, never shipped): runs fbo_fwd / fbo_delta /
 * fbo_bwd of blocked.c on ragged, rectangular, causal, masked and broadcast shapes with every
 * buffer allocated at its exact size, so that an index that leaves a tensor trips
 * AddressSanitizer and signed overflow / misaligned access trips UBSan.  Built by
 * `make -C oracle sanitize` (gcc -fsanitize=address,undefined); exit status 0 = clean.
 */
#include "blocked.c"

#include <stdio.h>

static float *fill(size_t n, unsigned *seed) {
    float *p = (float *)malloc(n * sizeof(float));
    for (size_t i = 0; i < n; ++i) {
        *seed = *seed * 1664525u + 1013904223u;
        p[i] = ((float)(*seed >> 8) / (float)(1u << 24) - 0.5f) * 2.f;
    }
    return p;
}

static fbo_t tensor(float *p, int L, int H, int c, int bcast_b, int bcast_h) {
    fbo_t t;
    t.p = p;
    t.ss = (int64_t)(bcast_h ? 1 : H) * c;
    t.sh = bcast_h ? 0 : c;
    t.sb = bcast_b ? 0 : (int64_t)L * t.ss;
    return t;
}

static int run_case(int B, int H, int Lq, int Lk, int d, int r, int causal, int mask_type, int bm, int bn, int bq_b,
                    int bk_h) {
    unsigned seed = 12345u + (unsigned)(Lq * 31 + Lk * 7 + d);
    fbo_params P;
    memset(&P, 0, sizeof(P));
    P.B = B; P.H = H; P.Lq = Lq; P.Lk = Lk; P.d = d; P.r = r;
    P.causal = causal; P.mask_type = mask_type; P.block_m = bm; P.block_n = bn;
    P.scale = 1.f / sqrtf((float)d);
    const size_t nq = (size_t)B * Lq * H * d, nk = (size_t)B * Lk * H * d;
    float *q = fill(nq, &seed), *k = fill(nk, &seed), *v = fill(nk, &seed), *dO = fill(nq, &seed);
    float *o = fill(nq, &seed), *dq = fill(nq, &seed), *dk = fill(nk, &seed), *dv = fill(nk, &seed);
    P.q = tensor(q, Lq, H, d, 0, 0); P.k = tensor(k, Lk, H, d, 0, 0); P.v = tensor(v, Lk, H, d, 0, 0);
    P.o = tensor(o, Lq, H, d, 0, 0); P.dO = tensor(dO, Lq, H, d, 0, 0);
    P.dq = tensor(dq, Lq, H, d, 0, 0); P.dk = tensor(dk, Lk, H, d, 0, 0); P.dv = tensor(dv, Lk, H, d, 0, 0);
    float *qb = NULL, *kb = NULL, *dqb = NULL, *dkb = NULL, *mask = NULL;
    if (r > 0) {
        const size_t nqb = (size_t)(bq_b ? 1 : B) * Lq * H * r, nkb = (size_t)B * Lk * (bk_h ? 1 : H) * r;
        qb = fill(nqb, &seed); kb = fill(nkb, &seed);
        dqb = (float *)calloc(nqb, sizeof(float)); dkb = (float *)calloc(nkb, sizeof(float));
        P.qb = tensor(qb, Lq, H, r, bq_b, 0); P.kb = tensor(kb, Lk, H, r, 0, bk_h);
        P.dqb = tensor(dqb, Lq, H, r, bq_b, 0); P.dkb = tensor(dkb, Lk, H, r, 0, bk_h);
    }
    if (mask_type == 1) {
        mask = fill((size_t)B * Lk, &seed);
        P.mask.p = mask; P.mask.sb = Lk; P.mask.sh = 0; P.mask.ss = 0;
    } else if (mask_type == 2) {
        mask = fill((size_t)H * Lq * Lk, &seed);
        P.mask.p = mask; P.mask.sb = 0; P.mask.sh = (int64_t)Lq * Lk; P.mask.ss = Lk;
    }
    P.lse = (float *)malloc((size_t)B * H * Lq * sizeof(float));
    P.delta = (float *)malloc((size_t)B * H * Lq * sizeof(float));
    int rc = fbo_fwd(&P);
    if (!rc) rc = fbo_delta(&P);
    if (!rc) rc = fbo_bwd(&P);
    double sum = 0;
    for (size_t i = 0; i < nq; ++i) sum += o[i] + dq[i];
    for (size_t i = 0; i < nk; ++i) sum += dk[i] + dv[i];
    free(q); free(k); free(v); free(dO); free(o); free(dq); free(dk); free(dv);
    free(qb); free(kb); free(dqb); free(dkb); free(mask); free(P.lse); free(P.delta);
    if (rc || sum != sum) {
        fprintf(stderr, "case B%d H%d Lq%d Lk%d d%d r%d causal%d mask%d: rc=%d sum=%f\n", B, H, Lq, Lk, d, r, causal,
                mask_type, rc, sum);
        return 1;
    }
    return 0;
}

int main(void) {
    int bad = 0;
    bad |= run_case(2, 3, 37, 37, 32, 8, 0, 0, 16, 16, 0, 0);
    bad |= run_case(1, 2, 50, 23, 20, 5, 1, 0, 16, 32, 0, 0);   /* rectangular, causal, ragged d and r */
    bad |= run_case(2, 2, 19, 70, 16, 3, 0, 1, 32, 16, 1, 0);   /* vector mask, q_bias shared by the batch */
    bad |= run_case(1, 3, 33, 33, 40, 2, 1, 2, 16, 16, 0, 1);   /* matrix mask, k_bias shared by the heads */
    bad |= run_case(1, 1, 1, 1, 8, 0, 0, 0, 16, 16, 0, 0);      /* a single pair, no factors */
    bad |= run_case(1, 2, 65, 129, 128, 16, 0, 0, 64, 64, 0, 0);
    if (!bad) puts("sanitize_check: clean");
    return bad;
}
