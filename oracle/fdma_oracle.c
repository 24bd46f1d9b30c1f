/*
 * TEST INFRASTRUCTURE ONLY -- CPU restatement of the dynamic-mask attention hot path.
 *
 * This file is the parity checker for the HIP kernels.  It is never linked into, called from
 * or shipped with the product library; only tests, the smoke check and the benchmark's CPU
 * baseline leg may load it.
 *
 * Algorithm restated (reference citations, paths relative to the reference checkout):
 *   forward   S = (Q K^T) * scale + bias ; S[~mask] = -inf ; P = softmax(S) ; O = P V
 *             benchmarks/forward_equivalence.py:117-124 (GQA expand :113-115, :55-67)
 *   causal    bottom-right aligned, key j visible to query i iff j <= i + Lk - Lq
 *             csrc/flash_sparse_attn/src/mask.h:39 ; flash_sparse_attn_interface.py:633-642
 *   empty row O = 0, LSE = +inf   csrc/flash_sparse_attn/src/softmax.h:210-214 ;
 *             flash_sparse_attn_interface.py:643
 *   LSE       log sum exp of the masked scores, natural log
 *             csrc/flash_sparse_attn/src/softmax.h:201-220
 *   backward  autograd of the same formula: benchmarks/backward_equivalence.py:123-135, i.e.
 *             dP = dO V^T ; D = rowsum(dO * O) ; dS = P * (dP - D) ; dQ = scale dS K ;
 *             dK = scale dS^T Q ; dV = P^T dO ; dBias = dS
 *             csrc/flash_sparse_attn/src/flash_bwd_kernel.h:764-790, 909-957, 1069-1070
 *   GQA       query head h uses kv head h / (H/Hkv); mask/bias head h / (H/Hm)
 *             csrc/flash_sparse_attn/src/flash_fwd_kernel.h:158, 178, 188
 *   dK,dV     summed over the query heads of a group; dBias summed over every broadcast
 *             dim of the bias  csrc/flash_sparse_attn/flash_api.cpp:1027-1047
 *
 * Pinning: checked in tests/test_oracle.py against closed forms (torch softmax / matmul /
 * scaled_dot_product_attention), a brute-force per-row gather, the literal causal matrices of
 * the reference docstring, invariances (bias row shift, key permutation, rows of P sum to 1),
 * torch autograd of the closed form and fp64 finite differences.
 *
 * All arithmetic is IEEE double on float inputs.  Tensors are dense row-major:
 *   q, out, dout, dq : [B, Lq, H, D]        k, v, dk, dv : [B, Lk, Hk, D]
 *   mask (uint8 0/1) : [mb, mh, mq, mk]     bias, dbias   : [bb, bh, bq, bk]
 * where each of mb/bb in {1,B}, mh/bh in {1,Hk,H}, mq/bq in {1,Lq}, mk/bk in {1,Lk};
 * a NULL mask or bias means "absent".
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

typedef struct {
    int32_t b, lq, lk, h, hk, d;
    int32_t mb, mh, mq, mk; /* mask dims  */
    int32_t bb, bh, bq, bk; /* bias dims  */
    float scale;
    int32_t causal;
} fdma_oracle_shape;

static inline size_t bcast_index(int dim_b, int dim_h, int dim_q, int dim_k, int B, int H, int Hk,
                                 int b, int h, int i, int j, int Lq, int Lk) {
    (void)B; (void)Lq; (void)Lk;
    int ib = dim_b == 1 ? 0 : b;
    int ih = dim_h == 1 ? 0 : (dim_h == H ? h : h / (H / dim_h));
    (void)Hk;
    int iq = dim_q == 1 ? 0 : i;
    int ik = dim_k == 1 ? 0 : j;
    return (((size_t)ib * dim_h + ih) * dim_q + iq) * dim_k + ik;
}

static inline int visible(const fdma_oracle_shape *s, const uint8_t *mask, int b, int h, int i, int j) {
    if (s->causal && j > i + s->lk - s->lq) return 0;
    if (mask) {
        size_t idx = bcast_index(s->mb, s->mh, s->mq, s->mk, s->b, s->h, s->hk, b, h, i, j, s->lq, s->lk);
        if (!mask[idx]) return 0;
    }
    return 1;
}

/* scores of row (b,h,i) into sc[0..lk) ; returns number of visible keys; masked entries = -INFINITY */
static int row_scores(const fdma_oracle_shape *s, const float *q, const float *k, const uint8_t *mask,
                      const float *bias, int b, int h, int i, double *sc) {
    int hk = h / (s->h / s->hk);
    const float *qr = q + (((size_t)b * s->lq + i) * s->h + h) * s->d;
    int n = 0;
    for (int j = 0; j < s->lk; j++) {
        if (!visible(s, mask, b, h, i, j)) { sc[j] = -INFINITY; continue; }
        const float *kr = k + (((size_t)b * s->lk + j) * s->hk + hk) * s->d;
        double acc = 0.0;
        for (int t = 0; t < s->d; t++) acc += (double)qr[t] * (double)kr[t];
        acc *= (double)s->scale;
        if (bias) acc += (double)bias[bcast_index(s->bb, s->bh, s->bq, s->bk, s->b, s->h, s->hk, b, h, i, j, s->lq, s->lk)];
        sc[j] = acc;
        n++;
    }
    return n;
}

/* returns lse (natural log); converts sc to probabilities in place; empty row -> +inf, p = 0 */
static double row_softmax(int lk, int nvis, double *sc) {
    if (nvis == 0) { for (int j = 0; j < lk; j++) sc[j] = 0.0; return INFINITY; }
    double mx = -INFINITY;
    for (int j = 0; j < lk; j++) if (sc[j] > mx) mx = sc[j];
    double sum = 0.0;
    for (int j = 0; j < lk; j++) { sc[j] = (sc[j] == -INFINITY) ? 0.0 : exp(sc[j] - mx); sum += sc[j]; }
    for (int j = 0; j < lk; j++) sc[j] /= sum;
    return mx + log(sum);
}

int fdma_oracle_fwd(const fdma_oracle_shape *s, const float *q, const float *k, const float *v,
                    const uint8_t *mask, const float *bias, float *out, float *lse) {
    if (s->h % s->hk) return -1;
    long rows = (long)s->b * s->h * s->lq;
#pragma omp parallel
    {
        double *sc = (double *)malloc(sizeof(double) * (size_t)(s->lk > 0 ? s->lk : 1));
        double *o = (double *)malloc(sizeof(double) * (size_t)s->d);
#pragma omp for schedule(dynamic, 16)
        for (long r = 0; r < rows; r++) {
            int i = (int)(r % s->lq); int h = (int)((r / s->lq) % s->h); int b = (int)(r / ((long)s->lq * s->h));
            int hk = h / (s->h / s->hk);
            int n = row_scores(s, q, k, mask, bias, b, h, i, sc);
            double l = row_softmax(s->lk, n, sc);
            for (int t = 0; t < s->d; t++) o[t] = 0.0;
            for (int j = 0; j < s->lk; j++) {
                if (sc[j] == 0.0) continue;
                const float *vr = v + (((size_t)b * s->lk + j) * s->hk + hk) * s->d;
                for (int t = 0; t < s->d; t++) o[t] += sc[j] * (double)vr[t];
            }
            float *orow = out + (((size_t)b * s->lq + i) * s->h + h) * s->d;
            for (int t = 0; t < s->d; t++) orow[t] = (float)o[t];
            if (lse) lse[((size_t)b * s->h + h) * s->lq + i] = (float)l; /* [B,H,Lq] */
        }
        free(sc); free(o);
    }
    return 0;
}

int fdma_oracle_bwd(const fdma_oracle_shape *s, const float *q, const float *k, const float *v,
                    const uint8_t *mask, const float *bias, const float *dout,
                    float *dq, float *dk, float *dv, float *dbias) {
    if (s->h % s->hk) return -1;
    const int G = s->h / s->hk;
    long rows = (long)s->b * s->h * s->lq;
    double *LSE = (double *)malloc(sizeof(double) * (size_t)(rows > 0 ? rows : 1));
    double *Dv = (double *)malloc(sizeof(double) * (size_t)(rows > 0 ? rows : 1));
    /* pass 1: row statistics and dQ (each row owned by one thread) */
#pragma omp parallel
    {
        double *sc = (double *)malloc(sizeof(double) * (size_t)(s->lk > 0 ? s->lk : 1));
        double *acc = (double *)malloc(sizeof(double) * (size_t)s->d);
#pragma omp for schedule(dynamic, 16)
        for (long r = 0; r < rows; r++) {
            int i = (int)(r % s->lq); int h = (int)((r / s->lq) % s->h); int b = (int)(r / ((long)s->lq * s->h));
            int hk = h / G;
            int n = row_scores(s, q, k, mask, bias, b, h, i, sc);
            double l = row_softmax(s->lk, n, sc);
            const float *dor = dout + (((size_t)b * s->lq + i) * s->h + h) * s->d;
            /* D = sum_j p_j dP_j = dO . O */
            double Dsum = 0.0;
            for (int j = 0; j < s->lk; j++) {
                if (sc[j] == 0.0) continue;
                const float *vr = v + (((size_t)b * s->lk + j) * s->hk + hk) * s->d;
                double dp = 0.0;
                for (int t = 0; t < s->d; t++) dp += (double)dor[t] * (double)vr[t];
                Dsum += sc[j] * dp;
            }
            for (int t = 0; t < s->d; t++) acc[t] = 0.0;
            for (int j = 0; j < s->lk; j++) {
                if (sc[j] == 0.0) continue;
                const float *vr = v + (((size_t)b * s->lk + j) * s->hk + hk) * s->d;
                const float *kr = k + (((size_t)b * s->lk + j) * s->hk + hk) * s->d;
                double dp = 0.0;
                for (int t = 0; t < s->d; t++) dp += (double)dor[t] * (double)vr[t];
                double ds = sc[j] * (dp - Dsum);
                for (int t = 0; t < s->d; t++) acc[t] += ds * (double)kr[t];
            }
            float *dqr = dq + (((size_t)b * s->lq + i) * s->h + h) * s->d;
            for (int t = 0; t < s->d; t++) dqr[t] = (float)(acc[t] * (double)s->scale);
            LSE[r] = l; Dv[r] = Dsum;
        }
        free(sc); free(acc);
    }
    /* pass 2: dK, dV, dBias; every key column j owned by one thread */
    size_t nb = bias ? (size_t)s->bb * s->bh * s->bq * s->bk : 0;
    double *dbacc = nb ? (double *)calloc(nb, sizeof(double)) : NULL;
    int bk1 = bias && s->bk == 1;  /* key-broadcast bias: every column adds to the same element */
#pragma omp parallel
    {
        double *ak = (double *)malloc(sizeof(double) * (size_t)s->d);
        double *av = (double *)malloc(sizeof(double) * (size_t)s->d);
#pragma omp for schedule(dynamic, 4)
        for (int j = 0; j < s->lk; j++) {
            for (int b = 0; b < s->b; b++) for (int hk = 0; hk < s->hk; hk++) {
                const float *kr = k + (((size_t)b * s->lk + j) * s->hk + hk) * s->d;
                const float *vr = v + (((size_t)b * s->lk + j) * s->hk + hk) * s->d;
                for (int t = 0; t < s->d; t++) { ak[t] = 0.0; av[t] = 0.0; }
                for (int g = 0; g < G; g++) {
                    int h = hk * G + g;
                    for (int i = 0; i < s->lq; i++) {
                        if (!visible(s, mask, b, h, i, j)) continue;
                        long r = ((long)b * s->h + h) * s->lq + i;
                        const float *qr = q + (((size_t)b * s->lq + i) * s->h + h) * s->d;
                        const float *dor = dout + (((size_t)b * s->lq + i) * s->h + h) * s->d;
                        double sc = 0.0, dp = 0.0;
                        for (int t = 0; t < s->d; t++) { sc += (double)qr[t] * (double)kr[t]; dp += (double)dor[t] * (double)vr[t]; }
                        sc *= (double)s->scale;
                        size_t bi = 0;
                        if (bias) { bi = bcast_index(s->bb, s->bh, s->bq, s->bk, s->b, s->h, s->hk, b, h, i, j, s->lq, s->lk); sc += (double)bias[bi]; }
                        double p = exp(sc - LSE[r]);
                        double ds = p * (dp - Dv[r]);
                        for (int t = 0; t < s->d; t++) { av[t] += p * (double)dor[t]; ak[t] += ds * (double)qr[t]; }
                        if (bias) {
                            if (bk1) {
#pragma omp atomic
                                dbacc[bi] += ds;
                            } else dbacc[bi] += ds;
                        }
                    }
                }
                float *dkr = dk + (((size_t)b * s->lk + j) * s->hk + hk) * s->d;
                float *dvr = dv + (((size_t)b * s->lk + j) * s->hk + hk) * s->d;
                for (int t = 0; t < s->d; t++) { dkr[t] = (float)(ak[t] * (double)s->scale); dvr[t] = (float)av[t]; }
            }
        }
        free(ak); free(av);
    }
    if (dbias) for (size_t t = 0; t < nb; t++) dbias[t] = (float)dbacc[t];
    free(dbacc); free(LSE); free(Dv);
    return 0;
}

/* LSE-weighted merge of split partial results: flash_fwd_kernel.h:1695-1782.
 * o_part [S, R, D], lse_part [S, R] -> o [R, D], lse [R]; an empty split carries lse = -inf. */
int fdma_oracle_combine(int nsplit, long rows, int d, const float *o_part, const float *lse_part,
                        float *o, float *lse) {
    for (long r = 0; r < rows; r++) {
        double mx = -INFINITY;
        for (int s = 0; s < nsplit; s++) { double l = lse_part[(size_t)s * rows + r]; if (l > mx) mx = l; }
        if (mx == -INFINITY) { for (int t = 0; t < d; t++) o[r * d + t] = 0.f; lse[r] = INFINITY; continue; }
        double sum = 0.0;
        for (int s = 0; s < nsplit; s++) sum += exp((double)lse_part[(size_t)s * rows + r] - mx);
        double L = mx + log(sum);
        for (int t = 0; t < d; t++) {
            double acc = 0.0;
            for (int s = 0; s < nsplit; s++) {
                double l = lse_part[(size_t)s * rows + r];
                if (l == -INFINITY) continue;
                acc += exp(l - L) * (double)o_part[((size_t)s * rows + r) * d + t];
            }
            o[r * d + t] = (float)acc;
        }
        lse[r] = (float)L;
    }
    return 0;
}
