/*
 * CPU oracle for bitfield-masked attention, plain C.  TEST INFRASTRUCTURE ONLY:
 * it is linked or loaded by the tests, the smoke check and the benchmark's CPU
 * baseline leg, never by the shipped library.
 *
 * Every function restates, with scalar loops and double accumulation, one piece of
 * cornstarch/kernel/bitfield_attention.py of the reference; the line ranges are
 * given at each function.  Tensors are dense row-major: q/o/do/dq (B,S,Hq,D),
 * k/v/dk/dv (B,S,Hkv,D), bitfield (B,S) int64, lse/delta (B,Hq,S).
 *
 * Pins (tests/test_oracle.py): bam_oracle_allow and bam_oracle_mask against the
 * closed-form masks of the reference's own test
 * (tests/test_kernel/test_bitfield_attention.py:55-110); bam_oracle_tile_flags
 * against the analytic histogram of the 1024-token plumbing layout and the
 * context-parallel test's per-row-block counts; bam_oracle_attn_fwd against library
 * SDPA and logsumexp; bam_oracle_attn_bwd against autograd through SDPA.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define BAM_BLOCK_M 128 /* bitfield_attention.py:53 */
#define BAM_BLOCK_N 32  /* bitfield_attention.py:54 */
#define BAM_MODALITY_MASK ((((int64_t)1) << 62) - 1)

/* Allow rule for one (query, key) pair; i, j are global positions
 * (bitfield_attention.py:86-101). */
int bam_oracle_allow(int64_t bf_q, int64_t bf_k, int64_t i, int64_t j) {
    int text = (bf_q & 1) != 0;
    int64_t qb = bf_q & BAM_MODALITY_MASK;
    int64_t kb = bf_k & BAM_MODALITY_MASK;
    if (text) return (i >= j) && ((qb & kb) != 0);
    return (qb == kb) && (qb != 0);
}

static int64_t bf_at(const int64_t *bf, int64_t S, int64_t pos) {
    return (pos >= 0 && pos < S) ? bf[pos] : 0; /* :86-87 out-of-range reads 0 */
}

/* out: uint8 (B,S,S). */
void bam_oracle_mask(const int64_t *bf, int64_t B, int64_t S, uint8_t *out) {
    for (int64_t b = 0; b < B; b++)
        for (int64_t i = 0; i < S; i++)
            for (int64_t j = 0; j < S; j++)
                out[(b * S + i) * S + j] =
                    (uint8_t)bam_oracle_allow(bf[b * S + i], bf[b * S + j], i, j);
}

/* Indexed variant (context-parallel callers, bitfield_attention.py:71-81): row r of
 * the local problem is global position idx_q[r], column c is idx_k[c]; bf has
 * S_total entries per sequence.  out: uint8 (B,Sq,Sk). */
void bam_oracle_mask_indexed(const int64_t *bf, int64_t B, int64_t S_total,
                             const int64_t *idx_q, int64_t Sq, const int64_t *idx_k,
                             int64_t Sk, uint8_t *out) {
    for (int64_t b = 0; b < B; b++)
        for (int64_t r = 0; r < Sq; r++)
            for (int64_t c = 0; c < Sk; c++) {
                int64_t i = idx_q[r], j = idx_k[c];
                out[(b * Sq + r) * Sk + c] = (uint8_t)bam_oracle_allow(
                    bf_at(bf + b * S_total, S_total, i), bf_at(bf + b * S_total, S_total, j), i, j);
            }
}

/* flags: int8 (B, ceil(S/128), ceil(S/32)); 0 empty, 1 partial, 2 full over the
 * in-range cells (bitfield_attention.py:105-156). */
void bam_oracle_tile_flags(const int64_t *bf, int64_t B, int64_t S, int8_t *flags) {
    int64_t nm = (S + BAM_BLOCK_M - 1) / BAM_BLOCK_M, nn = (S + BAM_BLOCK_N - 1) / BAM_BLOCK_N;
    for (int64_t b = 0; b < B; b++)
        for (int64_t m = 0; m < nm; m++)
            for (int64_t n = 0; n < nn; n++) {
                int64_t cnt = 0;
                for (int64_t i = m * BAM_BLOCK_M; i < (m + 1) * BAM_BLOCK_M; i++)
                    for (int64_t j = n * BAM_BLOCK_N; j < (n + 1) * BAM_BLOCK_N; j++)
                        cnt += bam_oracle_allow(bf_at(bf + b * S, S, i), bf_at(bf + b * S, S, j), i, j);
                int64_t rows = ((m + 1) * BAM_BLOCK_M > S) ? S % BAM_BLOCK_M : BAM_BLOCK_M;
                int64_t cols = ((n + 1) * BAM_BLOCK_N > S) ? S % BAM_BLOCK_N : BAM_BLOCK_N;
                int8_t f = 0;
                if (cnt > 0) f = 1;
                if (cnt == rows * cols) f = 2;
                flags[(b * nm + m) * nn + n] = f;
            }
}

/* Forward (bitfield_attention.py:285-293,389-390,435-495):
 *   s_ij = scale * q_i . k_j ; lse_i = log sum_{allowed j} exp(s_ij)
 *   o_i  = sum_{allowed j} exp(s_ij - lse_i) v_j ; rows allowing nothing: o = 0, lse = -inf
 *   kv head of q head h is h / (Hq/Hkv). */
void bam_oracle_attn_fwd(const float *q, const float *k, const float *v, const int64_t *bf,
                         int64_t B, int64_t S, int64_t Hq, int64_t Hkv, int64_t D, double scale,
                         float *o, float *lse) {
    int64_t G = Hq / Hkv;
    double *s = (double *)malloc(sizeof(double) * (size_t)S);
    double *acc = (double *)malloc(sizeof(double) * (size_t)D);
    for (int64_t b = 0; b < B; b++)
        for (int64_t h = 0; h < Hq; h++) {
            int64_t hk = h / G;
            for (int64_t i = 0; i < S; i++) {
                const float *qi = q + ((b * S + i) * Hq + h) * D;
                double mx = -INFINITY;
                for (int64_t j = 0; j < S; j++) {
                    if (!bam_oracle_allow(bf[b * S + i], bf[b * S + j], i, j)) { s[j] = -INFINITY; continue; }
                    const float *kj = k + ((b * S + j) * Hkv + hk) * D;
                    double d = 0;
                    for (int64_t t = 0; t < D; t++) d += (double)qi[t] * (double)kj[t];
                    s[j] = d * scale;
                    if (s[j] > mx) mx = s[j];
                }
                float *oi = o + ((b * S + i) * Hq + h) * D;
                if (mx == -INFINITY) {
                    memset(oi, 0, sizeof(float) * (size_t)D);
                    lse[(b * Hq + h) * S + i] = -INFINITY;
                    continue;
                }
                double sum = 0;
                for (int64_t j = 0; j < S; j++) if (s[j] != -INFINITY) sum += exp(s[j] - mx);
                double l = mx + log(sum);
                for (int64_t t = 0; t < D; t++) acc[t] = 0;
                for (int64_t j = 0; j < S; j++) {
                    if (s[j] == -INFINITY) continue;
                    double p = exp(s[j] - l);
                    const float *vj = v + ((b * S + j) * Hkv + hk) * D;
                    for (int64_t t = 0; t < D; t++) acc[t] += p * (double)vj[t];
                }
                for (int64_t t = 0; t < D; t++) oi[t] = (float)acc[t];
                lse[(b * Hq + h) * S + i] = (float)l;
            }
        }
    free(s);
    free(acc);
}

/* delta[b,h,i] = sum_d o*do (bitfield_attention.py:527-572). */
void bam_oracle_delta(const float *o, const float *dout, int64_t B, int64_t S, int64_t Hq, int64_t D,
                      float *delta) {
    for (int64_t b = 0; b < B; b++)
        for (int64_t i = 0; i < S; i++)
            for (int64_t h = 0; h < Hq; h++) {
                double d = 0;
                const float *oi = o + ((b * S + i) * Hq + h) * D, *gi = dout + ((b * S + i) * Hq + h) * D;
                for (int64_t t = 0; t < D; t++) d += (double)oi[t] * (double)gi[t];
                delta[(b * Hq + h) * S + i] = (float)d;
            }
}

/* Backward (bitfield_attention.py:840-886), given o-independent inputs lse and delta:
 *   p_ij = exp(s_ij - lse_i) for allowed pairs, else 0
 *   dv_j += p_ij do_i ; dp_ij = do_i . v_j ; ds_ij = p_ij (dp_ij - delta_i) scale
 *   dk_j += ds_ij q_i ; dq_i += ds_ij k_j       (dk, dv summed over the group's q heads)
 * dq/dk/dv are ACCUMULATED INTO (caller zeroes them, :1248-1250). */
void bam_oracle_attn_bwd(const float *q, const float *k, const float *v, const float *dout,
                         const float *lse, const float *delta, const int64_t *bf, int64_t B, int64_t S,
                         int64_t Hq, int64_t Hkv, int64_t D, double scale, float *dq, float *dk,
                         float *dv) {
    int64_t G = Hq / Hkv;
    double *aq = (double *)malloc(sizeof(double) * (size_t)D);
    double *ak = (double *)calloc((size_t)(S * Hkv * D), sizeof(double));
    double *av = (double *)calloc((size_t)(S * Hkv * D), sizeof(double));
    for (int64_t b = 0; b < B; b++) {
        memset(ak, 0, sizeof(double) * (size_t)(S * Hkv * D));
        memset(av, 0, sizeof(double) * (size_t)(S * Hkv * D));
        for (int64_t h = 0; h < Hq; h++) {
            int64_t hk = h / G;
            for (int64_t i = 0; i < S; i++) {
                const float *qi = q + ((b * S + i) * Hq + h) * D;
                const float *gi = dout + ((b * S + i) * Hq + h) * D;
                double li = lse[(b * Hq + h) * S + i], di = delta[(b * Hq + h) * S + i];
                for (int64_t t = 0; t < D; t++) aq[t] = 0;
                for (int64_t j = 0; j < S; j++) {
                    if (!bam_oracle_allow(bf[b * S + i], bf[b * S + j], i, j)) continue;
                    const float *kj = k + ((b * S + j) * Hkv + hk) * D;
                    const float *vj = v + ((b * S + j) * Hkv + hk) * D;
                    double s = 0, dp = 0;
                    for (int64_t t = 0; t < D; t++) { s += (double)qi[t] * (double)kj[t]; dp += (double)gi[t] * (double)vj[t]; }
                    double p = exp(s * scale - li);
                    double ds = p * (dp - di) * scale;
                    double *akj = ak + (j * Hkv + hk) * D, *avj = av + (j * Hkv + hk) * D;
                    for (int64_t t = 0; t < D; t++) {
                        avj[t] += p * (double)gi[t];
                        akj[t] += ds * (double)qi[t];
                        aq[t] += ds * (double)kj[t];
                    }
                }
                float *dqi = dq + ((b * S + i) * Hq + h) * D;
                for (int64_t t = 0; t < D; t++) dqi[t] += (float)aq[t];
            }
        }
        for (int64_t x = 0; x < S * Hkv * D; x++) {
            dk[b * S * Hkv * D + x] += (float)ak[x];
            dv[b * S * Hkv * D + x] += (float)av[x];
        }
    }
    free(aq);
    free(ak);
    free(av);
}
