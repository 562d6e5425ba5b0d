/* Plain-C fp64 restatement of the attention hot path and its dropout generator.
 * TEST INFRASTRUCTURE ONLY: nothing shipped links or loads this file.
 *
 * Follows, in the reference:
 *   forward semantics     trident/kernel/attention.py:115-165 (online softmax collapsed to the
 *                         two-pass form; causal rule row >= col :131-134; additive mask :135-138)
 *   saved statistic       trident/kernel/attention.py:164 (log2 domain)
 *   delta pre-pass        trident/kernel/softmax.py:223-238
 *   backward closed forms trident/kernel/attention.py:304-333
 *   comparison contract   tests/test_attention.py:22-84
 * Not followed: low-precision accumulators, dropout-on-O (see oracle/attention.py).
 *
 * Philox4x32-10: Random123 (Salmon et al. 2011), the generator behind tl.rand at
 * trident/kernel/attention.py:159; pinned by the Random123 known-answer vectors.
 * Layout per head: q,k,v,o,do,dq,dk,dv [S][D] row-major doubles; mask/dmask [S][S] or NULL.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>

void oracle_philox4x32_10(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4]) {
    uint32_t c0 = ctr[0], c1 = ctr[1], c2 = ctr[2], c3 = ctr[3];
    uint32_t k0 = key[0], k1 = key[1];
    for (int r = 0; r < 10; ++r) {
        uint64_t p0 = (uint64_t)0xD2511F53u * c0;
        uint64_t p1 = (uint64_t)0xCD9E8D57u * c2;
        uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0;
        uint32_t n1 = (uint32_t)p1;
        uint32_t n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
        uint32_t n3 = (uint32_t)p0;
        c0 = n0; c1 = n1; c2 = n2; c3 = n3;
        k0 += 0x9E3779B9u;
        k1 += 0xBB67AE85u;
    }
    out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}

/* keep decision for element (bh, i, j); thr8 in [0,256] */
int oracle_dropout_keep(uint64_t seed, uint32_t offset, uint32_t bh, uint32_t i, uint32_t j, int thr8) {
    uint32_t ctr[4] = {j >> 2, i >> 2, bh, offset};
    uint32_t key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
    uint32_t r[4];
    oracle_philox4x32_10(ctr, key, r);
    int u8 = (int)((r[i & 3] >> (8 * (j & 3))) & 0xffu);
    return u8 >= thr8;
}

void oracle_dropout_mask(uint64_t seed, uint32_t offset, uint32_t bh, int S, int thr8, uint8_t* keep) {
    for (int i = 0; i < S; ++i)
        for (int j = 0; j < S; ++j)
            keep[(size_t)i * S + j] = (uint8_t)oracle_dropout_keep(seed, offset, bh, (uint32_t)i, (uint32_t)j, thr8);
}

/* probabilities of one row i into p[0..S): returns natural-log LSE */
static double row_softmax(const double* q, const double* k, const double* mask, int S, int D, int i,
                          int causal, double scale, double* p) {
    double m = -INFINITY;
    for (int j = 0; j < S; ++j) {
        double s;
        if (causal && j > i) {
            s = -INFINITY;
        } else {
            s = 0.0;
            for (int d = 0; d < D; ++d) s += q[(size_t)i * D + d] * k[(size_t)j * D + d];
            s *= scale;
            if (mask && !causal) s += mask[(size_t)i * S + j];
        }
        p[j] = s;
        if (s > m) m = s;
    }
    double ms = isfinite(m) ? m : 0.0;
    double l = 0.0;
    for (int j = 0; j < S; ++j) { p[j] = exp(p[j] - ms); l += p[j]; }
    for (int j = 0; j < S; ++j) p[j] /= l;
    return ms + log(l);
}

/* one head forward; thr8 == 0 disables dropout */
void oracle_attn_fwd_head(const double* q, const double* k, const double* v, const double* mask,
                          int S, int D, int causal, double scale,
                          uint64_t seed, uint32_t offset, uint32_t bh, int thr8,
                          double* o, double* lse2) {
    double* p = (double*)malloc(sizeof(double) * (size_t)S);
    double zs = thr8 >= 256 ? 0.0 : 256.0 / (256.0 - thr8);
    for (int i = 0; i < S; ++i) {
        double lse = row_softmax(q, k, mask, S, D, i, causal, scale, p);
        lse2[i] = lse * 1.4426950408889634;
        for (int d = 0; d < D; ++d) o[(size_t)i * D + d] = 0.0;
        for (int j = 0; j < S; ++j) {
            double w = p[j];
            if (thr8 > 0) w *= oracle_dropout_keep(seed, offset, bh, (uint32_t)i, (uint32_t)j, thr8) ? zs : 0.0;
            if (w == 0.0) continue;
            for (int d = 0; d < D; ++d) o[(size_t)i * D + d] += w * v[(size_t)j * D + d];
        }
    }
    free(p);
}

/* one head backward; o is the forward output of the same call; dmask may be NULL */
void oracle_attn_bwd_head(const double* q, const double* k, const double* v, const double* mask,
                          const double* o, const double* d_o,
                          int S, int D, int causal, double scale,
                          uint64_t seed, uint32_t offset, uint32_t bh, int thr8,
                          double* dq, double* dk, double* dv, double* dmask, double* delta) {
    double* p = (double*)malloc(sizeof(double) * (size_t)S);
    double zs = thr8 >= 256 ? 0.0 : 256.0 / (256.0 - thr8);
    for (size_t n = 0; n < (size_t)S * D; ++n) { dq[n] = 0.0; dk[n] = 0.0; dv[n] = 0.0; }
    for (int i = 0; i < S; ++i) {
        row_softmax(q, k, mask, S, D, i, causal, scale, p);
        double dl = 0.0;
        for (int d = 0; d < D; ++d) dl += d_o[(size_t)i * D + d] * o[(size_t)i * D + d];
        delta[i] = dl;
        for (int j = 0; j < S; ++j) {
            double z = 1.0;
            if (thr8 > 0) z = oracle_dropout_keep(seed, offset, bh, (uint32_t)i, (uint32_t)j, thr8) ? zs : 0.0;
            double dp = 0.0;
            for (int d = 0; d < D; ++d) dp += d_o[(size_t)i * D + d] * v[(size_t)j * D + d];
            dp *= z;
            double ds = p[j] * (dp - dl);
            double pz = p[j] * z;
            for (int d = 0; d < D; ++d) {
                dv[(size_t)j * D + d] += pz * d_o[(size_t)i * D + d];
                dq[(size_t)i * D + d] += scale * ds * k[(size_t)j * D + d];
                dk[(size_t)j * D + d] += scale * ds * q[(size_t)i * D + d];
            }
            if (dmask) dmask[(size_t)i * S + j] = ds;
        }
    }
    free(p);
}
