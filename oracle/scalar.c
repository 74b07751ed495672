/*
 * Plain-C, double-precision, loop-per-element CPU oracle for the block-sparse
 * attention forward.  TEST INFRASTRUCTURE ONLY: the product (hbsattn_amd/) never
 * links or loads this file; tests/, the smoke check and bench.py's cpu_baseline
 * leg use it as the checker.
 *
 * It restates the semantics of the reference's golden implementation
 *   hbsattn/reference.py:23-107  (in-sequence mask :56-60, bottom-right causal
 *   :64-77, block-mask lookup :80-87, softmax over keys :92-95, rows with no
 *   visible key -> 0 :97-98, PV :100)
 * and the block geometry of hbsattn/utils.py:7-50, but derives the geometry from
 * first principles: a token at in-sequence position p of sequence b lies in global
 * block  (sum over earlier sequences of ceil(len/bs)) + p / bs.  It never reads a
 * cu_block / block_to_batch array, so agreement with oracle/dense.py (which goes
 * through calculate_blocks_oracle) also cross-checks that function.
 *
 * Pinned by tests/test_oracle_cross.py (agreement with oracle/dense.py) and
 * tests/test_oracle_dense.py (SDPA reductions run against both).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#ifdef _OPENMP
#include <omp.h>
#endif

static int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

/* hbsattn/utils.py:7-50: returns num_block; fills cu_block[nb+1], block_to_batch[nb],
 * cu_num_block[batch+1].  Pass NULL outputs to only count. */
int64_t hbsa_oracle_calculate_blocks(const int32_t *cu_seqlen, int32_t batch, int32_t block_size,
                                     int32_t *cu_block, int32_t *block_to_batch, int32_t *cu_num_block)
{
    int64_t nb = 0;
    if (cu_block) cu_block[0] = 0;
    if (cu_num_block) cu_num_block[0] = 0;
    for (int32_t b = 0; b < batch; ++b) {
        int64_t len = (int64_t)cu_seqlen[b + 1] - cu_seqlen[b];
        int64_t n = ceil_div(len, block_size);
        for (int64_t t = 0; t < n; ++t) {
            int64_t end = cu_seqlen[b] + (t + 1) * (int64_t)block_size;
            if (end > cu_seqlen[b + 1]) end = cu_seqlen[b + 1];
            if (cu_block) cu_block[nb + 1] = (int32_t)end;
            if (block_to_batch) block_to_batch[nb] = b;
            ++nb;
        }
        if (cu_num_block) cu_num_block[b + 1] = (int32_t)nb;
    }
    return nb;
}

/*
 * q   [total_q, nhead_q, headdim] float32 contiguous (bf16 inputs are widened exactly by the caller)
 * k,v [total_k, nhead_k, headdim]
 * block_mask [nhead_k, num_q_block, num_k_block] bytes (0 / non-0), global block indices
 * out [total_q, nhead_q, headdim] float32
 * row_begin/row_end: restrict to global query rows [row_begin, row_end) (others untouched).
 * Returns 0, or -1 on a geometry mismatch.
 */
int hbsa_oracle_fwd(const float *q, const float *k, const float *v, float *out,
                    const int32_t *cu_q, const int32_t *cu_k, const uint8_t *block_mask,
                    int32_t batch, int32_t nhead_q, int32_t nhead_k, int32_t headdim,
                    int32_t num_q_block, int32_t num_k_block,
                    int32_t q_block_size, int32_t k_block_size, int32_t causal, double softmax_scale,
                    int64_t row_begin, int64_t row_end)
{
    if (nhead_k <= 0 || nhead_q % nhead_k != 0) return -1;
    const int32_t ratio = nhead_q / nhead_k;
    int64_t qb_base = 0, kb_base = 0, max_klen = 0;
    for (int32_t b = 0; b < batch; ++b) {
        int64_t kl = (int64_t)cu_k[b + 1] - cu_k[b];
        if (kl > max_klen) max_klen = kl;
    }
    int status = 0;
    for (int32_t b = 0; b < batch; ++b) {
        const int64_t q0 = cu_q[b], qlen = (int64_t)cu_q[b + 1] - q0;
        const int64_t k0 = cu_k[b], klen = (int64_t)cu_k[b + 1] - k0;
        const int64_t shift = klen - qlen; /* bottom-right alignment */
        const int64_t qb0 = qb_base, kb0 = kb_base;
        if (qb0 + ceil_div(qlen, q_block_size) > num_q_block || kb0 + ceil_div(klen, k_block_size) > num_k_block) {
            status = -1;
            break;
        }
#pragma omp parallel
        {
            double *score = (double *)malloc(sizeof(double) * (size_t)(max_klen > 0 ? max_klen : 1));
            double *acc = (double *)malloc(sizeof(double) * (size_t)headdim);
#pragma omp for schedule(dynamic, 4) collapse(2)
            for (int64_t i = 0; i < qlen; ++i) {
                for (int32_t h = 0; h < nhead_q; ++h) {
                    const int64_t row = q0 + i;
                    if (row < row_begin || row >= row_end) continue;
                    const int32_t hk = h / ratio;
                    const int64_t qblk = qb0 + i / q_block_size;
                    const uint8_t *mrow = block_mask + ((int64_t)hk * num_q_block + qblk) * num_k_block;
                    const float *qv = q + (row * nhead_q + h) * (int64_t)headdim;
                    double best = -INFINITY;
                    for (int64_t j = 0; j < klen; ++j) {
                        int visible = mrow[kb0 + j / k_block_size] != 0;
                        if (causal && i + shift < j) visible = 0;
                        if (!visible) { score[j] = -INFINITY; continue; }
                        const float *kv = k + ((k0 + j) * nhead_k + hk) * (int64_t)headdim;
                        double s = 0.0;
                        for (int32_t d = 0; d < headdim; ++d) s += (double)qv[d] * (double)kv[d];
                        s *= softmax_scale;
                        score[j] = s;
                        if (s > best) best = s;
                    }
                    float *o = out + (row * nhead_q + h) * (int64_t)headdim;
                    for (int32_t d = 0; d < headdim; ++d) acc[d] = 0.0;
                    double denom = 0.0;
                    if (best > -INFINITY) {
                        for (int64_t j = 0; j < klen; ++j) {
                            if (score[j] == -INFINITY) continue;
                            const double p = exp(score[j] - best);
                            denom += p;
                            const float *vv = v + ((k0 + j) * nhead_k + hk) * (int64_t)headdim;
                            for (int32_t d = 0; d < headdim; ++d) acc[d] += p * (double)vv[d];
                        }
                    }
                    for (int32_t d = 0; d < headdim; ++d) o[d] = denom > 0.0 ? (float)(acc[d] / denom) : 0.0f;
                }
            }
            free(score);
            free(acc);
        }
        qb_base += ceil_div(qlen, q_block_size);
        kb_base += ceil_div(klen, k_block_size);
    }
    return status;
}

int hbsa_oracle_max_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
