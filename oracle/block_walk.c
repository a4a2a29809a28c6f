/*
 * Scalar CPU restatement of the reference's scalar kernel
 * omni_attn_simple_kernel_impl (omni-attn-mma/mma/attn_naive.cu:21-302).
 * TEST INFRASTRUCTURE ONLY: never linked into or called by the product.
 *
 * One loop iteration per query row, two passes over the listed KV blocks (row max,
 * then exp / sum / weighted V), everything in fp32 -- the structure of the reference
 * kernel, with the inputs given as fp32 values (already rounded to the 16-bit type
 * under test by the caller).  Also returns the natural-log logsumexp of each row,
 * which the reference does not have (-inf for rows with no allowed key).
 *
 * Build: gcc -O2 -fopenmp -shared -fPIC block_walk.c -o _build/libomni_oracle.so -lm
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>

#define BLOCK_MASK_MASKED 0  /* attn_naive.cu:4-7 */
#define BLOCK_MASK_CAUSAL 1
#define BLOCK_MASK_FULL 2
#define BLOCK_MASK_PARTIAL 3

static int imin(int a, int b) { return a < b ? a : b; }

/* Visit every allowed key of row q_idx; pass 0 finds the max, pass 1 accumulates. */
static void walk_row(const float* Q, const float* K, const float* V, float* out, float* max_score,
                     float* sum_exp, int pass, const int32_t* kv_indices, const int32_t* types,
                     const int32_t* partial_idx, const uint8_t* partial_masks, int num_partial,
                     int kv_nb, int q_idx, int q_block, int QB, int KB, int seqlen_orig, int D) {
  const float scale = 1.0f / sqrtf((float)D); /* attn_naive.cu:88 */
  const float* qrow = Q + (size_t)q_idx * D;
  for (int s = 0; s < kv_nb; ++s) {
    const int kv_block = kv_indices[s];
    const int mask_type = types[s];
    if (mask_type == BLOCK_MASK_MASKED) continue; /* :108-110 */
    if (mask_type != BLOCK_MASK_CAUSAL && mask_type != BLOCK_MASK_FULL &&
        mask_type != BLOCK_MASK_PARTIAL)
      continue;
    const int kv_start = kv_block * KB;
    int kv_end = imin(kv_start + KB, seqlen_orig); /* :113 */
    int pid = -1;
    if (mask_type == BLOCK_MASK_PARTIAL) { /* :119-131 */
      if (!partial_idx || !partial_masks) continue;
      pid = partial_idx[s];
      if (pid < 0) continue;
      /* the reference reads any index unchecked; the product's contract is that an index
       * beyond the stored tiles means "no bits stored", like a negative one */
      if (pid >= num_partial) continue;
    }
    if (mask_type == BLOCK_MASK_CAUSAL) { /* :134-140 */
      if (q_idx < kv_start) continue;
      kv_end = imin(kv_end, q_idx + 1);
    }
    for (int kv = kv_start; kv < kv_end; ++kv) {
      if (mask_type == BLOCK_MASK_PARTIAL) { /* :143-154 */
        const int local_q = q_idx - q_block * QB;
        const int local_kv = kv - kv_block * KB;
        if (!partial_masks[(size_t)pid * QB * KB + (size_t)local_q * KB + local_kv]) continue;
      }
      const float* krow = K + (size_t)kv * D;
      float score = 0.0f;
      for (int d = 0; d < D; ++d) score += qrow[d] * krow[d];
      score *= scale;
      if (pass == 0) {
        if (score > *max_score) *max_score = score;
      } else {
        const float w = expf(score - *max_score); /* :270-272 */
        *sum_exp += w;
        const float* vrow = V + (size_t)kv * D;
        for (int d = 0; d < D; ++d) out[d] += w * vrow[d];
      }
    }
  }
}

/*
 * q, k, v, o: [B, H, S, D] fp32; lse: [B, H, S] fp32; metadata as in the product ABI
 * (partial_idx indexed like block_mask_types, attn_naive.cu:124-127).
 * Returns 0, or -1 on a bad argument.
 */
int omni_oracle_block_walk(const float* q, const float* k, const float* v, float* o, float* lse,
                           const int32_t* kv_num_blocks, const int32_t* kv_indices,
                           const int32_t* block_mask_types, const int32_t* partial_idx,
                           const uint8_t* partial_masks, int B, int H, int S, int D, int Tq,
                           int max_blocks, int QB, int KB, int num_partial, int seqlen_orig) {
  if (!q || !k || !v || !o || !lse || !kv_num_blocks || !kv_indices || !block_mask_types) return -1;
  if (B <= 0 || H <= 0 || S <= 0 || D <= 0 || D > 256 || Tq <= 0 || max_blocks <= 0) return -1;
  if (seqlen_orig > S) seqlen_orig = S;
  const long total = (long)B * H * S;
#pragma omp parallel for schedule(dynamic, 16)
  for (long row = 0; row < total; ++row) {
    const int q_idx = (int)(row % S);
    const long bh = row / S;
    const size_t slab = (size_t)bh * S * D;
    float* orow = o + slab + (size_t)q_idx * D;
    for (int d = 0; d < D; ++d) orow[d] = 0.0f;
    lse[row] = -INFINITY;
    if (q_idx >= seqlen_orig) continue; /* padding row: zeros, :64-72 */
    int q_block = q_idx / QB;
    if (q_block >= Tq) q_block = Tq - 1; /* :75-78 */
    const size_t mrow = (size_t)bh * Tq + q_block;
    int kv_nb = kv_num_blocks[mrow];
    if (kv_nb > max_blocks) kv_nb = max_blocks;
    const int32_t* idx = kv_indices + mrow * max_blocks;
    const int32_t* tys = block_mask_types + mrow * max_blocks;
    const int32_t* pidx = partial_idx ? partial_idx + mrow * max_blocks : 0;
    float max_score = -INFINITY, sum_exp = 0.0f;
    float acc[256];
    for (int d = 0; d < D; ++d) acc[d] = 0.0f;
    walk_row(q + slab, k + slab, v + slab, acc, &max_score, &sum_exp, 0, idx, tys, pidx,
             partial_masks, num_partial, kv_nb, q_idx, q_block, QB, KB, seqlen_orig, D);
    if (max_score == -INFINITY) continue; /* everything masked: zeros, :177-183 */
    walk_row(q + slab, k + slab, v + slab, acc, &max_score, &sum_exp, 1, idx, tys, pidx,
             partial_masks, num_partial, kv_nb, q_idx, q_block, QB, KB, seqlen_orig, D);
    if (sum_exp <= 0.0f) continue; /* :283-288 */
    const float inv = 1.0f / sum_exp;
    for (int d = 0; d < D; ++d) orow[d] = acc[d] * inv;
    lse[row] = max_score + logf(sum_exp);
  }
  return 0;
}
