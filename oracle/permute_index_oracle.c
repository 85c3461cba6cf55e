/* CPU oracle for the integer part of the MoE token permute.  TEST
 * INFRASTRUCTURE ONLY: loaded by the test-suite and the smoke check through
 * ctypes, never by the product library.
 *
 * Restates mindspeed/core/transformer/moe/moe_utils.py:204-206 (flatten the
 * [T,k] expert ids token-major and stable-sort them) as a counting sort, the
 * unique stable order for integer keys:
 *
 *   forward[r]  = flat position t*k+j that lands in output row r
 *                 (the torch path's sorted_indices, moe_utils.py:206)
 *   inverse[i]  = output row of flat position i (the fused op's full-length
 *                 int32 map, mindspeed/ops/csrc/cann/
 *                 npu_moe_token_permute.cpp:81-85)
 *   counts[e]   = rows owned by expert e (tokens_per_expert)
 *
 * Pinned by tests against numpy.argsort(kind="stable"), a brute-force
 * sorted() and the torch restatement.
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

int ms_oracle_permute_index(const int64_t *flat, int64_t n, int64_t num_experts,
                            int32_t *forward, int32_t *inverse, int64_t *counts)
{
    if (n < 0 || num_experts <= 0) return 1;
    int64_t *offset = (int64_t *)calloc((size_t)num_experts + 1, sizeof(int64_t));
    if (!offset) return 2;
    for (int64_t i = 0; i < n; ++i) {
        if (flat[i] < 0 || flat[i] >= num_experts) { free(offset); return 3; }
        offset[flat[i] + 1]++;
    }
    if (counts) memcpy(counts, offset + 1, (size_t)num_experts * sizeof(int64_t));
    for (int64_t e = 0; e < num_experts; ++e) offset[e + 1] += offset[e];
    for (int64_t i = 0; i < n; ++i) {          /* ascending i => stable */
        int64_t r = offset[flat[i]]++;
        if (forward) forward[r] = (int32_t)i;
        if (inverse) inverse[i] = (int32_t)r;
    }
    free(offset);
    return 0;
}

/* Row gather of the permute: out[r] = tokens[forward[r] / k] for r < num_out
 * (moe_utils.py:207-209).  Rows are opaque byte strings of row_bytes. */
int ms_oracle_permute_rows(const unsigned char *tokens, const int32_t *forward,
                           int64_t num_out, int64_t topk, int64_t row_bytes,
                           unsigned char *out)
{
    if (topk <= 0) return 1;
    for (int64_t r = 0; r < num_out; ++r)
        memcpy(out + r * row_bytes, tokens + (int64_t)(forward[r] / topk) * row_bytes,
               (size_t)row_bytes);
    return 0;
}
