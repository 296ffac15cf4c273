/* CPU oracle for the routing segment pass.  TEST INFRASTRUCTURE ONLY: it is the checker for the
 * HIP kernels (tests/, the smoke check and the benchmark's CPU-baseline leg), never the product.
 *
 * Plain-C restatement of
 *   launch_count  + count_tokens_vectorized   hexa_moe_cuda/hexa_moe/kernels/shared_cuda_core.cu:31-182
 *   launch_assign + assign_tokens_vectorized  hexa_moe_cuda/hexa_moe/kernels/shared_cuda_core.cu:184-333
 * The reference pads every expert's segment to a multiple of 16 (BLOCK_SIZE, :17,:167-169) and lets
 * atomics decide the order inside a segment; here `pad` is a parameter (16 = the reference's
 * format, 1 = unpadded) and the order inside a segment is ascending token id, which is one of the
 * orders the reference can produce and the only deterministic one.
 *
 * Pinned (tests/test_oracle_route.py) against numpy bincount / stable argsort, brute force on tiny
 * inputs and the partition invariants; the reference holds no vectors for this path.
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* counts[E], expanded[E+1] for one routing slot.  Returns 0, or -1 on an out-of-range expert id. */
int oracle_token_count(const int32_t *routing, int num_tokens, int num_experts, int pad,
                       int32_t *counts, int32_t *expanded)
{
    memset(counts, 0, sizeof(int32_t) * (size_t)num_experts);
    for (int t = 0; t < num_tokens; ++t) {
        int32_t e = routing[t];
        if (e < 0 || e >= num_experts) return -1;
        counts[e] += 1;
    }
    int32_t run = 0;
    for (int e = 0; e < num_experts; ++e) {
        expanded[e] = run;
        int32_t c = counts[e];
        if (c % pad != 0) c = (1 + c / pad) * pad;   /* shared_cuda_core.cu:167-169 */
        run += c;
    }
    expanded[num_experts] = run;
    return 0;
}

/* token_idx_list[P], expert_idx_list[P] (P = expanded[E]); padding slots are set to -1, which is
 * what the reference's caller pre-fills them with (impls/layers.py:238-239). */
int oracle_token_assign(const int32_t *routing, int num_tokens, int num_experts,
                        const int32_t *expanded, int32_t *token_idx_list, int32_t *expert_idx_list)
{
    int32_t P = expanded[num_experts];
    for (int32_t i = 0; i < P; ++i) { token_idx_list[i] = -1; expert_idx_list[i] = -1; }
    int32_t *cursor = (int32_t *)malloc(sizeof(int32_t) * (size_t)num_experts);
    if (!cursor) return -2;
    memcpy(cursor, expanded, sizeof(int32_t) * (size_t)num_experts);
    for (int t = 0; t < num_tokens; ++t) {
        int32_t e = routing[t];
        if (e < 0 || e >= num_experts) { free(cursor); return -1; }
        int32_t pos = cursor[e]++;                   /* shared_cuda_core.cu: atomicAdd(&start[e],1) */
        token_idx_list[pos] = t;
        expert_idx_list[pos] = e;
    }
    free(cursor);
    return 0;
}

/* All k slots of routing[T,k] (row-major), unpadded: counts[k,E], offsets[k,E+1], token_ids[k,T]. */
int oracle_route_build(const int32_t *routing, int num_tokens, int top_k, int num_experts,
                       int32_t *counts, int32_t *offsets, int32_t *token_ids)
{
    int32_t *slot = (int32_t *)malloc(sizeof(int32_t) * (size_t)(num_tokens > 0 ? num_tokens : 1));
    int32_t *exp_scratch = (int32_t *)malloc(sizeof(int32_t) * (size_t)(num_tokens > 0 ? num_tokens : 1));
    if (!slot || !exp_scratch) { free(slot); free(exp_scratch); return -2; }
    int rc = 0;
    for (int s = 0; s < top_k && rc == 0; ++s) {
        for (int t = 0; t < num_tokens; ++t) slot[t] = routing[(size_t)t * top_k + s];
        rc = oracle_token_count(slot, num_tokens, num_experts, 1,
                                counts + (size_t)s * num_experts, offsets + (size_t)s * (num_experts + 1));
        if (rc == 0)
            rc = oracle_token_assign(slot, num_tokens, num_experts, offsets + (size_t)s * (num_experts + 1),
                                     token_ids + (size_t)s * num_tokens, exp_scratch);
    }
    free(slot); free(exp_scratch);
    return rc;
}
