/*
 * TEST INFRASTRUCTURE ONLY -- CPU restatement of the integer part of the reference's top-2 / switch gating in index
 * form: given every token's expert choices, the capacity slot each choice lands in.  Nothing outside tests/,
 * __graft_entry__.smoke() and the cpu_baseline leg of bench.py may link or call this file.
 *
 * Follows /root/reference/models.py:483-491 (top-2) and models.py:458-466 (switch):
 *   mask  = one_hot(index, E)                          [B, S, k, E]
 *   pos   = cumsum(mask, dim = 1) * mask               1-based position of a token among the row's earlier
 *                                                      tokens with the same choice number k and expert
 *   first = sum(pos[:, :, 0, :], dim = 1)              the SUM of an expert's first-choice positions,
 *                                                      n (n + 1) / 2 for n first choices (not the count n)
 *   pos[:, :, 1, :] += first                           second choices queue behind that sum
 *   keep  = pos < C;  pos *= keep                      positions C and above are dropped; slot 0 is never used
 * The dense [B, S, E, C] tensors of the reference hold gate_k at (b, s, index_k, slot_k) for every kept choice.
 *
 * Pinned by (tests/test_oracle_gating.py): the hand-worked routing vectors of tests/golden/gating_vectors.json,
 * equality with the dense PyTorch restatement (oracle/ops.py top_2_gating / switch_gating) at the benchmark's
 * full shape for C = 80 and C = 40, and the closed forms n(n+1)/2 + j of the second choices' positions.
 */
#include <stdint.h>
#include <stdlib.h>

/* index[B, S, top_k] (expert of every choice) -> slot[B, S, top_k] (0 = dropped), token_of_slot[B, E, C] (-1 = empty).
 * Returns 0, or -1 for an expert index outside [0, E) or a failed allocation. */
int oracle_gating_slots(const int64_t *index, int64_t B, int64_t S, int64_t E, int64_t C, int64_t top_k,
                        int64_t *slot, int64_t *token_of_slot)
{
    int64_t *count = (int64_t *)malloc((size_t)E * sizeof(int64_t));
    int64_t *offset = (int64_t *)malloc((size_t)E * sizeof(int64_t));
    if (!count || !offset) {
        free(count);
        free(offset);
        return -1;
    }
    for (int64_t i = 0; i < B * E * C; ++i) token_of_slot[i] = -1;
    for (int64_t b = 0; b < B; ++b) {
        for (int64_t e = 0; e < E; ++e) offset[e] = 0;
        for (int64_t k = 0; k < top_k; ++k) {
            for (int64_t e = 0; e < E; ++e) count[e] = 0;
            for (int64_t s = 0; s < S; ++s) {
                const int64_t at = (b * S + s) * top_k + k;
                const int64_t e = index[at];
                if (e < 0 || e >= E) {
                    free(count);
                    free(offset);
                    return -1;
                }
                const int64_t pos = ++count[e] + offset[e];          /* inclusive cumsum: 1-based */
                slot[at] = pos < C ? pos : 0;
                if (pos < C) token_of_slot[(b * E + e) * C + pos] = s;
            }
            /* what the next choice number queues behind: the sum of this one's positions (only the first
             * choices' sum is ever used: top_k is 1 or 2) */
            for (int64_t e = 0; e < E; ++e) offset[e] = count[e] * (count[e] + 1) / 2;
        }
    }
    free(count);
    free(offset);
    return 0;
}
