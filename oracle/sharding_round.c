/*
 * TEST INFRASTRUCTURE ONLY -- CPU restatement of the reference's integer
 * rounding rule.  Nothing outside tests/, __graft_entry__.smoke() and the
 * cpu_baseline leg of bench.py may link or call this file.
 *
 * Follows /root/reference/hap.rs:3536-3559 (fn sharding_round):
 *   - full_length == 1  -> every device gets 1 (broadcast hack, pairs with the
 *     size-1 skip in split_param_or_buffer, hap.rs:44-45);
 *   - len[i] = (usize)(ratio[i] * (f64)full_length)   (truncation);
 *   - assert sum <= full_length;
 *   - while sum < full_length: +1 at argmax_i (ratio[i] - len[i]/full_length),
 *     where Rust's Iterator::max_by_key returns the LAST maximal element and
 *     FloatOrd gives a total order on f64.
 *
 * Pinned by: hand-derived known answers, sum/floor invariants and a
 * brute-force largest-remainder cross-check (tests/test_sharding_round.py).
 */
#include <stdint.h>
#include <stddef.h>

/* returns 0 on success, -1 when the truncated lengths already exceed n
 * (the reference asserts in that case). */
int oracle_sharding_round(int64_t full_length, const double *ratios, int64_t n_dev,
                          int64_t *out)
{
    if (full_length == 1) {
        for (int64_t i = 0; i < n_dev; ++i) out[i] = 1;
        return 0;
    }
    int64_t sum = 0;
    for (int64_t i = 0; i < n_dev; ++i) {
        out[i] = (int64_t)(ratios[i] * (double)full_length);
        sum += out[i];
    }
    if (sum > full_length) return -1;
    while (sum < full_length) {
        int64_t best = 0;
        double best_key = ratios[0] - (double)out[0] / (double)full_length;
        for (int64_t i = 1; i < n_dev; ++i) {
            double key = ratios[i] - (double)out[i] / (double)full_length;
            if (key >= best_key) { /* ties go to the last index */
                best_key = key;
                best = i;
            }
        }
        out[best] += 1;
        sum += 1;
    }
    return 0;
}
