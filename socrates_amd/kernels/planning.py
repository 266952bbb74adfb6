"""Host arithmetic that shapes a launch: how a row's keys are split over waves."""

from __future__ import annotations

MAX_KEY_SPLITS = 256    # of the MFMA attention: 64 workgroups of four splits meet per task


def plan_key_splits(n_blocks, n_kv_heads, group, max_keys, target_waves=1024, min_keys=64, n_units=256):
    """(split_len, n_splits) for the MFMA attention kernel: enough waves to fill the GPU, no
    split shorter than 64 keys, at most MAX_KEY_SPLITS of them (a longer context gets longer
    splits), one split or a multiple of four (four share a workgroup; some of the last four
    may lie beyond the keys and are empty). Splits are over absolute key indices, a multiple of
    16 keys long, and cover keys 0 .. max_keys - 1. Host arithmetic only."""
    waves = n_blocks * n_kv_heads * ((group + 15) // 16)
    # from one wave per SIMD on (1,024) no split: a split costs a trip through LDS, or memory
    n = 1 if waves >= 1024 else max(1, min((target_waves + waves - 1) // waves,
                                           (max_keys + min_keys - 1) // min_keys, MAX_KEY_SPLITS))
    if n > 1:
        # splits that would each stream more than 2,048 keys are halved: twice the waves keep
        # more loads on their way, and walks that long pay for the larger meeting (measured
        # at 8 rows of 8 kv heads, 32,768 keys: a step of 8.86 ms with 32 splits of 1,024 keys
        # against 9.28 ms with 16 of 2,048; at 8,192 keys 16 splits of 512 stay the faster)
        twice = min((2 * target_waves + waves - 1) // waves, MAX_KEY_SPLITS)
        if twice > n and max_keys >= twice * 1024:
            n = twice
    if n == 1:
        return ((max_keys + 15) // 16 * 16), 1
    n = (n + 3) // 4 * 4
    # Four splits make a workgroup, and a compute unit holds two such workgroups. A launch a
    # little over a whole number of workgroups per compute unit (288 of them: 32 of the 256
    # units get a second one and finish last) is cut down to that whole number; measured on
    # an MI355X at 8 kv heads, ms per step of a 4B-sized model: 12 rows behind 2,048 keys 3.29
    # with 12 splits (288 workgroups) against 3.16 with 8 (192), behind 8,192 keys 5.82 against
    # 4.97; 6 rows 2.75 with 24 splits (288) against 2.65 with 16 (192), 3.96 against 3.55; 24
    # rows 4.40 with 8 splits (384) against 4.20 with 4 (192).
    tasks = waves                                   # (row block, kv head, chunk of heads)
    groups = tasks * (n // 4)
    if groups > n_units and groups % n_units and (groups % n_units) * 4 < n_units * 3:
        fewer = (n_units * (groups // n_units) // tasks) * 4
        if fewer >= 4:
            n = fewer
    split_len = ((max_keys + n - 1) // n + 15) // 16 * 16
    return split_len, ((max_keys + split_len - 1) // split_len + 3) // 4 * 4
