"""The library's synthetic-input generators (include/warp34_synth.h; SplitMix64 -> Box-Muller ->
bf16, x20 outlier channels, Fisher-Yates) against the oracle's sequential ones: same seeds, same
bits, from any starting row, whatever the number of threads that filled the tensor; plus what
the recipe fixes on its own (a permutation is a permutation, three outlier channels per head,
unit variance elsewhere)."""
import numpy as np

import oracle
from oracle import DT_BF16
from warp34_amd import ffi


def test_normal_stream_equals_the_oracle_and_restarts_anywhere():
    n = 300001
    want = oracle.fill_normal(n, 77, DT_BF16)
    got = ffi.synth_normal_bf16(n, 77)
    assert got.tobytes() == want.tobytes()
    part = ffi.synth_normal_bf16(5000, 77, first=123456)
    assert part.tobytes() == want[123456:128456].tobytes()


def test_kv_rows_equal_the_oracle_and_restart_at_any_row():
    rows, heads, dim = 700, 2, 256
    want = oracle.fill_kv_rows(rows, heads, dim, 5, DT_BF16, 3)
    got = ffi.synth_kv_rows_bf16(rows, heads, dim, 5, 3)
    assert got.tobytes() == want.tobytes()
    part = ffi.synth_kv_rows_bf16(100, heads, dim, 5, 3, first_row=333)
    assert part.tobytes() == want[333:433].tobytes()
    # a tensor large enough for several threads
    big = ffi.synth_kv_rows_bf16(4096, heads, dim, 9, 3)
    assert big.tobytes() == oracle.fill_kv_rows(4096, heads, dim, 9, DT_BF16, 3).tobytes()
    f = oracle.bf16_bits_to_f32(big)
    std = f.reshape(-1, heads * dim).std(axis=0).reshape(heads, dim)
    for h in range(heads):
        assert int((std[h] > 10).sum()) == 3 and abs(float(np.median(std[h])) - 1.0) < 0.05


def test_permutation_and_uniform_draws():
    for n, seed in ((1, 3), (2, 4), (64, 0), (32768, 11)):
        p = ffi.synth_permutation(n, seed)
        assert p.tobytes() == oracle.permutation(n, seed).tobytes()
        assert sorted(p.tolist()) == list(range(n))
    u = ffi.synth_uniform_i32(1000, 1024, 65536, 0)
    assert u.min() >= 1024 and u.max() <= 65536 and len(set(u.tolist())) > 900
    assert ffi.synth_uniform_i32(10, 1024, 65536, 0).tolist() == u[:10].tolist()
