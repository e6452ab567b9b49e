"""Pins of the oracle's output gate (ops/op_norms_rope_act.cu:742-759): out = a * sigmoid(g)."""
import numpy as np

import oracle


def _ulp_f16(x):
    return np.maximum(np.abs(x), 2.0 ** -14) * 2.0 ** -10


def test_matches_float64_sigmoid_within_one_fp16_ulp():
    rng = np.random.default_rng(0)
    a = (rng.standard_normal((7, 512)) * 3).astype(np.float16)
    g = (rng.standard_normal((7, 512)) * 4).astype(np.float16)
    got = oracle.apply_attn_output_gate_f16(a.view(np.uint16), g.view(np.uint16)).view(np.float16).astype(np.float64)
    want = a.astype(np.float64) / (1.0 + np.exp(-g.astype(np.float64)))
    assert (np.abs(got - want) <= 0.5 * _ulp_f16(want) * 1.01 + 1e-12).all()


def test_special_values():
    a = np.array([[1.5, -2.25, 3.0, 7.0, 7.0, 0.0]], np.float16)
    g = np.array([[0.0, 0.0, 0.0, 30.0, -30.0, 5.0]], np.float16)
    got = oracle.apply_attn_output_gate_f16(a.view(np.uint16), g.view(np.uint16)).view(np.float16)
    assert got[0, 0] == np.float16(0.75) and got[0, 1] == np.float16(-1.125) and got[0, 2] == np.float16(1.5)
    assert got[0, 3] == np.float16(7.0)          # sigmoid saturates to 1 in fp32
    assert abs(float(got[0, 4])) < 1e-10         # and to 0
    assert got[0, 5] == 0


def test_masked_rows_are_skipped():
    rng = np.random.default_rng(1)
    a = rng.standard_normal((4, 64)).astype(np.float16).view(np.uint16)
    g = rng.standard_normal((4, 64)).astype(np.float16).view(np.uint16)
    out = np.full((4, 64), 0x5500, np.uint16)
    oracle.apply_attn_output_gate_f16(a, g, out=out, valid_token_mask=[1, 0, 1, 0])
    assert (out[1] == 0x5500).all() and (out[3] == 0x5500).all()
    assert (out[0] != 0x5500).any() and (out[2] != 0x5500).any()
