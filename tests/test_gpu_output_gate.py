"""GPU parity: output gate through the C ABI vs the CPU oracle.  Both compute in fp32 with their
own expf (each within one fp32 ulp of the true value), so the fp16 results agree except where the
product sits on a rounding boundary: at most one fp16 ulp apart, and equal nearly everywhere."""
import ctypes as C

import numpy as np
import pytest

import oracle

pytestmark = pytest.mark.gpu


def _run(a_bits, g_bits, mask=None, sentinel=0x5500):
    import gpu_harness as G
    import torch

    l = G.lib()
    ex, _ = G.make_exec()
    da, dg = G.to_dev(a_bits), G.to_dev(g_bits)
    out = torch.full(a_bits.shape, sentinel, dtype=torch.int16, device=G.DEV)
    dm = None if mask is None else G.to_dev(np.asarray(mask, np.uint8))
    rc = l.warp34_apply_attn_output_gate_f16(C.byref(ex), G.ptr(da), G.ptr(dg), C.c_void_p(out.data_ptr()),
                                             None if dm is None else G.ptr(dm), a_bits.shape[0], a_bits.shape[1])
    torch.cuda.synchronize()
    return rc, out.cpu().numpy().view(np.uint16)


@pytest.mark.parametrize("tokens,dim", [(37, 4096), (5, 4100), (3, 7), (2048, 4096)])
def test_output_gate_matches_oracle(tokens, dim):
    rng = np.random.default_rng(tokens)
    a = (rng.standard_normal((tokens, dim)) * 2).astype(np.float16).view(np.uint16)
    g = (rng.standard_normal((tokens, dim)) * 3).astype(np.float16).view(np.uint16)
    rc, got = _run(a, g)
    assert rc == 0
    want = oracle.apply_attn_output_gate_f16(a, g)
    gf, wf = got.view(np.float16).astype(np.float64), want.view(np.float16).astype(np.float64)
    ulp = np.maximum(np.abs(wf), 2.0 ** -14) * 2.0 ** -10
    assert (np.abs(gf - wf) <= ulp * 1.001).all()
    assert (got == want).mean() > 0.999


def test_output_gate_mask_and_validation():
    from warp34_amd import ffi
    import gpu_harness as G

    rng = np.random.default_rng(9)
    a = rng.standard_normal((6, 256)).astype(np.float16).view(np.uint16)
    g = rng.standard_normal((6, 256)).astype(np.float16).view(np.uint16)
    mask = [1, 0, 1, 1, 0, 1]
    rc, got = _run(a, g, mask=mask)
    assert rc == 0
    want = oracle.apply_attn_output_gate_f16(a, g, out=np.full((6, 256), 0x5500, np.uint16), valid_token_mask=mask)
    assert (got[1] == 0x5500).all() and (got[4] == 0x5500).all()
    assert (got == want).mean() > 0.999
    l = G.lib()
    ex, _ = G.make_exec()
    d = G.to_dev(a)
    assert l.warp34_apply_attn_output_gate_f16(C.byref(ex), None, G.ptr(d), G.ptr(d), None, 6, 256) == ffi.HIP_ERROR_INVALID_VALUE
    assert l.warp34_apply_attn_output_gate_f16(C.byref(ex), G.ptr(d), G.ptr(d), G.ptr(d), None, 0, 256) == 0
