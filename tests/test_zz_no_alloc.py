"""GPU test of ll_nvfp4_quantize_noalloc, the entry point that allocates nothing: called through the C ABI twice
in a row (the second input smaller), its outputs must equal those of ll_nvfp4_quantize bit for bit."""
import ctypes

import numpy as np
import pytest
import torch

from helpers import activations, u8
from longlive_amd import _native

pytestmark = pytest.mark.gpu


def _quantize_both(lib, x, rule_id):
    M, K = x.shape
    Mp, Kp = _native.padded_shape((M, K))
    dev = x.device
    stream = torch.cuda.current_stream().cuda_stream
    outs = []
    for which in ("noalloc", "workspace"):
        values = torch.full((Mp, Kp // 2), 0xA5, dtype=torch.uint8, device=dev)
        scales = torch.full((Mp * Kp // 16,), 0xA5, dtype=torch.uint8, device=dev)
        amax = torch.full((1,), -1.0, dtype=torch.float32, device=dev)
        if which == "noalloc":
            rc = lib.ll_nvfp4_quantize_noalloc(x.data_ptr(), M, K, x.stride(0), rule_id, values.data_ptr(),
                                               scales.data_ptr(), amax.data_ptr(), stream)
        else:
            ws = torch.empty(lib.ll_nvfp4_quantize_workspace_floats(), dtype=torch.float32, device=dev)
            rc = lib.ll_nvfp4_quantize(x.data_ptr(), M, K, x.stride(0), rule_id, values.data_ptr(), scales.data_ptr(),
                                       amax.data_ptr(), 0, ws.data_ptr(), stream)
        assert rc == 0, lib.ll_last_error().decode()
        outs.append((values, scales, amax))
    torch.cuda.synchronize()
    return outs


@pytest.mark.parametrize("rule", ["mse", "static_6"])
def test_noalloc_quantize_matches_workspace_quantize_on_two_calls_in_a_row(gpu, rule):
    lib = _native.load()
    rule_id = _native.RULE_IDS[rule]
    # first a larger tensor with a large maximum, then a smaller one with a smaller maximum: partial maxima the
    # first call left in the shared scratch must not leak into the second
    first = (activations((1000, 1472), 11) * 8).to(gpu)
    second = (activations((200, 192), 12) * 0.25).to(gpu)
    for x in (first, second):
        (v0, s0, a0), (v1, s1, a1) = _quantize_both(lib, x, rule_id)
        assert float(a0.cpu()) == float(a1.cpu()) == float(x.float().abs().max().cpu())
        assert np.array_equal(u8(v0), u8(v1)) and np.array_equal(u8(s0), u8(s1))
