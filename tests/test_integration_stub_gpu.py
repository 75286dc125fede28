"""The ctypes binding written out in the integration notes for a maintainer of
the reference (the replacement of get_custom_kernels() and of the TorchScript
epilogues, oslo/fused_kernels_utils.py:219-232, :259-308) is executed as
written, against the built library, and must give what this package's own
front gives: the notes cannot drift from the ABI."""

import ctypes
import os
import re

import pytest
import torch

from oslo_amd import _lib, kernels

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def stub_namespace():
    text = open(os.path.join(ROOT, "INTEGRATION.md")).read()
    section_b = text[text.index("## B."):text.index("## Entry points")]
    blocks = re.findall(r"```python\n(.*?)```", section_b, flags=re.S)
    assert len(blocks) == 2
    ns = {}
    exec(blocks[0].replace('path="liboslo_amd.so"', f'path="{_lib.LIB_PATH}"'), ns)
    exec(blocks[1], ns)
    # the argument types the notes list for the epilogue entry points
    L = ns["get_custom_kernels"]().L
    P, I64, U64, F, I = ctypes.c_void_p, ctypes.c_int64, ctypes.c_uint64, ctypes.c_float, ctypes.c_int
    L.oslo_bias_gelu_fwd.argtypes = [P, P, P, I64, I64, I, P]
    L.oslo_bias_gelu_bwd.argtypes = [P, P, P, P, P, P, I64, I64, I, P]
    L.oslo_bias_dropout_add_fwd.argtypes = [P, P, P, P, F, U64, U64, I64, I64, I, P]
    L.oslo_bias_dropout_add_bwd.argtypes = [P, P, P, P, F, U64, U64, I64, I64, I, P]
    L.oslo_colsum_workspace_bytes.argtypes = [I64, I64]
    L.oslo_colsum_workspace_bytes.restype = I64
    return ns


def test_documented_binding_matches_the_package():
    ns = stub_namespace()
    K = ns["get_custom_kernels"]()
    g = torch.Generator(device=DEV).manual_seed(0)
    x3 = (torch.randn((6, 128, 128), generator=g, device=DEV) * 4).half()
    y3 = K.scaled_upper_triang_masked_softmax_forward(x3, 0.125)
    assert torch.equal(y3, kernels.scaled_upper_triang_masked_softmax_forward(x3, 0.125))
    go = torch.randn((6, 128, 128), generator=g, device=DEV).half()
    assert torch.equal(K.scaled_upper_triang_masked_softmax_backward(go.clone(), y3, 0.125),
                       kernels.scaled_upper_triang_masked_softmax_backward(go.clone(), y3, 0.125))
    x4 = torch.randn((2, 3, 40, 264), generator=g, device=DEV).bfloat16()
    mask = torch.rand((2, 1, 40, 264), generator=g, device=DEV) < 0.3
    y4 = K.scaled_masked_softmax_forward(x4, mask, 0.5)
    assert torch.equal(y4, kernels.scaled_masked_softmax_forward(x4, mask, 0.5))
    g4 = torch.randn((2, 3, 40, 264), generator=g, device=DEV).bfloat16()
    assert torch.equal(K.scaled_masked_softmax_backward(g4.clone(), y4, 0.5),
                       kernels.scaled_masked_softmax_backward(g4.clone(), y4, 0.5))
    assert K.get_batch_per_block(128, 128, 2, 3) == kernels.get_batch_per_block(128, 128, 2, 3)
    tokens = torch.randint(0, 9, (4, 12), generator=g, device=DEV)
    lp = torch.randn((4, 9), generator=g, device=DEV)
    assert torch.equal(K.ngram_repeat_block_forward(tokens, lp.clone(), 2, 11, 2, 3),
                       kernels.ngram_repeat_block_forward(tokens, lp.clone(), 2, 11, 2, 3))
    # the epilogues
    y = torch.randn((33, 768), generator=g, device=DEV).bfloat16()
    b = (torch.randn((768,), generator=g, device=DEV) * 0.1).bfloat16()
    assert torch.equal(ns["bias_gelu_fwb"](y, b), kernels.bias_gelu_forward(y, b))
    gy = torch.randn((33, 768), generator=g, device=DEV).bfloat16()
    dy, db = ns["bias_gelu_bwd"](gy, y, b)
    want_dy, want_db = kernels.bias_gelu_backward(gy, y, b)
    assert torch.equal(dy, want_dy) and torch.equal(db, want_db)
    res = torch.randn((33, 768), generator=g, device=DEV).bfloat16()
    gen = torch.cuda.default_generators[0]
    seed, offset = gen.initial_seed(), gen.get_offset()
    x = y.clone().requires_grad_(True)
    out = ns["_BiasDropoutAdd"].apply(x, b, res, 0.1)
    assert gen.get_offset() == offset + 4
    assert torch.equal(out, kernels.bias_dropout_add_forward(y, b, res, 0.1, seed, offset))
    out.backward(gy)
    want_dx, _ = kernels.bias_dropout_add_backward(gy, 0.1, seed, offset)
    assert torch.equal(x.grad, want_dx)
