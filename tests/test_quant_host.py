"""Host-side int4 quantizer and tiled packing (subspec_amd.quant) and the int4 oracle.  No GPU."""
import pytest
import torch
import torch.nn as nn

from oracle import int4 as oi
from subspec_amd import quant


def test_quantize_roundtrip_and_closed_forms():
    torch.manual_seed(0)
    W = torch.randn(32, 256) * 0.02
    codes, scale, zero = quant.quantize_int4_g64(W)
    assert codes.dtype == torch.uint8 and int(codes.max()) <= 15 and scale.dtype == torch.float16
    deq = oi.dequant(codes, scale, zero)
    assert torch.equal(deq, quant.dequantize(codes, scale, zero))        # two independent dequantizers agree
    # affine min/max quantization: error bounded by half a step (plus fp16 rounding of scale / zero)
    step = scale.float().repeat_interleave(64, dim=1)
    assert ((deq - W).abs() <= 0.51 * step + 1e-4).all()
    # special case scale = 1, zero = 0: the linear is an integer matmul
    ones, zeros = torch.ones_like(scale), torch.zeros_like(zero)
    x = torch.randint(-3, 4, (5, 256)).float()
    assert torch.equal(oi.linear(x, codes, ones, zeros), x @ codes.float().T)
    # shifting codes and zero point together changes nothing
    assert torch.allclose(oi.dequant(codes, scale, zero), oi.dequant(codes + 1, scale, zero.float() + 1), atol=1e-6)


def test_tiled_packing_is_lossless():
    torch.manual_seed(1)
    W = torch.randn(48, 192)
    codes, scale, zero = quant.quantize_int4_g64(W)
    wq, sz = quant.pack_tiled(codes, scale, zero)
    assert wq.shape == (3, 3, 4, 16, 2) and sz.shape == (3, 3, 16) and wq.dtype == torch.int32
    c2, s2, z2 = oi.unpack_tiled(wq, sz, 48, 192)
    assert torch.equal(c2, codes) and torch.equal(s2, scale) and torch.equal(z2, zero)


def test_quantizer_replaces_named_linears_and_rejects_other_configs():
    model = nn.Sequential()
    model.add_module("a", nn.Linear(128, 32, bias=True))
    model.add_module("b", nn.Linear(128, 32, bias=False))
    quant.HqqQuantizer.quantize_model(model, {"a": {"nbits": 4, "group_size": 64, "axis": 1}}, torch.bfloat16, "cpu")
    assert isinstance(model.a, quant.HqqInt4Linear) and isinstance(model.b, nn.Linear)
    assert model.a.bias.dtype == torch.bfloat16
    with pytest.raises(ValueError):
        quant.HqqQuantizer.quantize_model(model, {"b": {"nbits": 8, "group_size": 64}}, torch.bfloat16, "cpu")
    with pytest.raises(ValueError):
        quant.quantize_int4_g64(torch.zeros(16, 100))
    from subspec_amd._lib import SubspecHipError
    with pytest.raises(SubspecHipError):                   # no CPU fallback
        model.a(torch.zeros(1, 128, dtype=torch.bfloat16))
