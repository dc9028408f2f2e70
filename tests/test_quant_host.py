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


def test_hqq_tensor_layout_round_trip():
    """``from_hqq_tensors`` reads hqq's published 4-bit layout (first half of the 64-wide groups in the
    high nibble, second half in the low nibble).  hqq itself is absent, so the layout is restated here
    independently, element by element, and checked in both directions."""
    g = torch.Generator().manual_seed(7)
    N, K = 48, 256
    codes = torch.randint(0, 16, (N, K), generator=g, dtype=torch.uint8)
    scale = (torch.rand(N, K // 64, generator=g) * 0.01 + 1e-3).to(torch.float16)
    zero = (torch.rand(N, K // 64, generator=g) * 15).to(torch.float16)
    rows = N * K // 64
    flat = codes.reshape(rows, 64)
    packed = torch.empty(rows // 2, 64, dtype=torch.uint8)
    for r in range(rows // 2):                                   # element-wise restatement of pack_4bit_u8
        for c in range(64):
            packed[r, c] = (int(flat[r, c]) << 4) | int(flat[r + rows // 2, c])
    c2, s2, z2 = quant.from_hqq_tensors(packed, scale.reshape(rows, 1), zero.reshape(rows, 1), (N, K))
    assert torch.equal(c2, codes) and torch.equal(s2, scale) and torch.equal(z2, zero)
    W_q, s3, z3 = quant.to_hqq_tensors(codes, scale, zero)
    assert torch.equal(W_q, packed) and s3.shape == (rows, 1) and z3.shape == (rows, 1)
    # dequantization in hqq's own arrangement equals the [N, K] form
    deq_rows = (torch.cat([packed >> 4, packed & 15], 0).float() - zero.reshape(rows, 1).float()) * scale.reshape(rows, 1).float()
    assert torch.equal(deq_rows.reshape(N, K), quant.dequantize(codes, scale, zero))
    with pytest.raises(ValueError):
        quant.from_hqq_tensors(packed[:-1], scale, zero, (N, K))


def test_proximal_zero_refinement():
    """The restated hqq solver (parity unpinned against hqq itself): what can be checked is what it promises --
    the scale and the code range are untouched, the mean absolute reconstruction error never grows against the
    min/max rule and shrinks on weights with outliers, a group that the min/max rule already reproduces exactly is
    left alone, and with zero iterations nothing changes."""
    g = torch.Generator().manual_seed(0)
    W = torch.randn(96, 512, generator=g) * 0.02
    W[torch.rand(96, 512, generator=g) < 0.01] *= 6                      # heavy tails, as trained weights have
    c0, s0, z0 = quant.quantize_int4_g64(W)
    c1, s1, z1 = quant.quantize_int4_g64(W, optimize=True)
    assert torch.equal(s0, s1) and int(c1.max()) <= 15 and c1.dtype == torch.uint8
    e0 = (W - quant.dequantize(c0, s0, z0)).abs().mean().item()
    e1 = (W - quant.dequantize(c1, s1, z1)).abs().mean().item()
    assert e1 < 0.99 * e0, (e0, e1)
    assert not torch.equal(z0, z1)
    # per group the refined zero is never worse than the starting point by more than fp16 rounding of the zero
    g0 = (W - quant.dequantize(c0, s0, z0)).abs().reshape(96, 8, 64).mean(-1)
    g1 = (W - quant.dequantize(c1, s1, z1)).abs().reshape(96, 8, 64).mean(-1)
    assert (g1 <= g0 * 1.5 + 1e-6).all()
    # weights that sit exactly on a 16-level grid are reproduced exactly, refined or not
    levels = torch.randint(0, 16, (8, 128), generator=g).float()
    levels[:, 0], levels[:, 1], levels[:, 64], levels[:, 65] = 0, 15, 0, 15
    Wg = (levels - 7.0) * 0.5
    for opt in (False, True):
        c, s, z = quant.quantize_int4_g64(Wg, optimize=opt)
        assert torch.equal(quant.dequantize(c, s, z), Wg)
    c2, s2, z2 = quant.quantize_int4_g64(W, optimize=True, opt_params={"iters": 0})
    assert torch.equal(c2, c0) and torch.equal(z2, z0)
