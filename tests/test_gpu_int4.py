"""GPU parity: int4 g64 linear (GEMV for M = 1, MFMA GEMM for M = 2..64) through the C ABI against
x.float() @ ((Wq - z) * s).T on identical (Wq, scale, zero).  Tolerance 1e-2 relative
(max |diff| <= 1e-2 * max |ref|, outputs rounded to the activation dtype)."""
import pytest
import torch

pytestmark = pytest.mark.gpu

from oracle import int4 as oi
from subspec_amd import ops, quant

DEV = "cuda:0"


def _check(N, K, M, dtype, seed, bias=False):
    print("int4", N, K, M, dtype, flush=True)
    g = torch.Generator().manual_seed(seed)
    W = torch.randn(N, K, generator=g) * 0.02
    codes, scale, zero = quant.quantize_int4_g64(W)
    wq, sz = quant.pack_tiled(codes, scale, zero)
    x = torch.randn(M, K, generator=g).to(dtype)
    b = (torch.randn(N, generator=g) * 0.1).to(dtype) if bias else None
    y = ops.int4_linear(x.to(DEV), wq.to(DEV), sz.to(DEV), N, None if b is None else b.to(DEV))
    torch.cuda.synchronize()
    ref = oi.linear(x, codes, scale, zero, b)
    got = y.float().cpu()
    assert got.shape == ref.shape
    err = (got - ref).abs().amax().item()
    assert err <= 1e-2 * ref.abs().amax().item(), (N, K, M, err, ref.abs().amax().item())
    return got, ref


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_small_shapes(dtype):
    for seed, (N, K, M) in enumerate([(16, 64, 1), (48, 192, 1), (64, 256, 2), (80, 512, 16), (128, 1024, 17),
                                      (256, 2048, 33), (64, 3584, 64), (512, 128, 5), (96, 7168, 8), (32, 320, 3)]):
        _check(N, K, M, dtype, seed, bias=seed % 2 == 0)


@pytest.mark.parametrize("N,K", [(4608, 3584), (3584, 3584), (37888, 3584), (3584, 18944)])
@pytest.mark.parametrize("M", [1, 8, 16, 64])                 # 8: one draft level (top-k 8), the 8-row activation block
def test_config4_qwen_shapes(N, K, M):
    _check(N, K, M, torch.bfloat16, 100 + M)


def test_exact_integer_case_and_module():
    # scale = 1, zero = 0, small integer activations: every product is exact -> bit-exact result
    g = torch.Generator().manual_seed(3)
    N, K = 64, 256
    codes = torch.randint(0, 16, (N, K), generator=g, dtype=torch.uint8)
    scale = torch.ones(N, K // 64, dtype=torch.float16)
    zero = torch.zeros(N, K // 64, dtype=torch.float16)
    wq, sz = quant.pack_tiled(codes, scale, zero)
    for M in (1, 7, 64):
        x = torch.randint(-2, 3, (M, K), generator=g).to(torch.bfloat16)
        y = ops.int4_linear(x.to(DEV), wq.to(DEV), sz.to(DEV), N).float().cpu()
        assert torch.equal(y, (x.float() @ codes.float().T).to(torch.bfloat16).float())
    lin = torch.nn.Linear(256, 64, bias=True)
    q = quant.HqqInt4Linear.from_linear(lin, torch.bfloat16, DEV)
    x = torch.randn(2, 5, 256).to(torch.bfloat16)
    y = q(x.to(DEV))
    assert y.shape == (2, 5, 64) and y.dtype == torch.bfloat16
    ref = oi.linear(x.reshape(10, 256), *quant.quantize_int4_g64(lin.weight.data), lin.bias.data.to(torch.bfloat16))
    assert (y.float().cpu().reshape(10, 64) - ref).abs().amax() <= 1e-2 * ref.abs().amax()


def test_argument_errors():
    wq = torch.zeros(1, 1, 4, 16, 2, dtype=torch.int32, device=DEV)
    sz = torch.zeros(1, 1, 16, dtype=torch.int32, device=DEV)
    with pytest.raises(ValueError):
        ops.int4_linear(torch.zeros(1, 64, device=DEV), wq, sz, 16)                       # fp32 activations
    with pytest.raises(ValueError):
        ops.int4_linear(torch.zeros(1, 128, dtype=torch.bfloat16, device=DEV), wq, sz, 16)  # shape mismatch


def test_random_shape_sweep():
    """Ragged everything: tile counts that do not divide the grid, group counts that are not multiples of
    four (dead pipeline steps), every activation-row tile count, with and without bias."""
    g = torch.Generator().manual_seed(2024)
    for i in range(24):
        N = 16 * int(torch.randint(1, 700, (1,), generator=g))
        K = 64 * int(torch.randint(1, 40, (1,), generator=g))
        M = int(torch.randint(1, 65, (1,), generator=g))
        _check(N, K, M, torch.bfloat16 if i % 3 else torch.float16, 500 + i, bias=bool(i % 2))
    # a very wide layer: more tiles than one resident wave of workgroups covers with five tiles each
    _check(16 * 6000, 256, 64, torch.bfloat16, 900)
    _check(16 * 6000, 256, 7, torch.bfloat16, 901)
    # more than 64 rows (a whole large tree through the draft): several passes of 64 rows
    for i, (N, K, M) in enumerate([(16 * 40, 64 * 9, 65), (4608, 3584, 289), (3584, 18944, 130), (16 * 10, 64 * 3, 512)]):
        _check(N, K, M, torch.bfloat16 if i % 2 == 0 else torch.float16, 950 + i, bias=bool(i % 2))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_rows_up_to_16_long_k(dtype):
    """At most 16 rows and K > 2048 take the kernel that issues every request up front: every tile count per
    workgroup it is compiled for (1, 2, 3 in one round; 4, 6, 8, 10 in two), launches beyond one workgroup per
    compute unit, K ranges that are not multiples of 8 groups (dead steps), several K ranges, ragged last
    workgroups, with and without bias.  More than 56 groups over at least 128 tiles take the kernel that walks the
    whole of K in one workgroup per tile: one round, a last round with dead steps, wavefronts with different round
    counts, the tile count at its threshold; fewer tiles keep the K ranges over workgroups."""
    cases = [(16 * 7, 64 * 33, 3), (16 * 300, 64 * 40, 8), (16 * 601, 64 * 56, 5), (16 * 1000, 64 * 35, 2),
             (16 * 1501, 64 * 34, 8), (16 * 1900, 64 * 33, 1), (16 * 2400, 64 * 34, 7), (16 * 3001, 64 * 33, 8),
             (16 * 9, 64 * 57, 8), (16 * 130, 64 * 120, 4), (16 * 224, 64 * 296, 6), (16 * 40, 64 * 1000, 8),
             (16 * 128, 64 * 57, 8), (16 * 128, 64 * 61, 1), (16 * 200, 64 * 129, 3), (16 * 129, 64 * 200, 8),
             (16 * 127, 64 * 64, 8)]
    for i, (N, K, M) in enumerate(cases):
        _check(N, K, M, dtype, 1200 + i, bias=bool(i % 2))
    # 9 to 16 rows: the same kernel with activation blocks of 16 rows, every tile count again (and one shape whose
    # long K stays split over workgroups at these row counts)
    for i, (N, K, _) in enumerate(cases[:12]):
        _check(N, K, 9 + (5 * i) % 8, dtype, 1300 + i, bias=bool(i % 2))


def test_quantizer_default_refines_zero_points():
    """HqqQuantizer.quantize_model refines the zero points unless told not to (as hqq does); the module then
    computes the affine dequantization of those tensors, and its output is at least as close to the unquantized
    layer as with the min/max rule on weights with heavy tails."""
    g = torch.Generator().manual_seed(12)
    W = torch.randn(128, 512, generator=g) * 0.02
    W[torch.rand(128, 512, generator=g) < 0.01] *= 6
    x = torch.randn(16, 512, generator=g).to(torch.bfloat16)
    want = x.float() @ W.T
    errs = {}
    for optimize in (True, False):
        model = torch.nn.Sequential()
        lin = torch.nn.Linear(512, 128, bias=False)
        lin.weight.data.copy_(W)
        model.add_module("p", lin)
        cfg = {"nbits": 4, "group_size": 64, "axis": 1}
        if not optimize:
            cfg["optimize"] = False
        quant.HqqQuantizer.quantize_model(model, {"p": cfg}, torch.bfloat16, DEV)
        y = model.p(x.to(DEV)).float().cpu()
        ref = oi.linear(x, *quant.quantize_int4_g64(W, optimize=optimize))
        assert (y - ref).abs().amax() <= 1e-2 * ref.abs().amax()
        errs[optimize] = (y - want).pow(2).mean().item()
    assert errs[True] <= errs[False] * 1.02, errs


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_gate_up_projection_with_the_activation_in_its_output_stage(dtype):
    """The fused launch against the plain projection followed by the activation on the values it stored: the same
    accumulation per tile, the same roundings, so only the exponential (hardware exp against torch's) may differ --
    nearly every element is identical, the rest within one unit in the last place.  Every activation-row tile
    count, one and two tile pairs per workgroup, with and without bias."""
    for seed, (F, K, M, bias) in enumerate([(16, 64, 1, False), (48, 192, 5, True), (512, 256, 16, False), (1184, 128, 17, True),
                                            (18944, 3584, 8, False), (18944, 3584, 64, False), (2048, 512, 33, True),
                                            (40000, 64, 3, False),
                                            # 8 rows, K > 2048: one, three, four and five tile pairs per workgroup
                                            (16 * 500, 2112, 8, True), (9728, 2112, 8, False), (14336, 2240, 5, True),
                                            (16 * 1190, 2176, 1, False), (16 * 1500, 2112, 8, False),
                                            # 9 to 16 rows, K > 2048: the same tile counts with 16-row activation blocks
                                            (16 * 500, 2112, 16, True), (9728, 2112, 9, False), (14336, 2240, 13, True),
                                            (16 * 1190, 2176, 12, False), (18944, 3584, 16, False)]):
        print("gate|up + silu", dtype, F, K, M, bias, flush=True)
        g = torch.Generator().manual_seed(700 + seed)
        W = torch.randn(2 * F, K, generator=g) * (2.0 / K ** 0.5)
        codes, scale, zero = quant.quantize_int4_g64(W)
        wq, sz = quant.pack_tiled(codes, scale, zero)
        x = torch.randn(M, K, generator=g).to(dtype)
        b = (torch.randn(2 * F, generator=g) * 0.1).to(dtype) if bias else None
        bd = None if b is None else b.to(DEV)
        got = ops.int4_gate_up_silu(x.to(DEV), wq.to(DEV), sz.to(DEV), F, bd)
        gu = ops.int4_linear(x.to(DEV), wq.to(DEV), sz.to(DEV), 2 * F, bd)
        gate, up = gu[:, :F].float(), gu[:, F:].float()
        want = ((gate / (1 + torch.exp(-gate))).to(dtype).float() * up).to(dtype)
        assert got.shape == (M, F) and got.dtype == dtype
        differing = int((got != want).sum())
        # more than five tile pairs per compute unit: the fused launch stays on the four-wavefront kernel while the
        # plain projection of up to 16 rows takes the eight-wavefront one, so the partial sums are grouped differently
        same_grouping = not (M <= 16 and K > 2048 and F // 16 > 1280)
        if same_grouping:
            assert differing <= max(1, got.numel() // 1000), (F, K, M, differing)
        ulp = 2.0 ** (-7 if dtype == torch.bfloat16 else -10)
        # (with another grouping a projection that nearly cancels differs by its absolute rounding, not by a unit in
        # the last place: the bound is then absolute, against the largest output)
        atol = 1e-6 if same_grouping else 2e-3 * want.float().abs().amax().item()
        assert ((got.float() - want.float()).abs() <= (2 if same_grouping else 4) * ulp * want.float().abs() + atol).all()
    with pytest.raises(ValueError):
        ops.int4_gate_up_silu(torch.zeros(65, 64, dtype=dtype, device=DEV), torch.zeros(2 * 32 * 64 // 8, dtype=torch.int32, device=DEV),
                              torch.zeros(2 * 32, dtype=torch.int32, device=DEV), 32)          # more than 64 rows
