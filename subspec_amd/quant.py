"""int4 group-wise quantization of the substitute draft's linear layers and the module / quantizer
classes that plug it into a model.

Mirrors the reference's quantizer seam: ``HqqQuantizer.quantize_model(model, quant_config,
compute_dtype, device)`` (specdecodes/helpers/quantizers/hqq/__init__.py:17-120) replaces every
``nn.Linear`` named in ``quant_config`` by a quantized module; the per-layer config is the
``BaseQuantizeConfig(nbits=4, group_size=64, axis=1)`` of
specdecodes/helpers/recipes/subspec/hqq_4bit_postspec.py:17-58 (here a plain dict
``{"nbits": 4, "group_size": 64, "axis": 1}``).

The quantizer starts from the plain affine min/max rule of the benchmark definition: per (output row,
64-wide input group) ``s = (max - min) / 15``, ``z = -min / s`` (both stored as fp16),
``Wq = clamp(round(W / s + z), 0, 15)``.  With ``optimize=True`` the zero point is then refined by the
half-quadratic proximal iteration that hqq (``hqq==0.2.6`` in the reference's requirements, not part
of the reference tree and not installed here) applies by default: its published algorithm
(Badri & Shaji, "Half-Quadratic Quantization of Large Machine Learning Models", 2023;
``optimize_weights_proximal`` with lp_norm 0.7, beta 10, kappa 1.01, 20 iterations, stop when the mean
absolute error stops falling) restated, NOT checked against hqq's output: parity unpinned.  The
kernels only rely on the affine dequantization ``(Wq - z) * s``, whichever zero point is stored.
"""
from __future__ import annotations

from typing import Dict, Optional, Tuple

import torch
import torch.nn as nn

from . import ops

GROUP = 64


HQQ_OPT_PARAMS = {"lp_norm": 0.7, "beta": 1e1, "kappa": 1.01, "iters": 20}     # hqq's defaults


def refine_zero_proximal(w: torch.Tensor, s: torch.Tensor, zero: torch.Tensor, opt_params: Optional[dict] = None) -> torch.Tensor:
    """hqq's half-quadratic solver for the zero point, scale fixed: ``w`` [N, G, 64] fp32, ``s`` / ``zero`` [N, G] fp32.
    Alternates  W_e = shrink_lp(W - W_r)  (the generalized soft threshold of the l_p error, p < 1)  and
    zero = mean(Wq - (W - W_e) / s)  over the group, with beta growing by kappa, until the mean absolute
    reconstruction error stops falling.  Returns the refined zero [N, G] fp32."""
    p = dict(HQQ_OPT_PARAMS, **(opt_params or {}))
    lp, beta, kappa, iters = float(p["lp_norm"]), float(p["beta"]), float(p["kappa"]), int(p["iters"])
    inv_s = (1.0 / s).unsqueeze(-1)
    z = zero.unsqueeze(-1).clone()
    best_err, best_z = float("inf"), z
    for _ in range(iters):
        wq = torch.clamp(torch.round(w * inv_s + z), 0, 15)
        w_r = (wq - z) / inv_s
        err = float((w - w_r).abs().mean())
        if err < best_err:
            best_err, best_z = err, z
        else:
            break                                             # the error stopped falling: keep the best zero seen
        d = w - w_r
        if lp == 1.0:
            w_e = torch.sign(d) * torch.relu(d.abs() - 1.0 / beta)
        else:
            w_e = torch.sign(d) * torch.relu(d.abs() - (1.0 / beta) * d.abs().clamp_min(1e-30).pow(lp - 1.0))
        z = (wq - (w - w_e) * inv_s).mean(-1, keepdim=True)
        beta *= kappa
    return best_z.squeeze(-1)


def quantize_int4_g64(weight: torch.Tensor, optimize: bool = False,
                      opt_params: Optional[dict] = None) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """``weight`` [N, K] -> (codes uint8 [N, K] in 0..15, scale fp16 [N, K/64], zero fp16 [N, K/64]).
    ``optimize``: refine the zero point as hqq does (see the module text); the codes then follow the refined zero."""
    N, K = weight.shape
    if K % GROUP:
        raise ValueError(f"in_features={K} must be a multiple of {GROUP}")
    w = weight.detach().float().reshape(N, K // GROUP, GROUP)
    lo, hi = w.amin(-1), w.amax(-1)
    scale = ((hi - lo) / 15.0).clamp_min(1e-8).to(torch.float16)
    s = scale.float()
    zero = (-lo / s).to(torch.float16)
    if optimize:
        zero = refine_zero_proximal(w, s, zero.float(), opt_params).to(torch.float16)
    codes = torch.clamp(torch.round(w / s.unsqueeze(-1) + zero.float().unsqueeze(-1)), 0, 15).to(torch.uint8)
    return codes.reshape(N, K), scale, zero


def dequantize(codes: torch.Tensor, scale: torch.Tensor, zero: torch.Tensor) -> torch.Tensor:
    N, K = codes.shape
    c = codes.float().reshape(N, K // GROUP, GROUP)
    return ((c - zero.float().unsqueeze(-1)) * scale.float().unsqueeze(-1)).reshape(N, K)


def pack_tiled(codes: torch.Tensor, scale: torch.Tensor, zero: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """Tiled device layout consumed by the kernels (see include/subspec_hip.h): returns
    (wq int32 [N/16, K/64, 4, 16, 2], sz int32 [N/16, K/64, 16])."""
    N, K = codes.shape
    if N % 16 or K % GROUP:
        raise ValueError(f"[{N}, {K}]: out_features must be a multiple of 16 and in_features of {GROUP}")
    G = K // GROUP
    # [nt, r, g, c, j, i, parity] : k = 64 g + 16 c + 8 j + 2 i + parity
    q = codes.to(torch.int64).reshape(N // 16, 16, G, 4, 2, 4, 2)
    shifts = torch.tensor([0, 4, 8, 12], dtype=torch.int64, device=codes.device).view(1, 1, 1, 1, 1, 4)
    word = (q[..., 0] << shifts).sum(-1) | ((q[..., 1] << (shifts + 16)).sum(-1))        # [nt, r, g, c, j]
    word = word.permute(0, 2, 3, 1, 4).contiguous()                                        # [nt, g, c, r, j]
    wq = torch.where(word >= 2 ** 31, word - 2 ** 32, word).to(torch.int32)
    s_bits = scale.contiguous().view(torch.int16).to(torch.int64) & 0xFFFF
    z_bits = zero.contiguous().view(torch.int16).to(torch.int64) & 0xFFFF
    both = (s_bits | (z_bits << 16)).reshape(N // 16, 16, G).permute(0, 2, 1).contiguous()
    sz = torch.where(both >= 2 ** 31, both - 2 ** 32, both).to(torch.int32)
    return wq, sz


def from_hqq_tensors(W_q: torch.Tensor, scale: torch.Tensor, zero: torch.Tensor, shape: Tuple[int, int]
                     ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Convert the tensors an ``hqq.core.quantize.HQQLinear`` holds for ``nbits=4, group_size=64, axis=1``
    (the configuration of specdecodes/helpers/recipes/subspec/hqq_4bit_postspec.py:17-58) into
    ``(codes [N, K], scale [N, K/64], zero [N, K/64])`` for ``pack_tiled``.

    hqq (pinned at 0.2.6 by the reference's requirements.txt:7; not installed here, so this follows its
    published layout and is not checked against the package) quantizes ``W.reshape(-1, 64)``: row r of that
    matrix is group ``r % (K/64)`` of output row ``r // (K/64)``, with one ``scale`` / ``zero`` per row
    (``meta['scale']``, ``meta['zero']`` of shape ``[N*K/64, 1]``), and stores the codes with
    ``BitPack.pack_4bit_u8``: the first half of the rows in the high nibble, the second half in the low
    nibble of a uint8 matrix ``[N*K/128, 64]``."""
    N, K = int(shape[0]), int(shape[1])
    if K % GROUP:
        raise ValueError(f"in_features={K} must be a multiple of {GROUP}")
    rows = N * K // GROUP
    if rows % 2:
        raise ValueError("hqq 4-bit packing needs an even number of groups")
    if W_q.dtype != torch.uint8 or W_q.numel() != rows // 2 * GROUP:
        raise ValueError(f"W_q must be the uint8 [{rows // 2}, {GROUP}] matrix of pack_4bit_u8")
    if scale.numel() != rows or zero.numel() != rows:
        raise ValueError(f"scale and zero must hold {rows} entries (one per 64-wide group)")
    packed = W_q.reshape(rows // 2, GROUP)
    codes = torch.cat([packed >> 4, packed & 0x0F], dim=0).reshape(N, K)
    return codes, scale.reshape(N, K // GROUP).to(torch.float16), zero.reshape(N, K // GROUP).to(torch.float16)


def to_hqq_tensors(codes: torch.Tensor, scale: torch.Tensor, zero: torch.Tensor
                   ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Inverse of ``from_hqq_tensors``: (W_q uint8 [N*K/128, 64], scale [N*K/64, 1], zero [N*K/64, 1])."""
    N, K = codes.shape
    rows = N * K // GROUP
    flat = codes.reshape(rows, GROUP).to(torch.uint8)
    W_q = (flat[:rows // 2] << 4) | flat[rows // 2:]
    return W_q, scale.reshape(rows, 1), zero.reshape(rows, 1)


class HqqInt4Linear(nn.Module):
    """Drop-in for ``nn.Linear`` holding tiled int4 weights; forward runs the HIP GEMV / GEMM."""

    def __init__(self, in_features: int, out_features: int, wq: torch.Tensor, sz: torch.Tensor,
                 bias: Optional[torch.Tensor] = None):
        super().__init__()
        self.in_features, self.out_features = in_features, out_features
        self.register_buffer("wq", wq)
        self.register_buffer("sz", sz)
        self.register_buffer("bias", bias)

    @classmethod
    def from_linear(cls, linear: nn.Linear, compute_dtype: torch.dtype = torch.bfloat16, device=None,
                    optimize: bool = False):
        device = device or linear.weight.device
        codes, scale, zero = quantize_int4_g64(linear.weight.data.to(device), optimize=optimize)
        wq, sz = pack_tiled(codes, scale, zero)
        bias = None if linear.bias is None else linear.bias.data.to(device=device, dtype=compute_dtype)
        return cls(linear.in_features, linear.out_features, wq.to(device), sz.to(device), bias)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        rows = x.numel() // x.shape[-1]
        if rows <= 64:
            return ops.int4_linear(x, self.wq, self.sz, self.out_features, self.bias)
        # wider inputs (prefill) are processed in slabs of 64 rows
        flat = x.reshape(rows, x.shape[-1])
        out = [ops.int4_linear(flat[i:i + 64], self.wq, self.sz, self.out_features, self.bias)
               for i in range(0, rows, 64)]
        return torch.cat(out).reshape(*x.shape[:-1], self.out_features)

    def extra_repr(self) -> str:
        return f"in_features={self.in_features}, out_features={self.out_features}, nbits=4, group_size={GROUP}"


class HqqQuantizer:
    """``quantize_model(model, quant_config, compute_dtype, device)`` as the reference recipe calls it
    (specdecodes/helpers/recipes/base_recipe.py:43-52): ``quant_config`` maps module names to a
    per-layer config; every named ``nn.Linear`` is replaced in place.  A config may carry ``"optimize"``
    (default True, as hqq's ``Quantizer.quantize``): refine the zero points with hqq's proximal solver."""

    @staticmethod
    def _params(name: str, cfg) -> dict:
        """nbits / group_size / axis / optimize of one entry: a plain dict, the nested dict hqq's ``BaseQuantizeConfig``
        returns (``{"weight_quant_params": {...}}``), or an object with those attributes."""
        if isinstance(cfg, dict) and isinstance(cfg.get("weight_quant_params"), dict):
            cfg = dict(cfg["weight_quant_params"], **{k: v for k, v in cfg.items() if k == "optimize"})
        get = cfg.get if isinstance(cfg, dict) else (lambda k, d=None: getattr(cfg, k, d))
        p = {"nbits": int(get("nbits", 4)), "group_size": int(get("group_size", GROUP) or GROUP), "axis": int(get("axis", 1)),
             "optimize": bool(get("optimize", True))}
        if p["nbits"] != 4 or p["group_size"] != GROUP or p["axis"] != 1:
            raise ValueError(f"{name}: only nbits=4, group_size={GROUP}, axis=1 is supported "
                             f"(got {p['nbits']}, {p['group_size']}, {p['axis']})")
        return p

    @classmethod
    def quantize_model(cls, model: nn.Module, quant_config: Dict[str, dict], compute_dtype: torch.dtype, device):
        for name, cfg in quant_config.items():
            p = cls._params(name, cfg)
            parent_name, _, child = name.rpartition(".")
            parent = model.get_submodule(parent_name) if parent_name else model
            linear = getattr(parent, child)
            if not isinstance(linear, nn.Linear):
                raise TypeError(f"{name} is {type(linear).__name__}, expected nn.Linear")
            setattr(parent, child, HqqInt4Linear.from_linear(linear, compute_dtype, device, optimize=p["optimize"]))
        return model
