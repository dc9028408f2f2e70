"""Oracle: int4 group-wise dequantization and linear.  Test infrastructure only.

The arithmetic of the reference's quantized linear lives in un-vendored packages
(hqq==0.2.6 HQQLinear on HQQBackend.PYTORCH semantics, gemlite==0.5.1.post1; call sites
specdecodes/helpers/quantizers/hqq/__init__.py:65-66,120): W_r = (W_q - zero) * scale per group of
64 consecutive input features of one output row, then y = x @ W_r^T (+ bias).  The quantizer itself
is parity unpinned; parity is defined on the linear given identical (W_q, scale, zero).
"""
import torch


def dequant(codes: torch.Tensor, scale: torch.Tensor, zero: torch.Tensor, group: int = 64) -> torch.Tensor:
    N, K = codes.shape
    out = torch.empty(N, K, dtype=torch.float32)
    for g in range(K // group):                       # written group by group, independent of the product code
        sl = slice(g * group, (g + 1) * group)
        out[:, sl] = (codes[:, sl].float() - zero[:, g:g + 1].float()) * scale[:, g:g + 1].float()
    return out


def linear(x: torch.Tensor, codes, scale, zero, bias=None) -> torch.Tensor:
    y = x.float() @ dequant(codes, scale, zero).T
    if bias is not None:
        y = y + bias.float()
    return y


def unpack_tiled(wq: torch.Tensor, sz: torch.Tensor, N: int, K: int):
    """Inverse of the device layout, written from the layout's definition (bit positions), used
    to check that packing loses nothing."""
    G = K // 64
    w = wq.to(torch.int64) & 0xFFFFFFFF                 # [nt, g, c, r, j]
    codes = torch.zeros(N // 16, 16, G, 64, dtype=torch.uint8)   # [nt, r, g, k % 64]: row 16 nt + r, k = 64 g + ...
    for c in range(4):
        for j in range(2):
            word = w[:, :, c, :, j].permute(0, 2, 1)    # [nt, r, g]: all tiles and groups at once
            for i in range(4):
                k = 16 * c + 8 * j + 2 * i
                codes[:, :, :, k] = ((word >> (4 * i)) & 0xF).to(torch.uint8)
                codes[:, :, :, k + 1] = ((word >> (16 + 4 * i)) & 0xF).to(torch.uint8)
    codes = codes.reshape(N, K)
    b = sz.to(torch.int64) & 0xFFFFFFFF                 # [nt, g, r]
    s16 = (b & 0xFFFF).to(torch.int32).to(torch.int16) if False else (b & 0xFFFF)
    z16 = (b >> 16) & 0xFFFF
    def to_half(v):
        v = torch.where(v >= 2 ** 15, v - 2 ** 16, v).to(torch.int16)
        return v.view(torch.float16)
    scale = to_half(s16).permute(0, 2, 1).reshape(N, G)
    zero = to_half(z16).permute(0, 2, 1).reshape(N, G)
    return codes, scale, zero
