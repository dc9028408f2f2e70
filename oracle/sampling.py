"""Oracle: drawing the target token of a row (do_sample=True).  Test infrastructure only.

The reference warps the logits with HuggingFace's TemperatureLogitsWarper (``scores / temperature``, a
tensor op, so rounded to the logits dtype), takes ``torch.softmax`` in that dtype and draws
``torch.multinomial(probs, 1)`` (specdecodes/models/generators/base.py:116-132, classic_sd.py:111-116,
lossy_tree_verify.py:75-77).  For one sample ``torch.multinomial`` is an exponential race:
``argmax(probs / q)`` with ``q ~ Exp(1)`` per element.  The random stream of torch's generator is
not part of any interface, so the device path fixes its own: Philox4x32-10 (Salmon, Moraes, Dror,
Shaw: "Parallel random numbers: as easy as 1, 2, 3", SC'11; the generator of Random123 1.x) with

    counter = (i // 4, row, offset & 0xffffffff, offset >> 32),   key = (seed & 0xffffffff, seed >> 32)
    u_i     = ((word[i % 4] >> 9) + 0.5) * 2**-23,   E_i = -log(u_i),   token = argmax_i p_i / E_i

(first index on equal keys).  ``philox4x32_10`` is pinned by Random123's known-answer vectors,
``draw_tokens`` by a per-element python loop on tiny rows and by a chi-square test of the drawn
frequencies against the probabilities.
"""
from __future__ import annotations

from typing import Tuple

import numpy as np
import torch

_M0, _M1 = 0xD2511F53, 0xCD9E8D57
_W0, _W1 = 0x9E3779B9, 0xBB67AE85
_MASK = 0xFFFFFFFF


def philox4x32_10(counter, key) -> np.ndarray:
    """``counter`` [..., 4] and ``key`` [..., 2] of 32-bit words (broadcast) -> [..., 4] uint32."""
    c = np.asarray(counter, dtype=np.uint64) & _MASK
    k = np.asarray(key, dtype=np.uint64) & _MASK
    c, k = np.broadcast_arrays(c, k[..., [0, 1, 0, 1]])
    c0, c1, c2, c3 = (c[..., j].copy() for j in range(4))
    k0, k1 = k[..., 0].copy(), k[..., 1].copy()
    for _ in range(10):
        p0 = _M0 * c0                      # 32 x 32 -> 64 bit products fit uint64 exactly
        p1 = _M1 * c2
        c0, c1, c2, c3 = ((p1 >> 32) ^ c1 ^ k0) & _MASK, p1 & _MASK, ((p0 >> 32) ^ c3 ^ k1) & _MASK, p0 & _MASK
        k0, k1 = (k0 + _W0) & _MASK, (k1 + _W1) & _MASK
    return np.stack([c0, c1, c2, c3], axis=-1).astype(np.uint32)


def race_uniforms(row: int, vocab: int, seed: int, offset: int) -> np.ndarray:
    """u_i for every element of global row ``row``: float64 array [vocab], exact values in (0, 1)."""
    groups = (vocab + 3) // 4
    ctr = np.zeros((groups, 4), dtype=np.uint64)
    ctr[:, 0] = np.arange(groups, dtype=np.uint64)
    ctr[:, 1] = row
    ctr[:, 2] = offset & _MASK
    ctr[:, 3] = (offset >> 32) & _MASK
    words = philox4x32_10(ctr, np.array([seed & _MASK, (seed >> 32) & _MASK], dtype=np.uint64))
    w = words.reshape(-1)[:vocab].astype(np.uint64)
    return ((w >> np.uint64(9)).astype(np.float64) + 0.5) * 2.0 ** -23


def warp_probs(logits: torch.Tensor, temperature: float) -> torch.Tensor:
    """softmax(logits / T) in the logits dtype, the quotient rounded to that dtype first
    (TemperatureLogitsWarper is skipped when T == 1: generators/base.py:57-58)."""
    lg = logits.cpu()
    if temperature is not None and float(temperature) != 1.0:
        lg = lg / float(temperature)
    return torch.softmax(lg, dim=-1)


def draw_tokens(probs: torch.Tensor, seed: int, offset: int = 0, first_row: int = 0) -> Tuple[list, list]:
    """One draw per row of ``probs [rows, V]`` (row r is global row ``first_row + r`` of the call).

    Returns (tokens, margins): ``margins[r]`` = (best key - runner-up key) / best key, evaluated in
    float64; a device result computed in fp32 may only differ from ``tokens[r]`` when the margin
    is at rounding level.
    """
    p = probs.detach().cpu().double().numpy()
    rows, vocab = p.shape
    toks, margins = [], []
    for r in range(rows):
        u = race_uniforms(first_row + r, vocab, seed, offset)
        keys = p[r] / -np.log(u)
        best = int(np.argmax(keys))                      # numpy returns the first maximum
        top = keys[best]
        rest = np.delete(keys, best)
        second = float(rest.max()) if rest.size else 0.0
        toks.append(best)
        margins.append(float((top - second) / top) if top > 0 else 0.0)
    return toks, margins
