"""CPU: the float32 decoder-layer oracle against what the mathematics fixes."""
import torch

from oracle import attention as oa
from oracle import decoder as od


def _weights(g, H, Q, KV, F, scale=0.05):
    r = lambda *s: torch.randn(*s, generator=g) * scale
    return {"input_norm": torch.rand(H, generator=g) + 0.5, "post_norm": torch.rand(H, generator=g) + 0.5,
            "qkv": r(Q + 2 * KV, H), "qkv_bias": r(Q + 2 * KV), "o": r(H, Q), "gate_up": r(2 * F, H), "down": r(H, F)}


def test_rope_is_a_rotation_and_identity_at_position_zero():
    g = torch.Generator().manual_seed(0)
    t = torch.randn(5, 3, 128, generator=g)
    pos = torch.tensor([0, 1, 7, 100, 4000])
    r = od.rope(t, pos, 1e6)
    assert torch.equal(r[0], t[0])
    assert torch.allclose(r.norm(dim=-1), t.norm(dim=-1), rtol=1e-5)
    # relative-position property: <rope(a, p), rope(b, q)> depends on p - q only
    a, b = torch.randn(1, 1, 128, generator=g), torch.randn(1, 1, 128, generator=g)
    d1 = (od.rope(a, torch.tensor([10]), 1e4) * od.rope(b, torch.tensor([3]), 1e4)).sum()
    d2 = (od.rope(a, torch.tensor([107]), 1e4) * od.rope(b, torch.tensor([100]), 1e4)).sum()
    assert torch.allclose(d1, d2, rtol=1e-3, atol=1e-3)


def test_zero_output_projections_leave_the_stream_and_write_the_cache():
    g = torch.Generator().manual_seed(1)
    H, Hq, Hkv, D, F, n, prefix = 64, 2, 1, 32, 96, 4, 5
    w = _weights(g, H, Hq * D, Hkv * D, F)
    w["o"].zero_()
    w["down"].zero_()
    x = torch.randn(n, H, generator=g)
    kc, vc = torch.zeros(Hkv, 16, D), torch.zeros(Hkv, 16, D)
    pos, rows = torch.arange(prefix, prefix + n), torch.arange(prefix, prefix + n)
    y = od.decoder_layer(x, w, kc, vc, pos, rows, [1, 3, 7, 15], prefix, Hq, Hkv, D, 1e-6, 1e4)
    assert torch.equal(y, x)
    h = od.rms_norm(x, w["input_norm"], 1e-6)
    qkv = h @ w["qkv"].T + w["qkv_bias"]
    k = od.rope(qkv[:, Hq * D:Hq * D + Hkv * D].reshape(n, Hkv, D), pos, 1e4)
    assert torch.allclose(kc[:, prefix:prefix + n], k.transpose(0, 1))
    assert torch.equal(kc[:, :prefix], torch.zeros(Hkv, prefix, D)) and torch.equal(vc[:, prefix + n:], torch.zeros(Hkv, 16 - prefix - n, D))


def test_attention_block_matches_the_attention_oracle():
    g = torch.Generator().manual_seed(2)
    H, Hq, Hkv, D, F, n, prefix = 64, 4, 2, 32, 96, 6, 9
    w = _weights(g, H, Hq * D, Hkv * D, F)
    w["down"].zero_()
    w["o"] = torch.eye(H, Hq * D)                               # x + attention output, H <= Hq * D
    x = torch.randn(n, H, generator=g)
    kc, vc = torch.randn(Hkv, 32, D, generator=g), torch.randn(Hkv, 32, D, generator=g)
    parents = [-1, 0, 0, 1, 1, 3]
    bits = []
    for i, p in enumerate(parents):
        bits.append((1 << i) | (bits[p] if p >= 0 else 0))
    pos = torch.tensor([prefix + d for d in [0, 1, 1, 2, 2, 3]])
    rows = torch.arange(prefix, prefix + n)
    y = od.decoder_layer(x, w, kc, vc, pos, rows, bits, prefix, Hq, Hkv, D, 1e-6, 1e4)
    h = od.rms_norm(x, w["input_norm"], 1e-6)
    q = od.rope((h @ w["qkv"].T + w["qkv_bias"])[:, :Hq * D].reshape(n, Hq, D), pos, 1e4)
    ref = oa.tree_attention(q.transpose(0, 1)[None], kc[None], vc[None], parents, prefix)     # caches hold the new rows
    assert torch.allclose(y - x, ref.reshape(n, Hq * D)[:, :H], rtol=1e-4, atol=1e-5)


def test_many_row_form_equals_the_row_loop():
    """Above 64 rows the oracle evaluates attention for all rows at once (masked scores) instead of row by row; both forms
    on the same 70-row tree (slots beyond 64 in use), the loop form run as two calls' worth of rows over the same cache."""
    g = torch.Generator().manual_seed(7)
    H, Hq, Hkv, D, F, n, prefix = 64, 4, 2, 32, 96, 70, 11
    w = _weights(g, H, Hq * D, Hkv * D, F)
    x = torch.randn(n, H, generator=g)
    parents = [-1] + [int(torch.randint(max(0, i - 9), i, (1,), generator=g)) for i in range(1, n)]
    bits, depth = [], []
    for i, p in enumerate(parents):
        bits.append((1 << i) | (bits[p] if p >= 0 else 0))
        depth.append(0 if p < 0 else depth[p] + 1)
    assert max(b.bit_length() for b in bits) > 64
    pos = torch.tensor([prefix + d for d in depth])
    rows = torch.arange(prefix, prefix + n)
    kc0, vc0 = torch.randn(Hkv, 96, D, generator=g), torch.randn(Hkv, 96, D, generator=g)
    kc, vc = kc0.clone(), vc0.clone()
    y = od.decoder_layer(x, w, kc, vc, pos, rows, bits, prefix, Hq, Hkv, D, 1e-6, 1e4)
    # row loop: the K / V rows of all 70 nodes are in the cache already (kc, vc from the call above), so any window of at
    # most 64 rows sees what it saw in the one call
    parts = []
    for lo, hi in ((0, 40), (40, 70)):
        k2, v2 = kc.clone(), vc.clone()
        parts.append(od.decoder_layer(x[lo:hi], w, k2, v2, pos[lo:hi], rows[lo:hi], bits[lo:hi], prefix, Hq, Hkv, D, 1e-6, 1e4))
        assert torch.allclose(k2, kc, atol=1e-6) and torch.allclose(v2, vc, atol=1e-6)
    assert torch.allclose(torch.cat(parts), y, rtol=1e-5, atol=1e-5)
