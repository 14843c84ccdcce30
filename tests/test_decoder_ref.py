"""CPU: the float64 decoder the GPU tests compare with (tests/decoder_ref.py) against library
routines - torch's scaled_dot_product_attention, silu and repeat_interleave in float64 - and
against the properties a causal decoder has."""
import numpy as np
import torch
import torch.nn.functional as F

import decoder_ref


class _Cfg:
    hidden, heads, kv_heads, head_dim, ffn, vocab, eps, rope_theta = 64, 4, 2, 16, 96, 50, 1e-5, 10000.0


def _weights(rng, cfg):
    L = lambda o, i: rng.standard_normal((o, i)) / np.sqrt(i)
    kvd = cfg.kv_heads * cfg.head_dim
    layer = lambda: {"in_norm": 1 + 0.2 * rng.standard_normal(cfg.hidden), "post_norm": 1 + 0.2 * rng.standard_normal(cfg.hidden),
                     "q": L(cfg.hidden, cfg.hidden), "k": L(kvd, cfg.hidden), "v": L(kvd, cfg.hidden),
                     "o": L(cfg.hidden, cfg.hidden), "gate": L(cfg.ffn, cfg.hidden), "up": L(cfg.ffn, cfg.hidden),
                     "down": L(cfg.hidden, cfg.ffn)}
    return {"embed": rng.standard_normal((cfg.vocab, cfg.hidden)), "lm_head": L(cfg.vocab, cfg.hidden),
            "norm": 1 + 0.2 * rng.standard_normal(cfg.hidden), "layers": [layer(), layer()]}


def _torch_forward(W, cfg, ids):
    t = lambda a: torch.from_numpy(np.asarray(a))
    T, D = len(ids), cfg.head_dim
    x = t(W["embed"])[torch.from_numpy(np.asarray(ids))]
    norm = lambda v, w: v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + cfg.eps) * t(w)
    inv_freq = 1.0 / (cfg.rope_theta ** (torch.arange(0, D, 2, dtype=torch.float64) / D))
    emb = torch.outer(torch.arange(T, dtype=torch.float64), inv_freq).repeat(1, 2)
    cos, sin = emb.cos(), emb.sin()
    rot = lambda v: torch.cat((-v[..., D // 2:], v[..., :D // 2]), dim=-1)
    for w in W["layers"]:
        h = norm(x, w["in_norm"])
        q = (h @ t(w["q"]).T).view(T, cfg.heads, D).transpose(0, 1)
        k = (h @ t(w["k"]).T).view(T, cfg.kv_heads, D).transpose(0, 1)
        v = (h @ t(w["v"]).T).view(T, cfg.kv_heads, D).transpose(0, 1)
        q, k = q * cos + rot(q) * sin, k * cos + rot(k) * sin
        rep = cfg.heads // cfg.kv_heads
        a = F.scaled_dot_product_attention(q[None], k.repeat_interleave(rep, 0)[None], v.repeat_interleave(rep, 0)[None],
                                           is_causal=True)[0]
        x = x + a.transpose(0, 1).reshape(T, -1) @ t(w["o"]).T
        h = norm(x, w["post_norm"])
        x = x + (F.silu(h @ t(w["gate"]).T) * (h @ t(w["up"]).T)) @ t(w["down"]).T
    return (norm(x, W["norm"]) @ t(W["lm_head"]).T).numpy()


def test_float64_decoder_matches_library_routines_and_is_causal():
    cfg = _Cfg()
    rng = np.random.default_rng(0)
    W = _weights(rng, cfg)
    ids = rng.integers(0, cfg.vocab, 9)
    lg, caches = decoder_ref.forward(W, cfg, ids)
    assert lg.shape == (9, cfg.vocab) and len(caches) == 2 and caches[0][0].shape == (cfg.kv_heads, 9, cfg.head_dim)
    assert np.abs(lg - _torch_forward(W, cfg, ids)).max() < 1e-10
    # a prefix sees nothing of what follows it
    assert np.abs(decoder_ref.forward(W, cfg, ids[:5])[0] - lg[:5]).max() < 1e-12
    # position 0: rotary is the identity there, so its key is the plain projection
    h0 = W["embed"][ids[0]]
    h0 = h0 / np.sqrt((h0 * h0).mean() + cfg.eps) * W["layers"][0]["in_norm"]
    assert np.abs(caches[0][0][:, 0].reshape(-1) - W["layers"][0]["k"] @ h0).max() < 1e-12
