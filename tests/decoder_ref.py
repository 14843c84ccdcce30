"""A float64 Llama-architecture decoder on dense weights, written from the reference's model code
alone - it shares no code with qtip_amd.llama_decode, whose wiring it checks:

  decoder layer   residual + attention(input_layernorm(x)), then residual + mlp(post_attention_layernorm(.))
                  (model/llama.py:966-982)
  RMSNorm         x * rsqrt(mean(x^2) + eps) * weight             (model/llama.py:129-135)
  rotary          inv_freq = theta^(-2i/d); emb = [freqs, freqs]; q*cos + rotate_half(q)*sin with
                  rotate_half(x) = [-x2, x1]                        (model/llama.py:219-237, 264-295)
  attention       heads as (seq, heads, head_dim) views of the projections, key / value heads
                  repeated n_rep times in place (repeat_kv, model/llama.py:405-418), causal
                  softmax(q k^T / sqrt(d)) v, heads concatenated, o_proj (model/llama.py:831-898)
  MLP             down(silu(gate(x)) * up(x))                       (model/llama.py:399-400)
  logits          lm_head(norm(x))                                  (model/llama.py:1466-1467)

Every quantized projection enters as the dense matrix the reference's own formula gives for it
(oracle.dense_equivalent: lib/codebook/bitshift.py:389-413).  No rounding anywhere: the GPU paths
(fp16 activations) are compared with it by tolerance.
"""
import numpy as np

from oracle import c_oracle
from oracle import qtip_oracle as O


def dense_of(lin):
    """float64 (out, in) matrix of a QuantizedLinear module (or of a dense nn.Linear)."""
    if hasattr(lin, "trellis"):
        g = lambda t: t.detach().cpu().numpy()
        return O.dense_equivalent(g(lin.trellis), g(lin.SU), g(lin.SV), g(lin.tlut), int(lin.K),
                                  decode_fn=c_oracle.decode)
    return lin.weight.detach().cpu().numpy().astype(np.float64)


def weights_of(model):
    """The model's parameters as float64 arrays, per layer in the reference's separate form
    (q, k, v, o, gate, up, down); fused matrices are cut by rows."""
    cfg = model.cfg
    d, kvd = cfg.hidden, cfg.kv_heads * cfg.head_dim
    f64 = lambda t: t.detach().cpu().numpy().astype(np.float64)
    layers = []
    for layer in model.layers:
        w = {"in_norm": f64(layer.input_norm.weight), "post_norm": f64(layer.post_norm.weight)}
        if layer.fused:
            qkv = dense_of(layer.qkv)
            w["q"], w["k"], w["v"] = qkv[:d], qkv[d:d + kvd], qkv[d + kvd:]
            ug = dense_of(layer.up_gate)
            w["gate"], w["up"] = ug[:cfg.ffn], ug[cfg.ffn:]
        else:
            for name in ("q", "k", "v", "gate", "up"):
                w[name] = dense_of(getattr(layer, name + "_proj"))
        w["o"], w["down"] = dense_of(layer.o), dense_of(layer.down)
        layers.append(w)
    return {"embed": f64(model.embed), "lm_head": f64(model.lm_head), "norm": f64(model.norm.weight), "layers": layers}


def _rmsnorm(x, w, eps):
    return x / np.sqrt((x * x).mean(-1, keepdims=True) + eps) * w


def _rotate_half(x):
    h = x.shape[-1] // 2
    return np.concatenate([-x[..., h:], x[..., :h]], axis=-1)


def forward(W, cfg, ids):
    """ids: (T,) token ids at positions 0..T-1.  Returns (logits (T, vocab), per layer the rotated
    keys and the values, each (kv_heads, T, head_dim)) - everything float64."""
    T = len(ids)
    D, H, HK = cfg.head_dim, cfg.heads, cfg.kv_heads
    x = W["embed"][np.asarray(ids)]
    inv_freq = 1.0 / (cfg.rope_theta ** (np.arange(0, D, 2, dtype=np.float64) / D))
    freqs = np.arange(T, dtype=np.float64)[:, None] * inv_freq[None, :]
    emb = np.concatenate([freqs, freqs], axis=-1)
    cos, sin = np.cos(emb)[None], np.sin(emb)[None]            # (1, T, D): broadcast over heads
    causal = np.tril(np.ones((T, T), dtype=bool))
    caches = []
    for w in W["layers"]:
        h = _rmsnorm(x, w["in_norm"], cfg.eps)
        q = (h @ w["q"].T).reshape(T, H, D).transpose(1, 0, 2)   # (heads, T, D)
        k = (h @ w["k"].T).reshape(T, HK, D).transpose(1, 0, 2)
        v = (h @ w["v"].T).reshape(T, HK, D).transpose(1, 0, 2)
        q = q * cos + _rotate_half(q) * sin
        k = k * cos + _rotate_half(k) * sin
        caches.append((k, v))
        rep = H // HK
        kk, vv = np.repeat(k, rep, axis=0), np.repeat(v, rep, axis=0)   # head j reads kv head j // rep
        s = q @ kk.transpose(0, 2, 1) / np.sqrt(D)
        s = np.where(causal[None], s, -np.inf)
        p = np.exp(s - s.max(-1, keepdims=True))
        p /= p.sum(-1, keepdims=True)
        a = (p @ vv).transpose(1, 0, 2).reshape(T, H * D)
        x = x + a @ w["o"].T
        h = _rmsnorm(x, w["post_norm"], cfg.eps)
        g, u = h @ w["gate"].T, h @ w["up"].T
        x = x + ((g / (1.0 + np.exp(-g))) * u) @ w["down"].T
    x = _rmsnorm(x, W["norm"], cfg.eps)
    return x @ W["lm_head"].T, caches
