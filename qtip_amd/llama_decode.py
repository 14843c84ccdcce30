"""Minimal Llama-architecture decoder whose every projection is a QuantizedLinear.

Used to measure end-to-end bs=1 decode throughput of the quantized-linear path
(random-init weights; no tokenizer or checkpoint is involved).  The numerical
recipe follows the reference's vendored model:
  RMSNorm      fp32 statistics, cast back, then weight   (model/llama.py:129-135)
  RoPE         fp32 cos/sin cast to fp16, q*cos + rotate_half(q)*sin (model/llama.py:219-237,264-295)
  KV cache     static buffers written at cache_position (model/cache_utils.py:1173-1193)
  attention    scaled dot product over the cache        (model/llama.py:831-898)
  MLP          down(silu(gate(x)) * up(x))              (model/llama.py:399-400)
  logits       fp16 lm_head, returned in fp32            (model/llama.py:1466-1467)
q/k/v and up/gate are fused into single quantized matrices (the configuration
the reference's README quotes its decode speed on); lm_head and the embedding
stay dense fp16.  Decode steps are recorded into one HIP graph, as the
reference does with torch.compile(mode="max-autotune") (eval/interactive_gen.py:147-149).
"""
import math
import time

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import ops
from .linear.quantized_linear import QuantizedLinear
from .utils.matmul_had import had_bits


class LlamaConfig:

    def __init__(self, hidden=4096, heads=32, kv_heads=32, layers=32, ffn=11008, vocab=32000, rope_theta=10000.0,
                 eps=1e-5, K=2):
        self.hidden, self.heads, self.kv_heads, self.layers = hidden, heads, kv_heads, layers
        self.ffn, self.vocab, self.rope_theta, self.eps, self.K = ffn, vocab, rope_theta, eps, K
        self.head_dim = hidden // heads


def _qlinear(cfg, fin, fout, gen, device):
    lin = QuantizedLinear(fin, fout, 16, 16, 16, cfg.K, 2, 9, 'quantlut_sym', dtype=torch.float16)
    with torch.no_grad():
        lin.trellis.copy_(torch.randint(-32768, 32768, lin.trellis.shape, dtype=torch.int16, generator=gen))
        lin.tlut.copy_(torch.randn(512, 2, generator=gen).half())
        lin.SU.copy_(torch.sign(torch.randn(fin, generator=gen) + 1e-5).half())
        # decoded weights are ~N(0,1): scale so that the layer behaves like a 1/sqrt(fan_in) init
        lin.SV.copy_(torch.sign(torch.randn(fout, generator=gen) + 1e-5) / math.sqrt(fin))
    return lin.to(device)


class RMSNorm(nn.Module):

    def __init__(self, n, eps):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(n, dtype=torch.float16), requires_grad=False)
        self.eps = eps

    def forward(self, x):
        h = x.float()
        h = h * torch.rsqrt(h.pow(2).mean(-1, keepdim=True) + self.eps)
        return self.weight * h.to(x.dtype)


class DecoderLayer(nn.Module):

    def __init__(self, cfg, gen, device):
        super().__init__()
        d, kvd = cfg.hidden, cfg.kv_heads * cfg.head_dim
        self.cfg = cfg
        self.input_norm = RMSNorm(d, cfg.eps).to(device)
        self.post_norm = RMSNorm(d, cfg.eps).to(device)
        self.qkv = _qlinear(cfg, d, d + 2 * kvd, gen, device)
        self.o = _qlinear(cfg, d, d, gen, device)
        self.up_gate = _qlinear(cfg, d, 2 * cfg.ffn, gen, device)
        self.down = _qlinear(cfg, cfg.ffn, d, gen, device)

    def forward(self, x, cos, sin, k_cache, v_cache, cache_position, attn_mask):
        cfg = self.cfg
        q_len = x.shape[1]
        h = self.input_norm(x)
        qkv = self.qkv(h)
        d, kvd = cfg.hidden, cfg.kv_heads * cfg.head_dim
        q, k, v = qkv.split([d, kvd, kvd], dim=-1)
        q = q.view(1, q_len, cfg.heads, cfg.head_dim).transpose(1, 2)
        k = k.view(1, q_len, cfg.kv_heads, cfg.head_dim).transpose(1, 2)
        v = v.view(1, q_len, cfg.kv_heads, cfg.head_dim).transpose(1, 2)
        q = q * cos + _rotate_half(q) * sin
        k = k * cos + _rotate_half(k) * sin
        k_cache.index_copy_(2, cache_position, k)
        v_cache.index_copy_(2, cache_position, v)
        kk, vv = k_cache, v_cache
        if cfg.kv_heads != cfg.heads:
            rep = cfg.heads // cfg.kv_heads
            kk = kk.repeat_interleave(rep, dim=1)
            vv = vv.repeat_interleave(rep, dim=1)
        attn = F.scaled_dot_product_attention(q, kk, vv, attn_mask=attn_mask)
        attn = attn.transpose(1, 2).reshape(1, q_len, d)
        x = x + self.o(attn)
        h = self.post_norm(x)
        ug = self.up_gate(h)
        gate, up = ug.split([cfg.ffn, cfg.ffn], dim=-1)
        x = x + self.down(F.silu(gate) * up)
        return x

    def decode_fused(self, x, k_cache, v_cache, pos, inv_freq):
        """One new token, x (1, hidden) fp16: 13 launches (4 x [transform, matvec, transform] + attention)."""
        cfg = self.cfg
        if not hasattr(self, "_fused"):
            self._fused = [_FusedLinear(l) for l in (self.qkv, self.o, self.up_gate, self.down)]
        qkv_l, o_l, ug_l, down_l = self._fused
        qkv = qkv_l(x, ops.PRE_RMSNORM, self.input_norm.weight, cfg.eps)
        attn = ops.decode_attention(qkv.reshape(-1), k_cache, v_cache, pos, inv_freq, cfg.heads, cfg.kv_heads,
                                    cfg.head_dim)
        x = o_l(attn.reshape(1, -1), residual=x)
        ug = ug_l(x, ops.PRE_RMSNORM, self.post_norm.weight, cfg.eps)
        return down_l(ug, ops.PRE_SILU_MUL, residual=x)


class _FusedLinear:
    """The three launches of a bs=1 QuantizedLinear with the neighbouring element-wise work of
    the decoder layer folded into the two transforms (RMSNorm or SiLU*up on the way in, the
    residual addition on the way out)."""

    def __init__(self, lin):
        dev = lin.trellis.device
        self.lin = lin
        self.n, self.m, self.K = lin.in_features, lin.out_features, lin.K
        self.trellis = lin.trellis.reshape(-1)
        self.tlut = lin.tlut.data.reshape(-1).contiguous()
        self.SU, self.SV = lin.SU, lin.SV
        self.Kl, self.Kr = lin.K_left, lin.K_right
        self.bl = had_bits(lin.had_left, self.Kl, True, dev) if self.Kl > 1 else None
        self.br = had_bits(lin.had_right, self.Kr, False, dev) if self.Kr > 1 else None

    def __call__(self, x, pre_mode=ops.PRE_NONE, norm_weight=None, eps=0.0, residual=None):
        xt = ops.rht(x, order=self.Kl, had_bits=self.bl, pre=self.SU, scale=(self.n**-0.5) / 32.0,
                     out_dtype=torch.float16, pre_mode=pre_mode, norm_weight=norm_weight, eps=eps)
        parts = ops.decompress_matvec_parts(self.trellis, xt.reshape(-1), self.tlut, self.m, self.n, self.K)
        return ops.rht(parts if parts.shape[0] > 1 else parts.reshape(1, self.m), order=self.Kr, had_bits=self.br,
                       post=self.SV, scale=(self.m**-0.5) * 32.0, out_dtype=torch.float16, in_parts=parts.shape[0],
                       residual=residual)


def _rotate_half(x):
    x1, x2 = x[..., :x.shape[-1] // 2], x[..., x.shape[-1] // 2:]
    return torch.cat((-x2, x1), dim=-1)


class LlamaDecoder(nn.Module):

    def __init__(self, cfg, max_cache_len, seed=0, device="cuda"):
        super().__init__()
        self.cfg = cfg
        gen = torch.Generator().manual_seed(seed)
        self.embed = (torch.randn(cfg.vocab, cfg.hidden, generator=gen) * 0.02).half().to(device)
        self.layers = nn.ModuleList([DecoderLayer(cfg, gen, device) for _ in range(cfg.layers)])
        self.norm = RMSNorm(cfg.hidden, cfg.eps).to(device)
        self.lm_head = (torch.randn(cfg.vocab, cfg.hidden, generator=gen) * 0.02).half().to(device)
        self.max_cache_len = max_cache_len
        shape = (1, cfg.kv_heads, max_cache_len, cfg.head_dim)
        self.k_cache = [torch.zeros(shape, dtype=torch.float16, device=device) for _ in range(cfg.layers)]
        self.v_cache = [torch.zeros(shape, dtype=torch.float16, device=device) for _ in range(cfg.layers)]
        inv_freq = 1.0 / (cfg.rope_theta**(torch.arange(0, cfg.head_dim, 2, dtype=torch.float32) / cfg.head_dim))
        self.inv_freq = inv_freq.to(device)

    def rope(self, positions):
        freqs = positions.float()[:, None] * self.inv_freq[None, :]
        emb = torch.cat((freqs, freqs), dim=-1)
        return emb.cos().half()[None, None], emb.sin().half()[None, None]

    def forward(self, ids, cache_position):
        """ids (1, q_len) int64, cache_position (q_len,) int64 -> logits (1, q_len, vocab) fp32."""
        x = self.embed[ids]
        cos, sin = self.rope(cache_position)
        # a query at position p attends to cache slots <= p
        slots = torch.arange(self.max_cache_len, device=ids.device)
        mask = slots[None, :] <= cache_position[:, None]
        mask = mask[None, None]
        for i, layer in enumerate(self.layers):
            x = layer(x, cos, sin, self.k_cache[i], self.v_cache[i], cache_position, mask)
        x = self.norm(x)
        return (x @ self.lm_head.T).float()

    def decode_fused(self, tok, pos):
        """tok (1,1) int64, pos (1,) int64 device tensors -> logits (1, 1, vocab) fp32, fused kernels."""
        x = self.embed[tok.reshape(-1)]
        for i, layer in enumerate(self.layers):
            x = layer.decode_fused(x, self.k_cache[i], self.v_cache[i], pos, self.inv_freq)
        x = self.norm(x)
        return (x @ self.lm_head.T).float().reshape(1, 1, -1)


@torch.no_grad()
def generate(model, prompt_ids, max_new_tokens, use_graph=True, fused=True):
    """Greedy decode.  Returns (token ids, decode seconds, tokens per second);
    throughput is max_new_tokens / decode wall-clock as in eval/interactive_gen.py:71-85."""
    dev = prompt_ids.device
    n = prompt_ids.shape[1]
    logits = model(prompt_ids, torch.arange(n, device=dev))
    tok = logits[:, -1].argmax(-1, keepdim=True)
    static_tok = tok.clone()
    static_pos = torch.tensor([n], device=dev)
    out = [tok.clone()]

    def step():
        lg = model.decode_fused(static_tok, static_pos) if fused else model(static_tok, static_pos)
        return lg[:, -1].argmax(-1, keepdim=True)

    graph = None
    if use_graph:
        s = torch.cuda.Stream()
        s.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(s):
            for _ in range(2):
                step()
        torch.cuda.current_stream().wait_stream(s)
        # the warm-up wrote cache slot n with this token's k/v, which the timed step rewrites identically
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            static_next = step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(max_new_tokens - 1):
        if graph is not None:
            graph.replay()
            nxt = static_next
        else:
            nxt = step()
        static_tok.copy_(nxt)
        static_pos.add_(1)
        out.append(nxt.clone())
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    return torch.cat(out, dim=1), dt, (max_new_tokens - 1) / dt
