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
                 eps=1e-5, K=2, rope_scaling=None):
        self.hidden, self.heads, self.kv_heads, self.layers = hidden, heads, kv_heads, layers
        self.ffn, self.vocab, self.rope_theta, self.eps, self.K = ffn, vocab, rope_theta, eps, K
        self.head_dim = hidden // heads
        self.rope_scaling = dict(rope_scaling) if rope_scaling else None
        # key ranges per head of the fused decode attention; generate() sets it from the longest
        # context the run will reach (ops.attention_key_splits)
        self.attn_key_splits = 1


def rope_inv_freq(cfg):
    """Rotary frequencies of the model, fp32 (head_dim / 2,).  `rope_scaling` as in the Hugging Face
    config the reference's LlamaRotaryEmbedding reads (model/llama.py:150-190): none / "default",
    "linear" (frequencies divided by the factor) and "llama3" (the Llama-3.1 rule: long wavelengths
    divided by the factor, a smooth blend in the band between the two wavelength limits).  The types
    that change with the sequence length ("dynamic", ...) are not supported by the static tables of
    the decode loop."""
    inv_freq = 1.0 / (cfg.rope_theta**(torch.arange(0, cfg.head_dim, 2, dtype=torch.float32) / cfg.head_dim))
    rs = cfg.rope_scaling
    kind = (rs.get("rope_type", rs.get("type")) if rs else None) or "default"
    if kind == "default":
        return inv_freq
    if kind == "linear":
        return inv_freq / float(rs["factor"])
    if kind == "llama3":
        factor, lo, hi = float(rs["factor"]), float(rs["low_freq_factor"]), float(rs["high_freq_factor"])
        old_len = float(rs["original_max_position_embeddings"])
        wavelen = 2 * math.pi / inv_freq
        scaled = torch.where(wavelen > old_len / lo, inv_freq / factor, inv_freq)
        smooth = (old_len / wavelen - lo) / (hi - lo)
        blended = (1 - smooth) * scaled / factor + smooth * scaled
        medium = ~(wavelen < old_len / hi) & ~(wavelen > old_len / lo)
        return torch.where(medium, blended, scaled)
    raise NotImplementedError(f"rope_scaling type {kind!r}")


def _qlinear(cfg, fin, fout, gen, device, K=None):
    """A QuantizedLinear of the HYB code; seeded random contents when `gen` is given (the loader
    passes None and fills the buffers from a checkpoint)."""
    lin = QuantizedLinear(fin, fout, 16, 16, 16, K or cfg.K, 2, 9, 'quantlut_sym', dtype=torch.float16)
    if gen is not None:
        with torch.no_grad():
            lin.trellis.copy_(torch.randint(-32768, 32768, lin.trellis.shape, dtype=torch.int16, generator=gen))
            # quantlut_sym gives only the first value of a table entry a random sign
            # (lib/codebook/bitshift.py:72-80), so the second column's mean is the mean of half the
            # weights: a random table leaves a rank-one part mu * 1 1^T in the matrix, which the
            # output transform collects in element 0 of every layer's output (hundreds of sigma for
            # the widest layers; 80 layers of it overflow the fp16 residual).  Trained tables are
            # symmetric; centre the random one.
            tlut = torch.randn(512, 2, generator=gen)
            tlut[:, 1] -= tlut[:, 1].mean()
            lin.tlut.copy_(tlut.half())
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
    """fused=True: one quantized matrix for q/k/v and one for up/gate (the layout the reference's
    README quotes its speed on).  fused=False: the seven separate projections of the reference's
    model/llama.py (q_proj, k_proj, v_proj, o_proj, gate_proj, up_proj, down_proj), the layout of
    its published checkpoints; a projection named in `skip` stays a dense fp16 nn.Linear."""

    def __init__(self, cfg, gen, device, fused=True, skip=(), K_v=None):
        super().__init__()
        d, kvd = cfg.hidden, cfg.kv_heads * cfg.head_dim
        self.cfg = cfg
        self.fused = fused
        self.input_norm = RMSNorm(d, cfg.eps).to(device)
        self.post_norm = RMSNorm(d, cfg.eps).to(device)

        def proj(name, fin, fout, K=None):
            if name in skip:
                return nn.Linear(fin, fout, bias=False, dtype=torch.float16, device=device)
            return _qlinear(cfg, fin, fout, gen, device, K)

        if fused:
            self.qkv = proj('qkv', d, d + 2 * kvd)
            self.up_gate = proj('up_gate', d, 2 * cfg.ffn)
        else:
            self.q_proj = proj('q', d, d)
            self.k_proj = proj('k', d, kvd)
            self.v_proj = proj('v', d, kvd, K_v)
            self.gate_proj = proj('gate', d, cfg.ffn)
            self.up_proj = proj('up', d, cfg.ffn)
        self.o = proj('o', d, d)
        self.down = proj('down', cfg.ffn, d)

    def _qkv(self, h):
        if self.fused:
            return self.qkv(h)
        return torch.cat([self.q_proj(h), self.k_proj(h), self.v_proj(h)], dim=-1)

    def _gate_up(self, h):
        if self.fused:
            return self.up_gate(h)
        return torch.cat([self.gate_proj(h), self.up_proj(h)], dim=-1)

    def forward(self, x, cos, sin, k_cache, v_cache, cache_position, attn_mask):
        cfg = self.cfg
        q_len = x.shape[1]
        h = self.input_norm(x)
        qkv = self._qkv(h)
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
        ug = self._gate_up(h)
        gate, up = ug.split([cfg.ffn, cfg.ffn], dim=-1)
        x = x + self.down(F.silu(gate) * up)
        return x

    def _fused_linears(self):
        if not hasattr(self, "_fused"):
            names = ('qkv', 'o', 'up_gate', 'down') if self.fused else \
                ('q_proj', 'k_proj', 'v_proj', 'o', 'gate_proj', 'up_proj', 'down')
            self._fused = {n: _FusedLinear(getattr(self, n)) for n in names}
        return self._fused

    def decode_fused(self, x, k_cache, v_cache, pos, inv_freq, qkv_parts=None, next_layer=None):
        """One new token, x (1, hidden) fp16, on the fused transforms: 12 launches for the fused
        layout (4 x [transform, matvec, transform] + attention, the attention kernel doing the qkv
        output transform itself), 24 for the separate projections.
        With power-of-two hidden sizes the [transform-out + residual] of o / down and the
        [RMSNorm + transform-in] that follows are one launch and the o projection transforms its
        input inside the matvec (9 per layer); where it pays, that one launch is the following
        matvec itself (7 per layer): `qkv_parts` are then the partial sums of this layer's qkv matvec
        (launched by the previous layer with the layer boundary in its prologue) and `next_layer` the
        layer whose qkv matvec this one launches.  Returns (x, qkv partial sums for the next layer)."""
        cfg = self.cfg
        f = self._fused_linears()
        if self.grouped_ok():
            return self._decode_grouped(x, k_cache, v_cache, pos, inv_freq, qkv_parts, next_layer)
        if self.grouped_plain_ok():
            return self._decode_grouped_plain(x, k_cache, v_cache, pos, inv_freq), None
        if self.fused:
            if qkv_parts is None:
                qkv_parts = f['qkv'].matvec(f['qkv'].transform_in(x, ops.PRE_RMSNORM, self.input_norm.weight, cfg.eps))
            qkv = None if f['qkv'].out_transform_fits_attention(cfg.head_dim) else f['qkv'].transform_out(qkv_parts)
        else:
            qkv = torch.cat([f[n](x, ops.PRE_RMSNORM, self.input_norm.weight, cfg.eps)
                             for n in ('q_proj', 'k_proj', 'v_proj')], dim=-1)
        if qkv is None:
            # the attention kernel transforms the head-sized slices it needs itself
            q = f['qkv']
            attn = ops.decode_attention_rht(qkv_parts, q.SV, (q.m**-0.5) * 32.0, q.br, q.Kr, k_cache, v_cache, pos,
                                            inv_freq, cfg.heads, cfg.kv_heads, cfg.head_dim, key_splits=cfg.attn_key_splits)
        else:
            attn = ops.decode_attention(qkv.reshape(-1), k_cache, v_cache, pos, inv_freq, cfg.heads, cfg.kv_heads,
                                        cfg.head_dim, key_splits=cfg.attn_key_splits)
        if self.fused and f['o'].can_chain_into(f['up_gate']):
            parts = f['o'].matvec_from(attn.reshape(1, -1))
            x, ug_parts = f['o'].chain_matvec(parts, x, f['up_gate'], self.post_norm.weight, cfg.eps)
            ug = f['up_gate'].transform_out_silu(ug_parts)
        else:
            x = f['o'](attn.reshape(1, -1), residual=x)
            if self.fused and not f['up_gate'].dense:
                u = f['up_gate']
                ug = u.transform_out_silu(u.matvec(u.transform_in(x, ops.PRE_RMSNORM, self.post_norm.weight, cfg.eps)))
            elif self.fused:
                ug = f['up_gate'](x, ops.PRE_RMSNORM, self.post_norm.weight, cfg.eps)
            else:
                ug = torch.cat([f[n](x, ops.PRE_RMSNORM, self.post_norm.weight, cfg.eps)
                                for n in ('gate_proj', 'up_proj')], dim=-1)
        # ug: [gate | up], or already fp16(silu(gate)) * up where the output transform paired them
        pre = ops.PRE_SILU_MUL if ug.shape[-1] == 2 * cfg.ffn else ops.PRE_NONE
        nq = next_layer._fused_linears().get('qkv') if (next_layer is not None and next_layer.fused) else None
        if nq is not None and not f['down'].dense and f['down'].can_chain_into(nq):
            parts = f['down'].matvec(f['down'].transform_in(ug, pre))
            return f['down'].chain_matvec(parts, x, nq, next_layer.input_norm.weight, cfg.eps)
        return f['down'](ug, pre, residual=x), None

    # ---- separate projections (the layout of the published checkpoints) in grouped launches

    def grouped_ok(self):
        """Separate q / k / v and gate / up projections that the grouped launches cover: all
        quantized, power-of-two hidden size, equal bit widths inside a group, output transforms
        that fit the attention prologue."""
        if not hasattr(self, "_grouped"):
            ok = not self.fused
            if ok:
                f = self._fused_linears()
                cfg = self.cfg
                ok = (not any(l.dense or l.shard_in or l.shard_out for l in f.values())
                      and cfg.hidden in ops.RHT_IN_MATVEC_SIZES)
                if ok:
                    q, k, v, g, u, o, d = (f[n] for n in ('q_proj', 'k_proj', 'v_proj', 'gate_proj', 'up_proj', 'o',
                                                          'down'))
                    ok = (q.K == k.K == v.K and g.K == u.K and g.m == u.m and g.Kr == u.Kr
                          and all(l.Kl == 1 and l.n == cfg.hidden for l in (q, k, v, g, u))
                          and all(l.out_transform_fits_attention(cfg.head_dim) for l in (q, k, v))
                          and o.Kr == 1 and o.m == cfg.hidden and d.Kr == 1 and d.m == cfg.hidden
                          and all(l.SU.dtype == torch.float16 for l in (q, k, v, g, u)))
                    if ok:
                        self._sv_gate_up = torch.stack([g.SV, u.SV]).contiguous()
            self._grouped = ok
        return self._grouped

    def grouped_plain_ok(self):
        """Separate projections whose hidden size is not one the matvec transforms itself (e.g.
        5120 = 40 x 128): the transforms stay launches of their own, but the projections that
        share an input still share their launches."""
        if not hasattr(self, "_grouped_plain"):
            ok = not self.fused and not self.grouped_ok()
            if ok:
                f = self._fused_linears()
                cfg = self.cfg
                ok = not any(l.dense or l.shard_in or l.shard_out for l in f.values())
                if ok:
                    q, k, v, g, u = (f[n] for n in ('q_proj', 'k_proj', 'v_proj', 'gate_proj', 'up_proj'))
                    ok = (q.K == k.K == v.K and g.K == u.K and g.m == u.m and g.Kr == u.Kr
                          and all(l.n == cfg.hidden and l.Kl == q.Kl for l in (q, k, v, g, u))
                          and all(l.out_transform_fits_attention(cfg.head_dim) for l in (q, k, v))
                          and all(l.SU.dtype == torch.float16 for l in (q, k, v, g, u)))
                    if ok:
                        self._sv_gate_up = torch.stack([g.SV, u.SV]).contiguous()
                        self._su_qkv = torch.stack([q.SU, k.SU, v.SU]).contiguous()
                        self._su_gate_up = torch.stack([g.SU, u.SU]).contiguous()
            self._grouped_plain = ok
        return self._grouped_plain

    def _group_plain(self, names, x, su_rows, norm_weight):
        """Two launches: the input transforms (RMSNorm, one sign vector per projection) and the
        matvecs of the projections `names`, which read the same vector."""
        f = self._fused_linears()
        ls = [f[n] for n in names]
        l0 = ls[0]
        xt = ops.rht_fused_pre_rows(x, su_rows, norm_weight, self.cfg.eps, order=l0.Kl, had_bits=l0.bl,
                                    scale=(l0.n**-0.5) / 32.0)
        return ops.decompress_matvec_group([l.trellis for l in ls], [xt[i] for i in range(len(ls))],
                                           [l.tlut for l in ls], [l.m for l in ls], l0.n, l0.K)

    def _decode_grouped_plain(self, x, k_cache, v_cache, pos, inv_freq):
        """decode_fused for separate projections with a hidden size the matvec does not transform
        itself, 12 launches: [RMSNorm + three input transforms], [q, k, v matvecs], attention with
        the three output transforms in its prologue, o as transform / matvec / transform +
        residual, [RMSNorm + two input transforms], [gate, up matvecs], both output transforms
        (with SiLU * up in the same launch for vectors above 4096), and down as
        [SiLU * up +] transform / matvec / transform + residual."""
        cfg = self.cfg
        f = self._fused_linears()
        qkv = [f[n] for n in ('q_proj', 'k_proj', 'v_proj')]
        qkv_parts = self._group_plain(('q_proj', 'k_proj', 'v_proj'), x, self._su_qkv, self.input_norm.weight)
        views, off = [], 0
        for l in qkv:
            views.append(qkv_parts[:, off:off + l.m])
            off += l.m
        attn = ops.decode_attention_rht3(views, [l.SV for l in qkv], [(l.m**-0.5) * 32.0 for l in qkv],
                                         [l.br for l in qkv], [l.Kr for l in qkv], k_cache, v_cache, pos, inv_freq,
                                         cfg.heads, cfg.kv_heads, cfg.head_dim, key_splits=cfg.attn_key_splits)
        x = f['o'](attn.reshape(1, -1), residual=x)
        gu_parts = self._group_plain(('gate_proj', 'up_proj'), x, self._su_gate_up, self.post_norm.weight)
        h, pre = self._gate_up_out(gu_parts)
        return f['down'](h, pre, residual=x)

    def _gate_up_out(self, gu_parts):
        """(input of down, its pre_mode) from the partial sums (S, 2 * m) of the gate / up matvecs:
        both output transforms with SiLU(gate) * up in one launch where that form exists, else
        [gate | up] for the input transform of down to combine."""
        g = self._fused_linears()['gate_proj']
        parts = gu_parts.view(gu_parts.shape[0], 2, g.m)
        scale = (g.m**-0.5) * 32.0
        if ops.rht_silu_pair_ok(g.m, g.Kr, True):
            return ops.rht_silu_pair(parts, self._sv_gate_up, order=g.Kr, had_bits=g.br,
                                     scale=scale).reshape(1, -1), ops.PRE_NONE
        return ops.rht_post_rows(parts, self._sv_gate_up, order=g.Kr, had_bits=g.br,
                                 scale=scale).reshape(1, -1), ops.PRE_SILU_MUL

    def _group_chain(self, names, prev_parts, prev, residual, norm_weight):
        """One launch: boundary after `prev` (its output transform, residual, RMSNorm) and the
        matvecs of the projections `names`, which share that input."""
        f = self._fused_linears()
        ls = [f[n] for n in names]
        return ops.decompress_matvec_group_chain(
            [l.trellis for l in ls], [l.tlut for l in ls], [l.m for l in ls], ls[0].n, ls[0].K, prev_parts, prev.SV,
            (prev.m**-0.5) * 32.0, residual, norm_weight, self.cfg.eps, [l.SU for l in ls], (ls[0].n**-0.5) / 32.0)

    def _decode_grouped(self, x, k_cache, v_cache, pos, inv_freq, qkv_parts, next_layer):
        """decode_fused for separate projections, 8 launches: [boundary + q, k, v matvecs] (by the
        previous layer), attention with the three output transforms in its prologue, o matvec with
        its input transform, [boundary + gate, up matvecs], both output transforms (with SiLU * up in
        the same launch for vectors above 4096), [SiLU * up +] input transform of down, down
        matvec.  Returns (x, partial sums of the next layer's q, k, v)."""
        cfg = self.cfg
        f = self._fused_linears()
        qkv = [f[n] for n in ('q_proj', 'k_proj', 'v_proj')]
        if qkv_parts is None:  # first layer: no boundary in front of it
            vec = torch.cat([l(x, ops.PRE_RMSNORM, self.input_norm.weight, cfg.eps) for l in qkv], dim=-1)
            attn = ops.decode_attention(vec.reshape(-1), k_cache, v_cache, pos, inv_freq, cfg.heads, cfg.kv_heads,
                                        cfg.head_dim, key_splits=cfg.attn_key_splits)
        else:
            views, off = [], 0
            for l in qkv:
                views.append(qkv_parts[:, off:off + l.m])
                off += l.m
            attn = ops.decode_attention_rht3(views, [l.SV for l in qkv], [(l.m**-0.5) * 32.0 for l in qkv],
                                             [l.br for l in qkv], [l.Kr for l in qkv], k_cache, v_cache, pos, inv_freq,
                                             cfg.heads, cfg.kv_heads, cfg.head_dim, key_splits=cfg.attn_key_splits)
        po = f['o'].matvec_from(attn.reshape(1, -1))
        gu_parts, x = self._group_chain(('gate_proj', 'up_proj'), po, f['o'], x, self.post_norm.weight)
        h, pre = self._gate_up_out(gu_parts)
        pd = f['down'].matvec(f['down'].transform_in(h, pre))
        if next_layer is not None and next_layer.grouped_ok():
            parts, x = next_layer._group_chain(('q_proj', 'k_proj', 'v_proj'), pd, f['down'], x,
                                               next_layer.input_norm.weight)
            return x, parts
        return f['down'].transform_out(pd, residual=x), None


class _FusedLinear:
    """The three launches of a bs=1 QuantizedLinear with the neighbouring element-wise work of
    the decoder layer folded into the two transforms (RMSNorm or SiLU*up on the way in, the
    residual addition on the way out).  A dense nn.Linear (a projection the checkpoint left
    unquantized) gets the same interface on library kernels."""

    def __init__(self, lin):
        self.lin = lin
        self.dense = isinstance(lin, nn.Linear)
        self.shards, self.shard_in, self.shard_out = 1, False, False
        if self.dense:
            return
        if not lin.has_kernel:
            raise NotImplementedError("fused decode needs kernel-packed HYB layers")
        dev = lin.trellis.device
        self.n, self.m, self.K = lin.in_features, lin.out_features, lin.K
        # per-shard transforms (lib/codebook/bitshift.py:437-441,465-469): rcp 1 applies the input
        # transform to each of the tp_rank slices of the input, rcp 2 the output transform to each
        # slice of the output.  Such a side keeps its transform as a launch of its own (tp_rank rows
        # of a smaller transform) and takes no part in the launches that fold transforms into their
        # neighbours.
        rcp = int(lin.rcp)
        self.shards = int(lin.tp_rank) if rcp in (1, 2) else 1
        self.shard_in = rcp == 1 and self.shards > 1
        self.shard_out = rcp == 2 and self.shards > 1
        if (self.shard_in and self.n % self.shards) or (self.shard_out and self.m % self.shards):
            raise NotImplementedError("tp_rank does not divide the sharded side")
        self.trellis = lin.trellis.reshape(-1)
        self.tlut = lin.tlut.data.reshape(-1).contiguous()
        self.SU, self.SV = lin.SU, lin.SV
        self.Kl, self.Kr = lin.K_left, lin.K_right
        self.bl = had_bits(lin.had_left, self.Kl, True, dev) if self.Kl > 1 else None
        self.br = had_bits(lin.had_right, self.Kr, False, dev) if self.Kr > 1 else None

    def _dense(self, x, pre_mode, norm_weight, eps, residual):
        if pre_mode == ops.PRE_RMSNORM:
            h = x.float()
            x = norm_weight * (h * torch.rsqrt(h.pow(2).mean(-1, keepdim=True) + eps)).to(x.dtype)
        elif pre_mode == ops.PRE_SILU_MUL:
            gate, up = x.split(x.shape[-1] // 2, dim=-1)
            x = F.silu(gate) * up
        y = self.lin(x)
        return y if residual is None else residual + y

    def transform_in(self, x, pre_mode=ops.PRE_NONE, norm_weight=None, eps=0.0):
        if self.shard_in:
            if pre_mode == ops.PRE_RMSNORM:
                x = ops.rmsnorm(x.reshape(-1), norm_weight, eps)
            elif pre_mode == ops.PRE_SILU_MUL:
                gate, up = x.reshape(-1).split(x.numel() // 2)
                x = F.silu(gate) * up
            ns = self.n // self.shards
            xf = (x.reshape(-1).float() * self.SU).reshape(self.shards, ns)
            return ops.rht(xf, order=self.Kl, had_bits=self.bl, scale=(ns**-0.5) / 32.0,
                           out_dtype=torch.float16).reshape(1, self.n)
        return ops.rht(x, order=self.Kl, had_bits=self.bl, pre=self.SU, scale=(self.n**-0.5) / 32.0,
                       out_dtype=torch.float16, pre_mode=pre_mode, norm_weight=norm_weight, eps=eps)

    def matvec(self, xt):
        """(S, 1, m) fp32 partial sums."""
        return ops.decompress_matvec_parts(self.trellis, xt.reshape(-1), self.tlut, self.m, self.n, self.K).unsqueeze(1)

    def matvec_from(self, x):
        """matvec(transform_in(x)) for a plain input; one launch when the transform is a power of
        two the matvec kernel computes in its prologue."""
        if (self.Kl == 1 and self.n in ops.RHT_IN_MATVEC_SIZES and x.dtype == torch.float16
                and self.SU.dtype == torch.float16 and not self.shard_in):
            return ops.decompress_matvec_parts_rht(self.trellis, x.reshape(-1), self.SU, (self.n**-0.5) / 32.0,
                                                   self.tlut, self.m, self.n, self.K).unsqueeze(1)
        return self.matvec(self.transform_in(x))

    def transform_out(self, parts, residual=None):
        if self.shard_out:
            y = parts.reshape(parts.shape[0], self.m)
            y = y.sum(0) if y.shape[0] > 1 else y[0]
            ms = self.m // self.shards
            yt = ops.rht(y.reshape(self.shards, ms), order=self.Kr, had_bits=self.br, scale=ms**-0.5,
                         out_dtype=torch.float32).reshape(1, self.m)
            out = (yt * (self.SV * 32.0)).to(torch.float16)
            return out if residual is None else residual + out
        return ops.rht(parts if parts.shape[0] > 1 else parts.reshape(1, self.m), order=self.Kr, had_bits=self.br,
                       post=self.SV, scale=(self.m**-0.5) * 32.0, out_dtype=torch.float16, in_parts=parts.shape[0],
                       residual=residual)

    def transform_out_silu(self, parts):
        """Output transform of a fused up/gate projection; where one launch can pair the halves it
        also applies SiLU(gate) * up and returns (1, m / 2) instead of (1, m)."""
        if not self.shard_out and ops.rht_silu_pair_ok(self.m, self.Kr, False):
            return ops.rht_silu_pair(parts.reshape(parts.shape[0], self.m), self.SV, order=self.Kr, had_bits=self.br,
                                     scale=(self.m**-0.5) * 32.0).reshape(1, -1)
        return self.transform_out(parts)

    def out_transform_fits_attention(self, head_dim):
        """The output transform can run in the attention kernel's prologue (head-sized slices of a
        table-order x power-of-two transform)."""
        p2 = self.m // self.Kr
        return (not self.dense and not self.shard_out and head_dim in (64, 128) and p2 >= head_dim
                and p2 & (p2 - 1) == 0 and self.m <= 16384)

    def can_chain_into(self, nxt):
        """This layer's output transform and `nxt`'s input transform are plain power-of-two
        transforms of one hidden-size vector: one launch does both plus residual and RMSNorm."""
        return (not self.dense and not nxt.dense and self.Kr == 1 and nxt.Kl == 1 and self.m == nxt.n
                and self.m in (2048, 4096, 8192) and not self.shard_out and not nxt.shard_in)

    def chain(self, parts, residual, nxt, norm_weight, eps):
        """(x_new, xt): transform_out(parts) + residual, then nxt.transform_in(RMSNorm(x_new))."""
        return ops.rht_chain(parts, self.SV, (self.m**-0.5) * 32.0, residual, norm_weight, eps, nxt.SU,
                             (nxt.n**-0.5) / 32.0)

    def chain_matvec(self, parts, residual, nxt, norm_weight, eps):
        """(x_new, partial sums of nxt's matvec) from this layer's partial sums: the layer boundary
        runs inside nxt's matvec launch.  (Timed alone, the boundary as a launch of its own followed
        by the plain matvec is ~2 us faster in front of the largest 8192-wide matrices, since every
        workgroup repeats the boundary; inside the decode loop the saved launch wins there too:
        109.7 against 107.8 tok/s on the 70B architecture.)"""
        p, x_new = ops.decompress_matvec_parts_chain(nxt.trellis, nxt.tlut, nxt.m, nxt.n, nxt.K, parts, self.SV,
                                                     (self.m**-0.5) * 32.0, residual, norm_weight, eps, nxt.SU,
                                                     (nxt.n**-0.5) / 32.0)
        return x_new, p.unsqueeze(1)

    def __call__(self, x, pre_mode=ops.PRE_NONE, norm_weight=None, eps=0.0, residual=None):
        if self.dense:
            return self._dense(x, pre_mode, norm_weight, eps, residual)
        if pre_mode == ops.PRE_NONE:
            return self.transform_out(self.matvec_from(x), residual)
        return self.transform_out(self.matvec(self.transform_in(x, pre_mode, norm_weight, eps)), residual)


# the decode attention kernel keeps one score per cache slot in LDS
FUSED_MAX_CACHE_LEN = 4096


def _rotate_half(x):
    x1, x2 = x[..., :x.shape[-1] // 2], x[..., x.shape[-1] // 2:]
    return torch.cat((-x2, x1), dim=-1)


class LlamaDecoder(nn.Module):
    """gen=None (used by the checkpoint loader) leaves every tensor zero / identity."""

    def __init__(self, cfg, max_cache_len, seed=0, device="cuda", fused=True, skip=(), K_v=None, random_init=True):
        super().__init__()
        self.cfg = cfg
        self.fused = fused
        gen = torch.Generator().manual_seed(seed) if random_init else None

        def dense(rows, cols):
            if gen is None:
                return torch.zeros(rows, cols, dtype=torch.float16, device=device)
            return (torch.randn(rows, cols, generator=gen) * 0.02).half().to(device)

        self.embed = dense(cfg.vocab, cfg.hidden)
        self.layers = nn.ModuleList([
            DecoderLayer(cfg, gen, device, fused=fused,
                         skip={n.split('_', 1)[1] for n in skip if n.split('_', 1)[0] == str(i)}, K_v=K_v)
            for i in range(cfg.layers)])
        self.norm = RMSNorm(cfg.hidden, cfg.eps).to(device)
        self.lm_head = dense(cfg.vocab, cfg.hidden)
        self.max_cache_len = max_cache_len
        shape = (1, cfg.kv_heads, max_cache_len, cfg.head_dim)
        self.k_cache = [torch.zeros(shape, dtype=torch.float16, device=device) for _ in range(cfg.layers)]
        self.v_cache = [torch.zeros(shape, dtype=torch.float16, device=device) for _ in range(cfg.layers)]
        self.inv_freq = rope_inv_freq(cfg).to(device)

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

    def supports_fused_decode(self):
        """False when a layer needs what the fused decode step does not cover (a layer that is not
        kernel-packed, or a key / value cache longer than the attention kernel's
        FUSED_MAX_CACHE_LEN slots): generate() then decodes module by module."""
        if self.max_cache_len > FUSED_MAX_CACHE_LEN:
            return False
        try:
            for layer in self.layers:
                layer._fused_linears()
        except NotImplementedError:
            return False
        return True

    def decode_fused(self, tok, pos, float_logits=True):
        """tok (1,1) int64, pos (1,) int64 device tensors -> logits (1, 1, vocab), fused kernels;
        fp32 as the reference returns them, or the fp16 values the lm_head product yields
        (float_logits=False, what the greedy pick reads)."""
        if self.max_cache_len > FUSED_MAX_CACHE_LEN:
            raise ValueError(f"the fused decode step covers caches of up to {FUSED_MAX_CACHE_LEN} slots "
                             f"(this model has {self.max_cache_len}); decode module by module")
        x = self.embed[tok.reshape(-1)]
        qp = None
        for i, layer in enumerate(self.layers):
            nxt = self.layers[i + 1] if i + 1 < len(self.layers) else None
            x, qp = layer.decode_fused(x, self.k_cache[i], self.v_cache[i], pos, self.inv_freq, qp, nxt)
        x = ops.rmsnorm(x, self.norm.weight, self.norm.eps)
        lg = (x @ self.lm_head.T).reshape(1, 1, -1)
        return lg.float() if float_logits else lg


def logits_to_probs(logits, temperature=1.0, top_k=None):
    """softmax(logits / temperature) restricted to the top_k largest logits
    (eval/interactive_gen.py:23-33)."""
    logits = logits / max(temperature, 1e-5)
    if top_k is not None:
        v, _ = torch.topk(logits, min(top_k, logits.size(-1)))
        logits = torch.where(logits < v[..., -1:], float("-inf"), logits)
    return torch.softmax(logits, dim=-1)


def sample(logits, temperature=1.0, top_k=None):
    """One token per row from the last position's distribution, without a host
    synchronisation: argmax(p / Exp(1)) draws from p (eval/interactive_gen.py:15-40)."""
    probs = logits_to_probs(logits[:, -1], temperature, top_k)
    q = torch.empty_like(probs).exponential_(1)
    return torch.argmax(probs / q, dim=-1, keepdim=True), probs


@torch.no_grad()
def generate(model, prompt_ids, max_new_tokens, use_graph=True, fused=True, temperature=None, top_k=None,
             callback=None):
    """Decode max_new_tokens tokens after the prompt.  Returns (token ids, decode seconds, tokens
    per second); throughput is max_new_tokens / decode wall-clock as in
    eval/interactive_gen.py:71-85.  Greedy by default; with `temperature` (and optionally
    `top_k`) tokens are sampled as the reference's generation script does (it uses 0.6 / 5).
    `callback(token)` is called with every new (1, 1) token tensor as soon as it is queued -
    the streaming hook of the interactive script; reading the value synchronises."""
    dev = prompt_ids.device
    n = prompt_ids.shape[1]
    # the last token that is fed back sits at position n + max_new_tokens - 2; past the cache the
    # fused kernels would silently drop its key / value (the position is device memory, nothing
    # on the host sees it), so the whole request is checked here
    if n < 1 or n + max(max_new_tokens, 1) - 1 > model.max_cache_len:
        raise ValueError(f"prompt of {n} tokens + {max_new_tokens} new tokens does not fit the key / value cache "
                         f"of {model.max_cache_len} slots")
    sampling = temperature is not None
    fused = fused and model.supports_fused_decode()

    def pick(lg):
        if sampling:
            return sample(lg, temperature, top_k)[0]
        return lg[:, -1].argmax(-1, keepdim=True)

    logits = model(prompt_ids, torch.arange(n, device=dev))
    tok = pick(logits)
    static_tok = tok.clone()
    static_pos = torch.tensor([n], device=dev)
    # decoding on the fused kernels keeps its bookkeeping on the device: the pick kernel (greedy, or
    # the sampled draw with its counter-based random numbers) writes the next input token, the
    # history slot and the advanced position, so a step is one graph replay and nothing else
    device_sampling = sampling and (top_k is None or top_k <= ops.SAMPLE_PICK_MAX_TOP_K)
    on_device = fused and (not sampling or device_sampling)
    seed = int(torch.randint(0, 2**31 - 1, (1,)).item()) if sampling else 0  # follows torch.manual_seed
    draw_counter = torch.zeros(1, dtype=torch.int64, device=dev)
    history = torch.zeros(max(max_new_tokens, 1), dtype=torch.int64, device=dev)
    history[0] = tok.reshape(-1)[0]
    out = [tok.clone()]
    if callback is not None:
        callback(out[-1])

    def step():
        # (a draw by the framework's generator stays outside the captured graph: a replay would repeat it)
        if on_device:
            lg = model.decode_fused(static_tok, static_pos, float_logits=False)
            if sampling:
                ops.sample_pick(lg.reshape(-1), temperature, top_k, seed, draw_counter, static_tok, static_pos,
                                history, n - 1)
            else:
                ops.greedy_pick(lg.reshape(-1), static_tok, static_pos, history, n - 1)
            return None
        lg = model.decode_fused(static_tok, static_pos) if fused else model(static_tok, static_pos)
        return lg if sampling else pick(lg)

    def capture():
        """Two eager steps (allocations, set-up), then the step recorded into a graph; the decode
        state is put back afterwards, so a capture in the middle of a run leaves it untouched."""
        keep = (static_tok.clone(), static_pos.clone(), history.clone(), draw_counter.clone())
        s = torch.cuda.Stream()
        s.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(s):
            for _ in range(2):
                step()
                if on_device:  # the warm-up steps must not advance the decode
                    static_tok.copy_(keep[0])
                    static_pos.copy_(keep[1])
                    history.copy_(keep[2])
                    draw_counter.copy_(keep[3])
        torch.cuda.current_stream().wait_stream(s)
        # the warm-up wrote the cache slot of the current position with this token's k/v, which the
        # next step rewrites identically
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            nxt = step()
        if on_device:  # capture only records; restore in case the stream ran anything
            static_tok.copy_(keep[0])
            static_pos.copy_(keep[1])
            history.copy_(keep[2])
            draw_counter.copy_(keep[3])
        return g, nxt

    # the fused attention has two forms (one workgroup per head; key ranges for long contexts): a run
    # that crosses ops.ATTN_SPLIT_FROM records its step again there, so short contexts never pay
    # for the second launch of the long form
    splits_at = lambda ctx: ops.attention_key_splits(ctx) if fused else 1
    model.cfg.attn_key_splits = splits_at(n + 1)
    graph = static_next = None
    if use_graph:
        graph, static_next = capture()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    recapture_s = 0.0
    for i in range(max_new_tokens - 1):
        want = splits_at(n + i + 1)  # this step attends to n + i + 1 cache slots
        if want != model.cfg.attn_key_splits:
            model.cfg.attn_key_splits = want
            if graph is not None:
                torch.cuda.synchronize()
                t1 = time.perf_counter()
                graph, static_next = capture()
                torch.cuda.synchronize()
                recapture_s += time.perf_counter() - t1  # recording is set-up, not decoding
        if graph is not None:
            graph.replay()
            nxt = static_next
        else:
            nxt = step()
        if on_device:
            if callback is not None:
                callback(history[i + 1:i + 2].view(1, 1))
            continue
        if sampling:
            nxt = pick(nxt)
        static_tok.copy_(nxt)
        static_pos.add_(1)
        out.append(nxt.clone())
        if callback is not None:
            callback(out[-1])
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0 - recapture_s
    if on_device:
        return history[:max_new_tokens].view(1, -1).clone(), dt, (max_new_tokens - 1) / dt
    return torch.cat(out, dim=1), dt, (max_new_tokens - 1) / dt
