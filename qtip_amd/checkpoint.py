"""Checkpoints of QTIP-quantized Llama models.

Two on-disk forms of the reference are read:

* the Hugging Face directory its `quantize_llama/hfize_llama.py` writes with
  `save_pretrained(safe_serialization=True)` (the form of the published `relaxml/*-QTIP-*`
  models): `config.json` with a `quip_params` block (model/llama.py:306-315, 445-456) and one or
  more `*.safetensors` files whose keys are `model.layers.{i}.self_attn.{q,k,v,o}_proj.*`,
  `model.layers.{i}.mlp.{gate,up,down}_proj.*` with the QuantizedLinear buffers `trellis`, `SU`,
  `SV`, `tlut`, `rcp`, `tp_rank` (lib/linear/quantized_linear.py:41-81), the two RMSNorm weights
  per layer, `model.embed_tokens.weight`, `model.norm.weight` and `lm_head.weight`;
* the per-layer dictionaries of the quantiser (`{i}_{q,k,v,o,up,gate,down}.pt` contents) through
  `unpack_quip`, which folds `Wscale` into the sign vectors as lib/utils/data_utils.py:281-307 does.

Only safetensors and JSON are parsed (nothing is unpickled).  `save_llama` writes the same
Hugging Face form, which is what the tests round-trip through.
"""
import json
import os

import torch
from safetensors import safe_open
from safetensors.torch import save_file

from .linear.quantized_linear import QuantizedLinear
from .llama_decode import LlamaConfig, LlamaDecoder

_ATTN = {'q': 'q_proj', 'k': 'k_proj', 'v': 'v_proj', 'o': 'o_proj'}
_MLP = {'gate': 'gate_proj', 'up': 'up_proj', 'down': 'down_proj'}
_BUFFERS = ('trellis', 'SU', 'SV', 'tlut', 'rcp', 'tp_rank')


def unpack_quip(module, saved_layer):
    """Fill a QuantizedLinear from one quantiser output dictionary (lib/utils/data_utils.py:281-307):
    the scalar (or, for sharded layers, per-shard) `Wscale` is multiplied into SV, or into SU for
    row-parallel layers (rcp == 1)."""
    with torch.no_grad():
        module.trellis.copy_(saved_layer['trellis'])
        if module.tlut is not None:
            module.tlut.copy_(saved_layer['tlut'].float().to(torch.float16))
        SU, SV = saved_layer['SU'].float(), saved_layer['SV'].float()
        Wscale = saved_layer['Wscale'].float()
        if 'rcp' not in saved_layer:
            module.SU.copy_(saved_layer['SU'])
            module.SV.copy_(SV * Wscale)
            return
        rcp = int(saved_layer['rcp'])
        if isinstance(module.rcp, torch.Tensor):
            module.rcp.copy_(saved_layer['rcp'])
            module.tp_rank.copy_(saved_layer['tp_rank'])
        else:  # the module already ran once and holds python ints
            module.rcp, module.tp_rank = rcp, int(saved_layer['tp_rank'])
        shards = int(saved_layer['tp_rank'])
        if rcp == 1:
            module.SU.copy_((SU.reshape(shards, -1) * Wscale.reshape(-1, 1)).reshape(SU.shape))
            module.SV.copy_(SV)
        elif rcp == 2:
            module.SU.copy_(SU)
            module.SV.copy_((SV.reshape(shards, -1) * Wscale.reshape(-1, 1)).reshape(SV.shape))
        else:
            module.SU.copy_(SU)
            module.SV.copy_(SV * Wscale)


def read_config(path):
    """(LlamaConfig, quip_params dict) from a Hugging Face directory."""
    with open(os.path.join(path, 'config.json')) as f:
        c = json.load(f)
    if 'quip_params' not in c:
        raise ValueError(f"{path}/config.json has no quip_params block: not a QTIP checkpoint")
    qp = dict(c['quip_params'])
    want = dict(td_x=16, td_y=16, L=16, V=2, tlut_bits=9, decode_mode='quantlut_sym')
    for key, val in want.items():
        if qp.get(key) != val:
            raise NotImplementedError(f"quip_params[{key!r}] = {qp.get(key)!r}: the decoder is built for {val!r}")
    if qp.get('K') not in (2, 3, 4):
        raise NotImplementedError(f"quip_params['K'] = {qp.get('K')!r}")
    heads = c['num_attention_heads']
    cfg = LlamaConfig(hidden=c['hidden_size'], heads=heads, kv_heads=c.get('num_key_value_heads', heads),
                      layers=c['num_hidden_layers'], ffn=c['intermediate_size'], vocab=c['vocab_size'],
                      rope_theta=float(c.get('rope_theta', 10000.0)), eps=float(c.get('rms_norm_eps', 1e-5)),
                      K=qp['K'], rope_scaling=c.get('rope_scaling'))
    return cfg, qp


def _tensor_files(path):
    index = os.path.join(path, 'model.safetensors.index.json')
    if os.path.exists(index):
        with open(index) as f:
            files = sorted(set(json.load(f)['weight_map'].values()))
    else:
        files = sorted(f for f in os.listdir(path) if f.endswith('.safetensors'))
    if not files:
        raise FileNotFoundError(f"no .safetensors files in {path}")
    return [os.path.join(path, f) for f in files]


def _targets(model):
    """checkpoint key -> destination tensor (or (module, attribute) for scalars)."""
    out = {'model.embed_tokens.weight': model.embed, 'model.norm.weight': model.norm.weight,
           'lm_head.weight': model.lm_head}
    for i, layer in enumerate(model.layers):
        pre = f'model.layers.{i}.'
        out[pre + 'input_layernorm.weight'] = layer.input_norm.weight
        out[pre + 'post_attention_layernorm.weight'] = layer.post_norm.weight
        mods = {'self_attn.q_proj': layer.q_proj, 'self_attn.k_proj': layer.k_proj, 'self_attn.v_proj': layer.v_proj,
                'self_attn.o_proj': layer.o, 'mlp.gate_proj': layer.gate_proj, 'mlp.up_proj': layer.up_proj,
                'mlp.down_proj': layer.down}
        for name, mod in mods.items():
            if isinstance(mod, QuantizedLinear):
                for b in _BUFFERS:
                    out[f'{pre}{name}.{b}'] = getattr(mod, b)
            else:
                out[f'{pre}{name}.weight'] = mod.weight
    return out


def load_llama(path, max_cache_len=2048, device='cuda'):
    """Hugging Face directory of a QTIP Llama -> LlamaDecoder with the separate projections of
    the reference's model (model/llama.py:300-372, 437-531).  Projections in
    quip_params['skip_list'] ('{layer}_{q|k|v|o|up|gate|down}') are dense fp16."""
    cfg, qp = read_config(path)
    with open(os.path.join(path, 'config.json')) as f:
        tied = bool(json.load(f).get('tie_word_embeddings', False))
    skip = tuple(qp.get('skip_list') or ())
    model = LlamaDecoder(cfg, max_cache_len, device=device, fused=False, skip=skip, K_v=qp.get('K_v_proj'),
                         random_init=False)
    targets = _targets(model)
    seen = set()
    with torch.no_grad():
        for fname in _tensor_files(path):
            with safe_open(fname, framework='pt', device='cpu') as f:
                for key in f.keys():
                    if key.endswith('rotary_emb.inv_freq'):
                        continue
                    if key not in targets:
                        raise KeyError(f"{fname}: unexpected tensor {key}")
                    dst, src = targets[key], f.get_tensor(key)
                    if dst.shape != src.shape:
                        raise ValueError(f"{key}: checkpoint shape {tuple(src.shape)}, model {tuple(dst.shape)}")
                    dst.copy_(src.to(dst.dtype))
                    seen.add(key)
    if tied and 'lm_head.weight' not in seen and 'model.embed_tokens.weight' in seen:
        # tied output embedding (LlamaForCausalLM._tied_weights_keys, model/llama.py:1350): the file
        # holds the matrix once, under the embedding's name
        with torch.no_grad():
            model.lm_head.copy_(model.embed)
        seen.add('lm_head.weight')
    missing = sorted(set(targets) - seen)
    if missing:
        raise KeyError(f"checkpoint lacks {len(missing)} tensors, e.g. {missing[:3]}")
    return model


def save_llama(model, path, max_shard_bytes=4 << 30):
    """Write `model` (separate-projection layout) as a Hugging Face directory in the reference's
    key layout; shards like save_pretrained does when the tensors exceed max_shard_bytes."""
    if model.fused:
        raise ValueError("the reference's checkpoint layout has separate q/k/v and gate/up projections")
    os.makedirs(path, exist_ok=True)
    cfg = model.cfg
    skip = []
    for i, layer in enumerate(model.layers):
        for short, attr in (('q', 'q_proj'), ('k', 'k_proj'), ('v', 'v_proj'), ('o', 'o'), ('gate', 'gate_proj'),
                            ('up', 'up_proj'), ('down', 'down')):
            if not isinstance(getattr(layer, attr), QuantizedLinear):
                skip.append(f'{i}_{short}')
    config = dict(model_type='llama', architectures=['LlamaForCausalLM'], hidden_size=cfg.hidden,
                  num_attention_heads=cfg.heads, num_key_value_heads=cfg.kv_heads, num_hidden_layers=cfg.layers,
                  intermediate_size=cfg.ffn, vocab_size=cfg.vocab, rope_theta=cfg.rope_theta, rms_norm_eps=cfg.eps,
                  hidden_act='silu', torch_dtype='float16',
                  quip_params=dict(td_x=16, td_y=16, L=16, K=cfg.K, V=2, tlut_bits=9, decode_mode='quantlut_sym',
                                   skip_list=skip))
    if cfg.rope_scaling:
        config['rope_scaling'] = cfg.rope_scaling
    kv = [l.v_proj.K for l in model.layers if isinstance(l.v_proj, QuantizedLinear)]
    if kv and kv[0] != cfg.K:
        config['quip_params']['K_v_proj'] = kv[0]
    with open(os.path.join(path, 'config.json'), 'w') as f:
        json.dump(config, f, indent=1)
    tensors = {}
    for key, t in _targets(model).items():
        t = t if isinstance(t, torch.Tensor) else torch.tensor(t)
        tensors[key] = t.detach().cpu().contiguous()
    shards, cur, size = [], {}, 0
    for key in sorted(tensors):
        nb = tensors[key].numel() * tensors[key].element_size()
        if cur and size + nb > max_shard_bytes:
            shards.append(cur)
            cur, size = {}, 0
        cur[key] = tensors[key]
        size += nb
    shards.append(cur)
    if len(shards) == 1:
        save_file(shards[0], os.path.join(path, 'model.safetensors'), metadata={'format': 'pt'})
        return
    weight_map = {}
    for n, sh in enumerate(shards):
        name = f'model-{n + 1:05d}-of-{len(shards):05d}.safetensors'
        save_file(sh, os.path.join(path, name), metadata={'format': 'pt'})
        weight_map.update({k: name for k in sh})
    with open(os.path.join(path, 'model.safetensors.index.json'), 'w') as f:
        json.dump({'metadata': {}, 'weight_map': weight_map}, f, indent=1)
