"""Checkpoint reader/writer for the reference's Hugging Face layout and the quantiser's per-layer
dictionaries.  CPU tests cover the file format and the Wscale folding; the GPU tests run the
loaded model."""
import json
import os

import numpy as np
import pytest
import torch

from qtip_amd import checkpoint as C
from qtip_amd.linear.quantized_linear import QuantizedLinear
from qtip_amd.llama_decode import LlamaConfig, LlamaDecoder


def _tiny(device, skip=('1_k', '0_down'), seed=0, K_v=None):
    cfg = LlamaConfig(hidden=256, heads=4, kv_heads=2, layers=2, ffn=512, vocab=96, K=2)
    return LlamaDecoder(cfg, 64, seed=seed, device=device, fused=False, skip=skip, K_v=K_v)


def _state(model):
    return {k: (v.detach().cpu() if isinstance(v, torch.Tensor) else torch.tensor(v))
            for k, v in C._targets(model).items()}


@pytest.mark.parametrize("shard_bytes", [4 << 30, 100000])
def test_save_load_round_trip_cpu(tmp_path, shard_bytes):
    model = _tiny('cpu', K_v=3)
    l3 = {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
          "original_max_position_embeddings": 8192}
    model.cfg.rope_scaling = dict(l3)
    for layer in model.layers:  # skipped projections and norms get non-trivial values
        layer.input_norm.weight.data.uniform_(0.5, 1.5)
        for mod in layer.children():
            if isinstance(mod, torch.nn.Linear):
                mod.weight.data.normal_(0, 0.05)
    C.save_llama(model, str(tmp_path), max_shard_bytes=shard_bytes)
    files = sorted(os.listdir(tmp_path))
    assert 'config.json' in files
    if shard_bytes < 1 << 20:
        assert 'model.safetensors.index.json' in files and sum(f.endswith('.safetensors') for f in files) > 1
    cfg = json.load(open(tmp_path / 'config.json'))
    assert cfg['quip_params']['skip_list'] == ['0_down', '1_k'] and cfg['quip_params']['K_v_proj'] == 3
    loaded = C.load_llama(str(tmp_path), max_cache_len=64, device='cpu')
    assert cfg['rope_scaling'] == l3 and loaded.cfg.rope_scaling == l3
    from qtip_amd.llama_decode import rope_inv_freq
    assert torch.equal(loaded.inv_freq, rope_inv_freq(loaded.cfg))
    a, b = _state(model), _state(loaded)
    assert a.keys() == b.keys()
    for k in a:
        assert a[k].dtype == b[k].dtype and torch.equal(a[k], b[k]), k
    # reference key layout and dtypes
    assert a['model.layers.0.self_attn.q_proj.trellis'].dtype == torch.int16
    assert a['model.layers.0.self_attn.q_proj.SV'].dtype == torch.float32
    assert a['model.layers.0.self_attn.v_proj.trellis'].shape == (8 * 16, 16 * 3)
    assert 'model.layers.1.self_attn.k_proj.weight' in a and 'model.layers.0.mlp.down_proj.weight' in a


def test_load_rejects_foreign_and_incomplete_checkpoints(tmp_path):
    model = _tiny('cpu', skip=())
    C.save_llama(model, str(tmp_path))
    cfg = json.load(open(tmp_path / 'config.json'))
    bad = dict(cfg)
    bad['quip_params'] = dict(cfg['quip_params'], decode_mode='1mad')
    json.dump(bad, open(tmp_path / 'config.json', 'w'))
    with pytest.raises(NotImplementedError):
        C.load_llama(str(tmp_path), 64, 'cpu')
    bad = {k: v for k, v in cfg.items() if k != 'quip_params'}
    json.dump(bad, open(tmp_path / 'config.json', 'w'))
    with pytest.raises(ValueError):
        C.load_llama(str(tmp_path), 64, 'cpu')
    bad = dict(cfg, num_hidden_layers=3)  # tensors of a third layer are missing
    json.dump(bad, open(tmp_path / 'config.json', 'w'))
    with pytest.raises(KeyError):
        C.load_llama(str(tmp_path), 64, 'cpu')
    bad = dict(cfg, intermediate_size=1024)
    json.dump(bad, open(tmp_path / 'config.json', 'w'))
    with pytest.raises(ValueError):
        C.load_llama(str(tmp_path), 64, 'cpu')


@pytest.mark.parametrize("rcp", [None, 0, 1, 2])
def test_unpack_quip_folds_wscale(rcp):
    """lib/utils/data_utils.py:281-307: Wscale goes into SV (plain / column-parallel, per shard for
    rcp 2) or into SU per shard (row-parallel, rcp 1)."""
    fin, fout, shards = 256, 128, 8
    g = torch.Generator().manual_seed(1)
    lin = QuantizedLinear(fin, fout, 16, 16, 16, 2, 2, 9, 'quantlut_sym')
    SU = torch.sign(torch.randn(fin, generator=g)).half()
    SV = torch.sign(torch.randn(fout, generator=g)).half()
    saved = dict(trellis=torch.randint(-32768, 32768, lin.trellis.shape, dtype=torch.int16, generator=g),
                 tlut=torch.randn(512, 2, generator=g), SU=SU, SV=SV)
    if rcp in (1, 2):
        saved['Wscale'] = torch.rand(shards, generator=g) + 0.5
    else:
        saved['Wscale'] = torch.tensor(0.37)
    if rcp is not None:
        saved['rcp'] = torch.tensor(rcp)
        saved['tp_rank'] = torch.tensor(shards)
    C.unpack_quip(lin, saved)
    assert torch.equal(lin.trellis, saved['trellis'])
    assert torch.equal(lin.tlut.data, saved['tlut'].half())
    w = saved['Wscale'].float()
    if rcp == 1:
        assert torch.equal(lin.SU.float(), (SU.float() * w.repeat_interleave(fin // shards)).half().float())
        assert torch.equal(lin.SV, SV.float())
    elif rcp == 2:
        assert torch.equal(lin.SU, SU)
        assert torch.equal(lin.SV, SV.float() * w.repeat_interleave(fout // shards))
    else:
        assert torch.equal(lin.SU, SU)
        assert torch.equal(lin.SV, SV.float() * w)
    if rcp is not None:
        assert int(lin.rcp) == rcp and int(lin.tp_rank) == shards


def _reference_schema_checkpoint(tmp_path, tie=False):
    """A checkpoint written WITHOUT this package's key map: the keys come from
    tests/golden/checkpoint_keys.json (derived from the text of the reference's model/llama.py and
    lib/linear/quantized_linear.py by tests/golden/make_checkpoint_keys.py), the shapes and dtypes
    from QuantizedLinear's constructor in the reference (lib/linear/quantized_linear.py:41-67)."""
    from safetensors.torch import save_file
    schema = json.load(open(os.path.join(os.path.dirname(os.path.abspath(__file__)), 'golden', 'checkpoint_keys.json')))
    ex = schema['example']
    hidden, heads, kv_heads, ffn, vocab, K = 256, 4, 2, 512, 96, 2
    kvd = hidden // heads * kv_heads
    dims = {'q_proj': (hidden, hidden), 'k_proj': (hidden, kvd), 'v_proj': (hidden, kvd), 'o_proj': (hidden, hidden),
            'gate_proj': (hidden, ffn), 'up_proj': (hidden, ffn), 'down_proj': (ffn, hidden)}
    g = torch.Generator().manual_seed(5)
    tensors = {}
    for key in ex['keys']:
        parts = key.split('.')
        leaf, owner = parts[-1], parts[-2]
        if owner in dims:
            fin, fout = dims[owner]
            if leaf == 'trellis':
                t = torch.randint(-32768, 32768, (fout // 16 * (fin // 16), 16 * K), dtype=torch.int16, generator=g)
            elif leaf == 'tlut':
                t = torch.randn(512, 2, generator=g).half()
            elif leaf == 'SU':
                t = torch.sign(torch.randn(fin, generator=g) + 1e-5).half()
            elif leaf == 'SV':
                t = torch.sign(torch.randn(fout, generator=g) + 1e-5) * 0.05
            elif leaf == 'rcp':
                t = torch.tensor(0)
            elif leaf == 'tp_rank':
                t = torch.tensor(8)
            elif leaf == 'weight':  # a projection named in skip_list: dense nn.Linear (out, in)
                t = (torch.randn(fout, fin, generator=g) * 0.05).half()
            else:
                raise AssertionError(key)
        elif owner in ('embed_tokens', 'lm_head'):
            t = (torch.randn(vocab, hidden, generator=g) * 0.02).half()
        else:  # RMSNorm weights
            t = (torch.rand(hidden, generator=g) + 0.5).half()
        tensors[key] = t
    if tie:
        del tensors['lm_head.weight']
    # a buffer older transformers versions wrote and newer ones do not (non-persistent in the reference)
    tensors['model.layers.0.self_attn.rotary_emb.inv_freq'] = torch.ones(hidden // heads // 2)
    save_file(tensors, str(tmp_path / 'model.safetensors'), metadata={'format': 'pt'})
    config = dict(model_type='llama', hidden_size=hidden, num_attention_heads=heads, num_key_value_heads=kv_heads,
                  num_hidden_layers=ex['num_hidden_layers'], intermediate_size=ffn, vocab_size=vocab,
                  rope_theta=10000.0, rms_norm_eps=1e-5, tie_word_embeddings=tie,
                  quip_params=dict(td_x=16, td_y=16, L=16, K=K, V=2, tlut_bits=9, decode_mode='quantlut_sym',
                                   skip_list=ex['skip_list']))
    json.dump(config, open(tmp_path / 'config.json', 'w'))
    return ex, tensors


@pytest.mark.parametrize("tie", [False, True])
def test_loader_reads_the_reference_key_schema(tmp_path, tie):
    ex, tensors = _reference_schema_checkpoint(tmp_path, tie)
    model = C.load_llama(str(tmp_path), max_cache_len=64, device='cpu')
    # the loader's own key map names exactly the reference's state-dict keys
    assert set(C._targets(model)) == set(ex['keys'])
    # and every tensor sits where the reference's module tree puts it
    l0, l1 = model.layers
    t = lambda k: tensors[k]
    assert torch.equal(l0.q_proj.trellis, t('model.layers.0.self_attn.q_proj.trellis'))
    assert torch.equal(l0.v_proj.SU, t('model.layers.0.self_attn.v_proj.SU'))
    assert torch.equal(l0.o.SV, t('model.layers.0.self_attn.o_proj.SV'))
    assert torch.equal(l0.gate_proj.tlut.data, t('model.layers.0.mlp.gate_proj.tlut'))
    assert torch.equal(l1.up_proj.trellis, t('model.layers.1.mlp.up_proj.trellis'))
    assert torch.equal(l1.down.SV, t('model.layers.1.mlp.down_proj.SV'))
    assert isinstance(l1.k_proj, torch.nn.Linear) and torch.equal(l1.k_proj.weight, t('model.layers.1.self_attn.k_proj.weight'))
    assert isinstance(l0.down, torch.nn.Linear) and torch.equal(l0.down.weight, t('model.layers.0.mlp.down_proj.weight'))
    assert torch.equal(l0.input_norm.weight, t('model.layers.0.input_layernorm.weight'))
    assert torch.equal(l1.post_norm.weight, t('model.layers.1.post_attention_layernorm.weight'))
    assert torch.equal(model.norm.weight, t('model.norm.weight'))
    assert torch.equal(model.embed, t('model.embed_tokens.weight'))
    assert torch.equal(model.lm_head, t('model.embed_tokens.weight' if tie else 'lm_head.weight'))
    assert int(l0.q_proj.rcp) == 0 and int(l0.q_proj.tp_rank) == 8


def test_untied_checkpoint_without_lm_head_is_incomplete(tmp_path):
    _reference_schema_checkpoint(tmp_path, tie=True)
    cfg = json.load(open(tmp_path / 'config.json'))
    cfg['tie_word_embeddings'] = False
    json.dump(cfg, open(tmp_path / 'config.json', 'w'))
    with pytest.raises(KeyError):
        C.load_llama(str(tmp_path), 64, 'cpu')


@pytest.mark.gpu
@pytest.mark.parametrize("tie", [False, True])
def test_reference_schema_checkpoint_on_the_gpu_runs_like_its_dense_model(tmp_path, tie):
    """The reference-keyed checkpoint loaded onto the GPU: the logits of the loaded model (module
    path over a prompt, then the fused decode step) against a float64 dense model assembled from the
    checkpoint's own tensors by key - a tensor the loader put in the wrong place changes them."""
    import numpy as np
    import decoder_ref
    from oracle import c_oracle
    from oracle import qtip_oracle as O
    ex, tensors = _reference_schema_checkpoint(tmp_path, tie)
    dev = torch.device('cuda:0')
    model = C.load_llama(str(tmp_path), max_cache_len=32, device=dev)
    assert model.embed.is_cuda and model.layers[0].q_proj.trellis.is_cuda
    f64 = lambda k: tensors[k].numpy().astype(np.float64)

    def dense(prefix):
        if prefix + '.weight' in tensors:
            return f64(prefix + '.weight')
        g = lambda leaf: tensors[prefix + '.' + leaf].numpy()
        return O.dense_equivalent(g('trellis'), g('SU'), g('SV'), g('tlut'), 2, decode_fn=c_oracle.decode)

    layers = []
    for i in range(ex['num_hidden_layers']):
        a, m = f'model.layers.{i}.self_attn.', f'model.layers.{i}.mlp.'
        layers.append({"in_norm": f64(f'model.layers.{i}.input_layernorm.weight'),
                       "post_norm": f64(f'model.layers.{i}.post_attention_layernorm.weight'),
                       "q": dense(a + 'q_proj'), "k": dense(a + 'k_proj'), "v": dense(a + 'v_proj'), "o": dense(a + 'o_proj'),
                       "gate": dense(m + 'gate_proj'), "up": dense(m + 'up_proj'), "down": dense(m + 'down_proj')})
    W = {"embed": f64('model.embed_tokens.weight'), "norm": f64('model.norm.weight'), "layers": layers,
         "lm_head": f64('model.embed_tokens.weight' if tie else 'lm_head.weight')}
    ids = torch.randint(0, 96, (8,), generator=torch.Generator().manual_seed(2))
    ref, _ = decoder_ref.forward(W, model.cfg, ids.numpy())

    def close(got, want):
        d = np.abs(got.astype(np.float64) - want)
        assert d.max() <= 2e-2 * np.abs(want).max() and d.mean() <= 5e-3 * np.abs(want).mean()

    with torch.no_grad():
        lg = model(ids[None, :7].to(dev), torch.arange(7, device=dev))
        close(lg[0].cpu().numpy(), ref[:7])
        got = model.decode_fused(ids[7].view(1, 1).to(dev), torch.tensor([7], device=dev))
        close(got[0, 0].cpu().numpy(), ref[7])


@pytest.mark.gpu
def test_loaded_model_runs_like_the_original(tmp_path):
    from qtip_amd.llama_decode import generate
    dev = torch.device('cuda:0')
    model = _tiny(dev, skip=('1_k',), seed=3)
    C.save_llama(model, str(tmp_path))
    loaded = C.load_llama(str(tmp_path), max_cache_len=64, device=dev)
    ids = torch.randint(0, 96, (1, 9), generator=torch.Generator().manual_seed(0)).to(dev)
    pos = torch.arange(9, device=dev)
    with torch.no_grad():
        a = model(ids, pos)
        b = loaded(ids, pos)
    assert torch.equal(a, b)
    # fused transforms on the separate-projection layout follow the module path
    with torch.no_grad():
        tok = torch.tensor([[5]], device=dev)
        p = torch.tensor([9], device=dev)
        ref = model(tok, p)
        got = loaded.decode_fused(tok, p)
    err = (got - ref).abs().max() / ref.abs().max()
    assert err < 2e-2
    out, _, _ = generate(loaded, ids, 6, use_graph=True, fused=True)
    assert out.shape == (1, 6)
