"""GPU: the whole decoder (module-by-module forward and the fused decode step) against a float64
dense model written from the reference's model code (tests/decoder_ref.py), teacher-forced over
a prompt and several decode steps - logits and key / value caches at every step."""
import numpy as np
import pytest
import torch

import decoder_ref

pytestmark = pytest.mark.gpu


def _rel(got, ref):
    d = np.abs(np.asarray(got, dtype=np.float64) - ref)
    return d.max() / np.abs(ref).max(), d.mean() / np.abs(ref).mean()


# (hidden, heads, kv_heads, ffn, fused): grouped-query heads everywhere; 12 * 64 and 12 * 256 make the
# up / gate and down transforms table orders; hidden 2048 takes the launches with the layer boundary
# inside the matvec and the transforms inside the attention prologue, 256 the launch-per-step path
CASES = [(256, 4, 2, 12 * 64, True), (2048, 16, 4, 12 * 256, True), (2048, 16, 4, 12 * 256, False)]


@pytest.mark.parametrize("hidden,heads,kv_heads,ffn,fused", CASES)
def test_decoder_against_float64_dense_model(hidden, heads, kv_heads, ffn, fused):
    from qtip_amd.llama_decode import LlamaConfig, LlamaDecoder
    cfg = LlamaConfig(hidden=hidden, heads=heads, kv_heads=kv_heads, layers=2, ffn=ffn, vocab=320)
    model = LlamaDecoder(cfg, max_cache_len=32, seed=hidden + fused, fused=fused)
    g = torch.Generator().manual_seed(7)
    with torch.no_grad():
        # norm weights away from 1 and different per norm, so that a norm feeding the wrong
        # projection (or a skipped one) shows
        for mod in [model.norm] + [n for l in model.layers for n in (l.input_norm, l.post_norm)]:
            mod.weight.copy_((1.0 + 0.3 * torch.randn(hidden, generator=g)).half())
    W = decoder_ref.weights_of(model)
    n_prompt, n_steps = 6, 5
    ids = torch.randint(0, cfg.vocab, (n_prompt + n_steps,), generator=g)
    ref_logits, ref_caches = decoder_ref.forward(W, cfg, ids.numpy())

    def check_caches(upto):
        for i, (k_ref, v_ref) in enumerate(ref_caches):
            for got, ref in ((model.k_cache[i], k_ref), (model.v_cache[i], v_ref)):
                mx, mn = _rel(got[0, :, :upto].float().cpu().numpy(), ref[:, :upto])
                assert mx <= 2e-2 and mn <= 5e-3, (i, upto, mx, mn)

    dev_ids = ids.cuda()
    with torch.no_grad():
        lg = model(dev_ids[None, :n_prompt], torch.arange(n_prompt, device="cuda"))
        mx, mn = _rel(lg[0].cpu().numpy(), ref_logits[:n_prompt])
        assert mx <= 2e-2 and mn <= 5e-3, ("prompt", mx, mn)
        check_caches(n_prompt)
        # teacher-forced decode steps: the same token goes through both GPU paths at every position
        for t in range(n_prompt, n_prompt + n_steps):
            tok = dev_ids[t].view(1, 1)
            pos = torch.tensor([t], device="cuda")
            a = model(tok, pos)
            mx, mn = _rel(a[0, 0].cpu().numpy(), ref_logits[t])
            assert mx <= 2e-2 and mn <= 5e-3, ("module", t, mx, mn)
            check_caches(t + 1)
            for c in model.k_cache + model.v_cache:   # the fused step must write this slot itself
                c[:, :, t].zero_()
            b = model.decode_fused(tok, pos)
            mx, mn = _rel(b[0, 0].cpu().numpy(), ref_logits[t])
            assert mx <= 2e-2 and mn <= 5e-3, ("fused", t, mx, mn)
            check_caches(t + 1)
