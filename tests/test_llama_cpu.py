"""CPU checks of the end-to-end row: the oracle's glue around the linears is pinned by properties that a wrong
index, sign or mask would break, the product's module wiring is compared with the oracle's on dense weights, and the
packed checkpoint layout round-trips.  No GPU, no HIP library."""
import math

import pytest
import torch

from oracle import llama_oracle as lo
from quest_amd import checkpoint, llama

CFG = dict(n_layer=2, n_embd=256, n_head=4, vocab_size=384, sequence_length=48)


def tiny_model(dtype=torch.float32, seed=0):
    torch.manual_seed(seed)
    cfg = llama.LlamaConfig(**CFG)
    return llama.Llama(cfg).to(dtype), cfg


def test_config_matches_the_benchmark_model():
    cfg = llama.LlamaConfig()
    assert cfg.hidden_dim == 2816                               # 256 * ceil((2 * 4096 / 3) / 256)
    assert cfg.linear_ops_per_token() == 2 * 12 * 12_845_056    # 12.85 M weights per layer
    assert abs(cfg.linear_ops_per_token() * 32 * 512 - 5.05e12) < 0.01e12


def test_rope_is_a_rotation_that_depends_on_relative_position():
    torch.manual_seed(1)
    hs, t = 32, 24
    fc = lo.precompute_freqs_cis(hs, t)
    q = torch.randn(1, t, 2, hs)
    k = torch.randn(1, t, 2, hs)
    q[0, :, :, :] = q[0, 0]                                      # the same vector at every position
    k[0, :, :, :] = k[0, 0]
    rq, rk = lo.apply_rotary_emb(q, k, fc)
    assert torch.allclose(rq[0, 0], q[0, 0], atol=1e-6)          # position 0: identity
    pair_norm = lambda x: x.reshape(*x.shape[:-1], -1, 2).norm(dim=-1)      # noqa: E731
    assert torch.allclose(pair_norm(rq), pair_norm(q), atol=1e-5)
    dots = torch.einsum('thd,shd->hts', rq[0], rk[0])            # (head, m, n)
    for s in (1, 5):
        assert torch.allclose(dots[:, :-s, :-s], dots[:, s:, s:], atol=1e-4)   # <R_m q, R_n k> depends on m - n only
    # first pair rotates by exactly `position` radians (theta^0 = 1)
    ang = torch.atan2(rq[0, :, 0, 1], rq[0, :, 0, 0]) - math.atan2(q[0, 0, 0, 1], q[0, 0, 0, 0])
    want = torch.arange(t, dtype=torch.float32)
    assert torch.allclose(torch.remainder(ang - want + math.pi, 2 * math.pi) - math.pi, torch.zeros(t), atol=1e-4)


def test_rmsnorm_closed_forms():
    w = torch.linspace(0.5, 1.5, 8)
    x = torch.full((3, 8), -2.0)
    assert torch.allclose(lo.rmsnorm(x, w, 0.0), -w.expand(3, 8))
    x = torch.randn(5, 8)
    y = lo.rmsnorm(x, torch.ones(8), 0.0)
    assert torch.allclose(y.pow(2).mean(-1), torch.ones(5), atol=1e-5)
    assert torch.allclose(lo.rmsnorm(3 * x, w, 0.0), lo.rmsnorm(x, w, 0.0), atol=1e-5)


def test_oracle_forward_is_causal():
    model, cfg = tiny_model()
    weights = {k: v.detach() for k, v in model.state_dict().items()}
    g = torch.Generator().manual_seed(3)
    ids = torch.randint(0, cfg.vocab_size, (2, 16), generator=g)
    a = lo.forward(weights, ids, cfg.n_layer, cfg.n_head, cfg.rmsnorm_eps, linear='dense')
    ids2 = ids.clone()
    ids2[:, 10:] = torch.randint(0, cfg.vocab_size, (2, 6), generator=g)
    b = lo.forward(weights, ids2, cfg.n_layer, cfg.n_head, cfg.rmsnorm_eps, linear='dense')
    assert torch.equal(a[:, :10], b[:, :10])
    assert not torch.equal(a[:, 10:], b[:, 10:])


def test_product_wiring_equals_oracle_wiring_on_dense_weights():
    """Same parameter names, same op order: the dense fp32 forward of quest_amd.llama on the CPU against the oracle."""
    model, cfg = tiny_model()
    weights = {k: v.detach() for k, v in model.state_dict().items()}
    ids = torch.randint(0, cfg.vocab_size, (2, 24), generator=torch.Generator().manual_seed(4))
    want = lo.forward(weights, ids, cfg.n_layer, cfg.n_head, cfg.rmsnorm_eps, linear='dense')
    with torch.no_grad():
        got = model(ids, all_logits=True)['logits']
        last = model(ids)['logits']
    assert torch.allclose(got, want, atol=2e-5, rtol=1e-4)
    assert torch.allclose(last, got[:, [-1], :], atol=1e-5)


def test_w4a4_oracle_forward_tracks_the_dense_forward():
    """INT4 weights and activations perturb the logits, they do not scramble them (a wrong nibble order, a missing
    Hadamard on one side or a misplaced scale would)."""
    model, cfg = tiny_model(torch.bfloat16)
    weights = {k: v.detach() for k, v in model.state_dict().items()}
    ids = torch.randint(0, cfg.vocab_size, (2, 16), generator=torch.Generator().manual_seed(5))
    dense = lo.forward(weights, ids, cfg.n_layer, cfg.n_head, cfg.rmsnorm_eps, linear='dense').double()
    for had in (False, True):
        q = lo.forward(weights, ids, cfg.n_layer, cfg.n_head, cfg.rmsnorm_eps, use_hadamard=had).double()
        cos = torch.nn.functional.cosine_similarity(q.flatten(), dense.flatten(), dim=0)
        assert cos > 0.93, (had, float(cos))          # measured 0.96: INT4 noise of two layers, not scrambling


@pytest.mark.parametrize('fuse', [True, False])
def test_packed_checkpoint_round_trip(tmp_path, fuse):
    cfg = llama.LlamaConfig(**CFG)
    model = checkpoint._skeleton(cfg, torch.bfloat16, 'cpu', True, fuse)
    g = torch.Generator().manual_seed(6)
    with torch.no_grad():
        for k, v in model.state_dict().items():
            if v.dtype == torch.uint8:
                v.copy_(torch.randint(0, 256, v.shape, generator=g, dtype=torch.uint8))
            elif v.dtype == torch.int32:
                v.copy_(torch.randint(-4000, 4000, v.shape, generator=g, dtype=torch.int32))
            else:
                v.copy_(torch.randn(v.shape, generator=g).to(v.dtype))
    path = str(tmp_path / 'model.safetensors')
    checkpoint.save_llama(path, model, use_hadamard=True, fuse_gate_up=fuse)
    meta = checkpoint.read_metadata(path)
    assert meta['format'] == 'quest-w4a4-v1' and meta['hadamard'] == '1' and meta['hadamard_block'] == '128'
    back = checkpoint.load_llama(path, 'cpu')
    a, b = model.state_dict(), back.state_dict()
    assert list(a.keys()) == list(b.keys())
    for k in a:
        assert a[k].dtype == b[k].dtype and torch.equal(a[k], b[k]), k
    packed = [k for k in a if k.endswith('w_int_packed')]
    assert len(packed) == cfg.n_layer * (4 if fuse else 5)
    d, h = cfg.n_embd, cfg.hidden_dim
    assert a['transformer.h.0.attn.c_attn.w_int_packed'].shape == (3 * d, d // 2)
    assert a['transformer.h.0.mlp.c_proj.w_int_packed'].shape == (d, h // 2)
    assert a['transformer.h.0.attn.c_attn.w_add'].dtype == torch.int32
    assert back.config == cfg


def test_load_rejects_other_files(tmp_path):
    from safetensors.torch import save_file
    path = str(tmp_path / 'x.safetensors')
    save_file({'a': torch.zeros(2)}, path, metadata={'format': 'something-else'})
    with pytest.raises(ValueError):
        checkpoint.read_metadata(path)


def test_reference_checkpoint_names_load():
    model, cfg = tiny_model()
    src, _ = tiny_model(seed=9)
    sd = {'_orig_mod.module.' + k: v for k, v in src.state_dict().items()}
    sd['_orig_mod.module.transformer.h.0.attn.c_attn.weight_quantizer.some_buffer'] = torch.zeros(1)
    llama.load_reference_state_dict(model, sd)
    for (ka, va), (kb, vb) in zip(model.state_dict().items(), src.state_dict().items()):
        assert ka == kb and torch.equal(va, vb)
    del sd['_orig_mod.module.lm_head.weight']
    with pytest.raises(KeyError):
        llama.load_reference_state_dict(model, sd)


def test_reference_checkpoint_file_loads_weights_only(tmp_path):
    """A file as the reference's training loop writes it (src/optim/utils.py:245-256: model / optimizer / scheduler /
    itr, parameter names behind the training wrapper's prefix), read back with the weights-only loader."""
    torch.manual_seed(3)
    cfg = llama.LlamaConfig(n_layer=1, n_embd=128, n_head=2, vocab_size=64, sequence_length=16)
    donor = llama.Llama(cfg)
    state = {'_orig_mod.module.' + k: v.detach().clone() for k, v in donor.state_dict().items()}
    path = tmp_path / 'main.pt'
    torch.save({'model': state, 'optimizer': {'state': {}, 'param_groups': [{'lr': 1e-3}]}, 'scheduler': {'last_epoch': 7}, 'itr': 7}, path)
    torch.manual_seed(4)
    model = llama.Llama(cfg)
    llama.load_reference_checkpoint(model, str(path))
    for k, v in donor.state_dict().items():
        assert torch.equal(model.state_dict()[k], v), k
    # a bare state dict is accepted too
    torch.save(state, tmp_path / 'bare.pt')
    torch.manual_seed(5)
    other = llama.Llama(cfg)
    llama.load_reference_checkpoint(other, str(tmp_path / 'bare.pt'))
    assert torch.equal(other.lm_head.weight, donor.lm_head.weight)
