"""Packed W4A4 checkpoints: the on-disk form of what `preprocess_weight` produces.

The reference keeps packed weights only in memory, as the buffers `w_int_packed`, `w_scale`, `w_add` of its
`Linear4bit` (gemm-quest/benchmarks/bench_e2e.py:53-56, produced by gemm-quest/benchmarks/utils.py:20-49); this
module gives those buffers a stable file layout so that a model is packed once and served many times.

File: one safetensors file.  Tensors, per packed linear `<name>`:
    <name>.w_int_packed   uint8  (N, K/2)   byte j of a row = (q[2j+1] << 4) | (q[2j] & 0xF), two's-complement nibbles
    <name>.w_scale        bf16 or fp16 (N, 1)   step of the INT4 grid of that output channel
    <name>.w_add          int32  (N, 1)     sum of the row's codes + K/2
    <name>.bias           optional, as in the dense model
plus every other parameter of the model under its usual name (embeddings, norms, lm_head).
Metadata (strings): format = "quest-w4a4-v1", hadamard = "1" if the weights were rotated by the block-128
Hadamard transform with factor 2^-3.5 before quantisation (activations must then be rotated too), hadamard_block =
"128", fuse_gate_up, dtype, and the model configuration as JSON under "config".
"""
from __future__ import annotations

import json
from dataclasses import asdict

import torch
from safetensors import safe_open
from safetensors.torch import save_file

from . import harness
from .llama import Llama, LlamaConfig

FORMAT = 'quest-w4a4-v1'


def save_llama(path: str, model: Llama, use_hadamard: bool, fuse_gate_up: bool) -> None:
    """Write a model whose transformer linears are `Linear4bit` (see `llama.quantize_model`)."""
    tensors = {k: v.detach().to('cpu').contiguous() for k, v in model.state_dict().items()}
    dtype = next(model.parameters()).dtype
    meta = {'format': FORMAT, 'hadamard': '1' if use_hadamard else '0', 'hadamard_block': '128',
            'fuse_gate_up': '1' if fuse_gate_up else '0', 'dtype': str(dtype).replace('torch.', ''),
            'config': json.dumps(asdict(model.config))}
    save_file(tensors, path, metadata=meta)


def read_metadata(path: str) -> dict:
    with safe_open(path, framework='pt', device='cpu') as f:
        meta = f.metadata() or {}
    if meta.get('format') != FORMAT:
        raise ValueError(f'{path}: not a {FORMAT} file (format = {meta.get("format")!r})')
    return meta


def load_llama(path: str, device) -> Llama:
    """Rebuild the model around the packed buffers: no dense weight of a packed linear is ever materialised."""
    meta = read_metadata(path)
    config = LlamaConfig(**json.loads(meta['config']))
    dtype = getattr(torch, meta['dtype'])
    use_hadamard = meta['hadamard'] == '1'
    fuse = meta['fuse_gate_up'] == '1'
    model = _skeleton(config, dtype, device, use_hadamard, fuse)
    state = {}
    with safe_open(path, framework='pt', device='cpu') as f:
        for k in f.keys():
            state[k] = f.get_tensor(k)
    model.load_state_dict(state, strict=True)
    return model


def _skeleton(config: LlamaConfig, dtype, device, use_hadamard: bool, fuse_gate_up: bool) -> Llama:
    """The module tree of a packed model with unset storage: dense parts on `device` in `dtype`, linears as empty
    `Linear4bit`."""
    model = Llama(LlamaConfig(**{**asdict(config), 'n_layer': 0})).to(device=device, dtype=dtype)   # embeddings, final norm, lm_head
    model.config = config
    d, h = config.n_embd, config.hidden_dim
    mk = lambda i, o: harness.Linear4bit.empty(i, o, bias=config.bias, device=device, dtype=dtype,   # noqa: E731
                                               use_hadamard=use_hadamard)
    from .llama import LlamaBlock
    for _ in range(config.n_layer):
        with torch.device('meta'):
            block = LlamaBlock(config)
        block.ln_1 = type(block.ln_1)(d, eps=config.rmsnorm_eps).to(device=device, dtype=dtype)
        block.ln_2 = type(block.ln_2)(d, eps=config.rmsnorm_eps).to(device=device, dtype=dtype)
        block.attn.c_attn, block.attn.c_proj = mk(d, 3 * d), mk(d, d)
        if fuse_gate_up:
            block.mlp.w12, block.mlp.w1, block.mlp.w2 = harness.Linear4bit.empty(d, 2 * h, False, device, dtype, use_hadamard), None, None
        else:
            block.mlp.w1 = harness.Linear4bit.empty(d, h, False, device, dtype, use_hadamard)
            block.mlp.w2 = harness.Linear4bit.empty(d, h, False, device, dtype, use_hadamard)
        block.mlp.c_proj = harness.Linear4bit.empty(h, d, False, device, dtype, use_hadamard)
        model.transformer.h.append(block)
    return model
