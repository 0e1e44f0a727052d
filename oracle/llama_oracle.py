"""CPU restatement of the reference's Llama forward with W4A4 linears.  TEST INFRASTRUCTURE ONLY: imported by
tests/ and nothing else; the product (quest_amd/) never imports this package.

Follows /root/reference/src/models/llama.py:17-62 (RoPE), 65-77 (RMSNorm), 79-118 (SwiGLU MLP), 121-177 (attention,
block), 229-262 (forward) and src/models/base.py:32-60 (fused QKV), with every linear under `transformer` run as
gemm-quest/benchmarks/utils.py:56-101 through `quest_oracle.linear_forward` on weights packed by
`quest_oracle.preprocess_weight` (utils.py:20-49), as gemm-quest/benchmarks/bench_e2e.py:41-70 wires them.

Parity status: the linears are pinned (see quest_oracle.py).  The glue between them (RMSNorm, RoPE, softmax
attention, SiLU, residual adds) is plain torch on the CPU in the reference's op order; torch's CPU and GPU kernels
round bf16 intermediates differently, and a code that sits within that noise of a quantisation step flips, so a
GPU forward is compared with this one to a tolerance on the logits, not bit for bit.
"""
from __future__ import annotations

import math

import torch
from torch.nn import functional as F

from . import quest_oracle as qo


def precompute_freqs_cis(dim: int, end: int, theta: float = 10000.0) -> torch.Tensor:
    """llama.py:17-24."""
    freqs = 1.0 / (theta ** (torch.arange(0, dim, 2)[: dim // 2].float() / dim))
    t = torch.arange(end)
    freqs = torch.outer(t, freqs).float()
    return torch.stack((torch.cos(freqs), torch.sin(freqs)), dim=-1)


def apply_rotary_emb(q, k, freqs_cis):
    """llama.py:43-62, q and k of shape (B, T, nh, hs)."""
    orig = q.dtype
    q = q.float().reshape(*q.shape[:-1], -1, 2)
    k = k.float().reshape(*k.shape[:-1], -1, 2)
    fc = freqs_cis.view(1, q.shape[1], 1, q.shape[3], 2)
    q_cos = q[..., 0] * fc[..., 0] - q[..., 1] * fc[..., 1]
    q_sin = q[..., 0] * fc[..., 1] + q[..., 1] * fc[..., 0]
    k_cos = k[..., 0] * fc[..., 0] - k[..., 1] * fc[..., 1]
    k_sin = k[..., 0] * fc[..., 1] + k[..., 1] * fc[..., 0]
    q_out = torch.stack((q_cos, q_sin), dim=-1).reshape(q.shape).flatten(3)
    k_out = torch.stack((k_cos, k_sin), dim=-1).reshape(k.shape).flatten(3)
    return q_out.to(orig), k_out.to(orig)


def rmsnorm(x, weight, eps):
    """llama.py:71-77."""
    xf = x.float()
    return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)).type_as(x) * weight


class W4A4Linear:
    """bench_e2e.py:41-70: packed once, applied with linear_forward."""

    def __init__(self, weight: torch.Tensor, use_hadamard: bool):
        self.use_hadamard = use_hadamard
        self.packed, self.scale, self.add, _ = qo.preprocess_weight(weight, use_hadamard=use_hadamard)

    def __call__(self, x: torch.Tensor) -> torch.Tensor:
        a = x.contiguous().flatten(end_dim=-2)
        y = qo.linear_forward(a, self.packed, self.scale, self.add, use_hadamard=self.use_hadamard, hadamard='matmul',
                              via='fp32')
        return y.unflatten(0, x.shape[:-1])


class DenseLinear:
    """The unquantised layer (bench_e2e.py:85, mode 'bf16'), for judging the quantised forward against."""

    def __init__(self, weight: torch.Tensor, use_hadamard: bool = False):
        self.weight = weight

    def __call__(self, x: torch.Tensor) -> torch.Tensor:
        return F.linear(x, self.weight)


class FakeQuantLinear:
    """The layer a QuEST-trained checkpoint is evaluated with (src/eval_hswag.py:156-217 of the reference): both
    operands fake-quantised in the rotated space, dense fp32 product, result in the activation dtype."""

    def __init__(self, weight: torch.Tensor, use_hadamard: bool = True):
        self.weight = weight

    def __call__(self, x: torch.Tensor) -> torch.Tensor:
        return qo.fake_quant_linear(x, self.weight).to(x.dtype)


def forward(weights: dict, idx: torch.Tensor, n_layer: int, n_head: int, eps: float, use_hadamard: bool = True,
            all_logits: bool = True, linear: str = 'w4a4') -> torch.Tensor:
    """Logits for ids (B, T).  `weights` maps the reference's parameter names (`transformer.wte.weight`,
    `transformer.h.0.attn.c_attn.weight`, ..., `lm_head.weight`) to CPU tensors in the model dtype.
    linear = 'w4a4' (packed INT4 layers), 'fake_quant' (the training-side evaluation layer) or 'dense'."""
    W4A4Linear = {'w4a4': globals()['W4A4Linear'], 'dense': DenseLinear, 'fake_quant': FakeQuantLinear}[linear]     # noqa: N806
    wte = weights['transformer.wte.weight']
    b, t = idx.shape
    d = wte.size(1)
    x = F.embedding(idx, wte)
    freqs_cis = precompute_freqs_cis(d // n_head, t)
    for i in range(n_layer):
        p = f'transformer.h.{i}.'
        lin = {n: W4A4Linear(weights[p + n + '.weight'], use_hadamard)
               for n in ('attn.c_attn', 'attn.c_proj', 'mlp.w1', 'mlp.w2', 'mlp.c_proj')}
        h = rmsnorm(x, weights[p + 'ln_1.weight'], eps)
        q, k, v = lin['attn.c_attn'](h).split(d, dim=2)
        k = k.view(b, t, n_head, d // n_head)
        q = q.view(b, t, n_head, d // n_head)
        q, k = apply_rotary_emb(q, k, freqs_cis)
        q, k = q.transpose(1, 2), k.transpose(1, 2)
        v = v.view(b, t, n_head, d // n_head).transpose(1, 2)
        att = (q.float() @ k.float().transpose(-2, -1)) * (1.0 / math.sqrt(k.size(-1)))
        mask = torch.tril(torch.ones(t, t, dtype=torch.bool))
        att = F.softmax(att.masked_fill(~mask, float('-inf')), dim=-1)
        y = (att @ v.float()).to(x.dtype).transpose(1, 2).contiguous().view(b, t, d)
        x = x + lin['attn.c_proj'](y)
        h = rmsnorm(x, weights[p + 'ln_2.weight'], eps)
        x = x + lin['mlp.c_proj'](F.silu(lin['mlp.w1'](h)) * lin['mlp.w2'](h))
    x = rmsnorm(x, weights['transformer.ln_f.weight'], eps)
    if not all_logits:
        x = x[:, [-1], :]
    return F.linear(x.float(), weights['lm_head.weight'].float())
