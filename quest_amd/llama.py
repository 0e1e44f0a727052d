"""The Llama-style decoder the reference benchmarks end to end, with every transformer projection as a W4A4
linear on the HIP kernels.

Mirrors the model the reference builds for gemm-quest/benchmarks/bench_e2e.py (src/models/llama.py:17-62 RoPE,
65-77 RMSNorm, 79-118 SwiGLU MLP, 121-177 attention and block, 180-247 model; src/models/base.py:32-60 fused
QKV `c_attn` + `c_proj`; init src/models/base.py:98-104 and llama.py:213-217) and the layer swap of
bench_e2e.py:73-99: only the linears under `transformer` are replaced, `lm_head` stays a dense bf16 matmul.
Module names follow the reference (`transformer.h.<i>.attn.c_attn`, `mlp.w1`, ...), so a state dict of the
reference's model loads by name.

Modes (bench_e2e.py:84-95): 'bf16' dense torch linears, 'int4' packed INT4 weights and the W4A4 kernels,
'noop' the same modules returning zeros (everything but the linears).  Two things differ from the reference's
'int4' wiring, both switchable: gate and up projections (`w1`, `w2`) read the same tensor, so it is quantised
once and multiplied by the concatenated weights in one GEMM (`fuse_gate_up`); the reference launches them
separately (llama.py:89-106, 117-118); and with `fuse_producers` the RMSNorms and the SwiGLU product run inside
the quantising kernels of the linears they feed.
"""
from __future__ import annotations

import math
from dataclasses import dataclass

import torch
from torch import nn
from torch.nn import functional as F

from . import api as quest
from . import harness


@dataclass
class LlamaConfig:
    """Defaults: the 12-layer, d=1024 model of the end-to-end benchmark row."""
    n_layer: int = 12
    n_embd: int = 1024
    n_head: int = 16
    multiple_of: int = 256
    vocab_size: int = 32000
    sequence_length: int = 512
    rmsnorm_eps: float = 1e-5
    init_std: float = 0.02
    bias: bool = False

    @property
    def hidden_dim(self) -> int:
        """llama.py:83-87: 2/3 of 4 d, rounded up to a multiple of `multiple_of` (2816 for d=1024)."""
        h = int(2 * self.n_embd * 4 / 3)
        return self.multiple_of * ((h + self.multiple_of - 1) // self.multiple_of)

    def linear_ops_per_token(self) -> int:
        """Integer operations (2 per multiply-add) of the transformer linears for one token."""
        d, h = self.n_embd, self.hidden_dim
        return 2 * self.n_layer * (d * 3 * d + d * d + 2 * d * h + h * d)


def precompute_freqs_cis(dim: int, end: int, theta: float = 10000.0) -> torch.Tensor:
    """llama.py:17-24: (end, dim/2, 2) cos / sin table."""
    freqs = 1.0 / (theta ** (torch.arange(0, dim, 2)[: dim // 2].float() / dim))
    ang = torch.outer(torch.arange(end), freqs).float()
    return torch.stack((torch.cos(ang), torch.sin(ang)), dim=-1)


def apply_rotary_emb(q: torch.Tensor, k: torch.Tensor, freqs_cis: torch.Tensor):
    """llama.py:43-62: rotate interleaved pairs of q, k (B, T, nh, hs) in fp32, back to the input dtype."""
    dtype = q.dtype
    cos = freqs_cis[..., 0].view(1, q.size(1), 1, -1)
    sin = freqs_cis[..., 1].view(1, q.size(1), 1, -1)

    def rot(x):
        x = x.float().reshape(*x.shape[:-1], -1, 2)
        re = x[..., 0] * cos - x[..., 1] * sin
        im = x[..., 0] * sin + x[..., 1] * cos
        return torch.stack((re, im), dim=-1).flatten(3).to(dtype)

    return rot(q), rot(k)


class RMSNorm(nn.Module):
    """llama.py:65-77."""

    def __init__(self, dim: int, eps: float = 1e-6):
        super().__init__()
        self.eps = eps
        self.weight = nn.Parameter(torch.ones(dim))

    def forward(self, x):
        xf = x.float()
        return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + self.eps)).type_as(x) * self.weight


class LlamaMLP(nn.Module):
    """llama.py:79-118: c_proj(silu(w1 x) * w2 x)."""

    def __init__(self, config: LlamaConfig):
        super().__init__()
        self.w1 = nn.Linear(config.n_embd, config.hidden_dim, bias=False)
        self.w2 = nn.Linear(config.n_embd, config.hidden_dim, bias=False)
        self.c_proj = nn.Linear(config.hidden_dim, config.n_embd, bias=False)
        self.w12 = None          # set by quantize_model(..., fuse_gate_up=True): one module for both
        self.glu = None          # enable_swiglu_epilogue(): w12's packed rows in the order the gated-unit GEMM reads
        self.glu_tiles = None

    def enable_swiglu_epilogue(self):
        """A second copy of the fused gate/up weights with the rows interleaved in eights (four gate rows, then the four
        up rows of the same outputs; `quest.swiglu_interleave_rows`), which lets the GEMM apply silu(gate) * up in
        its epilogue.  Plain tensors, not buffers: they are derived data and stay out of checkpoints."""
        w = self.w12
        p = quest.swiglu_interleave_rows(w.w_int_packed.size(0) // 2, device=w.w_int_packed.device)
        self.glu = (w.w_int_packed[p].contiguous(), w.w_scale[p].contiguous(), w.w_add[p].contiguous())
        self.glu_tiles = None            # the interleaved rows as E2M3 tiles, built on first use

    def swiglu_quantized(self, a_scale, a_int_packed, a_int_row_sum):
        """silu(w1 x) * w2 x, (M, hidden), from the codes of x; the gated unit runs in the GEMM's epilogue when that
        kernel takes the shape, otherwise in the torch expression on the plain GEMM's output."""
        m = a_int_packed.size(0)
        if self.w12.use_noop:
            return torch.zeros(m, self.c_proj.weight.size(1), dtype=a_scale.dtype, device=a_scale.device)
        if self.glu is not None and m > 64 and a_int_packed.size(1) % 64 == 0 and self.w12.bias is None:
            w_packed, w_scale, w_add = self.glu
            return quest.fused_matmul_dequantize_swiglu_int4_int4t(a_int_packed, w_packed, a_int_row_sum, w_add, a_scale, w_scale)
        gate_up = self.w12.forward_quantized(a_scale, a_int_packed, a_int_row_sum)
        h = gate_up.size(-1) // 2
        return F.silu(gate_up[..., :h]) * gate_up[..., h:]

    def swiglu_tiles(self, a_scale, a_tiles):
        """The same from the E2M3 tiles of x, on the FP6 matrix instructions (needs enable_swiglu_epilogue())."""
        w_packed, w_scale, _ = self.glu
        if self.w12.use_noop:
            return torch.zeros(a_scale.numel(), self.c_proj.weight.size(1), dtype=a_scale.dtype, device=a_scale.device)
        if self.glu_tiles is None:
            self.glu_tiles = harness.weight_tiles(w_packed)
        return quest.fused_matmul_dequantize_e2m3(a_tiles, self.glu_tiles, a_scale, w_scale, w_packed.size(1) * 2, swiglu=True)

    def forward(self, x):
        if self.w12 is not None:
            gate_up = self.w12(x)
            h = gate_up.size(-1) // 2
            return self.c_proj(F.silu(gate_up[..., :h]) * gate_up[..., h:])
        return self.c_proj(F.silu(self.w1(x)) * self.w2(x))


class LlamaAttention(nn.Module):
    """base.py:32-60 and llama.py:121-163: fused QKV projection, RoPE on q and k, causal attention, output projection."""

    def __init__(self, config: LlamaConfig):
        super().__init__()
        assert config.n_embd % config.n_head == 0
        self.c_attn = nn.Linear(config.n_embd, 3 * config.n_embd, bias=config.bias)
        self.c_proj = nn.Linear(config.n_embd, config.n_embd, bias=config.bias)
        self.n_head, self.n_embd = config.n_head, config.n_embd
        self.fused_rope = False          # set by quantize_model(..., fuse_producers=True)

    def forward(self, x, freqs_cis):
        return self.attend(self.c_attn(x), freqs_cis)

    def attend(self, qkv, freqs_cis, rotated=False):
        """Everything after the QKV projection: qkv (B, T, 3 d) -> (B, T, d)."""
        return self.c_proj(self.attention_core(qkv, freqs_cis, rotated))

    def attention_core(self, qkv, freqs_cis, rotated=False):
        """Rotary embedding (unless the projection has `rotated` q and k already) and causal attention: qkv (B, T, 3 d)
        -> the input of the output projection (B, T, d)."""
        b, t, c3 = qkv.size()
        c = c3 // 3
        if (rotated or self.fused_rope) and qkv.is_cuda and qkv.is_contiguous():
            # q and k rotated where they lie in the projection's output (one kernel, bit-identical to apply_rotary_emb)
            if not rotated:
                quest.rope_interleaved_(qkv, freqs_cis.contiguous(), 2 * c, c // self.n_head)
            q, k, v = (z.view(b, t, self.n_head, c // self.n_head).transpose(1, 2) for z in qkv.split(self.n_embd, dim=2))
            y = F.scaled_dot_product_attention(q, k, v, attn_mask=None, dropout_p=0.0, is_causal=True)
            return y.transpose(1, 2).contiguous().view(b, t, c)
        q, k, v = qkv.split(self.n_embd, dim=2)
        k = k.view(b, t, self.n_head, c // self.n_head)
        q = q.view(b, t, self.n_head, c // self.n_head)
        q, k = apply_rotary_emb(q, k, freqs_cis)
        q, k = q.transpose(1, 2), k.transpose(1, 2)
        v = v.view(b, t, self.n_head, c // self.n_head).transpose(1, 2)
        y = F.scaled_dot_product_attention(q, k, v, attn_mask=None, dropout_p=0.0, is_causal=True)
        return y.transpose(1, 2).contiguous().view(b, t, c)


class LlamaBlock(nn.Module):
    """llama.py:166-177."""

    def __init__(self, config: LlamaConfig):
        super().__init__()
        self.ln_1 = RMSNorm(config.n_embd, eps=config.rmsnorm_eps)
        self.attn = LlamaAttention(config)
        self.ln_2 = RMSNorm(config.n_embd, eps=config.rmsnorm_eps)
        self.mlp = LlamaMLP(config)

        self.fuse_producers = False      # set by quantize_model: norms and SwiGLU product folded into the quantiser

    def forward(self, x, freqs_cis):
        if self.fuse_producers:
            x, branch = self.forward_fused(x, freqs_cis)
            return x if branch is None else x + branch
        x = x + self.attn(self.ln_1(x), freqs_cis)
        return x + self.mlp(self.ln_2(x))

    def forward_fused(self, x, freqs_cis, branch=None):
        """The same block with each W4A4 linear fed by the kernel that also computes its input: RMSNorm -> codes for
        c_attn and for the fused gate/up projection, silu(gate) * up -> codes for the MLP's c_proj.  Three bf16
        tensors per block (two normalised activations, one SwiGLU product) are never written or re-read, and the
        residual additions run inside the norm kernels: x is the residual stream, updated IN PLACE; `branch`, if
        given, is the previous block's MLP output still to be added to it.  Returns (x, this block's MLP output or
        None): the caller adds the last one (or hands it to the next block); None when the output projection's GEMM has
        added it already."""
        b, t, c = x.shape
        m = b * t
        x2 = x.view(m, c)
        hidden = self.mlp.c_proj.weight.size(1)
        # each producer writes the operand form its GEMM runs fastest on: E2M3 tiles for the FP6 kernel, or packed
        # nibbles and row sums for the INT8 kernels (same codes, same output bits either way)
        rotated = False
        if harness.prefers_e2m3(m, c, 3 * c):
            if branch is None:
                q = quest.rmsnorm_hadamard_quantize_e2m3(x2, self.ln_1.weight, self.ln_1.eps)
            else:
                q = quest.add_rmsnorm_hadamard_quantize_e2m3(x2, branch.view(m, c), self.ln_1.weight, self.ln_1.eps)
            # ... whose GEMM also rotates q and k where the shapes allow (the bits of the separate rotary kernel)
            head_dim = c // self.attn.n_head
            c_attn = self.attn.c_attn
            if (harness.GEMM_ROTATES_QK and self.attn.fused_rope and isinstance(c_attn, harness.Linear4bit)
                    and c_attn.bias is None and not c_attn.use_noop and quest.rope_gemm_fuses(t, 3 * c, 2 * c, head_dim)):
                qkv = c_attn.forward_tiles(*q, rope=(freqs_cis.contiguous(), 2 * c, head_dim))
                rotated = True
            else:
                qkv = c_attn.forward_tiles(*q)
        else:
            if branch is None:
                q = quest.rmsnorm_hadamard_quantize_int4(x2, self.ln_1.weight, self.ln_1.eps)
            else:
                q = quest.add_rmsnorm_hadamard_quantize_int4(x2, branch.view(m, c), self.ln_1.weight, self.ln_1.eps)
            c_attn = self.attn.c_attn
            if (harness.GEMM_ROTATES_QK and self.attn.fused_rope and isinstance(c_attn, harness.Linear4bit)
                    and c_attn.bias is None and not c_attn.use_noop and m % t == 0):
                # (in the GEMM's launch where a tiled kernel takes the shape, as a second launch for a handful of tokens)
                qkv = c_attn.forward_quantized(*q, rope=(freqs_cis.contiguous(), 2 * c, c // self.attn.n_head))
                rotated = True
            else:
                qkv = c_attn.forward_quantized(*q)
        # the attention's output projection: on the FP6 path its GEMM adds into the residual stream itself (the bits of
        # x + c_proj(...)) and the second norm has no addition left to do; otherwise the norm kernel adds
        att = None
        gemm_adds = harness.GEMM_ADDS_RESIDUAL
        o_proj = self.attn.c_proj
        packed_adds = (isinstance(o_proj, harness.Linear4bit) and o_proj.use_hadamard and o_proj.bias is None
                       and not o_proj.quantize_from_fp32)
        if gemm_adds and harness.prefers_e2m3(m, c, c) and isinstance(o_proj, harness.Linear4bit) and o_proj.use_hadamard:
            core = self.attn.attention_core(qkv.view(b, t, 3 * c), freqs_cis, rotated)
            o_proj.forward_tiles(*quest.hadamard_quantize_e2m3(core.view(m, c)), out=x2, add_to_out=True)
        elif gemm_adds and harness.GEMM_ADDS_RESIDUAL_PACKED and packed_adds and quest.gemm_add_fuses(m, c, c, x.device):
            # the same on packed nibbles where the INT8 large-tile kernel takes the projection
            core = self.attn.attention_core(qkv.view(b, t, 3 * c), freqs_cis, rotated)
            o_proj.forward_quantized(*quest.hadamard_quantize_int4(core.view(m, c)), out=x2, add_to_out=True)
        else:
            att = self.attn.attend(qkv.view(b, t, 3 * c), freqs_cis, rotated)
        down_tiles = harness.prefers_e2m3(m, hidden, c)

        def second_norm(tiles: bool):
            if att is None:
                f = quest.rmsnorm_hadamard_quantize_e2m3 if tiles else quest.rmsnorm_hadamard_quantize_int4
                return f(x2, self.ln_2.weight, self.ln_2.eps)
            f = quest.add_rmsnorm_hadamard_quantize_e2m3 if tiles else quest.add_rmsnorm_hadamard_quantize_int4
            return f(x2, att.view(m, c), self.ln_2.weight, self.ln_2.eps)

        if harness.prefers_e2m3(m, c, 2 * hidden):
            q = second_norm(True)
            if self.mlp.glu is not None:
                act = self.mlp.swiglu_tiles(*q)
                q = quest.hadamard_quantize_e2m3(act) if down_tiles else quest.hadamard_quantize_int4(act)
            else:
                gate_up = self.mlp.w12.forward_tiles(*q)
                q = quest.silu_mul_hadamard_quantize_e2m3(gate_up) if down_tiles else quest.silu_mul_hadamard_quantize_int4(gate_up)
        else:
            q = second_norm(False)
            if self.mlp.glu is not None:
                act = self.mlp.swiglu_quantized(*q)
                q = quest.hadamard_quantize_e2m3(act) if down_tiles else quest.hadamard_quantize_int4(act)
            else:
                gate_up = self.mlp.w12.forward_quantized(*q)
                q = quest.silu_mul_hadamard_quantize_e2m3(gate_up) if down_tiles else quest.silu_mul_hadamard_quantize_int4(gate_up)
        if down_tiles and gemm_adds:
            # the MLP's output projection adds into the residual stream as well: nothing is left for the caller to add
            self.mlp.c_proj.forward_tiles(*q, out=x2, add_to_out=True)
            return x, None
        down = self.mlp.c_proj
        if (not down_tiles and gemm_adds and harness.GEMM_ADDS_RESIDUAL_PACKED and isinstance(down, harness.Linear4bit) and down.use_hadamard and down.bias is None
                and not down.quantize_from_fp32 and quest.gemm_add_fuses(m, hidden, c, x.device)):
            down.forward_quantized(*q, out=x2, add_to_out=True)
            return x, None
        y = self.mlp.c_proj.forward_tiles(*q) if down_tiles else self.mlp.c_proj.forward_quantized(*q)
        return x, y.view(b, t, c)


class Llama(nn.Module):
    """llama.py:180-247 without tokenizer, dropout (0 at inference) and loss."""

    def __init__(self, config: LlamaConfig):
        super().__init__()
        self.config = config
        self.freqs_cis = precompute_freqs_cis(config.n_embd // config.n_head, config.sequence_length)
        self.transformer = nn.ModuleDict(dict(
            wte=nn.Embedding(config.vocab_size, config.n_embd),
            h=nn.ModuleList([LlamaBlock(config) for _ in range(config.n_layer)]),
            ln_f=RMSNorm(config.n_embd, eps=config.rmsnorm_eps),
        ))
        self.lm_head = nn.Linear(config.n_embd, config.vocab_size, bias=False)
        self.apply(self._init_weights)
        for name, p in self.named_parameters():
            if name.endswith('c_proj.weight'):
                nn.init.normal_(p, mean=0.0, std=config.init_std / math.sqrt(2 * config.n_layer))

    def _init_weights(self, module):
        if isinstance(module, nn.Linear):
            nn.init.normal_(module.weight, mean=0.0, std=self.config.init_std)
            if module.bias is not None:
                nn.init.zeros_(module.bias)
        elif isinstance(module, nn.Embedding):
            nn.init.normal_(module.weight, mean=0.0, std=self.config.init_std)

    def hidden_states(self, idx: torch.Tensor) -> torch.Tensor:
        """Everything up to and including the final norm: (B, T) ids -> (B, T, d)."""
        t = idx.size(1)
        assert t <= self.config.sequence_length
        x = self.transformer.wte(idx)
        if self.freqs_cis.device != x.device:          # moved once, outside any graph capture (the table stays fp32)
            self.freqs_cis = self.freqs_cis.to(x.device)
        freqs_cis = self.freqs_cis[:t]
        branch = None                                  # a fused block's MLP output, not yet added to the stream
        for block in self.transformer.h:
            if block.fuse_producers and x.is_contiguous():
                x, branch = block.forward_fused(x, freqs_cis, branch)
            else:
                if branch is not None:
                    x, branch = x + branch, None
                x = block(x, freqs_cis)
        if branch is not None:
            x = x + branch
        return self.transformer.ln_f(x)

    def forward(self, idx: torch.Tensor, all_logits: bool = False) -> dict:
        """Logits of the last position (llama.py:253-262, the reference's inference default) or of all positions."""
        x = self.hidden_states(idx)
        logits = self.lm_head(x) if all_logits else self.lm_head(x[:, -1:, :])      # a slice: index lists copy from the host
        return {'logits': logits}


def _pack(linear: nn.Linear, use_hadamard: bool, use_noop: bool, from_fp32: bool = False) -> harness.Linear4bit:
    m = harness.Linear4bit.from_weight(linear.weight.data, bias=None if linear.bias is None else linear.bias.data,
                                       use_hadamard=use_hadamard, quantize_from_fp32=from_fp32)
    m.use_noop = use_noop
    return m


@torch.no_grad()
def quantize_model(model: Llama, mode: str = 'int4', use_hadamard: bool = True, fuse_gate_up: bool = True,
                   fuse_producers: bool = False, swiglu_epilogue: bool = True, quantize_from_fp32: bool = False) -> Llama:
    """bench_e2e.py:77-97 on an existing model: every linear under `transformer` becomes a `Linear4bit` holding the
    packed INT4 form of that linear's own weight ('int4'), or the same module in no-op mode ('noop'); 'bf16' leaves
    the dense linears.  The model must already sit on the GPU in bf16 or fp16.  quantize_from_fp32: weights and
    activations are quantised from the fp32 transform, as the reference's evaluation-side fake quantiser does
    (src/eval_hswag.py:201-214), not from its 16-bit rounding: the mode for checking a packed model against its
    fake-quantised original (not available together with fuse_producers)."""
    if quantize_from_fp32 and fuse_producers:
        raise NotImplementedError('quantize_from_fp32 runs the unfused blocks: the producer-fused kernels quantise the 16-bit transform')
    if mode == 'bf16':
        for block in model.transformer.h:          # dense linears; only the rotary kernel replaces torch glue
            block.attn.fused_rope = bool(fuse_producers)
        return model
    if mode not in ('int4', 'noop'):
        raise NotImplementedError(mode)
    noop = mode == 'noop'
    for block in model.transformer.h:
        block.attn.c_attn = _pack(block.attn.c_attn, use_hadamard, noop, quantize_from_fp32)
        block.attn.c_proj = _pack(block.attn.c_proj, use_hadamard, noop, quantize_from_fp32)
        mlp = block.mlp
        if fuse_gate_up:
            both = nn.Linear(mlp.w1.in_features, 2 * mlp.w1.out_features, bias=False, device=mlp.w1.weight.device,
                             dtype=mlp.w1.weight.dtype)
            both.weight.data = torch.cat([mlp.w1.weight.data, mlp.w2.weight.data], dim=0)
            mlp.w12 = _pack(both, use_hadamard, noop, quantize_from_fp32)
            mlp.w1 = mlp.w2 = None
        else:
            mlp.w1 = _pack(mlp.w1, use_hadamard, noop, quantize_from_fp32)
            mlp.w2 = _pack(mlp.w2, use_hadamard, noop, quantize_from_fp32)
        mlp.c_proj = _pack(mlp.c_proj, use_hadamard, noop, quantize_from_fp32)
        # the producer-fused kernels exist for the Hadamard variant, rows up to 32768 and the fused gate/up layout
        # (in no-op mode the fused blocks keep their producers -- norms, residual additions, quantisers, rotary kernel --
        # and only the GEMMs return zeros: the twin that prices the GEMMs of the producer-fused model)
        block.attn.fused_rope = bool(fuse_producers)
        block.fuse_producers = bool(fuse_producers and use_hadamard and fuse_gate_up and
                                    model.config.n_embd <= 32768 and model.config.hidden_dim <= 32768)
        if fuse_producers and not block.fuse_producers:
            import warnings
            warnings.warn('quantize_model: fuse_producers asked for, but this configuration (no Hadamard, separate gate / up '
                          'projections or rows over 32768) has no producer-fused kernels: the blocks run with torch glue')
        if block.fuse_producers and swiglu_epilogue and model.config.hidden_dim % 4 == 0:
            mlp.enable_swiglu_epilogue()
    return model


def load_reference_checkpoint(model: Llama, path: str) -> Llama:
    """Load a checkpoint file written by the reference's training loop (src/optim/utils.py:245-256: a dict with the
    model's state dict under "model", next to optimizer, scheduler and iteration) into a dense model of this module.
    The file is read with torch's weights-only loader, which unpickles tensors and plain containers and executes
    nothing from the file; a bare state dict is accepted as well."""
    ckpt = torch.load(path, map_location='cpu', weights_only=True)
    state = ckpt['model'] if isinstance(ckpt, dict) and 'model' in ckpt and isinstance(ckpt['model'], dict) else ckpt
    return load_reference_state_dict(model, state)


@torch.no_grad()
def load_reference_state_dict(model: Llama, state_dict: dict) -> Llama:
    """Copy the weights of a checkpoint of the reference's model (src/models/llama.py; parameter names
    `transformer.wte.weight`, `transformer.h.<i>.attn.c_attn.weight`, ..., `lm_head.weight`, possibly behind the
    `_orig_mod.module.` prefix its training wrapper adds, src/eval_hswag.py:187-195) into a dense model of this
    module; quantiser buffers and other non-parameter entries are ignored.  `quantize_model` then packs the linears:
    the weight quantiser the reference trains with (Hadamard, Gaussian clip, 16 levels) is the grid
    `preprocess_weight(use_hadamard=True)` produces, so the trained weights map to INT4 codes directly."""
    own = model.state_dict()
    picked = {}
    for name, value in state_dict.items():
        for prefix in ('_orig_mod.module.', 'module.', ''):
            if name.startswith(prefix) and name[len(prefix):] in own:
                picked[name[len(prefix):]] = value
                break
    missing = [k for k in own if k not in picked]
    if missing:
        raise KeyError(f'checkpoint lacks {len(missing)} parameters, e.g. {missing[:3]}')
    for k, v in picked.items():
        if own[k].shape != v.shape:
            raise ValueError(f'{k}: checkpoint shape {tuple(v.shape)} != model shape {tuple(own[k].shape)}')
        own[k].copy_(v)
    return model


@torch.inference_mode()
def bench_forward(model: Llama, batch_size: int, seq_len: int, n_warmup: int = 5, n_iter: int = 10) -> dict:
    """bench_e2e.py:99-121: seconds per forward, eagerly and as a replayed HIP graph (the smaller is the
    reference's figure); the graph's logits are checked against the eager ones on fresh ids."""
    dev = next(model.parameters()).device
    g = torch.Generator(device='cpu').manual_seed(0)
    input_ids = torch.randint(0, model.config.vocab_size, (batch_size, seq_len), generator=g).to(dev)
    f = lambda: model(input_ids)['logits']           # noqa: E731
    t_eager = harness.do_bench(f, n_iter=n_iter, n_warmup=n_warmup)
    graph = torch.cuda.CUDAGraph()
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        for _ in range(n_warmup):
            f()
    torch.cuda.current_stream().wait_stream(s)
    with torch.cuda.graph(graph):
        out = f()
    t_graph = harness.do_bench(graph.replay, n_iter=n_iter, n_warmup=n_warmup)
    input_ids.copy_(torch.randint(0, model.config.vocab_size, (batch_size, seq_len), generator=g).to(dev))
    graph.replay()
    torch.cuda.synchronize()
    graph_ok = bool(torch.equal(out, f()))
    return {'eager_s': t_eager, 'graph_s': t_graph, 'best_s': min(t_eager, t_graph), 'graph_matches_eager': graph_ok}
