"""End-to-end prefill benchmark: the counterpart of the reference's gemm-quest/benchmarks/bench_e2e.py.

The reference builds its 1600M Llama (config_1600M.json: 20 layers, d = 2560, 20 heads, SwiGLU hidden 6912, vocabulary
50304, sequence length 512; bench_e2e.py:21-38), swaps every linear under `transformer` (bench_e2e.py:79-96) and times one
forward at batch sizes 1, 2, 4, 8 x 512 tokens for four modes (bench_e2e.py:124-136): dense bf16, INT4, INT4 with the
Hadamard transform, and "no-op" linears (everything but the linears).  The LM head is never run there (its forward returns
no logits by default, src/models/llama.py:256-266), so this script times `Llama.hidden_states`.

Columns here, per batch size, milliseconds per forward (the smaller of plain launches and a replayed HIP graph, as the
reference takes it):

  bf16            dense linears, torch glue                                   (reference: bf16)
  int4            W4A4 linears without the transform, torch glue              (reference: int4)
  int4_had        W4A4 linears with the Hadamard transform, torch glue        (reference: int4 + HT)
  noop            no-op linears (they still rotate their input), torch glue   (reference: noop)
  fused           int4_had with the producer-fused blocks: norm / residual / SwiGLU inside the quantisers, rotary kernel
  fused_noop      the same blocks with the GEMMs returning zeros (an output projection that would add into the residual
                  stream leaves it untouched): what of `fused` is not GEMM time

    python -m quest_amd.bench_e2e [--model 1600m|213m] [--batch-sizes 1 2 4 8] [--matrix-path fp6|int8] [--json F] [--markdown F]

The published RTX 4090 figures (the arrays the authors left in bench_e2e.py:146 and notebooks/plots.ipynb) are printed
beside the 1600M rows.
"""
from __future__ import annotations

import argparse
import json

import torch

from . import harness, llama

MODELS = {
    # gemm-quest/benchmarks/config_1600M.json
    '1600m': dict(n_layer=20, n_embd=2560, n_head=20, vocab_size=50304, sequence_length=512),
    # the 12-layer model of the whole-model row of bench.py
    '213m': dict(n_layer=12, n_embd=1024, n_head=16, vocab_size=32000, sequence_length=512),
}
MODES = ('bf16', 'int4', 'int4_had', 'noop', 'fused', 'fused_noop')

# batch size -> (bf16, int4, int4 + HT, noop) milliseconds on an RTX 4090 for the 1600M model, notebooks/plots.ipynb cell 25
RTX4090_1600M_MS = {1: (14.58, 9.56, 10.24, 4.04), 2: (26.80, 15.66, 16.74, 6.42), 4: (52.50, 29.03, 31.31, 13.67),
                    8: (115.81, 69.99, 75.39, 43.61)}


def build(mode: str, cfg: llama.LlamaConfig, device) -> llama.Llama:
    torch.manual_seed(0)
    model = llama.Llama(cfg).to(torch.bfloat16).to(device).eval()
    if mode == 'bf16':
        return llama.quantize_model(model, 'bf16')
    if mode == 'int4':
        return llama.quantize_model(model, 'int4', use_hadamard=False, fuse_gate_up=True)
    if mode == 'int4_had':
        return llama.quantize_model(model, 'int4', use_hadamard=True, fuse_gate_up=True)
    if mode == 'noop':
        return llama.quantize_model(model, 'noop', use_hadamard=True, fuse_gate_up=True)
    if mode == 'fused':
        return llama.quantize_model(model, 'int4', use_hadamard=True, fuse_gate_up=True, fuse_producers=True)
    if mode == 'fused_noop':
        return llama.quantize_model(model, 'noop', use_hadamard=True, fuse_gate_up=True, fuse_producers=True)
    raise NotImplementedError(mode)


@torch.inference_mode()
def time_forward(model: llama.Llama, batch_size: int, seq_len: int, n_warmup: int = 5, n_iter: int = 10) -> float:
    """bench_e2e.py:99-121: seconds per forward (without the LM head), min of plain launches and graph replay."""
    dev = next(model.parameters()).device
    g = torch.Generator(device='cpu').manual_seed(0)
    ids = torch.randint(0, model.config.vocab_size, (batch_size, seq_len), generator=g).to(dev)
    f = lambda: model.hidden_states(ids)            # noqa: E731
    t_eager = harness.do_bench(f, n_iter=n_iter, n_warmup=n_warmup)
    graph = torch.cuda.CUDAGraph()
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        for _ in range(n_warmup):
            f()
    torch.cuda.current_stream().wait_stream(s)
    with torch.cuda.graph(graph):
        f()
    t_graph = harness.do_bench(graph.replay, n_iter=n_iter, n_warmup=n_warmup)
    return min(t_eager, t_graph)


def get_timing(model_name: str = '1600m', batch_sizes=(1, 2, 4, 8), modes=MODES, device=None, progress=None) -> list:
    """bench_e2e.py:124-136: one record per batch size, milliseconds per forward for every mode."""
    device = torch.device('cuda') if device is None else device
    cfg = llama.LlamaConfig(**MODELS[model_name])
    times = {b: {} for b in batch_sizes}
    for mode in modes:                               # one model per mode, every batch size on it
        model = build(mode, cfg, device)
        for b in batch_sizes:
            times[b][mode] = time_forward(model, b, cfg.sequence_length) * 1e3
            if progress is not None:
                progress(mode, b, times[b][mode])
        del model
        torch.cuda.empty_cache()
    records = []
    for b in batch_sizes:
        rec = {'model': model_name, 'batch_size': b, 'tokens': b * cfg.sequence_length, 'ms': times[b],
               'matrix_path': harness.MATRIX_PATH}
        t = times[b]
        if 'bf16' in t and 'fused' in t:
            rec['speedup_fused_over_bf16'] = t['bf16'] / t['fused']
        if 'bf16' in t and 'int4_had' in t:
            rec['speedup_int4_had_over_bf16'] = t['bf16'] / t['int4_had']
        if 'fused' in t and 'fused_noop' in t:
            gemm_ms = t['fused'] - t['fused_noop']
            rec['fused_gemm_ms'] = gemm_ms
            rec['fused_gemm_frac_of_int8_peak'] = cfg.linear_ops_per_token() * b * cfg.sequence_length / (gemm_ms * 1e-3) / 5.0e15
        if model_name == '1600m' and b in RTX4090_1600M_MS:
            rec['rtx4090_ms'] = dict(zip(('bf16', 'int4', 'int4_had', 'noop'), RTX4090_1600M_MS[b]))
        records.append(rec)
    return records


def markdown_table(records: list) -> str:
    lines = ['| model | batch x 512 | bf16 | int4 | int4+HT | noop | fused | fused, no-op GEMMs | fused vs bf16 | GEMMs of fused: ms (of INT8 peak) | RTX 4090: bf16 / int4 / int4+HT / noop |',
             '|---|---|---|---|---|---|---|---|---|---|---|']
    for r in records:
        t = r['ms']
        cell = lambda k: f"{t[k]:.2f}" if k in t else ''                         # noqa: E731
        ref = r.get('rtx4090_ms')
        ref_s = ' / '.join(f"{ref[k]:.2f}" for k in ('bf16', 'int4', 'int4_had', 'noop')) if ref else ''
        gemm = f"{r['fused_gemm_ms']:.2f} ({r['fused_gemm_frac_of_int8_peak']:.2f})" if 'fused_gemm_ms' in r else ''
        sp = f"{r['speedup_fused_over_bf16']:.2f}x" if 'speedup_fused_over_bf16' in r else ''
        lines.append(f"| {r['model']} | {r['batch_size']} | {cell('bf16')} | {cell('int4')} | {cell('int4_had')} | {cell('noop')} | "
                     f"{cell('fused')} | {cell('fused_noop')} | {sp} | {gemm} | {ref_s} |")
    return '\n'.join(lines)


def main():
    ap = argparse.ArgumentParser(description=__doc__.split('\n\n')[0])
    ap.add_argument('--model', choices=sorted(MODELS), default='1600m')
    ap.add_argument('--batch-sizes', type=int, nargs='+', default=[1, 2, 4, 8])
    ap.add_argument('--modes', nargs='+', default=list(MODES), choices=MODES)
    ap.add_argument('--matrix-path', choices=('fp6', 'int8'), default=None, help='force the GEMM path of large layers (default: harness.MATRIX_PATH)')
    ap.add_argument('--json', help='write the records to this file')
    ap.add_argument('--markdown', help='write the table to this file')
    ap.add_argument('--min-k', type=int, default=None, help='shortest rows that take the FP6 path (default: harness.E2M3_MIN_K)')
    ap.add_argument('--no-gemm-add', action='store_true', help='residual additions in the norm kernels instead of the output projections\' GEMMs')
    ap.add_argument('--no-packed-gemm-add', action='store_true', help='no residual additions in the INT8 large-tile GEMM (the FP6 GEMM keeps its own)')
    ap.add_argument('--no-gemm-rope', action='store_true', help='rotary embedding in its own kernel instead of the QKV projection\'s GEMM')
    args = ap.parse_args()
    if args.no_gemm_add:
        harness.GEMM_ADDS_RESIDUAL = False
    if args.no_packed_gemm_add:
        harness.GEMM_ADDS_RESIDUAL_PACKED = False
    if args.no_gemm_rope:
        harness.GEMM_ROTATES_QK = False
    if args.min_k is not None:
        harness.E2M3_MIN_K = args.min_k
    if args.matrix_path is not None:
        harness.MATRIX_PATH = args.matrix_path

    def progress(mode, b, ms):
        print(f'{args.model} {mode} batch {b}: {ms:.2f} ms', flush=True)

    records = get_timing(args.model, tuple(args.batch_sizes), tuple(args.modes), progress=progress)
    table = markdown_table(records)
    print(table)
    if args.json:
        with open(args.json, 'w') as f:
            json.dump(records, f, indent=1)
    if args.markdown:
        with open(args.markdown, 'w') as f:
            f.write(table + '\n')


if __name__ == '__main__':
    main()
