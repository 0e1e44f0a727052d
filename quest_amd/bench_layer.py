"""Layer benchmark: the counterpart of the reference's gemm-quest/benchmarks/bench_layer.py.

For each (N, K) of the reference's eight layer shapes (bench_layer.py:14; the 800M model's and
Llama-7B's qkv / o / gate-up / down projections) and each token count M in 32 ... 16384
(bench_layer.py:13) it times, through `harness.do_bench_network` (20 layers back to back on one
buffer, plain launches and a replayed HIP graph, the smaller of the two):

  dense     torch.matmul(a_in, weight.t(), out=a_out) in bf16          (bench_layer.py:31-36)
  int4      harness.linear_forward(..., use_hadamard=False)             (bench_layer.py:37-42)
  int4_had  harness.linear_forward(..., use_hadamard=True)              (bench_layer.py:43-48)

The reference leaves its operands uninitialised (bench_layer.py:22-29).  Here the activation pool is filled with
Gaussian values, the weight codes are random and the weight scales lie in [0.01, 0.1]: the run time of these kernels
does depend on the values -- the activation kernel takes a slower, clamping path for rows whose scale is zero, Inf or
NaN, which garbage memory can produce, and the matrix cores' clock follows the power that the operands' bit patterns
draw -- so finite, realistic data is what keeps the figures honest.  Layer i + 1 still quantises what layer i wrote
(one buffer serves as input and output, as in the reference), which stays finite.  With enough tokens the INT4 columns
run the FP6 matrix-core kernel on E2M3 tiles (`harness.prefers_e2m3`), otherwise the INT8 kernels on packed nibbles.

    python -m quest_amd.bench_layer [--quick] [--json out.json] [--markdown out.md]

The reference's RTX 4090 times (the array its authors left in bench_layer.py:139) are quoted in
RTX4090_US for the rows that the published table of this repository's baseline uses, so that the
printed table shows them beside the MI355X figures.
"""
from __future__ import annotations

import argparse
import json

import torch

from . import harness

HIDDEN_SIZES = [(6144, 2048), (2048, 2048), (11264, 2048), (2048, 5632),
                (12288, 4096), (4096, 4096), (22016, 4096), (4096, 11008)]          # (N, K), bench_layer.py:14
BATCH_SIZES = [2 ** e for e in range(5, 15)]                                          # bench_layer.py:13

# (N, K, M) -> (dense, int4, int4 + Hadamard) microseconds on an RTX 4090, from gemm-quest/benchmarks/bench_layer.py:139
RTX4090_US = {
    (22016, 4096, 4096): (4251., 1090., 1132.),
    (4096, 11008, 4096): (2151., 621., 804.),
    (12288, 4096, 4096): (2379., 670., 717.),
    (4096, 4096, 4096): (800.5, 281.6, 351.0),
    (4096, 4096, 32): (17.5, 47.6, 49.0),
    (4096, 11008, 32): (108.2, 85.0, 91.0),
    (22016, 4096, 16384): (16895., 4288., 4573.),
}


def time_layer(n: int, k: int, m: int, dtype=torch.bfloat16, device=None, n_layers: int = 20, n_warmup: int = 3):
    """Seconds per layer for (dense, int4, int4_had) at one shape."""
    device = torch.device('cuda') if device is None else device
    g = torch.Generator(device=device).manual_seed(0)
    weight = torch.randn(n, k, dtype=dtype, device=device, generator=g) * 0.02
    w_scale = (torch.rand(n, 1, device=device, generator=g) * 0.09 + 0.01).to(dtype)
    w_int_packed = torch.randint(0, 256, (n, k // 2), dtype=torch.uint8, device=device, generator=g)
    w_add = (harness.unpack_int4(w_int_packed).to(torch.int32).sum(-1, keepdim=True) + k // 2).to(torch.int32)
    use_tiles = harness.prefers_e2m3(m, k, n)
    w_tiles = harness.weight_tiles(w_int_packed) if use_tiles else None
    a_tiles = torch.empty(harness.quest.e2m3_tiles_bytes(m, k), dtype=torch.uint8, device=device) if use_tiles else None
    a_scale = torch.empty(m, 1, dtype=dtype, device=device)
    a_int_packed = torch.empty(m, k // 2, dtype=torch.uint8, device=device)
    a_int_row_sum = torch.empty(m, 1, dtype=torch.int32, device=device)

    def dense(a_in, a_out):
        torch.matmul(a_in, weight.t(), out=a_out)

    def int4(use_hadamard):
        def layer(a_in, a_out):
            harness.linear_forward(activation=a_in, w_int_packed=w_int_packed, w_scale=w_scale, w_add=w_add, w_meta_e=None,
                                   out=a_out, _a_scale=a_scale, _a_int_packed=a_int_packed, _a_int_row_sum=a_int_row_sum,
                                   use_hadamard=use_hadamard, w_tiles=w_tiles, _a_tiles=a_tiles)
        return layer

    kw = dict(dtype=dtype, device=device, n_layers=n_layers, n_warmup=n_warmup)
    return (harness.do_bench_network(dense, m, k, n, **kw),
            harness.do_bench_network(int4(False), m, k, n, **kw),
            harness.do_bench_network(int4(True), m, k, n, **kw))


def get_timing(hidden_sizes=None, batch_sizes=None, dtype=torch.bfloat16, device=None, n_layers: int = 20, progress=None):
    """bench_layer.py:12-54: {(N, K): [(M, t_dense, t_int4, t_int4_had), ...]}, times in seconds per layer."""
    runtime = {}
    for n, k in (HIDDEN_SIZES if hidden_sizes is None else hidden_sizes):
        rows = []
        for m in (BATCH_SIZES if batch_sizes is None else batch_sizes):
            rows.append((float(m), *time_layer(n, k, int(m), dtype=dtype, device=device, n_layers=n_layers)))
            if progress is not None:
                progress(n, k, rows[-1])
        runtime[n, k] = rows
    return runtime


def as_records(runtime: dict) -> list:
    out = []
    for (n, k), rows in runtime.items():
        for m, t_dense, t_int4, t_had in rows:
            m = int(m)
            rec = {'N': n, 'K': k, 'M': m, 'dense_us': t_dense * 1e6, 'int4_us': t_int4 * 1e6, 'int4_had_us': t_had * 1e6,
                   'speedup_int4': t_dense / t_int4, 'speedup_int4_had': t_dense / t_had,
                   'int4_had_TOPS': 2. * m * n * k / t_had / 1e12}
            ref = RTX4090_US.get((n, k, m))
            if ref is not None:
                rec['rtx4090_us'] = list(ref)
                rec['rtx4090_speedup'] = [ref[0] / ref[1], ref[0] / ref[2]]
            out.append(rec)
    return out


def markdown_table(records: list) -> str:
    lines = ['| N | K | M | dense bf16 us | INT4 us | INT4+HT us | speed-up INT4 / +HT | eff. TOPS (+HT) | RTX 4090 us (dense / INT4 / +HT) | RTX 4090 speed-up |',
             '|---|---|---|---|---|---|---|---|---|---|']
    for r in records:
        ref = r.get('rtx4090_us')
        ref_s = ' / '.join(f'{v:g}' for v in ref) if ref else ''
        ref_x = ' / '.join(f'{v:.2f}x' for v in r['rtx4090_speedup']) if ref else ''
        lines.append(f"| {r['N']} | {r['K']} | {r['M']} | {r['dense_us']:.1f} | {r['int4_us']:.1f} | {r['int4_had_us']:.1f} | "
                     f"{r['speedup_int4']:.2f}x / {r['speedup_int4_had']:.2f}x | {r['int4_had_TOPS']:.0f} | {ref_s} | {ref_x} |")
    return '\n'.join(lines)


def main():
    ap = argparse.ArgumentParser(description=__doc__.split('\n\n')[0])
    ap.add_argument('--quick', action='store_true', help='only the token counts 32, 512, 4096 and 16384')
    ap.add_argument('--json', help='write the records to this file')
    ap.add_argument('--markdown', help='write the table to this file')
    args = ap.parse_args()
    batch = [32, 512, 4096, 16384] if args.quick else None

    def progress(n, k, row):
        print(f'N={n} K={k} M={int(row[0])}: dense {row[1] * 1e6:.1f} us, int4 {row[2] * 1e6:.1f} us, '
              f'int4+had {row[3] * 1e6:.1f} us', flush=True)

    records = as_records(get_timing(batch_sizes=batch, progress=progress))
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
