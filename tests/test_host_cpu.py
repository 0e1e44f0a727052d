"""CPU checks of host-side pieces that need no GPU: the layer benchmark's record / table code, the packed layer's
module structure, and the arithmetic of the kernels' clamp-free quantiser, emulated in fp32 with numpy against the
IEEE-divide statement of the reference (gemm-quest/quest/quantize_kernel.cu:155-158, benchmarks/utils.py:342)."""
import numpy as np
import pytest
import torch

from quest_amd import bench_layer, harness


def test_bench_layer_records_and_table():
    runtime = {(4096, 4096): [(32.0, 17.5e-6, 47.6e-6, 49.0e-6), (4096.0, 800.5e-6, 281.6e-6, 351.0e-6)],
               (2048, 5632): [(64.0, 1e-5, 2e-5, 4e-5)]}
    rec = bench_layer.as_records(runtime)
    assert [(r['N'], r['K'], r['M']) for r in rec] == [(4096, 4096, 32), (4096, 4096, 4096), (2048, 5632, 64)]
    assert rec[0]['rtx4090_us'] == [17.5, 47.6, 49.0] and 'rtx4090_us' not in rec[2]
    assert rec[1]['speedup_int4'] == pytest.approx(800.5 / 281.6)
    assert rec[2]['int4_had_TOPS'] == pytest.approx(2 * 64 * 2048 * 5632 / 4e-5 / 1e12)
    table = bench_layer.markdown_table(rec).splitlines()
    assert len(table) == 2 + 3 and table[2].startswith('| 4096 | 4096 | 32 | 17.5 | 47.6 | 49.0 |')
    # the reference's eight shapes and ten token counts (bench_layer.py:13-14)
    assert len(bench_layer.HIDDEN_SIZES) == 8 and bench_layer.BATCH_SIZES == [2 ** e for e in range(5, 15)]
    assert all(k % 128 == 0 for _, k in bench_layer.HIDDEN_SIZES)


def test_linear4bit_module_structure():
    layer = harness.Linear4bit.empty(256, 64, bias=True, dtype=torch.bfloat16, use_hadamard=True)
    sd = layer.state_dict()
    assert set(sd) == {'bias', 'w_int_packed', 'w_scale', 'w_add'}
    assert sd['w_int_packed'].shape == (64, 128) and sd['w_int_packed'].dtype == torch.uint8
    assert sd['w_scale'].shape == (64, 1) and sd['w_add'].dtype == torch.int32
    assert layer.weight.device.type == 'meta' and layer.weight.shape == (64, 256)
    assert not layer.bias.requires_grad
    assert harness.Linear4bit.empty(256, 64, bias=False, dtype=torch.float16).bias is None
    with pytest.raises(NotImplementedError):
        harness.Linear4bit(128, 64, use_sparse=True)
    with pytest.raises(NotImplementedError):
        harness.find_scale_int4(torch.zeros(1, 128), backend='pytorch')


def _all16(dtype):
    x = torch.arange(0, 65536, dtype=torch.int32).to(torch.int16).view(dtype).float().numpy()
    return x[np.isfinite(x)]


def _reference_codes(x, s):
    with np.errstate(all='ignore'):
        q = np.floor(x / s)                                   # fp32 IEEE divide
        return np.fmin(np.fmax(q, -8), 7).astype(np.int32)


def _clamp_free_codes(x, s):
    """common.h: quant_inv28 / quant_top_nibble_any, then the arithmetic shift that reads the top nibble."""
    with np.errstate(all='ignore'):
        inv28 = ((np.float32(1) / s).astype(np.float32) * np.float32(2.0 ** 28)).astype(np.float32)
        t = (x * inv28).astype(np.float32)
        tn = (np.abs(t).astype(np.float64) * 2.0 ** -21 + t.astype(np.float64)).astype(np.float32)      # one rounding: an fma
        tn = np.where(np.isnan(tn), np.float32(-3.4028234663852886e38), tn)                            # v_max_f32 drops the NaN
        n = np.clip(np.floor(tn.astype(np.float64)), -2.0 ** 31, 2.0 ** 31 - 1).astype(np.int64)       # v_cvt_flr_i32_f32 saturates
    return (n >> 28).astype(np.int32)


@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float16])
def test_clamp_free_quantiser_equals_the_divide_form(dtype):
    """Every finite 16-bit x against a spread of scales over the whole fast range [2^-99, 2^15] (every 97th positive
    16-bit pattern, the range's two ends and a few scales with short mantissas, where exact-integer quotients abound)."""
    xs = _all16(dtype)
    pos = torch.arange(1, 32768, dtype=torch.int32).to(torch.int16).view(dtype).float().numpy()
    pos = pos[np.isfinite(pos) & (pos >= 2.0 ** -99) & (pos <= 2.0 ** 15)]
    scales = np.unique(np.concatenate([pos[::97], pos[:2], pos[-2:],
                                       np.array([0.25, 0.5, 1.0, 1.5, 3.0, 0.375, 2.0 ** -20, 2.0 ** 15], dtype=np.float32)]))
    scales = scales[(scales >= 2.0 ** -99) & (scales <= 2.0 ** 15)]
    assert len(scales) > 100
    for s in scales:
        s = np.float32(s)
        assert np.array_equal(_clamp_free_codes(xs, s), _reference_codes(xs, s)), float(s)
