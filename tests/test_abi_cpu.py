"""CPU-only checks of the boundary: the C-ABI library loads without a GPU and exports every symbol
the header declares; the host layer rejects what it must without touching the device."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, 'include', 'quest_hip.h')).read()
    text = re.sub(r'/\*.*?\*/', '', text, flags=re.S)
    return sorted(set(re.findall(r'\b(quest_[a-z0-9_]+)\s*\(', text)))


def test_header_declares_the_expected_entry_points():
    names = declared_symbols()
    for n in ['quest_version', 'quest_status_string', 'quest_find_scale_int4', 'quest_quantize_int4',
              'quest_add_mul_vv', 'quest_matmul_int4_int4t_int32', 'quest_fused_matmul_dequantize_int4_int4t', 'quest_fused_matmul_dequantize_swiglu_int4_int4t',
              'quest_hadamard128', 'quest_hadamard_quantize_int4', 'quest_hadamard_quantize_int4_rule',
              'quest_rmsnorm_hadamard_quantize_int4', 'quest_add_rmsnorm_hadamard_quantize_int4', 'quest_silu_mul_hadamard_quantize_int4', 'quest_rope_interleaved']:
        assert n in names


def test_library_exports_every_declared_symbol():
    from quest_amd import _lib
    lib = _lib.load()
    for name in declared_symbols():
        assert hasattr(lib, name), name
        assert name in _lib.SIGNATURES, f'{name} has no ctypes signature'
    assert set(_lib.SIGNATURES) == set(declared_symbols())
    assert lib.quest_version() >= 100
    assert lib.quest_status_string(0) == b'ok'
    assert b'NULL' in lib.quest_status_string(-1)


def test_argument_errors_need_no_gpu():
    from quest_amd import _lib
    lib = _lib.load()
    null = ctypes.c_void_p(0)
    fake = ctypes.c_void_p(0x1000)
    assert lib.quest_find_scale_int4(null, fake, 128, 1, 0, null) == -1
    assert lib.quest_find_scale_int4(fake, fake, 12, 1, 0, null) == -2
    assert lib.quest_find_scale_int4(fake, fake, 128, 1, 5, null) == -3
    assert lib.quest_find_scale_int4(fake, ctypes.c_void_p(0x1004), 128, 1, 0, null) == -4
    assert lib.quest_quantize_int4(fake, null, null, null, null, 128, 1, 0, 0, null) == -1
    assert lib.quest_hadamard128(fake, fake, 64, 1, 0.1, 0, null) == -2
    assert lib.quest_hadamard_quantize_int4(fake, fake, null, null, null, 128 * 1024, 1, 0.1, 0, null) == -5
    assert lib.quest_matmul_int4_int4t_int32(fake, fake, fake, 0, 128, 4, null) == -2
    assert lib.quest_matmul_int4_int4t_int32(fake, fake, fake, 4, 100, 4, null) == -2
    assert lib.quest_matmul_int4_int4t_int32(fake, fake, fake, 4, 1 << 18, 4, null) == -5
    assert lib.quest_fused_matmul_dequantize_int4_int4t(fake, fake, fake, null, fake, fake, fake, 4, 128, 4, 0, null) == -1
    assert lib.quest_add_mul_vv(fake, fake, fake, fake, fake, fake, 4, 4, 2, null) == -3


def test_host_layer_refuses_cpu_tensors_and_foreign_backends():
    import quest
    import quest_amd
    from quest_amd import harness
    assert quest.find_scale_int4 is quest_amd.find_scale_int4
    x = torch.zeros(4, 128, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match='GPU only'):
        quest_amd.find_scale_int4(x)
    with pytest.raises(AssertionError):
        quest_amd.find_scale_int4(x.float())
    with pytest.raises(NotImplementedError):
        harness.find_scale_int4(x, backend='pytorch')
    with pytest.raises(NotImplementedError):
        harness.preprocess_weight(x, use_sparse=True)
    with pytest.raises(NotImplementedError):
        quest_amd.generate_random_meta48_int4(4, 64)


def test_unpack_int4_host_helper_matches_oracle():
    from oracle import quest_oracle as qo
    from quest_amd import harness
    b = torch.arange(256, dtype=torch.int32).to(torch.uint8).view(2, 128)
    assert torch.equal(harness.unpack_int4(b), qo.unpack_int4(b))
