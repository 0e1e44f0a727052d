"""The decode GEMM entry point that allocates nothing (its split-K workspace is an array inside the library) against the
entry point that takes a caller-owned workspace, through the C ABI: same bits, on calls in a row that share the library's
array, the later ones with smaller inputs; torch's allocator sees no request during the calls."""
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = 'cuda:0'


def _inputs(m, k, n, seed, dtype):
    g = torch.Generator().manual_seed(seed)
    ap = torch.randint(0, 256, (m, k // 2), generator=g, dtype=torch.uint8)
    bp = torch.randint(0, 256, (n, k // 2), generator=g, dtype=torch.uint8)
    a_add = torch.randint(-4000, 4000, (m, 1), generator=g, dtype=torch.int32)
    b_add = torch.randint(-4000, 4000, (n, 1), generator=g, dtype=torch.int32)
    a_mul = (torch.rand(m, 1, generator=g) * 0.09 + 0.01).to(dtype)
    b_mul = (torch.rand(n, 1, generator=g) * 0.09 + 0.01).to(dtype)
    return [t.to(DEV) for t in (ap, bp, a_add, b_add, a_mul, b_mul)]


def test_no_alloc_decode_gemm_matches_the_workspace_entry_point():
    from quest_amd import _lib
    lib = _lib.load()
    assert torch.cuda.is_available()
    limit = lib.quest_gemm_noalloc_scratch_bytes()
    work = torch.zeros(limit, dtype=torch.uint8, device=DEV)
    stream = _lib.stream_of(work)
    # two shapes that split K (the second smaller in every dimension), one that does not, then the first again
    cases = [(16, 32768, 2048, torch.bfloat16), (3, 16384, 1000, torch.float16), (5, 4096, 4096, torch.bfloat16),
             (16, 32768, 2048, torch.bfloat16)]
    for i, (m, k, n, dtype) in enumerate(cases):
        assert lib.quest_gemm_workspace_bytes(m, k, n) <= limit
        assert (lib.quest_gemm_workspace_bytes(m, k, n) > 0) == (k >= 16384)
        ap, bp, a_add, b_add, a_mul, b_mul = _inputs(m, k, n, 20 + i, dtype)
        want = torch.full((m, n), 7, dtype=dtype, device=DEV)
        got = torch.full((m, n), 9, dtype=dtype, device=DEV)
        code = _lib.DTYPE_CODE[dtype]
        torch.cuda.synchronize()
        requests = torch.cuda.memory_stats(DEV)['allocation.all.allocated']
        rc = lib.quest_fused_matmul_dequantize_int4_int4t_noalloc(
            _lib.ptr(got), _lib.ptr(ap), _lib.ptr(bp), _lib.ptr(a_add), _lib.ptr(b_add), _lib.ptr(a_mul), _lib.ptr(b_mul),
            m, k, n, code, stream)
        assert rc == 0, lib.quest_status_string(rc)
        assert torch.cuda.memory_stats(DEV)['allocation.all.allocated'] == requests
        rc = lib.quest_fused_matmul_dequantize_int4_int4t_ws(
            _lib.ptr(want), _lib.ptr(ap), _lib.ptr(bp), _lib.ptr(a_add), _lib.ptr(b_add), _lib.ptr(a_mul), _lib.ptr(b_mul),
            m, k, n, code, _lib.ptr(work), work.numel(), stream)
        assert rc == 0, lib.quest_status_string(rc)
        torch.cuda.synchronize()
        assert torch.equal(got.view(torch.int16), want.view(torch.int16)), (m, k, n)
        assert torch.isfinite(got.float()).all()


def test_no_alloc_decode_gemm_refuses_what_it_does_not_serve():
    from quest_amd import _lib
    lib = _lib.load()
    m, k, n = 17, 4096, 4096
    ap, bp, a_add, b_add, a_mul, b_mul = _inputs(m, k, n, 1, torch.bfloat16)
    out = torch.empty(m, n, dtype=torch.bfloat16, device=DEV)
    args = (_lib.ptr(out), _lib.ptr(ap), _lib.ptr(bp), _lib.ptr(a_add), _lib.ptr(b_add), _lib.ptr(a_mul), _lib.ptr(b_mul))
    rc = lib.quest_fused_matmul_dequantize_int4_int4t_noalloc(*args, m, k, n, _lib.DTYPE_CODE[torch.bfloat16], _lib.stream_of(out))
    assert rc == -5 and b'shape outside' in lib.quest_status_string(rc)
    assert lib.quest_fused_matmul_dequantize_int4_int4t_noalloc(None, *args[1:], 4, k, n, _lib.DTYPE_CODE[torch.bfloat16], _lib.stream_of(out)) == -1
