"""tracea_gemm_noalloc (split-K workspace in a static device array, no device allocation)
against tracea_gemm on the same operands, through the C ABI: bit-identical outputs on two
calls in a row, the second on a smaller problem (the workspace keeps the first call's
contents), for half and fp32 operands; an unsplit launch; the refusal of a split whose
partial products exceed the workspace."""
import ctypes as C

import numpy as np
import pytest

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu

STATIC_SCRATCH_BYTES = 16 << 20


def _pair(tracea_gpu, capi, m, n, k, dtype, seed, epilogue="bias+relu"):
    g = torch.Generator(device="cuda").manual_seed(seed)
    a = (torch.randn(m, k, device="cuda", generator=g) / np.sqrt(k)).to(dtype)
    bt = torch.randn(n, k, device="cuda", generator=g).to(dtype)
    b = bt.t() if dtype != torch.float32 else bt.t().contiguous()
    bias = torch.randn(n, device="cuda", generator=g)
    want = tracea_gpu.gemm(a, b, bias=bias, epilogue=epilogue)
    splits_ref = capi.lib().tracea_last_split_k()
    out = torch.full_like(want, float("nan"))
    torch.cuda.synchronize()
    before = (torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0])   # torch's pool, and the device as a whole
    tracea_gpu.gemm_noalloc(a, b, out, bias=bias, epilogue=epilogue)
    splits = capi.lib().tracea_last_split_k()
    torch.cuda.synchronize()
    assert (torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]) == before
    assert splits == splits_ref
    assert torch.equal(out.view(torch.uint8), want.view(torch.uint8)), "%dx%dx%d differs" % (m, n, k)
    return splits


def test_two_calls_in_a_row_match_tracea_gemm(tracea_gpu):
    from tracea_amd import capi
    capi.lib().tracea_set_split_k(1)  # (on: the library's default, stated here because these shapes rely on it)
    for dtype in (torch.float16, torch.bfloat16):
        assert _pair(tracea_gpu, capi, 196, 256, 2304, dtype, 1) >= 2      # split, 196*256*4*splits bytes
        assert _pair(tracea_gpu, capi, 49, 136, 2120, dtype, 2) >= 2       # smaller, K tail, on the stale workspace
    assert _pair(tracea_gpu, capi, 512, 512, 1024, torch.float32, 3, "bias") >= 2
    assert _pair(tracea_gpu, capi, 100, 36, 2052, torch.float32, 4, "bias") >= 2


def test_unsplit_launch_needs_no_workspace(tracea_gpu):
    from tracea_amd import capi
    assert _pair(tracea_gpu, capi, 2048, 2048, 512, torch.float16, 5) == 1


def test_split_beyond_the_workspace_is_refused(tracea_gpu):
    from tracea_amd import capi
    m, n, k = 2048, 1024, 16384          # 32 tiles of 256x256: split 8 ways -> 64 MiB of partials
    a = torch.zeros(m, k, device="cuda", dtype=torch.float16)
    b = torch.zeros(n, k, device="cuda", dtype=torch.float16).t()
    out = torch.empty(m, n, device="cuda", dtype=torch.float16)
    tracea_gpu.gemm(a, b)
    splits = capi.lib().tracea_last_split_k()
    if splits * m * n * 4 <= STATIC_SCRATCH_BYTES:
        pytest.skip("the selector did not split this shape beyond the workspace")
    with pytest.raises(capi.TraceaError) as err:
        tracea_gpu.gemm_noalloc(a, b, out)
    assert err.value.status == capi.UNSUPPORTED_CONFIG
    assert "static workspace" in str(err.value)
