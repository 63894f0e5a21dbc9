"""The entry point of libdinfer_gemm_mid that allocates nothing (its partial sums live in a device array inside the
library), called through ctypes as a caller without torch's wrappers would, against the entry point that takes a
workspace: two calls in a row, the second with a smaller input, so that what the first left in the array must not
show in the second."""
import ctypes
from ctypes import c_int, c_int64, c_void_p

import pytest
import torch

pytestmark = pytest.mark.gpu

ARGS_STATIC = [c_int, c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_int64, c_int64, c_int64, c_int, c_int, c_int,
               c_void_p]
ARGS_WORKSPACE = ARGS_STATIC[:-1] + [c_void_p, c_int64, c_void_p]


def _library():
    from dinfer_amd.csrc import build
    path = build.find_built("gemm_mid") or build.build("gemm_mid")
    lib = ctypes.CDLL(str(path))
    lib.dinfer_gemm_mid_m_static.argtypes, lib.dinfer_gemm_mid_m_static.restype = ARGS_STATIC, c_int
    lib.dinfer_gemm_mid_m.argtypes, lib.dinfer_gemm_mid_m.restype = ARGS_WORKSPACE, c_int
    lib.dinfer_gemm_mid_m_workspace.argtypes = [c_int64, c_int64, c_int64, c_int, c_int, c_int, ctypes.POINTER(c_int64)]
    lib.dinfer_gemm_mid_m_workspace.restype = c_int
    lib.dinfer_gemm_mid_m_static_init.argtypes, lib.dinfer_gemm_mid_m_static_init.restype = [], c_int
    lib.dinfer_gemm_mid_m_static_capacity.argtypes, lib.dinfer_gemm_mid_m_static_capacity.restype = [], c_int64
    return lib


def test_static_scratch_product_equals_the_workspace_one():
    lib = _library()
    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    assert lib.dinfer_gemm_mid_m_static_init() == 0
    capacity = lib.dinfer_gemm_mid_m_static_capacity()
    assert capacity == 32 << 20
    stream = torch.cuda.current_stream(dev).cuda_stream
    gen = torch.Generator(device="cpu").manual_seed(5)
    # (M, N, K, gated): a large product, then smaller ones in every size, then one that needs float output
    cases = [(64, 1536, 4096, False, False), (23, 640, 1160, False, False), (40, 384, 2048, True, False),
             (17, 128, 520, False, True)]
    for M, N, K, gated, out_f32 in cases:
        rows = 2 * N if gated else N
        a = (torch.randn(M, K, generator=gen) * 0.5).to(torch.bfloat16).to(dev)
        w = (torch.randn(rows, K, generator=gen) * 0.05).to(torch.bfloat16).to(dev)
        out_dtype = torch.float32 if out_f32 else torch.bfloat16
        got = torch.full((M, N), 7.0, dtype=out_dtype, device=dev)
        want = torch.full((M, N), -7.0, dtype=out_dtype, device=dev)
        need = c_int64(0)
        assert lib.dinfer_gemm_mid_m_workspace(M, N, K, int(gated), 0, 0, ctypes.byref(need)) == 0
        assert 0 < need.value <= capacity
        ws = torch.empty(need.value // 4, dtype=torch.float32, device=dev)
        common = (int(out_f32), a.data_ptr(), a.stride(0), w.data_ptr(), w.stride(0))
        sizes = (M, N, K, int(gated), 0, 0)
        torch.cuda.synchronize()
        before = torch.cuda.memory_stats(dev)["allocation.all.allocated"], torch.cuda.mem_get_info(dev)[0]
        rc = lib.dinfer_gemm_mid_m_static(*common, got.data_ptr(), got.stride(0), *sizes, stream)
        assert rc == 0, f"case {(M, N, K, gated)}: status {rc}"
        torch.cuda.synchronize()
        after = torch.cuda.memory_stats(dev)["allocation.all.allocated"], torch.cuda.mem_get_info(dev)[0]
        assert after[0] == before[0] and after[1] >= before[1], "the call took device memory"
        assert lib.dinfer_gemm_mid_m(*common, want.data_ptr(), want.stride(0), *sizes, ws.data_ptr(), need.value, stream) == 0
        torch.cuda.synchronize()
        assert torch.equal(got, want), f"case {(M, N, K, gated)}: differs from the workspace entry point"
        # and both are the product
        ref = a.double() @ w.double().t()
        if gated:
            ref = torch.nn.functional.silu(ref[:, :N]) * ref[:, N:]
        torch.testing.assert_close(got.double(), ref, rtol=2e-2, atol=2e-2)


def test_static_scratch_refuses_what_does_not_fit():
    lib = _library()
    torch.cuda.set_device(0)
    dev = torch.device("cuda", 0)
    stream = torch.cuda.current_stream(dev).cuda_stream
    M, N, K = 64, 8192, 8192 + 4096   # 12 slices of 1,024 x 64 x 8,192 floats = 25 MB fits; gated doubles it
    need = c_int64(0)
    assert lib.dinfer_gemm_mid_m_workspace(M, N, K, 1, 1024, 2, ctypes.byref(need)) == 0
    assert need.value > lib.dinfer_gemm_mid_m_static_capacity()
    a = torch.zeros(M, K, dtype=torch.bfloat16, device=dev)
    w = torch.zeros(2 * N, K, dtype=torch.bfloat16, device=dev)
    out = torch.full((M, N), 3.0, dtype=torch.bfloat16, device=dev)
    rc = lib.dinfer_gemm_mid_m_static(0, a.data_ptr(), K, w.data_ptr(), K, out.data_ptr(), N, M, N, K, 1, 1024, 2, stream)
    assert rc == 6
    torch.cuda.synchronize()
    assert bool((out == 3.0).all()), "a refused call wrote its output"
