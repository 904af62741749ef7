"""The GEMM entry point that allocates nothing (its packed activations go to an array inside
the library's device image) against the entry point that takes a workspace: same bits, on two
calls in a row, the second with fewer rows, and a clear refusal beyond the array's size."""
import ctypes

import numpy as np
import pytest

from conftest import bf16_words, weight_like

pytestmark = pytest.mark.gpu


def _call(t, lib, x, y, fn, *extra):
    import torch
    t.error.zero_()
    status = fn(ctypes.byref(t.fused), ctypes.byref(t._gemm_tiling()[0]), x.data_ptr(), x.stride(0), x.shape[0],
                y.data_ptr(), y.stride(0), None, *extra, t.error.data_ptr(),
                torch.cuda.current_stream(t.device).cuda_stream)
    return status, y


def test_noalloc_gemm_matches_the_workspace_entry_point_twice():
    import torch
    from georefine_amd import bitexact_context_codec as codec
    from georefine_amd.bitexact_context_gpu import HipContextTensor
    rng = np.random.default_rng(11)
    words = weight_like(rng, 200, 1280)
    t = HipContextTensor(codec.encode(words), stride=1024, device="cuda:0")
    assert t.fused is not None, t.fused_reason
    lib = t._lib
    for rows in (96, 17):  # the second call is smaller: rows of the first must not show through
        print(f"rows={rows}", flush=True)
        x = torch.from_numpy(bf16_words(rng.normal(0, 1, size=(rows, 1280)))).view(torch.bfloat16).cuda()
        size = lib.grf_gemm_workspace_bytes_split(1280, t.shape[0], t._gemm_tiling()[0].k_parts, rows)
        workspace = torch.empty(size, device="cuda:0", dtype=torch.uint8)
        want, got = (torch.zeros((rows, t.shape[0]), device="cuda:0", dtype=torch.bfloat16) for _ in range(2))
        status, _ = _call(t, lib, x, want, lib.grf_bctx_gemm, workspace.data_ptr(), size)
        assert status == 0, lib.grf_last_error()
        torch.cuda.synchronize()
        assert t.error.item() == 0
        free_before = torch.cuda.mem_get_info()[0]  # device memory as the driver counts it
        status, _ = _call(t, lib, x, got, lib.grf_bctx_gemm_noalloc)
        assert status == 0, lib.grf_last_error()
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == free_before  # nothing was allocated or freed
        assert t.error.item() == 0
        assert torch.equal(got.view(torch.uint16), want.view(torch.uint16))
        dense = torch.nn.functional.linear(x.float(), t.decode().float())
        assert torch.allclose(got.float(), dense, rtol=1e-2, atol=1e-2 * float(dense.abs().max()))


def test_noalloc_gemm_refuses_sizes_beyond_its_scratch():
    import torch
    from georefine_amd import bitexact_context_codec as codec
    from georefine_amd.bitexact_context_gpu import HipContextTensor
    t = HipContextTensor(codec.encode(weight_like(np.random.default_rng(2), 64, 256)), stride=1024, device="cuda:0")
    lib = t._lib
    limit = lib.grf_gemm_noalloc_limit_bytes()
    assert limit == 8 << 20 and lib.grf_gemm_workspace_bytes(32752, 128) <= limit < lib.grf_gemm_workspace_bytes(32768, 128)
    wide = ctypes.pointer(type(t.fused).from_buffer_copy(t.fused))  # the same frame, claimed to be wider than the scratch allows
    wide.contents.cols = 40000
    x = torch.zeros((128, 256), device="cuda:0", dtype=torch.bfloat16)
    y = torch.empty((128, 64), device="cuda:0", dtype=torch.bfloat16)
    status = lib.grf_bctx_gemm_noalloc(wide, ctypes.byref(t._gemm_tiling()[0]), x.data_ptr(), 256, 128, y.data_ptr(), 64,
                                       None, t.error.data_ptr(), None)
    assert status != 0 and b"scratch" in lib.grf_last_error()
