"""The entry point that allocates nothing (pam_hip_pam_matmul_fwd_noalloc) against pam_hip_pam_matmul_fwd with a
caller-provided workspace: bit-identical outputs, two calls in a row, the second one smaller (the library's own
scratch array keeps the first call's contents)."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _both(m, n, k, seed):
    from pam_amd import _abi
    g = torch.Generator().manual_seed(seed)
    A = torch.randn(m, k, generator=g).cuda()
    B = (torch.randn(k, n, generator=g) * 0.05).cuda()
    lib = _abi.load_library()
    need = lib.pam_hip_gemm_workspace_bytes(1, m, n, k)
    ws = torch.empty(max(need, 4) // 4, dtype=torch.float32, device="cuda")
    want = torch.full((m, n), float("nan"), device="cuda")
    got = torch.full((m, n), float("nan"), device="cuda")
    st = _abi._stream()
    _abi._call("pam_hip_pam_matmul_fwd", A.data_ptr(), k, 1, B.data_ptr(), n, 1, want.data_ptr(), n, 1, m, n, k, 1.0,
               ws.data_ptr() if need else None, need, st)
    _abi._call("pam_hip_pam_matmul_fwd_noalloc", A.data_ptr(), k, 1, B.data_ptr(), n, 1, got.data_ptr(), n, 1, m, n, k, 1.0, st)
    torch.cuda.synchronize()
    return need, want.cpu().numpy(), got.cpu().numpy()


def test_noalloc_matches_workspace_variant_twice():
    # a weight-gradient shape (k split in many chunks, scratch in use), then a smaller one of the same kind
    for (m, n, k, seed) in [(192, 768, 12608, 1), (128, 192, 4096, 2)]:
        need, want, got = _both(m, n, k, seed)
        assert need > 0, "the shape was meant to use the scratch array"
        assert not np.isnan(want).any()
        assert np.array_equal(want.view(np.uint32), got.view(np.uint32)), f"{m}x{n}x{k}"
    # and a shape that needs no scratch at all
    need, want, got = _both(640, 512, 64, 3)
    assert np.array_equal(want.view(np.uint32), got.view(np.uint32))


def test_noalloc_call_allocates_nothing():
    """Device memory in use is the same before and after a call (the first call on a device has looked up the scratch
    array's address by then, which may load the code object: callers under graph capture make one call beforehand)."""
    from pam_amd import _abi
    m, n, k = 192, 768, 12608
    g = torch.Generator().manual_seed(5)
    A = torch.randn(m, k, generator=g).cuda(); B = torch.randn(k, n, generator=g).cuda(); Y = torch.empty(m, n, device="cuda")
    call = lambda: _abi._call("pam_hip_pam_matmul_fwd_noalloc", A.data_ptr(), k, 1, B.data_ptr(), n, 1, Y.data_ptr(), n, 1, m, n, k, 1.0, _abi._stream())
    call(); torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info(); held0 = torch.cuda.memory_allocated(); reserved0 = torch.cuda.memory_reserved()
    call(); call(); torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info()
    assert free1 == free0 and torch.cuda.memory_allocated() == held0 and torch.cuda.memory_reserved() == reserved0


def test_noalloc_refuses_what_does_not_fit():
    from pam_amd import _abi
    lib = _abi.load_library()
    m, n, k = 320, 19648, 2048                         # 1535 tiles, k cut in two: just more pieces than the array holds
    assert lib.pam_hip_gemm_workspace_bytes(1, m, n, k) > (48 << 20)
    x = torch.zeros(8, device="cuda")
    with pytest.raises(RuntimeError, match="scratch"):
        _abi._call("pam_hip_pam_matmul_fwd_noalloc", x.data_ptr(), k, 1, x.data_ptr(), n, 1, x.data_ptr(), n, 1, m, n, k, 1.0, _abi._stream())
