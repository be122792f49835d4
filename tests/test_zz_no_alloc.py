"""cfp_gemm_dh_noalloc: the variant of cfp_gemm_dh for callers that cannot allocate.
Its W mirror lives in a device array inside the library; results must equal
cfp_gemm_dh's bit for bit (same kernel, same arithmetic), on two calls in a row, the
second with a smaller input (the array keeps the first call's contents)."""
import numpy as np
import pytest

from parity_util import HIDDEN, TOL_FP32, assert_close

pytestmark = pytest.mark.gpu


def _r(shape, cuda, seed, scale=1.0):
    import torch
    g = torch.Generator(device="cpu").manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(cuda)


def test_noalloc_dh_equals_gemm_dh_twice(pkg, cuda):
    """The allocation check reads the driver's free-memory figure (hipMemGetInfo), which
    sees a hipMalloc made inside the library; torch's own allocator statistics would not.
    The no-alloc call comes first for each shape, so that nothing it could lean on (the
    seam's workspace) has been made for it by cfp_gemm_dh."""
    import torch
    for call, (m3, cols) in enumerate([(768, 4096), (48, 96)]):
        W, d = _r((m3, HIDDEN), cuda, 50 + call, 0.1), _r((cols, m3), cuda, 60 + call)
        got = torch.full((cols, HIDDEN), float("nan"), device=cuda)
        if call == 0:      # resolves the device array's address (first use on this GPU)
            pkg.policy.gemm_dh_noalloc(W, d, got)
            got.fill_(float("nan"))
        torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info()[0]
        pkg.policy.gemm_dh_noalloc(W, d, got)
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == free_before, "device memory was allocated inside the call"
        want = pkg.policy.gemm_dh(W, d)
        assert torch.equal(got, want), f"call {call}: ({m3}, {cols})"
        ref = (d.double() @ W.double()).cpu().numpy()
        assert_close(got.cpu().numpy(), ref, TOL_FP32, f"noalloc dh ({m3}, {cols})")


def test_noalloc_dh_rejects_what_does_not_fit(pkg, cuda):
    import torch
    out = torch.zeros((64, HIDDEN), device=cuda)
    for m3, cols, word in ((784, 64, "exceeds"), (40, 64, "multiple of 16"), (768, 40, "multiple of 16")):
        W, d = torch.zeros((m3, HIDDEN), device=cuda), torch.zeros((cols, m3), device=cuda)
        with pytest.raises(pkg._lib.CfpError, match=word):
            pkg.policy.gemm_dh_noalloc(W, d, out)
