"""hyc_rmsnorm_bwd_static, the entry point that allocates nothing (its dw partial rows live in a device array of the
library), against hyc_rmsnorm_bwd with a caller workspace: same kernels, so dx and dw must be identical bit for bit.
Two calls in a row, the second on a smaller input: the array keeps the first call's contents."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def K(hyc):
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return hyc.kernels


def _ptr(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _both_ways(hyc, K, M, H, bits, group, k, wdt, quirk, seed):
    lib, abi = hyc._abi.load(), hyc._abi
    gen = torch.Generator().manual_seed(seed)
    x = torch.randn(M, H, generator=gen)
    x[:, torch.randperm(H, generator=gen)[:max(k // 2, 1)]] *= 30
    x = x.bfloat16().cuda()
    w = (1 + 0.1 * torch.randn(H, generator=gen)).to(wdt).cuda()
    dy = (0.02 * torch.randn(M, H, generator=gen)).bfloat16().cuda()
    plan = K.select_channels(K.channel_absmax(x), k)
    _, rstd, c = K.rmsnorm_fwd_compress_channel(x, w, 1e-6, plan, bits, group)
    d = c.desc()
    wcode = abi.DTYPE_F32 if wdt == torch.float32 else abi.DTYPE_BF16
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    P = lib.hyc_rmsnorm_bwd_partials(M, H)
    partials = torch.empty((max(P, 1), H), dtype=torch.float32, device="cuda")
    dx_a, dw_a = torch.empty_like(dy), torch.empty(H, dtype=wdt, device="cuda")
    dx_b, dw_b = torch.full_like(dy, 7.0), torch.full((H,), 7.0, dtype=wdt, device="cuda")
    rc = lib.hyc_rmsnorm_bwd(_ptr(dy), _ptr(c.stored), _ptr(c.vals), _ptr(c.scales), _ptr(w), wcode, _ptr(rstd), M, H,
                             ctypes.byref(d), quirk, _ptr(dx_a), _ptr(partials), _ptr(dw_a), stream)
    assert rc == 0, lib.hyc_last_error()
    before = torch.cuda.memory_allocated()
    rc = lib.hyc_rmsnorm_bwd_static(_ptr(dy), _ptr(c.stored), _ptr(c.vals), _ptr(c.scales), _ptr(w), wcode, _ptr(rstd), M, H,
                                    ctypes.byref(d), quirk, _ptr(dx_b), _ptr(dw_b), stream)
    assert rc == 0, lib.hyc_last_error()
    assert torch.cuda.memory_allocated() == before
    torch.cuda.synchronize()
    assert torch.equal(dx_a.view(torch.int16), dx_b.view(torch.int16))
    assert torch.equal(dw_a.view(torch.int16 if wdt == torch.bfloat16 else torch.int32),
                       dw_b.view(torch.int16 if wdt == torch.bfloat16 else torch.int32))
    assert not bool(torch.isnan(dw_b.float()).any())


def test_static_workspace_backward_equals_the_caller_workspace_one(hyc, K):
    # a large call first, then a smaller one (fewer tokens, narrower rows, other code width): stale partial rows of the
    # first call stay in the array and must not leak into the second
    _both_ways(hyc, K, 4096, 4096, 4, 128, 41, torch.float32, 1, seed=1)
    _both_ways(hyc, K, 300, 2048, 2, 64, 20, torch.bfloat16, 0, seed=2)
    # rows that take the generic kernel (1-bit codes), again smaller than what the array last held
    _both_ways(hyc, K, 40, 1024, 1, 64, 10, torch.float32, 1, seed=3)


def test_static_workspace_limits(hyc, K):
    lib, abi = hyc._abi.load(), hyc._abi
    H, M = 16384, 8192                                   # 8-bit codes: 2048 chunks per segment, up to 1024 partial rows
    plan = K.select_channels(torch.zeros(H, device="cuda"), 0)
    d = K.channel_desc(plan, 8, 128)
    rows = lib.hyc_rmsnorm_bwd_partial_rows(M, H, ctypes.byref(d))
    assert rows * H > abi.RMSNORM_BWD_STATIC_MAX_FLOATS
    one = ctypes.c_void_p(0x1000)
    rc = lib.hyc_rmsnorm_bwd_static(one, one, one, one, one, abi.DTYPE_F32, one, M, H, ctypes.byref(d), 1, one, one, None)
    assert rc == abi.EINVAL and b"static workspace" in lib.hyc_last_error()
    d4 = K.channel_desc(plan, 4, 128)
    assert lib.hyc_rmsnorm_bwd_partial_rows(1 << 20, 8192, ctypes.byref(d4)) * 8192 <= abi.RMSNORM_BWD_STATIC_MAX_FLOATS
    rc = lib.hyc_rmsnorm_bwd_static(one, one, one, one, one, abi.DTYPE_F32, one, 64, 4096, ctypes.byref(d4), 1, one, None, None)
    assert rc == abi.EFAULT                               # dw is required
