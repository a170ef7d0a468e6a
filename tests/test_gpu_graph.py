"""The entry points under HIP graph capture: a captured sequence (fused RMSNorm forward + save, its backward with the
column sum, the LoRA-A weight gradient with its workspace, an activation backward) is replayed several times, with
eager work and synchronisations of the program's own between the replays and with fresh input data, and every replay
must reproduce the eager results bit for bit.  Nothing in the sequence allocates, clears memory or reads back."""
import ctypes
import importlib

import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def pkg():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return importlib.import_module("hyc-lora_amd")


class Sequence:
    """device buffers and prebuilt C-ABI calls; run() launches the whole sequence on the current stream"""

    def __init__(self, pkg, M, H, bits, group, r):
        K, abi = pkg.kernels, pkg._abi
        self.lib, self.abi, self.M, self.H = abi.load(), abi, M, H
        gen = torch.Generator(device="cuda").manual_seed(7)
        k = K.num_outlier_channels(H, 0.01)
        self.x = torch.randn(M, H, generator=gen, device="cuda").bfloat16()
        hot = torch.randperm(H, generator=gen, device="cuda")[:k]
        self.x[:, hot] *= 25.0
        self.w = 1 + 0.1 * torch.randn(H, generator=gen, device="cuda")
        self.dy = (0.02 * torch.randn(M, H, generator=gen, device="cuda")).bfloat16()
        self.dyA = (0.01 * torch.randn(M, r, generator=gen, device="cuda")).bfloat16()
        self.plan = K.select_channels(K.channel_absmax(self.x), k)
        self.c = K.alloc_channel(M, H, self.plan, bits, group, self.x.device)
        self.desc = self.c.desc()
        self.y = torch.empty_like(self.x)
        self.rstd = torch.empty(M, dtype=torch.float32, device="cuda")
        self.dx = torch.empty_like(self.x)
        self.dact = torch.empty_like(self.x)
        self.partials = torch.empty((self.lib.hyc_rmsnorm_bwd_partials(M, H), H), dtype=torch.float32, device="cuda")
        self.dw = torch.empty(H, dtype=torch.float32, device="cuda")
        self.dwA = torch.empty(r, H, dtype=torch.bfloat16, device="cuda")
        self.ws = torch.empty(max(self.lib.hyc_gradw_workspace_bytes(M, r, H) // 4, 1), dtype=torch.float32, device="cuda")
        self.r = r

    def outputs(self):
        return (self.y, self.rstd, self.c.stored, self.c.vals, self.c.scales, self.dx, self.dw, self.dwA, self.dact)

    def run(self):
        p = lambda t: ctypes.c_void_p(t.data_ptr())
        st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        lib, abi, M, H, c, d = self.lib, self.abi, self.M, self.H, self.c, ctypes.byref(self.desc)
        abi.check(lib.hyc_rmsnorm_fwd_compress(p(self.x), p(self.w), abi.DTYPE_F32, ctypes.c_float(1e-6), M, H, d, p(self.y),
                                               p(self.rstd), p(c.stored), p(c.vals), p(c.scales), None, st))
        abi.check(lib.hyc_rmsnorm_bwd(p(self.dy), p(c.stored), p(c.vals), p(c.scales), p(self.w), abi.DTYPE_F32, p(self.rstd),
                                      M, H, d, 1, p(self.dx), p(self.partials), p(self.dw), st))
        abi.check(lib.hyc_gradw_gemm(p(self.dyA), self.r, p(c.stored), p(c.vals), p(c.scales), M, self.r, H, d,
                                     ctypes.c_float(1.0), ctypes.c_float(0.0), p(self.dwA), abi.DTYPE_BF16, p(self.ws), st))
        abi.check(lib.hyc_act_bwd(abi.ACT_SILU, p(self.dy), p(c.stored), p(c.vals), p(c.scales), M, H, d, p(self.dact), st))


@pytest.mark.parametrize("M,H,bits,group,r", [(600, 1024, 4, 128, 16), (1500, 4096, 2, 64, 64)])
def test_replays_equal_the_eager_sequence(pkg, M, H, bits, group, r):
    seq = Sequence(pkg, M, H, bits, group, r)
    seq.run()
    torch.cuda.synchronize()
    want = [t.clone() for t in seq.outputs()]
    # capture (after a run on a side stream, as the framework's capture asks)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        seq.run()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        seq.run()
    for rep in range(4):
        if rep == 2:                                    # fresh input: the graph reads the buffers, not a snapshot
            seq.x.mul_(-0.5)
            seq.dy.mul_(1.5)
            seq.run()
            torch.cuda.synchronize()
            want = [t.clone() for t in seq.outputs()]
        for t in seq.outputs():
            t.view(torch.uint8).fill_(0x5A)             # stale results cannot pass for fresh ones
        # eager work of the program's own and a synchronisation between the replays
        noise = torch.randn(1 << 16, device="cuda").cumsum(0).sum()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.isfinite(noise)
        for got, ref in zip(seq.outputs(), want):
            assert torch.equal(got.view(torch.uint8), ref.view(torch.uint8)), "replay %d" % rep
