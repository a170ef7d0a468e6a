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


def _channel_tensors(c):
    return [c.stored, c.vals, c.scales]


@pytest.mark.parametrize("M,H,bits,group", [(520, 2048, 4, 128), (1030, 4096, 2, 64)])
def test_the_other_channel_entry_points_replay(pkg, M, H, bits, group):
    """compress / decompress, the one-pass forwards (activation, product, gated), their backwards, LayerNorm forward
    and backward and the wide weight gradient (codes decoded in the kernel, and the restored operand) through the
    package's wrappers: their output tensors come from the graph's memory pool, the kernels are the captured ones"""
    K = pkg.kernels
    gen = torch.Generator(device="cuda").manual_seed(11)
    k = K.num_outlier_channels(H, 0.01)

    def mk(scale):
        t = scale * torch.randn(M, H, generator=gen, device="cuda")
        t[:, torch.randperm(H, generator=gen, device="cuda")[:k]] *= 20.0
        return t.bfloat16()

    gate, up, g = mk(1.0), mk(1.0), mk(0.02)
    dyN = (0.01 * torch.randn(M, 256, generator=gen, device="cuda")).bfloat16()
    w = 1 + 0.1 * torch.randn(H, generator=gen, device="cuda")
    b = 0.1 * torch.randn(H, generator=gen, device="cuda")
    plans = [K.select_channels(K.channel_absmax(t), k) for t in (torch.nn.functional.silu(gate), up, gate)]
    gated = K.gated_act_fwd_supported(H, bits, group)
    product = K.hadamard_fwd_compress_supported(H, bits, group, bits, group)

    def run():
        out = []
        c = K.compress_channel(gate, plans[2], bits, group)
        out += _channel_tensors(c) + [K.decompress_channel(c)]
        y, cx = K.act_fwd_compress("gelu", gate, plans[2], bits, group)
        out += [y] + _channel_tensors(cx) + [K.act_bwd("gelu", g, cx)]
        if product:
            y, ca, cb = K.hadamard_fwd_compress(gate, up, plans[2], plans[1], bits, group)
            out += [y] + _channel_tensors(ca) + _channel_tensors(cb) + list(K.hadamard_bwd(g, ca, cb))
        if gated:
            h, c_act, c_up, c_gate = K.gated_act_fwd("silu", gate, up, plans[0], plans[1], plans[2], bits, group)
            out += [h] + _channel_tensors(c_act) + _channel_tensors(c_up) + _channel_tensors(c_gate)
            out += list(K.gated_act_bwd("silu", g, c_act, c_up, c_gate))
        y, mean, rstd, cl = K.layernorm_fwd_compress_channel(gate, w, b, 1e-5, plans[2], bits, group)
        out += [y, mean, rstd] + _channel_tensors(cl) + list(K.layernorm_bwd(g, cl, w, mean, rstd))
        out += [K.gradw_gemm(dyN, c, staged=False), K.gradw_gemm(dyN, c, staged=True)]
        return out

    want = [t.clone() for t in run()]
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        got = run()
    for rep in range(3):
        if rep == 1:                                    # fresh input in the same buffers
            gate.mul_(-0.75)
            g.mul_(2.0)
            want = [t.clone() for t in run()]
        for t in got:
            t.view(torch.uint8).fill_(0xA5)
        noise = torch.randn(1 << 16, device="cuda").cumsum(0).sum()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.isfinite(noise)
        assert len(got) == len(want)
        for i, (a, r) in enumerate(zip(got, want)):
            assert torch.equal(a.view(torch.uint8), r.view(torch.uint8)), "replay %d, output %d" % (rep, i)


def test_softmax_module_replays_once_calibrated(pkg):
    """EfficientMemorySoftmax forward + backward from its fourth call on never waits for the GPU (the kept entries are
    sized from the site's budget, kernels.KeptBudget), so the pair can be captured; replays on fresh scores and
    gradients equal the eager module bit for bit, and the device-side total shows that nothing was dropped."""
    ops, K = pkg.operators, pkg.kernels
    gen = torch.Generator(device="cuda").manual_seed(21)
    shape = (2, 4, 256, 256)
    mk = lambda s: (s * torch.randn(*shape, generator=gen, device="cuda")).bfloat16()
    mod = ops.EfficientMemorySoftmax(outlier_ratio=0.02)
    for _ in range(3):                                   # two calibration calls, one steady call that measures the budget
        x = mk(3.0).requires_grad_(True)
        mod(x).backward(mk(0.1))
    assert mod.iteration == 3 and K.kept_budget(mod.static_value).ready
    x, g = mk(3.0), mk(0.1)

    def run():
        xi = x.detach().clone().requires_grad_(True)
        y = mod(xi)
        kept = y.grad_fn.kept
        y.backward(g)
        return [y.detach(), xi.grad, kept.row_ptr, kept.total.view(1)]

    def eager():
        y, sp = K.softmax_fwd(x, K.threshold_value(mod.static_value))
        return [y, K.softmax_bwd(g, sp), sp.row_ptr, sp.total.view(1)]

    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        got = run()
    for rep in range(3):
        if rep:
            x.copy_(mk(2.0 + rep))
            g.copy_(mk(0.1 * rep))
        want = [t.clone() for t in eager()]
        for t in got[:2]:
            t.view(torch.uint8).fill_(0xA5)
        noise = torch.randn(1 << 16, device="cuda").cumsum(0).sum()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.isfinite(noise)
        for i, (a, r) in enumerate(zip(got, want)):
            assert torch.equal(a.view(torch.uint8), r.view(torch.uint8)), "replay %d, output %d" % (rep, i)
