"""Benchmark of the hybrid activation-compression hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step = one pass of the path over one batch of synthetic input, BASELINE config 2: fused RMSNorm forward +
compress (1 % outlier channels, INT4, group 128) of x [4,1024,4096] bf16, then the RMSNorm backward that
decompresses it.  Inputs are resident in HBM before the timed region.  Prints ONE JSON line.
"""
import argparse
import ctypes
import importlib
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
MFMA_BF16_PEAK_TFLOPS = 2500.0
# HBM bytes per launch at the bench workload, from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of
# `bench.py --pmc-probe`, each scaled by what the same counter reads for a plain copy of known size
# (profiles/rmsnorm_fwd_bwd_config2.md).  The figures belong to one state of the kernel sources: TRAFFIC_SOURCES_SHA
# is the digest of those files when the counters were taken, and `roofline.traffic` is null whenever the files on
# disk differ (a changed kernel needs new counter runs, not an old number).
TRAFFIC_FWD = int((16507.71 * 1.99841 + 41792.96) * 1024)    # FETCH_SIZE KiB x copy factor + WRITE_SIZE KiB
TRAFFIC_BWD = int((21030.41 * 1.99841 + 36866.62) * 1024)
TRAFFIC_SOURCES = ("norm.hip", "row_kernels.hpp", "row_codec.hpp")
TRAFFIC_SOURCES_SHA = "fc680345caa21d65"


def sources_sha():
    import hashlib
    h = hashlib.sha256()
    for name in TRAFFIC_SOURCES:
        with open(os.path.join(ROOT, "hyc-lora_amd", "csrc", name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def algorithmic_bytes(M, H, bits, group, k):
    """per-launch bytes a perfect kernel must move (every tensor read or written once): per token the forward reads x
    and writes y, the packed codes, the outlier values, the group scales and rstd; the backward reads dy and that side
    data and writes dx"""
    side = H * bits // 8 + 2 * k + 2 * (H // group)          # packed codes + outlier values + group scales
    fwd = M * (2 * H + 2 * H + side + 4)                       # read x, write y, side data, rstd
    bwd = M * (2 * H + side + 4 + 2 * H)                       # read dy, side data, rstd; write dx
    return fwd, bwd, M * side


class Workload:
    """device buffers + prebuilt ctypes calls for fwd and bwd of the fused RMSNorm path"""

    def __init__(self, pkg, torch, M, H, bits, group, n_hot, gain, seed=0):
        K, abi = pkg.kernels, pkg._abi
        self.torch, self.lib, self.M, self.H = torch, abi.load(), M, H
        gen = torch.Generator().manual_seed(seed)
        k = K.num_outlier_channels(H, 0.01)
        self.k, self.bits, self.group = k, bits, group
        # generate on the host in slabs (identical bits for the oracle), then move to the device
        xs = []
        hot = torch.randperm(H, generator=gen)[:n_hot]
        for r in range(0, M, 4096):
            m = min(4096, M - r)
            xs_ = torch.randn(m, H, generator=gen)
            xs_[:, hot] *= gain
            xs.append(xs_.bfloat16())
        self.x_host = xs[0] if len(xs) == 1 else None
        self.x = torch.cat([t.cuda() for t in xs])
        self.w_host = 1 + 0.1 * torch.randn(H, generator=gen)
        self.w = self.w_host.cuda()
        self.dy = torch.cat([(0.02 * torch.randn(min(4096, M - r), H, generator=gen)).bfloat16().cuda()
                             for r in range(0, M, 4096)])
        self.plan = K.select_channels(K.channel_absmax(self.x), k)
        self.c = K.alloc_channel(M, H, self.plan, bits, group, self.x.device)
        self.y = torch.empty_like(self.x)
        self.rstd = torch.empty(M, dtype=torch.float32, device="cuda")
        self.dx = torch.empty_like(self.x)
        P = self.lib.hyc_rmsnorm_bwd_partials(M, H)
        self.partials = torch.empty((P, H), dtype=torch.float32, device="cuda")
        self.dw = torch.empty(H, dtype=torch.float32, device="cuda")
        self.desc = self.c.desc()
        p = lambda t: ctypes.c_void_p(t.data_ptr())
        self._fwd_args = (p(self.x), p(self.w), abi.DTYPE_F32, ctypes.c_float(1e-6), M, H, ctypes.byref(self.desc),
                          p(self.y), p(self.rstd), p(self.c.stored), p(self.c.vals), p(self.c.scales), None)
        self._bwd_args = (p(self.dy), p(self.c.stored), p(self.c.vals), p(self.c.scales), p(self.w), abi.DTYPE_F32,
                          p(self.rstd), M, H, ctypes.byref(self.desc), 1, p(self.dx), p(self.partials), p(self.dw))
        self._bwd_main_args = self._bwd_args[:-1] + (None,)     # dw = NULL: the row kernel alone, no column sum
        self._check = abi.check

    def _stream(self):
        return ctypes.c_void_p(self.torch.cuda.current_stream().cuda_stream)

    def fwd(self):
        self._check(self.lib.hyc_rmsnorm_fwd_compress(*self._fwd_args, self._stream()))

    def bwd(self):
        self._check(self.lib.hyc_rmsnorm_bwd(*self._bwd_args, self._stream()))

    def bwd_main(self):
        self._check(self.lib.hyc_rmsnorm_bwd(*self._bwd_main_args, self._stream()))

    def step(self):
        self.fwd()
        self.bwd()


def time_events(torch, fn, iters, warmup):
    """average milliseconds of fn() over `iters` back-to-back launches, HIP events on the launch stream"""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(iters):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / iters


def time_graph(torch, fn, calls=10, replays=20):
    """average milliseconds of fn(): `calls` invocations captured into one HIP graph (so that the host cost of the
    Python wrapper does not space the launches out), replayed `replays` times between two events"""
    fn()
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        fn()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for _ in range(calls):
            fn()
    for _ in range(3):
        graph.replay()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(replays):
        graph.replay()
    e1.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / (calls * replays)
    del graph
    return ms


def side_bytes(H, bits, group, k):
    """bytes per token of a channel-compressed activation: packed codes + outlier values + group scales"""
    return H * bits // 8 + 2 * k + 2 * (H // group)


def hbm(nbytes, ms):
    return {"ms": round(ms, 5), "algorithmic_bytes": int(nbytes), "GBps": round(nbytes / ms / 1e6, 1),
            "frac_of_hbm_peak": round(nbytes / ms / 1e6 / HBM_PEAK_GBPS, 4)}


def make_activation(torch, M, H, hot, gain, seed):
    gen = torch.Generator(device="cuda").manual_seed(seed)
    x = torch.randn(M, H, generator=gen, device="cuda")
    x[:, torch.randperm(H, generator=gen, device="cuda")[:hot]] *= gain
    return x.bfloat16(), gen


def time_steady(torch, fn, iters, seconds=0.3):
    """like time_events, after `seconds` of the same launches: a matrix-core kernel on an idle GPU runs at clocks it
    does not hold (the first 20 ms read 15-20 % faster than the steady state), so every GEMM leg is timed warm"""
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        for _ in range(20):
            fn()
        torch.cuda.synchronize()
    return time_events(torch, fn, iters, 5)


def time_sustained(torch, fn, ms_estimate, seconds=2.5, iters=100):
    """milliseconds per launch after `seconds` of back-to-back launches with no pause at all (queued ahead, never
    synchronised): a matrix-core kernel that runs for seconds brings the GPU to its power limit and the clocks down,
    which 0.3 s of launches do not"""
    for _ in range(int(seconds / (ms_estimate * 1e-3))):
        fn()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(iters):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / iters


def gradw_extra(pkg, torch, c, sustained=False, shapes=(("full_w", 4096, 100, 30), ("lora_a_r16", 16, 300, 30), ("lora_a_r64", 64, 300, 30))):
    """weight-gradient GEMM dW = dY^T . x_hat on the channel-compressed activation `c`: x_hat decoded inside the GEMM,
    the staged route (restore x_hat once, then the dense form of the same kernel) and the framework's library GEMM on
    the restored activation; every leg warmed before it is timed"""
    K, abi = pkg.kernels, pkg._abi
    lib = abi.load()
    M, H = c.M, c.H
    desc = c.desc()
    out = {}
    p = lambda t: ctypes.c_void_p(t.data_ptr()) if t is not None else None
    stream = lambda: ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    xh = K.decompress_channel(c)
    # chunks of 8 channels that hold more than two outlier channels take the fused GEMM's rare (slow) splice path,
    # and one such chunk column delays the whole launch: say whether this plan has one
    seg = H * c.bits // 8
    idx = c.plan.idx.cpu().long()
    crowd = int(torch.bincount((idx // seg) * (seg // 8) + (idx % seg) // 8).max()) if idx.numel() else 0
    for name, N, iters, warm in shapes:
        dy = (0.01 * torch.randn(M, N, device="cuda")).bfloat16()
        dw = torch.empty(N, H, dtype=torch.bfloat16, device="cuda")
        ws_bytes = lib.hyc_gradw_workspace_bytes(M, N, H)
        ws = torch.empty(max(ws_bytes // 4, 1), dtype=torch.float32, device="cuda")
        args = (p(dy), N, p(c.stored), p(c.vals), p(c.scales), M, N, H, ctypes.byref(desc),
                ctypes.c_float(1.0), ctypes.c_float(0.0), p(dw), abi.DTYPE_BF16, p(ws))
        fn = lambda: abi.check(lib.hyc_gradw_gemm(*args, stream()))
        flop = 2.0 * M * N * H
        ms = time_steady(torch, fn, iters) if N > 64 else time_events(torch, fn, iters, warm)
        rec = {"M": M, "N_out": N, "H": H, "bits": c.bits, "group": c.group, "most_outlier_channels_in_a_chunk": crowd,
               "flop": int(flop), "ms": round(ms, 5),
               "TFLOPs": round(flop / ms / 1e9, 1), "frac_of_bf16_mfma_peak": round(flop / ms / 1e9 / MFMA_BF16_PEAK_TFLOPS, 4)}
        if N <= 64:
            # few output rows: the product is bound by reading the compressed activation and dY once
            nbytes = M * (side_bytes(H, c.bits, c.group, c.plan.k) + 2 * N) + 2 * N * H
            rec.update({"algorithmic_bytes": int(nbytes), "GBps": round(nbytes / ms / 1e6, 1),
                        "frac_of_hbm_peak": round(nbytes / ms / 1e6 / HBM_PEAK_GBPS, 4)})
        else:
            ms_staged = time_steady(torch, lambda: K.gradw_gemm(dy, c, staged=True), iters)
            ms_dense = time_steady(torch, lambda: K.gradw_gemm(dy, xh), iters)
            rec.update({"staged_ms": round(ms_staged, 5), "staged_TFLOPs": round(flop / ms_staged / 1e9, 1),
                        "staged_frac_of_bf16_mfma_peak": round(flop / ms_staged / 1e9 / MFMA_BF16_PEAK_TFLOPS, 4),
                        "dense_operand_ms": round(ms_dense, 5), "dense_operand_TFLOPs": round(flop / ms_dense / 1e9, 1),
                        "dense_operand_frac_of_bf16_mfma_peak": round(flop / ms_dense / 1e9 / MFMA_BF16_PEAK_TFLOPS, 4),
                        "default_route": "staged" if K.gradw_staged_by_default(N, H) else "fused"})
            if sustained:
                # the same launches after 2.5 s without a pause: the GPU at its power limit
                ms_s = time_sustained(torch, fn, ms)
                ms_ds = time_sustained(torch, lambda: K.gradw_gemm(dy, xh, out=dw), ms_dense)
                ms_ls = time_sustained(torch, lambda: torch.matmul(dy.t(), xh, out=dw), ms_dense)
                # the matrix cores' power follows the operand bits, and the clocks follow the power: the same launches
                # on an activation of zeros (what an unfilled buffer holds) show the kernels' ceiling at full clocks
                z = torch.zeros_like(xh)
                ms_dz = time_steady(torch, lambda: K.gradw_gemm(dy, z, out=dw), iters)
                ms_lz = time_steady(torch, lambda: torch.matmul(dy.t(), z, out=dw), iters)
                del z
                rec["on_an_activation_of_zeros"] = {
                    "dense_operand_ms": round(ms_dz, 5),
                    "dense_operand_frac_of_bf16_mfma_peak": round(flop / ms_dz / 1e9 / MFMA_BF16_PEAK_TFLOPS, 4),
                    "library_gemm_ms": round(ms_lz, 5)}
                rec["after_2.5_s_of_launches"] = {
                    "ms": round(ms_s, 5), "frac_of_bf16_mfma_peak": round(flop / ms_s / 1e9 / MFMA_BF16_PEAK_TFLOPS, 4),
                    "dense_operand_ms": round(ms_ds, 5),
                    "dense_operand_frac_of_bf16_mfma_peak": round(flop / ms_ds / 1e9 / MFMA_BF16_PEAK_TFLOPS, 4),
                    "library_gemm_on_decompressed_ms": round(ms_ls, 5)}
        ms_lib = (time_steady(torch, lambda: torch.matmul(dy.t(), xh), iters) if N > 64 else
                  time_events(torch, lambda: torch.matmul(dy.t(), xh), iters, warm))
        rec["library_gemm_on_decompressed_ms"] = round(ms_lib, 5)
        out[name] = rec
        del dy, dw, ws
    del xh
    return out


def hbm_yardstick(torch):
    """what the framework's own streaming kernels reach on this GPU in this run, on tensors that do not fit the
    Infinity Cache (512 MiB each): a device copy (1 read + 1 write per byte) and c = a + b (2 reads + 1 write)"""
    n = 256 << 20                                               # bf16 elements: 512 MiB per tensor
    a = torch.empty(n, dtype=torch.bfloat16, device="cuda").normal_()
    b = torch.empty_like(a).normal_()
    c = torch.empty_like(a)
    t_copy = time_events(torch, lambda: c.copy_(a), 20, 3)
    t_add = time_events(torch, lambda: torch.add(a, b, out=c), 20, 3)
    out = {"tensor_bytes": 2 * n, "copy": hbm(4 * n, t_copy), "add": hbm(6 * n, t_add)}
    del a, b, c
    torch.cuda.empty_cache()
    return out


def config1_extra(pkg, torch):
    """BASELINE configs[0] on the GPU: standalone compress + decompress of x [4,512,4096] (41 outlier channels x50,
    INT4, group 128), and the same at 16x the tokens"""
    K = pkg.kernels
    out = {}
    for tag, M in (("tokens_2048", 2048), ("tokens_32768", 32768)):
        H, bits, G, k = 4096, 4, 128, 41
        x, _ = make_activation(torch, M, H, k, 50.0, seed=11)
        plan = K.select_channels(K.channel_absmax(x), k)
        c = K.compress_channel(x, plan, bits, G)
        side = side_bytes(H, bits, G, k)
        t_c = time_graph(torch, lambda: K.compress_channel(x, plan, bits, G))
        t_d = time_graph(torch, lambda: K.decompress_channel(c))
        t_p = time_graph(torch, lambda: K.select_channels(K.channel_absmax(x), k))
        assert torch.equal(K.decompress_channel(K.compress_channel(x, plan, bits, G)), K.decompress_channel(c))
        out[tag] = {"compress": hbm(M * (2 * H + side), t_c), "decompress": hbm(M * (2 * H + side), t_d),
                    "round_trip": hbm(2 * M * (2 * H + side), t_c + t_d),
                    "channel_absmax_and_select_ms": round(t_p, 5)}
        del x, c
    return out


def config4_extra(pkg, torch):
    """BASELINE configs[3]: gate / up [4,1024,11008] with 1 % outlier channels x20, INT4 group 128: SiLU backward,
    the one-pass backward and forward of SiLU(gate)*up, the forwards with their saves, and the down_proj weight gradient (dY [4096,4096], 369 GFLOP) with its
    LoRA-A (r = 16) companion"""
    K = pkg.kernels
    M, H, bits, G = 4096, 11008, 4, 128
    k = K.num_outlier_channels(H, 0.01)
    gate, gen = make_activation(torch, M, H, k, 20.0, seed=41)
    up, _ = make_activation(torch, M, H, k, 20.0, seed=42)
    act = torch.nn.functional.silu(gate.float()).bfloat16()
    prod = (act.float() * up.float()).bfloat16()
    g = (0.02 * torch.randn(M, H, generator=gen, device="cuda")).bfloat16()
    cg, cu, ca, cp = [K.compress_channel(t, K.select_channels(K.channel_absmax(t), k), bits, G) for t in (gate, up, act, prod)]
    side = side_bytes(H, bits, G, k)
    out = {"silu_bwd": hbm(M * (4 * H + side), time_graph(torch, lambda: K.act_bwd("silu", g, cg))),
           "gated_silu_bwd": hbm(M * (6 * H + 3 * side), time_graph(torch, lambda: K.gated_act_bwd("silu", g, ca, cu, cg))),
           "silu_fwd_compress": hbm(M * (4 * H + side), time_graph(torch, lambda: K.act_fwd_compress("silu", gate, cg.plan, bits, G))),
           # SiLU(gate) * up and the three saves (act(gate), up, gate) in one pass: reads gate and up, writes the product
           "gated_silu_fwd": hbm(M * (6 * H + 3 * side), time_graph(torch, lambda: K.gated_act_fwd("silu", gate, up, ca.plan, cu.plan, cg.plan, bits, G))),
           "product_fwd_compress": hbm(M * (6 * H + 2 * side), time_graph(torch, lambda: K.hadamard_fwd_compress(act, up, ca.plan, cu.plan, bits, G)))}
    del gate, up, act, prod, g, cg, cu, ca
    out["down_proj"] = gradw_extra(pkg, torch, cp, shapes=(("full_w", 4096, 60, 20), ("lora_a_r16", 16, 300, 30), ("lora_a_r64", 64, 300, 30)))
    return out


def kernel_tour(pkg, torch, reps=5):
    """every kernel of the path at the BASELINE config shapes (INT4 / group 128 and INT2 / group 64, 1 % outlier
    channels): compress, decompress, activation / Hadamard / gated backward and forward, weight gradient"""
    K = pkg.kernels
    gen = torch.Generator(device="cuda").manual_seed(0)

    def mk(M, H, hot):
        x = torch.randn(M, H, generator=gen, device="cuda")
        x[:, torch.randperm(H, generator=gen, device="cuda")[:hot]] *= 30
        return x.bfloat16()

    for (M, H, bits, G) in ((4096, 4096, 4, 128), (4096, 4096, 2, 64), (4096, 11008, 4, 128)):
        k = K.num_outlier_channels(H, 0.01)
        x, up = mk(M, H, k // 2), mk(M, H, k // 2)
        a = torch.nn.functional.silu(x)
        g = (0.02 * torch.randn(M, H, generator=gen, device="cuda")).bfloat16()
        cs = [K.compress_channel(t, K.select_channels(K.channel_absmax(t), k), bits, G) for t in (x, up, a)]
        plan = K.select_channels(K.channel_absmax(x), k)
        dy16 = (0.01 * torch.randn(M, 16, generator=gen, device="cuda")).bfloat16()
        dyN = (0.01 * torch.randn(M, 4096, generator=gen, device="cuda")).bfloat16()
        for _ in range(reps):
            K.compress_channel(x, plan, bits, G)
            K.decompress_channel(cs[0])
            K.act_bwd("silu", g, cs[0])
            K.act_bwd("gelu", g, cs[0])
            K.hadamard_bwd(g, cs[2], cs[1])
            K.gated_act_bwd("silu", g, cs[2], cs[1], cs[0])
            if K.gated_act_fwd_supported(H, bits, G):
                K.gated_act_fwd("silu", x, up, cs[2].plan, cs[1].plan, cs[0].plan, bits, G)
            K.act_fwd_compress("silu", x, plan, bits, G)
            K.act_fwd_compress("gelu", x, plan, bits, G)
            if K.hadamard_fwd_compress_supported(H, bits, G, bits, G):
                K.hadamard_fwd_compress(a, up, cs[2].plan, cs[1].plan, bits, G)
            K.gradw_gemm(dy16, cs[0])
            K.gradw_gemm(dyN, cs[0], staged=False)        # x_hat decoded inside the GEMM
            K.gradw_gemm(dyN, cs[0], staged=True)         # x_hat restored once, then the dense form of the kernel
        torch.cuda.synchronize()
        del x, up, a, g, cs
    # the trained shape of the weight gradient (LoRA-A, 16 features) at 16x config 2's tokens, INT4 and INT2 / group 64
    M, H = 65536, 4096
    x = mk(M, H, 20)
    plan = K.select_channels(K.channel_absmax(x), 41)
    dy16 = (0.01 * torch.randn(M, 16, generator=gen, device="cuda")).bfloat16()
    for bits, G in ((4, 128), (2, 64)):
        c = K.compress_channel(x, plan, bits, G)
        for _ in range(reps):
            K.gradw_gemm(dy16, c)
        torch.cuda.synchronize()
        del c
    del x, dy16
    # the reference snapshot's own scheme (element threshold, static scale) at config 2's shape: 1 % outlier
    # elements, INT4, per-token and per-channel scales; consumers take the restored activation
    M, H, S = 4096, 4096, 1024
    x = mk(M, H, 20)
    g = (0.02 * torch.randn(M, H, generator=gen, device="cuda")).bfloat16()
    w = 1 + 0.1 * torch.randn(H, generator=gen, device="cuda")
    thr = float(x.float().abs().flatten()[::7].kthvalue(int(M * H / 7 * 0.99)).values)
    xf = x.float()
    for scale in (((xf.amax(-1, keepdim=True) - xf.amin(-1, keepdim=True)) / 15)[:S].bfloat16().contiguous(),
                  ((xf.amax(0, keepdim=True) - xf.amin(0, keepdim=True)) / 15).bfloat16().contiguous()):
        for _ in range(reps):
            c = K.compress_threshold(x, S, thr, scale, 4)
            xh = K.decompress_threshold(c)
            y, rstd, c2 = K.rmsnorm_fwd_compress_threshold(x, w, 1e-6, S, thr, scale, 4)
            K.rmsnorm_bwd(g, xh, w, rstd)
            K.act_bwd("silu", g, xh)
            K.hadamard_bwd(g, xh, xh)
        torch.cuda.synchronize()
    del x, xf, g, c, c2, xh, y
    # softmax at config 5's shape: probabilities [1, 32, 2048, 2048], 5 % kept
    x = (2.0 * torch.randn(1, 32, 2048, 2048, generator=gen, device="cuda")).bfloat16()
    g = (0.01 * torch.randn(1, 32, 2048, 2048, generator=gen, device="cuda")).bfloat16()
    y, _ = K.softmax_fwd(x)
    thr = float(y.float().flatten()[::101].kthvalue(int(y.numel() / 101 * 0.95)).values)
    for _ in range(reps):
        y, sp = K.softmax_fwd(x, thr)
        K.softmax_bwd(g, sp)
    torch.cuda.synchronize()
    print(json.dumps({"kernel_tour": True}))


def layer_report(pkg, torch, steps=6, attentions=("eager", "flash"), quiet=False, compressions=(True, False)):
    """full LLaMA-2-7B-shaped decoder layer (hidden 4096, 32 x 128 heads, intermediate 11008, NF4 base, LoRA r=16 on
    all seven projections), forward + backward, at batch 1 x seq 2048 and batch 4 x seq 1024: what the forward keeps
    for the backward, the peak above the resident weights, and the step time - with every saved activation compressed
    (1 % outlier channels, INT2 for linear inputs, INT4 elsewhere) and with the same layer keeping bf16; each with the
    attention the reference wires into its models (scores, softmax, kept probabilities) and with the library's fused
    attention kernel around compressed q, k, v and output."""
    DL = importlib.import_module("hyc-lora_amd.decoder_layer")
    out = []
    for compress, attention in [(c, a) for c in compressions for a in attentions]:
        layer = DL.DecoderLayer(DL.LayerConfig(compress=compress, attention=attention))
        torch.cuda.synchronize()
        for (B, S) in ((1, 2048), (4, 1024)):
            gen = torch.Generator(device="cuda").manual_seed(B * 7 + S)
            x = torch.randn(B, S, 4096, generator=gen, device="cuda")
            x[..., torch.randperm(4096, generator=gen, device="cuda")[:20]] *= 30
            x = x.bfloat16()
            g = (0.01 * torch.randn(B, S, 4096, generator=gen, device="cuda")).bfloat16()
            for mod in layer.modules():                      # a new sequence length calibrates again
                if hasattr(mod, "iteration"):
                    mod.iteration = 0
            layer.attention.static_value = None
            times, held, peak = [], 0, 0
            for it in range(3 + steps):
                for p in layer.parameters():
                    p.grad = None
                xg = x.clone().requires_grad_(True)
                torch.cuda.synchronize()
                torch.cuda.reset_peak_memory_stats()
                base = torch.cuda.memory_allocated()
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                y = layer(xg)
                if it == 3 + steps - 1:
                    torch.cuda.synchronize()
                    held = torch.cuda.memory_allocated() - base - y.numel() * 2
                y.backward(g)
                e1.record()
                torch.cuda.synchronize()
                if it >= 3:
                    times.append(e0.elapsed_time(e1))
                    peak = max(peak, torch.cuda.max_memory_allocated() - base)
                del y, xg
            times.sort()
            # the same steps issued back to back, as a training loop issues them (no synchronisation between steps, so
            # the host's launch latency after an idle GPU is paid once, not per step)
            xg = x.clone().requires_grad_(True)
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            torch.cuda.synchronize()
            e0.record()
            for it in range(steps):
                for p in layer.parameters():
                    p.grad = None
                xg.grad = None
                layer(xg).backward(g)
            e1.record()
            torch.cuda.synchronize()
            rec = {"layer_report": True, "compress": compress, "attention": attention, "batch": B, "seq": S,
                   "saved_for_backward_bytes": int(held), "peak_above_weights_bytes": int(peak),
                   "step_ms": round(times[len(times) // 2], 3),
                   "step_ms_back_to_back": round(e0.elapsed_time(e1) / steps, 3)}
            del xg
            if compress:
                rec["saved_analytic_bytes"] = int(layer.saved_activation_bytes(B, S))
            out.append(rec)
            if not quiet:
                print(json.dumps(rec), flush=True)
        del layer
        torch.cuda.empty_cache()
    return out


def cpu_baseline(torch, wl, rows, seconds):
    """the oracle (CPU PyTorch restatement of the path) on the host cores, bounded sample of the same workload"""
    from oracle import hyc_oracle as O
    threads = min(os.cpu_count() or 1, 16)
    torch.set_num_threads(threads)
    x = wl.x[:rows].cpu()
    dy = wl.dy[:rows].cpu()
    w = wl.w_host
    idx = wl.plan.idx.cpu()
    H, bits, group = wl.H, wl.bits, wl.group

    def one():
        y, rstd = O.rmsnorm_fwd(x, w, 1e-6)
        vals, stored, scales = O.hyc_compress(x, idx, bits, group)
        xh = O.hyc_decompress(vals, stored, idx, scales, bits, group)
        return O.rmsnorm_bwd(dy, xh, w, rstd)

    one()
    t0 = time.perf_counter()
    reps = 0
    while time.perf_counter() - t0 < seconds:
        one()
        reps += 1
    dt = (time.perf_counter() - t0) / reps
    fwd_b, bwd_b, _ = algorithmic_bytes(rows, H, bits, group, wl.k)
    return {"value": round((fwd_b + bwd_b) / dt / 1e9, 4), "unit": "GB/s", "cores": threads, "kind": "port",
            "sample": "oracle rmsnorm_fwd + hyc_compress + hyc_decompress + rmsnorm_bwd on the first %d of %d tokens "
                      "(H=%d), mean of %d passes, %.3f s per pass" % (rows, wl.M, H, reps, dt),
            "round_trip": cpu_round_trip(torch, O, threads)}


def cpu_round_trip(torch, O, threads):
    """the standalone compress -> decompress round trip of the oracle at configs[0]'s size (2048 x 4096, 41 channels
    x50) and at configs[1]'s (4096 x 4096): 3 warm-ups, median of 10, algorithmic GB/s (20 772 B per token)"""
    out = {}
    for tag, M, gain in (("config1_2048x4096", 2048, 50.0), ("config2_size_4096x4096", 4096, 50.0)):
        H, bits, group, k = 4096, 4, 128, 41
        gen = torch.Generator().manual_seed(0)
        x = torch.randn(M, H, generator=gen)
        x[:, torch.randperm(H, generator=gen)[:k]] *= gain
        x = x.bfloat16()
        idx = O.hyc_select_channels(O.hyc_channel_scores(x), k)

        def trip():
            vals, stored, scales = O.hyc_compress(x, idx, bits, group)
            return O.hyc_decompress(vals, stored, idx, scales, bits, group)

        for _ in range(3):
            trip()
        times = []
        for _ in range(10):
            t0 = time.perf_counter()
            trip()
            times.append(time.perf_counter() - t0)
        times.sort()
        med = 0.5 * (times[4] + times[5])
        nbytes = 2 * M * (2 * H + side_bytes(H, bits, group, k))
        out[tag] = {"ms": round(med * 1e3, 2), "GBps": round(nbytes / med / 1e9, 3), "bytes": nbytes, "cores": threads}
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-scaled", action="store_true", help="skip the 16x token-scaled run")
    ap.add_argument("--no-extras", action="store_true", help="skip the legs of the other BASELINE configurations")
    ap.add_argument("--kernel-tour", action="store_true",
                    help="for rocprofv3 --kernel-trace: run every kernel of the path a few times at the config shapes, then exit")
    ap.add_argument("--pmc-probe", action="store_true",
                    help="for rocprofv3 --pmc: 5x a plain 32 MiB device copy, 5x fwd, 5x bwd, then exit")
    ap.add_argument("--layer-report", action="store_true",
                    help="full decoder layer (the fifth BASELINE configuration): saved bytes, peak memory, step time; then exit")
    ap.add_argument("--layer-compress", choices=["on", "off", "both"], default="both",
                    help="with --layer-report: the layer with compressed activations, the same layer keeping bf16, or both")
    ap.add_argument("--layer-attention", choices=["eager", "flash", "both"], default="both",
                    help="with --layer-report: which attention form(s) of the layer to run")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.exit("bench.py: this path runs on ONE GPU (no sharding, no collectives); run with --gpus 1")

    import torch
    pkg = importlib.import_module("hyc-lora_amd")
    if not os.path.exists(pkg._abi.LIB_PATH):
        import __graft_entry__
        __graft_entry__.build()
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)

    M, H, bits, group = 4 * 1024, 4096, 4, 128
    wl = Workload(pkg, torch, M, H, bits, group, n_hot=20, gain=30.0)
    fwd_b, bwd_b, saved_b = algorithmic_bytes(M, H, bits, group, wl.k)

    if args.kernel_tour:
        kernel_tour(pkg, torch)
        return
    if args.layer_report:
        del wl
        layer_report(pkg, torch, attentions=("eager", "flash") if args.layer_attention == "both" else (args.layer_attention,),
                     compressions={"on": (True,), "off": (False,), "both": (True, False)}[args.layer_compress])
        return
    if args.pmc_probe:
        dst = torch.empty_like(wl.x)
        for _ in range(5):
            dst.copy_(wl.x)          # reads 2*M*H bytes, writes 2*M*H bytes: the counters' yardstick
        for _ in range(5):
            wl.fwd()
        for _ in range(5):
            wl.bwd()
        for case in (("silu", 4), ("gelu", 4)):
            for _ in range(5):
                pkg.kernels.act_bwd(case[0], wl.dy, wl.c)
        torch.cuda.synchronize()
        print(json.dumps({"pmc_probe": True, "copy_bytes_each_way": 2 * M * H, "fwd_bytes": fwd_b, "bwd_bytes": bwd_b}))
        return

    # ---- the other configurations and the long runs first: they also bring the clocks up before the short timed
    # region (a cold 20-step loop of 15-microsecond kernels reads 10-15 % slower than the same loop on a busy GPU)
    extra = {}
    # the weight-gradient legs read the activation that the forward saves: fill it first (a matrix-core kernel on an
    # operand of zeros, which freshly allocated memory holds, draws less power and reads 20-25 % faster than on data)
    wl.fwd()
    torch.cuda.synchronize()
    assert int(wl.c.stored.view(torch.uint8).max()) > 0, "the compressed activation is empty"
    extra["gradw_gemm_int4"] = gradw_extra(pkg, torch, wl.c, sustained=not args.no_extras)
    if not args.no_extras:
        extra["config1_compress_decompress"] = config1_extra(pkg, torch)
        K = pkg.kernels
        x3, _ = make_activation(torch, M, H, wl.k, 30.0, seed=31)
        c3 = K.compress_channel(x3, K.select_channels(K.channel_absmax(x3), wl.k), 2, 64)
        extra["config3_gradw_int2_g64"] = gradw_extra(pkg, torch, c3)
        del x3, c3
        extra["config4_mlp_h11008"] = config4_extra(pkg, torch)
    if not args.no_scaled:
        extra["hbm_yardstick"] = hbm_yardstick(torch)
        # the config-size working set (~150 MB) fits the 256 MB Infinity Cache; 16x the tokens does not
        Ms = 16 * M
        wls = Workload(pkg, torch, Ms, H, bits, group, n_hot=20, gain=30.0, seed=1)
        fs, bs, _ = algorithmic_bytes(Ms, H, bits, group, wls.k)
        f_ms = time_events(torch, wls.fwd, 60, 10)
        b_ms = time_events(torch, wls.bwd, 60, 10)
        bm_ms = time_events(torch, wls.bwd_main, 60, 10)
        extra["scaled16x"] = {"tokens": Ms, "fwd_ms": round(f_ms, 4), "fwd_GBps": round(fs / f_ms / 1e6, 1),
                              "bwd_ms": round(b_ms, 4), "bwd_GBps": round(bs / b_ms / 1e6, 1),
                              "bwd_row_kernel_ms": round(bm_ms, 4),
                              "fwd_frac_of_hbm_peak": round(fs / f_ms / 1e6 / HBM_PEAK_GBPS, 4),
                              "bwd_frac_of_hbm_peak": round(bs / b_ms / 1e6 / HBM_PEAK_GBPS, 4),
                              "bwd_row_kernel_frac_of_hbm_peak": round(bs / bm_ms / 1e6 / HBM_PEAK_GBPS, 4)}
        if not args.no_extras:
            # the trained shape of the weight gradient (LoRA-A, 16 features) on the same 16x activation: INT4 with
            # 128-channel groups (what the fused norm saved) and INT2 with 64-channel groups (configs[2]'s width)
            lora = (("lora_a_r16", 16, 100, 20),)
            extra["scaled16x"]["gradw_int4_g128"] = gradw_extra(pkg, torch, wls.c, shapes=lora)["lora_a_r16"]
            c2s = pkg.kernels.compress_channel(wls.x, wls.plan, 2, 64)
            extra["scaled16x"]["gradw_int2_g64"] = gradw_extra(pkg, torch, c2s, shapes=lora)["lora_a_r16"]
            del c2s
        del wls
        torch.cuda.empty_cache()
    if not args.no_extras:
        # configs[4]: the decoder layer with the reference's attention wiring, every saved activation compressed / kept bf16
        extra["config5_decoder_layer"] = layer_report(pkg, torch, steps=4, attentions=("eager",), quiet=True)
        torch.cuda.empty_cache()

    # the step as a HIP graph (three launches; removes the host launch cost from the timed loop)
    wl.step()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        wl.step()
    torch.cuda.current_stream().wait_stream(side)
    with torch.cuda.graph(graph):
        wl.step()

    def wall(fn):
        for _ in range(args.warmup):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3 / args.steps

    # per-kernel durations with events on the launch stream, over enough launches for a steady clock; they come
    # before the timed region so that it starts on a busy GPU
    n_ev = max(args.steps, 500)
    fwd_ms = time_events(torch, wl.fwd, n_ev, 50)
    bwd_ms = time_events(torch, wl.bwd, n_ev, 50)
    bwd_main_ms = time_events(torch, wl.bwd_main, n_ev, 50)                  # the row kernel alone
    eager_ms = time_events(torch, wl.step, n_ev, 50)

    # the timed region: W warm-up steps, then exactly K steps between two synchronisations, launched back to back on
    # one stream (the kernels of a step are short enough that a graph replay per step costs more than it saves)
    ms_step = wall(wl.step)
    ms_graph = wall(graph.replay)
    del graph

    value = (fwd_b + bwd_b) / (ms_step * 1e-3) / 1e9
    fresh = TRAFFIC_SOURCES_SHA != "" and sources_sha() == TRAFFIC_SOURCES_SHA
    if bwd_main_ms >= fwd_ms:
        dom_name, dom_ms, dom_b, dom_traffic = "hyc::k_rmsnorm_bwd_fast<4, true, true, 1024, false>", bwd_main_ms, bwd_b, TRAFFIC_BWD
    else:
        dom_name, dom_ms, dom_b, dom_traffic = "hyc::k_rmsnorm_fwd_fast<4, 16, true, 256, 1>", fwd_ms, fwd_b, TRAFFIC_FWD
    achieved = dom_b / (dom_ms * 1e-3) / 1e9
    extra.update({
        "graph_replay_ms_per_step": round(ms_graph, 5), "event_ms_per_step": round(eager_ms, 5),
        "event_loop_launches": n_ev,
        "fwd_kernel_ms": round(fwd_ms, 5), "fwd_GBps": round(fwd_b / fwd_ms / 1e6, 1),
        "fwd_frac_of_hbm_peak": round(fwd_b / fwd_ms / 1e6 / HBM_PEAK_GBPS, 4),
        "bwd_kernels_ms": round(bwd_ms, 5), "bwd_GBps": round(bwd_b / bwd_ms / 1e6, 1),
        "bwd_row_kernel_ms": round(bwd_main_ms, 5), "bwd_row_kernel_GBps": round(bwd_b / bwd_main_ms / 1e6, 1),
        "bwd_row_kernel_frac_of_hbm_peak": round(bwd_b / bwd_main_ms / 1e6 / HBM_PEAK_GBPS, 4),
        "act_mem_bytes_saved_tensor": saved_b + 4 * M, "act_mem_bytes_bf16": 2 * M * H,
        "act_mem_ratio": round(2 * M * H / (saved_b + 4 * M), 3),
        "scale_rule": "absmax",
        "traffic_note": ("HBM bytes per launch from rocprofv3 FETCH_SIZE / WRITE_SIZE runs of `bench.py --pmc-probe` "
                         "(profiles/rmsnorm_fwd_bwd_config2.md), taken with these kernel sources" if fresh else
                         "null: the kernel sources differ from the ones the committed counter runs were taken with"),
    })
    out = {
        "metric": "compress+decompress GB/s", "value": round(value, 2), "unit": "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_step, 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "BASELINE configs[1]: fused RMSNorm fwd+compress and bwd(decompress), x bf16 [4,1024,4096], "
                               "20 hot channels x30, 1% outlier channels kept bf16, INT4 codes, group 128, w fp32, eps 1e-6",
                   "tokens": M, "hidden": H, "bits": bits, "group": group, "outlier_channels": wl.k,
                   "launch": "fwd + bwd (+ dw column sum) entry points back to back on one stream"},
        "roofline": {"bound": "hbm", "kernel": dom_name, "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4), "algorithmic_bytes": dom_b,
                     "traffic": dom_traffic if fresh else None},
        "extra": extra,
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(torch, wl, rows=M, seconds=12.0)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
