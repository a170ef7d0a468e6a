"""Writes the golden vectors under tests/golden/ by running the reference's own CPU-runnable
functions.  Runs only where the reference checkout is mounted (REFERENCE_ROOT, default
/root/reference); the fixtures it writes are committed, the reference never is.

    python tests/golden/make_golden.py

Covered (functions that nothing but the reference itself pins against transcription error):
  * get_statistics                       operators/compress_function.py:292-340
  * true_divide_outlier_suboutlier_svd_compress / _decompress   :136-261
  * get_statistics_softmax, true_compress_softmax, true_decompress_softmax   :264-347
  * EfficientMemorySiLU / GELU / Hadamard / Softmax modules: three calls each (two calibration
    calls + one steady-state call) with backward, which pins the running-mean protocol and
    the op-by-op bf16 backward formulas.
bf16 tensors are stored as their uint16 bit patterns (numpy has no bf16).
"""
import os
import sys

import numpy as np
import torch

REFERENCE_ROOT = os.environ.get("REFERENCE_ROOT", "/root/reference")
HERE = os.path.dirname(os.path.abspath(__file__))


def bits_of(t):
    """tensor -> numpy array; bf16 as uint16 bit patterns."""
    t = t.detach().cpu().contiguous()
    if t.dtype == torch.bfloat16:
        return t.view(torch.int16).numpy().view(np.uint16)
    return t.numpy()


def make_input(gen, shape, n_hot, gain):
    x = torch.randn(*shape, generator=gen)
    H = shape[-1]
    hot = torch.randperm(H, generator=gen)[:n_hot]
    x[..., hot] *= gain
    return x.bfloat16()


def main():
    sys.path.insert(0, REFERENCE_ROOT)
    import operators.compress_function as cf                 # noqa: E402
    from operators.efficient_silu import EfficientMemorySiLU  # noqa: E402
    from operators.efficient_gelu import EfficientMemoryGELU  # noqa: E402
    from operators.efficient_hadamard import EfficientMemoryHadamard  # noqa: E402
    from operators.efficient_softmax import EfficientMemorySoftmax    # noqa: E402

    # ---------------------------------------------------------------- compress / decompress
    out = {}
    case = 0
    for shape in [(2, 16, 64), (1, 8, 256)]:
        for bits in (1, 2, 4, 8):
            for method in ('per-tensor', 'per-channel', 'per-token'):
                for rank in (0, 2):
                    gen = torch.Generator().manual_seed(1000 + case)
                    x = make_input(gen, shape, 2, 20.0)
                    torch.manual_seed(2000 + case)              # svd_lowrank draws from the global RNG
                    thr, L, R, scale = cf.get_statistics(x, 0, 0.05, 1.0, bits, method, rank)
                    coo, stored, scale2 = cf.true_divide_outlier_suboutlier_svd_compress(
                        x, thr, scale, bits, 1.0, L, R)
                    coo = coo.coalesce() if not coo.is_coalesced() else coo
                    xhat = cf.true_divide_outlier_suboutlier_svd_decompress(
                        coo, stored, bits, scale2, L=L, R=R)
                    p = f"c{case}_"
                    out[p + "meta"] = np.array([bits, rank, 1000 + case, 2000 + case] + list(shape), dtype=np.int64)
                    out[p + "method"] = np.array(method)
                    out[p + "x"] = bits_of(x)
                    out[p + "thr"] = bits_of(thr)
                    out[p + "L"] = bits_of(L)
                    out[p + "R"] = bits_of(R)
                    out[p + "scale"] = bits_of(scale)
                    out[p + "coo_idx"] = bits_of(coo.indices())
                    out[p + "coo_val"] = bits_of(coo.values())
                    out[p + "stored"] = bits_of(stored)
                    out[p + "xhat"] = bits_of(xhat)
                    case += 1
    # one head-shaped [B, nh, S, hd] case per bit width (is_head path, :138-141, :258-259)
    for bits in (2, 4, 8):
        gen = torch.Generator().manual_seed(1000 + case)
        x = make_input(gen, (2, 4, 8, 16), 1, 10.0)
        torch.manual_seed(2000 + case)
        thr, L, R, scale = cf.get_statistics(x, 0, 0.05, 1.0, bits, 'per-channel', 0)
        coo, stored, scale2 = cf.true_divide_outlier_suboutlier_svd_compress(x, thr, scale, bits, 1.0, L, R)
        xhat = cf.true_divide_outlier_suboutlier_svd_decompress(coo, stored, bits, scale2, is_head=True,
                                                                num_heads=4, L=L, R=R)
        p = f"c{case}_"
        out[p + "meta"] = np.array([bits, 0, 1000 + case, 2000 + case, 2, 4, 8, 16], dtype=np.int64)
        out[p + "method"] = np.array('per-channel')
        out[p + "x"] = bits_of(x)
        out[p + "thr"] = bits_of(thr)
        out[p + "L"] = bits_of(L)
        out[p + "R"] = bits_of(R)
        out[p + "scale"] = bits_of(scale)
        out[p + "coo_idx"] = bits_of(coo.indices())
        out[p + "coo_val"] = bits_of(coo.values())
        out[p + "stored"] = bits_of(stored)
        out[p + "xhat"] = bits_of(xhat)
        case += 1
    out["n_cases"] = np.array(case)
    np.savez_compressed(os.path.join(HERE, "compress_cases.npz"), **out)
    print("compress_cases:", case, "cases")

    # ---------------------------------------------------------------- softmax helpers
    out = {}
    gen = torch.Generator().manual_seed(31)
    logits = (3 * torch.randn(2, 2, 8, 16, generator=gen)).bfloat16()
    y = torch.softmax(logits, dim=-1)
    thr = cf.get_statistics_softmax(y, 0, 0.05)
    sp = cf.true_compress_softmax(y, thr).coalesce()
    out["y"] = bits_of(y)
    out["thr"] = bits_of(thr)
    out["coo_idx"] = bits_of(sp.indices())
    out["coo_val"] = bits_of(sp.values())
    out["dense"] = bits_of(cf.true_decompress_softmax(sp))
    out["pruned"] = bits_of(cf.prune_softmax(y, thr))
    np.savez_compressed(os.path.join(HERE, "softmax_cases.npz"), **out)

    # ---------------------------------------------------------------- module protocols
    out = {}

    def run_module(tag, mod, n_inputs, shape, bits_list):
        for call in range(3):
            gen = torch.Generator().manual_seed(500 + call + 17 * len(tag))
            xs = [make_input(gen, shape, 2, 8.0).requires_grad_(True) for _ in range(n_inputs)]
            g = (0.1 * torch.randn(*shape, generator=gen)).bfloat16()
            torch.manual_seed(900 + call)
            y = mod(*xs)
            y.backward(g)
            p = f"{tag}_call{call}_"
            for i, xi in enumerate(xs):
                out[p + f"x{i}"] = bits_of(xi)
                out[p + f"dx{i}"] = bits_of(xi.grad)
            out[p + "g"] = bits_of(g)
            out[p + "y"] = bits_of(y)
            statics = [mod.static_value] if n_inputs == 1 else [mod.static_value_1, mod.static_value_2]
            for i, sv in enumerate(statics):
                out[p + f"s{i}_thr"] = bits_of(sv[0])
                out[p + f"s{i}_L"] = bits_of(sv[1])
                out[p + f"s{i}_scale"] = bits_of(sv[2])
                out[p + f"s{i}_R"] = bits_of(sv[3])
            out[p + "iteration"] = np.array(mod.iteration)

    shape = (2, 8, 64)
    run_module("silu_b4_pc_r0", EfficientMemorySiLU(0.05, 1.0, 4, 'per-channel', 0), 1, shape, [4])
    run_module("silu_b8_pt_r2", EfficientMemorySiLU(0.05, 1.0, 8, 'per-token', 2), 1, shape, [8])
    run_module("gelu_b2_pt_r0", EfficientMemoryGELU(0.05, 1.0, 2, 'per-tensor', 0), 1, shape, [2])
    run_module("gelu_b4_pc_r0", EfficientMemoryGELU(0.05, 1.0, 4, 'per-channel', 0), 1, shape, [4])
    run_module("had_b4_b2_r0", EfficientMemoryHadamard(0.05, 1.0, 4, 'per-channel', 0.05, 1.0, 2, 'per-token', 0),
               2, shape, [4, 2])

    sm = EfficientMemorySoftmax(0.05)
    for call in range(3):
        gen = torch.Generator().manual_seed(700 + call)
        x = (3 * torch.randn(2, 2, 8, 16, generator=gen)).bfloat16().requires_grad_(True)
        g = (0.1 * torch.randn(2, 2, 8, 16, generator=gen)).bfloat16()
        y = sm(x)
        y.backward(g)
        p = f"softmax_call{call}_"
        out[p + "x"] = bits_of(x)
        out[p + "g"] = bits_of(g)
        out[p + "y"] = bits_of(y)
        out[p + "dx"] = bits_of(x.grad)
        out[p + "thr"] = bits_of(sm.static_value)
    np.savez_compressed(os.path.join(HERE, "module_cases.npz"), **out)
    for f in ("compress_cases.npz", "softmax_cases.npz", "module_cases.npz"):
        print(f, os.path.getsize(os.path.join(HERE, f)), "bytes")


if __name__ == "__main__":
    main()
