"""The CPU oracle against the golden vectors written from the reference (tests/golden/make_golden.py)."""
import numpy as np
import pytest
import torch

from conftest import bits_equal, from_bits
from oracle import hyc_oracle as O


def _case(gc, i):
    p = f"c{i}_"
    meta = gc[p + "meta"]
    return dict(bits=int(meta[0]), rank=int(meta[1]), seed_svd=int(meta[3]), shape=tuple(int(v) for v in meta[4:]),
                method=str(gc[p + "method"]), x=from_bits(gc[p + "x"]), thr=from_bits(gc[p + "thr"]),
                L=from_bits(gc[p + "L"]), R=from_bits(gc[p + "R"]), scale=from_bits(gc[p + "scale"]),
                coo_idx=from_bits(gc[p + "coo_idx"]), coo_val=from_bits(gc[p + "coo_val"]),
                stored=from_bits(gc[p + "stored"]), xhat=from_bits(gc[p + "xhat"]))


def test_case_count(golden_compress):
    assert int(golden_compress["n_cases"]) == 51


@pytest.mark.parametrize("i", range(51))
def test_get_statistics(golden_compress, i):
    c = _case(golden_compress, i)
    torch.manual_seed(c["seed_svd"])
    thr, L, R, scale = O.get_statistics(c["x"], 0, 0.05, 1.0, c["bits"], c["method"], c["rank"])
    assert thr.dtype == torch.float32 and torch.equal(thr, c["thr"])
    assert bits_equal(L, c["L"]) and bits_equal(R, c["R"])
    assert bits_equal(scale, c["scale"])


@pytest.mark.parametrize("i", range(51))
def test_compress_decompress(golden_compress, i):
    c = _case(golden_compress, i)
    coo, stored, scale = O.ref_compress(c["x"], c["thr"], c["scale"], c["bits"], 1.0, c["L"], c["R"])
    coo = coo.coalesce()
    assert torch.equal(coo.indices(), c["coo_idx"])
    assert bits_equal(coo.values(), c["coo_val"])
    assert stored.dtype == c["stored"].dtype and torch.equal(stored, c["stored"])
    is_head = len(c["shape"]) == 4
    xhat = O.ref_decompress(coo, stored, c["bits"], scale, is_head=is_head,
                            num_heads=c["shape"][1] if is_head else 1, L=c["L"], R=c["R"])
    assert bits_equal(xhat, c["xhat"])


def test_softmax_helpers(golden_softmax):
    g = golden_softmax
    y = from_bits(g["y"])
    thr = O.get_statistics_softmax(y, 0, 0.05)
    assert torch.equal(thr, from_bits(g["thr"]))
    sp = O.true_compress_softmax(y, thr).coalesce()
    assert torch.equal(sp.indices(), from_bits(g["coo_idx"]))
    assert bits_equal(sp.values(), from_bits(g["coo_val"]))
    assert bits_equal(O.true_decompress_softmax(sp), from_bits(g["dense"]))
    assert bits_equal(O.prune_softmax(y, thr), from_bits(g["pruned"]))


MODS = {
    "silu_b4_pc_r0": ("silu", [(0.05, 1.0, 4, 'per-channel')], 0),
    "silu_b8_pt_r2": ("silu", [(0.05, 1.0, 8, 'per-token')], 2),
    "gelu_b2_pt_r0": ("gelu", [(0.05, 1.0, 2, 'per-tensor')], 0),
    "gelu_b4_pc_r0": ("gelu", [(0.05, 1.0, 4, 'per-channel')], 0),
    "had_b4_b2_r0": ("had", [(0.05, 1.0, 4, 'per-channel'), (0.05, 1.0, 2, 'per-token')], 0),
}


@pytest.mark.parametrize("tag", sorted(MODS))
def test_module_protocol(golden_modules, tag):
    """three calls of an operator assembled from oracle pieces: forward value, calibration running
    mean, compress -> decompress -> backward formula, all bit-exact with the reference modules."""
    gm = golden_modules
    kind, knobs, rank = MODS[tag]
    statics = [[None] * 4 for _ in knobs]
    for call in range(3):
        p = f"{tag}_call{call}_"
        xs = [from_bits(gm[p + f"x{i}"]) for i in range(len(knobs))]
        g = from_bits(gm[p + "g"])
        torch.manual_seed(900 + call)
        hats = []
        for i, (ratio, sub, bits, method) in enumerate(knobs):
            if call < 2:
                thr, L, R, scale = O.get_statistics(xs[i], call, ratio, sub, bits, method, rank)
            else:
                thr, L, scale, R = statics[i]
            coo, stored, scale_o = O.ref_compress(xs[i], thr, scale, bits, sub, L, R)
            hats.append(O.ref_decompress(coo, stored, bits, scale_o, L=L, R=R))
            statics[i] = O.running_mean_update(statics[i], [thr, L, scale, R], call)
        if kind == "silu":
            y, dxs = torch.nn.functional.silu(xs[0]), [O.silu_bwd(hats[0], g)]
        elif kind == "gelu":
            y, dxs = torch.nn.functional.gelu(xs[0]), [O.gelu_bwd(hats[0], g)]
        else:
            y, dxs = xs[0] * xs[1], list(O.hadamard_bwd(hats[0], hats[1], g))
        assert bits_equal(y, from_bits(gm[p + "y"]))
        for i, dx in enumerate(dxs):
            assert bits_equal(dx, from_bits(gm[p + f"dx{i}"])), (tag, call, i)
        for i, sv in enumerate(statics):
            assert torch.equal(sv[0], from_bits(gm[p + f"s{i}_thr"]))
            assert bits_equal(sv[1], from_bits(gm[p + f"s{i}_L"]))
            assert bits_equal(sv[2], from_bits(gm[p + f"s{i}_scale"]))
            assert bits_equal(sv[3], from_bits(gm[p + f"s{i}_R"]))


def test_softmax_module(golden_modules):
    gm = golden_modules
    static = None
    for call in range(3):
        p = f"softmax_call{call}_"
        x, g = from_bits(gm[p + "x"]), from_bits(gm[p + "g"])
        y = torch.softmax(x, dim=-1)
        thr = O.get_statistics_softmax(y, call, 0.05) if call < 2 else static
        y_hat = O.true_decompress_softmax(O.true_compress_softmax(y, thr))
        if call < 2:
            static = thr if static is None else (call * static + thr) / (call + 1)
        assert bits_equal(y, from_bits(gm[p + "y"]))
        assert bits_equal(O.softmax_bwd(y_hat, g), from_bits(gm[p + "dx"]))
        assert torch.equal(static, from_bits(gm[p + "thr"]))
