"""GPU parity of the fused operators (RMSNorm forward + compress, RMSNorm backward, activation backward)
against the CPU oracle.  Tolerances: compressed outputs bit-exact; y and dx within 1 bf16 ulp of the oracle
(fp32 reduction order differs), gradients within rtol 1e-2 / atol 1e-3."""
import pytest
import torch

from conftest import bf16_ulp_diff, bits_equal
from oracle import hyc_oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def K(hyc):
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return hyc.kernels


def make_x(seed, M, H, n_hot, gain):
    gen = torch.Generator().manual_seed(seed)
    x = torch.randn(M, H, generator=gen)
    hot = torch.randperm(H, generator=gen)[:n_hot]
    x[:, hot] *= gain
    return x.bfloat16(), gen


def close_bf16(got, want, max_ulp=1, frac=1e-3):
    """all elements within max_ulp bf16 ulps, or (for values rounding to different binades near zero) tiny abs error"""
    d = bf16_ulp_diff(got, want)
    bad = (d > max_ulp) & ((got.float() - want.float()).abs() > 1e-6)
    return int(bad.sum()) <= frac * got.numel() and torch.allclose(got.float(), want.float(), rtol=1e-2, atol=1e-3)


NORM_CASES = [(4, 128, 96, 4096, 41, torch.float32), (4, 128, 96, 4096, 41, torch.bfloat16),
              (2, 64, 40, 4096, 41, torch.float32), (4, 128, 20, 11008, 110, torch.float32),
              (8, 128, 33, 2048, 20, torch.bfloat16), (1, 64, 16, 1024, 10, torch.float32),
              (4, 128, 5, 16384, 164, torch.float32), (8, 256, 3, 32768, 300, torch.float32),
              # rows whose chunks do not fill the last wave; two threads per packed word (2-bit)
              (2, 64, 40, 11008, 110, torch.float32), (2, 128, 21, 13824, 138, torch.bfloat16),
              (8, 128, 12, 11008, 110, torch.float32),
              # more rows than workgroups: every workgroup walks several rows with the next one requested ahead
              (4, 128, 2300, 4096, 41, torch.float32), (4, 64, 1100, 11008, 110, torch.bfloat16),
              (2, 64, 2300, 4096, 41, torch.bfloat16),
              # the longest rows of 4-bit codes: the backward's queue holds two stages beside the 64 KB weight row
              (4, 128, 700, 16384, 164, torch.float32)]


@pytest.mark.parametrize("rule", ["absmax", "range"])
@pytest.mark.parametrize("bits,group,M,H,k,wdt", NORM_CASES)
def test_rmsnorm_channel(K, bits, group, M, H, k, wdt, rule):
    x, gen = make_x(H + bits, M, H, k // 2, 30.0)
    w = (1 + 0.1 * torch.randn(H, generator=gen)).to(wdt)
    dy = (0.02 * torch.randn(M, H, generator=gen)).bfloat16()
    eps = 1e-6
    xd = x.cuda()
    plan = K.select_channels(K.channel_absmax(xd), k, rule)
    idx = plan.idx.cpu()
    assert torch.equal(idx, O.hyc_select_channels(O.hyc_channel_scores(x), k))
    y, rstd, c = K.rmsnorm_fwd_compress_channel(xd, w.cuda(), eps, plan, bits, group)
    y_o, rstd_o = O.rmsnorm_fwd(x, w, eps)
    assert torch.allclose(rstd.cpu(), rstd_o, rtol=2e-6, atol=0)
    assert bf16_ulp_diff(y.cpu(), y_o).max() <= 1
    vals, stored, scales = O.hyc_compress(x, idx, bits, group, rule)
    assert torch.equal(c.stored.cpu(), stored) and bits_equal(c.scales.cpu(), scales) and bits_equal(c.vals.cpu(), vals)
    # backward
    xh = O.hyc_decompress(vals, stored, idx, scales, bits, group)
    for quirk in (True, False):
        dx, dw = K.rmsnorm_bwd(dy.cuda(), c, w.cuda(), rstd, c2_quirk=quirk)
        dx_o, dw_o = O.rmsnorm_bwd(dy, xh, w, rstd_o, c2_quirk=quirk)
        assert close_bf16(dx.cpu(), dx_o)
        assert dw.dtype == w.dtype
        assert torch.allclose(dw.cpu().float(), dw_o.float(), rtol=1e-2, atol=1e-3)
    # the dense-source variant gives the same result as the fused one
    dx2, dw2 = K.rmsnorm_bwd(dy.cuda(), xh.cuda(), w.cuda(), rstd, c2_quirk=True)
    dx1, dw1 = K.rmsnorm_bwd(dy.cuda(), c, w.cuda(), rstd, c2_quirk=True)
    # the two variants may split the row over a different number of waves: sums agree to fp32 rounding
    assert close_bf16(dx1.cpu(), dx2.cpu(), frac=1e-5)
    assert torch.allclose(dw1.float(), dw2.float(), rtol=1e-2 if wdt == torch.bfloat16 else 1e-4, atol=1e-5)


@pytest.mark.parametrize("bits,M,H", [(4, 300, 4096), (2, 50, 11008), (1, 40, 1024)])
def test_rmsnorm_bwd_partial_rows(K, bits, M, H):
    """dw == NULL leaves the column sum to the caller: the partial rows add up to the dw of the full call"""
    x, gen = make_x(3, M, H, 10, 30.0)
    w = 1 + 0.1 * torch.randn(H, generator=gen)
    dy = (0.02 * torch.randn(M, H, generator=gen)).bfloat16()
    plan = K.select_channels(K.channel_absmax(x.cuda()), 10)
    y, rstd, c = K.rmsnorm_fwd_compress_channel(x.cuda(), w.cuda(), 1e-6, plan, bits, 64)
    dx, dw = K.rmsnorm_bwd(dy.cuda(), c, w.cuda(), rstd)
    dx2, part = K.rmsnorm_bwd_partial(dy.cuda(), c, w.cuda(), rstd)
    assert bits_equal(dx, dx2) and part.shape[0] >= 1
    assert torch.allclose(part.sum(0), dw, rtol=1e-5, atol=1e-6)


def test_rmsnorm_bwd_is_deterministic(K):
    x, gen = make_x(9, 512, 4096, 20, 30.0)
    w = (1 + 0.1 * torch.randn(4096, generator=gen))
    dy = (0.02 * torch.randn(512, 4096, generator=gen)).bfloat16().cuda()
    xd = x.cuda()
    plan = K.select_channels(K.channel_absmax(xd), 41)
    y, rstd, c = K.rmsnorm_fwd_compress_channel(xd, w.cuda(), 1e-6, plan, 4, 128)
    a = K.rmsnorm_bwd(dy, c, w.cuda(), rstd)
    b = K.rmsnorm_bwd(dy, c, w.cuda(), rstd)
    assert bits_equal(a[0], b[0]) and torch.equal(a[1], b[1])


@pytest.mark.parametrize("bits,method,rank", [(8, "per-channel", 2), (4, "per-token", 0), (2, "per-tensor", 0), (1, "per-channel", 0)])
def test_rmsnorm_threshold(K, bits, method, rank):
    B, S, H = 2, 24, 1024
    gen = torch.Generator().manual_seed(bits)
    x = torch.randn(B, S, H, generator=gen)
    x[..., :3] *= 15
    x = x.bfloat16()
    w = (1 + 0.1 * torch.randn(H, generator=gen))
    dy = (0.02 * torch.randn(B * S, H, generator=gen)).bfloat16()
    torch.manual_seed(1)
    thr, L, R, scale = O.get_statistics(x, 0, 0.005, 1.0, bits, method, rank)
    coo, stored, _ = O.ref_compress(x, thr, scale, bits, 1.0, L, R)
    xh = O.ref_decompress(coo, stored, bits, scale, L=L, R=R).reshape(-1, H)
    y, rstd, c = K.rmsnorm_fwd_compress_threshold(x.reshape(-1, H).cuda(), w.cuda(), 1e-6, S, float(thr), scale.cuda(), bits,
                                                  L.cuda() if rank else None, R.cuda() if rank else None)
    y_o, rstd_o = O.rmsnorm_fwd(x.reshape(-1, H), w, 1e-6)
    assert bf16_ulp_diff(y.cpu(), y_o).max() <= 1
    assert torch.equal(c.stored.cpu().reshape(stored.shape), stored)
    assert c.cols.numel() == coo.coalesce().values().numel()
    assert bits_equal(K.decompress_threshold(c).cpu(), xh)
    dx, dw = K.rmsnorm_bwd(dy.cuda(), c, w.cuda(), rstd)
    dx_o, dw_o = O.rmsnorm_bwd(dy, xh, w, rstd_o)
    assert close_bf16(dx.cpu(), dx_o)
    assert torch.allclose(dw.cpu(), dw_o, rtol=1e-2, atol=1e-3)


ACT_CASES = [(4, 128, 40, 11008, 110), (4, 128, 64, 4096, 41), (2, 64, 16, 4096, 41), (8, 32, 9, 512, 5), (1, 64, 9, 512, 5),
             (2, 64, 16, 11008, 110),
             # more rows than workgroups (rows are walked with the next one requested ahead)
             (4, 128, 4133, 4096, 41), (4, 128, 800, 11008, 110), (2, 64, 2100, 11008, 110)]


@pytest.mark.parametrize("bits,group,M,H,k", ACT_CASES)
def test_act_bwd_channel(K, bits, group, M, H, k):
    x, gen = make_x(bits + H, M, H, k, 20.0)
    g = (0.1 * torch.randn(M, H, generator=gen)).bfloat16()
    xd = x.cuda()
    plan = K.select_channels(K.channel_absmax(xd), k)
    c = K.compress_channel(xd, plan, bits, group)
    xh = K.decompress_channel(c).cpu()
    for act, fn in (("silu", O.silu_bwd), ("gelu", O.gelu_bwd)):
        got = K.act_bwd(act, g.cuda(), c).cpu()
        want = fn(xh, g)
        # exp / tanh differ in the last fp32 bit between the host and device math libraries: allow 1 bf16 ulp on a
        # small fraction of elements through each rounding of the chain, never more than the stated tolerance
        assert close_bf16(got, want, max_ulp=2, frac=2e-3), act
        same = (bf16_ulp_diff(got, want) == 0).float().mean()
        assert same > 0.99, (act, float(same))
        assert bits_equal(K.act_bwd(act, g.cuda(), xh.cuda()), K.act_bwd(act, g.cuda(), c))


@pytest.mark.parametrize("M,H,b1,g1,b2,g2", [(48, 4096, 4, 128, 2, 64),      # different code widths: two passes
                                              (48, 4096, 4, 128, 4, 64),      # same width: one fused pass
                                              (2100, 11008, 2, 64, 2, 32),    # partial last wave, several rows per workgroup
                                              (33, 2048, 8, 128, 8, 128)])
def test_hadamard_bwd(K, M, H, b1, g1, b2, g2):
    k = K.num_outlier_channels(H, 0.01)
    x1, gen = make_x(1, M, H, k, 20.0)
    x2, _ = make_x(2, M, H, k, 20.0)
    g = (0.1 * torch.randn(M, H, generator=gen)).bfloat16()
    p1 = K.select_channels(K.channel_absmax(x1.cuda()), k)
    p2 = K.select_channels(K.channel_absmax(x2.cuda()), k)
    c1 = K.compress_channel(x1.cuda(), p1, b1, g1)
    c2 = K.compress_channel(x2.cuda(), p2, b2, g2)
    d1, d2 = K.hadamard_bwd(g.cuda(), c1, c2)
    w1, w2 = O.hadamard_bwd(K.decompress_channel(c1).cpu(), K.decompress_channel(c2).cpu(), g)
    assert bits_equal(d1.cpu(), w1) and bits_equal(d2.cpu(), w2)


@pytest.mark.parametrize("act", ["silu", "gelu"])
@pytest.mark.parametrize("M,H,bits,group", [(40, 4096, 4, 128), (2100, 11008, 2, 64), (33, 2048, 8, 64),
                                            (2100, 11008, 4, 128),       # three 704-thread rows per workgroup: derivative table
                                            (900, 14336, 4, 128), (70, 16384, 4, 64),   # two workgroups per row
                                            (50, 13824, 4, 128), (300, 13824, 4, 64),   # 864 chunks: two workgroups of 432 threads
                                            (40, 12544, 4, 128)])        # 784 chunks: one workgroup of 1024 threads
def test_gated_act_bwd_equals_the_two_steps(K, act, M, H, bits, group):
    """one pass over (act(gate), up, gate) = hadamard backward followed by the activation backward, bit for bit"""
    k = K.num_outlier_channels(H, 0.01)
    gate, gen = make_x(5, M, H, k, 10.0)
    up, _ = make_x(6, M, H, k, 10.0)
    a = torch.nn.functional.silu(gate.float()).bfloat16() if act == "silu" else torch.nn.functional.gelu(gate.float()).bfloat16()
    g = (0.1 * torch.randn(M, H, generator=gen)).bfloat16().cuda()
    cs = []
    for t in (a, up, gate):
        td = t.cuda()
        cs.append(K.compress_channel(td, K.select_channels(K.channel_absmax(td), k), bits, group))
    d_h, d_up = K.hadamard_bwd(g, cs[0], cs[1])
    d_gate = K.act_bwd(act, d_h, cs[2])
    f_gate, f_up = K.gated_act_bwd(act, g, cs[0], cs[1], cs[2])
    assert bits_equal(f_up, d_up) and bits_equal(f_gate, d_gate)


def test_config2_shape(K):
    """BASELINE config 2: x [4,1024,4096] with 20 channels x30, w ~ N(1, 0.1), eps 1e-6, dy ~ N(0, 0.02), 1 % / INT4 / 128."""
    M, H = 4096, 4096
    x, gen = make_x(0, M, H, 20, 30.0)
    w = 1 + 0.1 * torch.randn(H, generator=gen)
    dy = (0.02 * torch.randn(M, H, generator=gen)).bfloat16()
    xd = x.cuda()
    plan = K.select_channels(K.channel_absmax(xd), 41)
    y, rstd, c = K.rmsnorm_fwd_compress_channel(xd, w.cuda(), 1e-6, plan, 4, 128)
    idx = plan.idx.cpu()
    vals, stored, scales = O.hyc_compress(x, idx, 4, 128)
    assert torch.equal(c.stored.cpu(), stored) and bits_equal(c.scales.cpu(), scales) and bits_equal(c.vals.cpu(), vals)
    y_o, rstd_o = O.rmsnorm_fwd(x, w, 1e-6)
    assert bf16_ulp_diff(y.cpu(), y_o).max() <= 1
    xh = O.hyc_decompress(vals, stored, idx, scales, 4, 128)
    dx, dw = K.rmsnorm_bwd(dy.cuda(), c, w.cuda(), rstd)
    dx_o, dw_o = O.rmsnorm_bwd(dy, xh, w, rstd_o)
    assert torch.allclose(dx.cpu().float(), dx_o.float(), rtol=1e-2, atol=1e-3)
    assert torch.allclose(dw.cpu(), dw_o, rtol=1e-2, atol=1e-3)


@pytest.mark.parametrize("act", ["silu", "gelu"])
def test_gated_forward_activation_matches_the_framework_for_every_bf16_value(K, act):
    """h = act(gate) * 1 from the one-pass forward against F.silu / F.gelu on all 65 536 bf16 patterns (NaN aside):
    the compressed act(gate) is only the framework's if every value is"""
    H = 512
    bits16 = torch.arange(65536, dtype=torch.int32)
    gate = bits16.to(torch.int16).view(torch.bfloat16).view(-1, H).cuda()
    up = torch.ones_like(gate)
    M = gate.shape[0]
    plan = K.select_channels(torch.zeros(H, device="cuda"), 0)
    h, _, _, _ = K.gated_act_fwd(act, gate, up, plan, plan, plan, 4, 128)
    want = torch.nn.functional.silu(gate) if act == "silu" else torch.nn.functional.gelu(gate)
    ok = torch.isnan(want) & torch.isnan(h) | (h.view(torch.int16) == want.view(torch.int16))
    assert bool(ok.all()), [(hex(int(b) & 0xFFFF)) for b in gate.view(torch.int16)[~ok][:8].cpu()]


@pytest.mark.parametrize("act,M,H,bits,group,k", [("silu", 333, 11008, 4, 128, 110), ("gelu", 64, 4096, 4, 128, 41),
                                                  ("silu", 2100, 4096, 4, 64, 41), ("silu", 40, 512, 8, 64, 5),
                                                  ("gelu", 130, 2048, 8, 128, 300),
                                                  # 2-bit codes: four segments per thread (128 and 344 threads per row)
                                                  ("silu", 300, 4096, 2, 128, 41), ("gelu", 77, 11008, 2, 64, 110),
                                                  ("silu", 1030, 11008, 2, 64, 110),
                                                  # three rows of 704 threads per workgroup: the activation table is in use
                                                  ("silu", 2100, 11008, 4, 128, 110), ("gelu", 1600, 11008, 4, 128, 110),
                                                  # rows of 896 and 1024 chunks: two workgroups per row
                                                  ("silu", 700, 14336, 4, 128, 143), ("gelu", 130, 16384, 4, 64, 164),
                                                  ("silu", 90, 28672, 2, 128, 287),
                                                  # 864 chunks: two workgroups of 432 threads, the last wave partly filled
                                                  ("gelu", 210, 13824, 4, 128, 138), ("silu", 130, 13824, 4, 64, 138)])
def test_gated_forward_equals_the_separate_calls(K, act, M, H, bits, group, k):
    """one pass = F.silu / F.gelu, three hyc_compress calls and a product, bit for bit; gate and up are column slices of
    one wider matrix, as a fused gate/up projection hands them over"""
    gen = torch.Generator().manual_seed(M + H + bits)
    both = torch.randn(M, 2 * H, generator=gen)
    both[:, torch.randperm(2 * H, generator=gen)[:2 * k]] *= 15
    both = both.bfloat16().cuda()
    gate, up = both[:, :H], both[:, H:]
    a = torch.nn.functional.silu(gate) if act == "silu" else torch.nn.functional.gelu(gate)
    # each site carries its own scale rule
    rules = ("absmax", "range", "absmax") if M % 2 else ("range", "absmax", "range")
    plans = [K.select_channels(K.channel_absmax(t), k, r) for t, r in zip((a, up, gate), rules)]
    want = [K.compress_channel(t, p, bits, group) for t, p in zip((a, up, gate), plans)]
    h, c_a, c_u, c_g = K.gated_act_fwd(act, gate, up, plans[0], plans[1], plans[2], bits, group)
    assert bits_equal(h, a * up)
    for got, ref in zip((c_a, c_u, c_g), want):
        assert torch.equal(got.stored.view(torch.uint8), ref.stored.view(torch.uint8))
        assert bits_equal(got.scales, ref.scales) and bits_equal(got.vals, ref.vals)
    assert K.gated_act_fwd_supported(4096, 2, 64) and K.gated_act_fwd_supported(11008, 4, 128)
    assert K.gated_act_fwd_supported(14336, 4, 128)              # 896 chunks per segment: two workgroups per row
    assert K.gated_act_fwd_supported(13824, 4, 128)              # 864 chunks: two parts of 27 scale groups
    assert not K.gated_act_fwd_supported(12544, 4, 128)          # 784 chunks = 49 groups: no 2 to 4 equal parts, separate calls
    assert not K.gated_act_fwd_supported(32832, 2, 64) and not K.gated_act_fwd_supported(4096, 1, 64)


@pytest.mark.parametrize("bits,group,M,H,k,wdt,with_bias", [
    (4, 64, 80, 768, 8, torch.float32, True), (4, 128, 33, 1024, 10, torch.bfloat16, True),
    (2, 64, 2100, 4096, 41, torch.float32, False), (8, 32, 9, 512, 5, torch.bfloat16, True),
    (1, 64, 17, 1024, 0, torch.float32, True), (4, 128, 20, 11008, 110, torch.float32, True),
    (4, 128, 9000, 768, 8, torch.float32, True), (8, 128, 5000, 1024, 10, torch.bfloat16, False)])   # many rows per workgroup
def test_layernorm_forward_channel(K, bits, group, M, H, k, wdt, with_bias):
    """one pass = the reference's two-pass statistics and y (efficient_layernorm.py:15-61) plus hyc_compress of x"""
    gen = torch.Generator().manual_seed(bits + M + H)
    x = 0.7 + torch.randn(M, H, generator=gen)
    x[:, torch.randperm(H, generator=gen)[:max(k, 1)]] *= 12
    x = x.bfloat16()
    w = (1 + 0.1 * torch.randn(H, generator=gen)).to(wdt)
    b = (0.1 * torch.randn(H, generator=gen)).to(wdt) if with_bias else None
    xd = x.cuda()
    plan = K.select_channels(K.channel_absmax(xd), k)
    y, mean, rstd, c = K.layernorm_fwd_compress_channel(xd, w.cuda(), None if b is None else b.cuda(), 1e-5, plan, bits, group)
    y_o, mean_o, rstd_o = O.layernorm_fwd(x, w, b, 1e-5)
    assert torch.allclose(mean.cpu(), mean_o, rtol=1e-5, atol=1e-6) and torch.allclose(rstd.cpu(), rstd_o, rtol=1e-5, atol=0)
    # one bf16 ulp, or the absolute error that 1e-5 relative in mean / rstd leaves where (x - mean) * rstd * w + b cancels
    diff = (y.cpu().float() - y_o.float()).abs()
    assert bool(((bf16_ulp_diff(y.cpu(), y_o) <= 1) | (diff <= 2e-3)).all())
    ref = K.compress_channel(xd, plan, bits, group)
    assert torch.equal(c.stored.view(torch.uint8), ref.stored.view(torch.uint8))
    assert bits_equal(c.scales, ref.scales) and bits_equal(c.vals, ref.vals)
    with pytest.raises(ValueError):
        K.layernorm_fwd_compress_channel(xd, w.cuda(), torch.zeros(H - 8, dtype=wdt, device="cuda"), 1e-5, plan, bits, group)


@pytest.mark.parametrize("rule", ["absmax", "range"])
@pytest.mark.parametrize("group,M,H,k", [(64, 2100, 11008, 110), (128, 2051, 13824, 138), (64, 2300, 16384, 164)])
def test_long_rows_of_2bit_codes_with_several_rows_per_workgroup(K, group, M, H, k, rule):
    """Rows of 2-bit codes with more than 256 chunks per segment travel through a queue of two stages (three do not fit
    the LDS); with more rows than workgroups every workgroup walks several rows, so the entry of the next row is
    requested while the current one is encoded.  RMSNorm and LayerNorm forward, codes / scales / outlier values bit for
    bit against the oracle."""
    x, gen = make_x(H + M, M, H, k // 2, 30.0)
    x = (x.float() + 0.25).bfloat16()
    w = 1 + 0.1 * torch.randn(H, generator=gen)
    b = 0.1 * torch.randn(H, generator=gen)
    xd = x.cuda()
    plan = K.select_channels(K.channel_absmax(xd), k, rule)
    idx = plan.idx.cpu()
    vals, stored, scales = O.hyc_compress(x, idx, 2, group, rule)
    y, rstd, c = K.rmsnorm_fwd_compress_channel(xd, w.cuda(), 1e-6, plan, 2, group)
    y_o, rstd_o = O.rmsnorm_fwd(x, w, 1e-6)
    assert torch.allclose(rstd.cpu(), rstd_o, rtol=2e-6, atol=0)
    assert bf16_ulp_diff(y.cpu(), y_o).max() <= 1
    assert torch.equal(c.stored.cpu(), stored) and bits_equal(c.scales.cpu(), scales) and bits_equal(c.vals.cpu(), vals)
    y, mean, rstd, c = K.layernorm_fwd_compress_channel(xd, w.cuda(), b.cuda(), 1e-5, plan, 2, group)
    y_o, mean_o, rstd_o = O.layernorm_fwd(x, w, b, 1e-5)
    assert torch.allclose(mean.cpu(), mean_o, rtol=1e-5, atol=1e-6) and torch.allclose(rstd.cpu(), rstd_o, rtol=1e-5, atol=0)
    diff = (y.cpu().float() - y_o.float()).abs()
    assert bool(((bf16_ulp_diff(y.cpu(), y_o) <= 1) | (diff <= 2e-3)).all())
    assert torch.equal(c.stored.cpu(), stored) and bits_equal(c.scales.cpu(), scales) and bits_equal(c.vals.cpu(), vals)


@pytest.mark.parametrize("bits,method,rank", [(8, "per-channel", 2), (4, "per-token", 0), (2, "per-tensor", 0)])
def test_layernorm_forward_threshold(K, bits, method, rank):
    B, S, H = 2, 24, 768
    gen = torch.Generator().manual_seed(40 + bits)
    x = 0.3 + torch.randn(B, S, H, generator=gen)
    x[..., :3] *= 15
    x = x.bfloat16()
    w = 1 + 0.1 * torch.randn(H, generator=gen)
    b = 0.1 * torch.randn(H, generator=gen)
    torch.manual_seed(1)
    thr, L, R, scale = O.get_statistics(x, 0, 0.005, 1.0, bits, method, rank)
    coo, stored, _ = O.ref_compress(x, thr, scale, bits, 1.0, L, R)
    xh = O.ref_decompress(coo, stored, bits, scale, L=L, R=R).reshape(-1, H)
    y, mean, rstd, c = K.layernorm_fwd_compress_threshold(x.reshape(-1, H).cuda(), w.cuda(), b.cuda(), 1e-5, S, float(thr),
                                                          scale.cuda(), bits, L.cuda() if rank else None,
                                                          R.cuda() if rank else None)
    y_o, mean_o, rstd_o = O.layernorm_fwd(x.reshape(-1, H), w, b, 1e-5)
    assert torch.allclose(mean.cpu(), mean_o, rtol=1e-5, atol=1e-6) and torch.allclose(rstd.cpu(), rstd_o, rtol=1e-5, atol=0)
    diff = (y.cpu().float() - y_o.float()).abs()
    assert bool(((bf16_ulp_diff(y.cpu(), y_o) <= 1) | (diff <= 2e-3)).all())
    assert torch.equal(c.stored.cpu().reshape(stored.shape), stored)
    assert bits_equal(K.decompress_threshold(c).cpu(), xh)


@pytest.mark.parametrize("act,M,H,bits,group,k", [("silu", 333, 11008, 4, 128, 110), ("gelu", 64, 4096, 4, 128, 41),
                                                  ("silu", 2100, 4096, 2, 64, 41), ("gelu", 40, 512, 8, 64, 5),
                                                  ("silu", 17, 2048, 2, 128, 300)])
@pytest.mark.parametrize("rule", ["absmax", "range"])
def test_activation_forward_with_the_save_fused_in(K, act, M, H, bits, group, k, rule):
    """y = F.silu / F.gelu bit for bit and the compressed x equal to hyc_compress of x; x is a column slice"""
    gen = torch.Generator().manual_seed(M + H + bits)
    wide = torch.randn(M, H + 64, generator=gen)
    wide[:, torch.randperm(H, generator=gen)[:k]] *= 15
    x = wide.bfloat16().cuda()[:, :H]
    plan = K.select_channels(K.channel_absmax(x), k, rule)
    y, c = K.act_fwd_compress(act, x, plan, bits, group)
    want = torch.nn.functional.silu(x) if act == "silu" else torch.nn.functional.gelu(x)
    assert bits_equal(y, want)
    ref = K.compress_channel(x, plan, bits, group)
    assert torch.equal(c.stored.view(torch.uint8), ref.stored.view(torch.uint8))
    assert bits_equal(c.scales, ref.scales) and bits_equal(c.vals, ref.vals)
    assert not K.act_fwd_compress_supported(4096, 1, 128) and not K.act_fwd_compress_supported(4096, 4, 32)


@pytest.mark.parametrize("M,H,bits,group,k", [(333, 11008, 4, 128, 110), (2100, 4096, 4, 64, 41), (40, 512, 8, 64, 5),
                                              (9, 2048, 8, 128, 300), (300, 4096, 2, 128, 41), (1030, 11008, 2, 64, 110)])
def test_product_forward_with_the_saves_fused_in(K, M, H, bits, group, k):
    gen = torch.Generator().manual_seed(M + H + bits + 1)
    both = torch.randn(M, 2 * H, generator=gen)
    both[:, torch.randperm(2 * H, generator=gen)[:2 * k]] *= 15
    both = both.bfloat16().cuda()
    a, b = both[:, :H], both[:, H:]
    pa, pb = (K.select_channels(K.channel_absmax(t), k, r) for t, r in ((a, "absmax"), (b, "range")))
    y, ca, cb = K.hadamard_fwd_compress(a, b, pa, pb, bits, group)
    assert bits_equal(y, a * b)
    for got, t, p in ((ca, a, pa), (cb, b, pb)):
        ref = K.compress_channel(t, p, bits, group)
        assert torch.equal(got.stored.view(torch.uint8), ref.stored.view(torch.uint8))
        assert bits_equal(got.scales, ref.scales) and bits_equal(got.vals, ref.vals)
    assert K.hadamard_fwd_compress_supported(4096, 2, 64, 2, 64) and not K.hadamard_fwd_compress_supported(4096, 4, 64, 8, 64)
    assert not K.hadamard_fwd_compress_supported(20480, 2, 64, 2, 64)


def test_rows_beyond_two_gibi_elements(K):
    """525 288 rows x 4096 channels = 2^31 + 4 M elements (4.3 GB): element offsets no longer fit 32 bits.  Rows are
    independent, so the last rows (all of them past the 2^31-element mark) are checked against the oracle run on
    those rows alone: codec, fused RMSNorm forward and backward, SiLU backward."""
    M, H, k, bits, group = (1 << 31) // 4096 + 1000, 4096, 41, 4, 128
    gen = torch.Generator(device="cuda").manual_seed(7)
    x = torch.randn(M, H, generator=gen, device="cuda", dtype=torch.bfloat16)
    x[:, 5::100] *= 20
    tail = slice(M - 48, M)
    xt = x[tail].cpu()
    w = (1 + 0.1 * torch.randn(H, generator=torch.Generator().manual_seed(1)))
    plan = K.select_channels(K.channel_absmax(x[:4096].contiguous()), k)
    idx = plan.idx.cpu().long()
    y, rstd, c = K.rmsnorm_fwd_compress_channel(x, w.cuda(), 1e-6, plan, bits, group)
    vals, stored, scales = O.hyc_compress(xt, idx, bits, group)
    assert torch.equal(c.stored[tail].cpu(), stored) and bits_equal(c.scales[tail].cpu(), scales)
    assert bits_equal(c.vals[tail].cpu(), vals)
    y_o, rstd_o = O.rmsnorm_fwd(xt, w, 1e-6)
    assert bf16_ulp_diff(y[tail].cpu(), y_o).max() <= 1
    del y
    c2 = K.compress_channel(x, plan, bits, group)
    assert torch.equal(c2.stored[tail], c.stored[tail]) and bits_equal(c2.vals[tail], c.vals[tail])
    del c2
    xh = K.decompress_channel(c)
    xh_o = O.hyc_decompress(vals, stored, idx, scales, bits, group)
    assert bits_equal(xh[tail].cpu(), xh_o)
    del xh, x
    dy = torch.zeros(M, H, device="cuda", dtype=torch.bfloat16)
    dyt = (0.02 * torch.randn(48, H, generator=torch.Generator().manual_seed(2))).bfloat16()
    dy[tail] = dyt.cuda()
    dx, dw = K.rmsnorm_bwd(dy, c, w.cuda(), rstd)
    dx_o, dw_o = O.rmsnorm_bwd(dyt, xh_o, w, rstd_o)            # every other row has dy = 0 and adds nothing to dw
    assert torch.allclose(dx[tail].cpu().float(), dx_o.float(), rtol=1e-2, atol=1e-3)
    assert torch.allclose(dw.cpu(), dw_o, rtol=1e-2, atol=1e-3)
    assert float(dx[:M - 48].abs().max()) == 0.0
    del dx
    ds = K.act_bwd("silu", dy, c)
    assert bits_equal(ds[tail].cpu(), O.silu_bwd(xh_o, dyt))


def test_empty_batches_pass_through_every_launcher(K):
    """M = 0: every launcher returns tensors of the right shape without a launch"""
    H, k = 512, 5
    e = torch.zeros(0, H, dtype=torch.bfloat16, device="cuda")
    plan = K.select_channels(torch.zeros(H, device="cuda"), k)
    w = torch.ones(H, device="cuda")
    y, rstd, c = K.rmsnorm_fwd_compress_channel(e, w, 1e-6, plan, 4, 128)
    assert y.shape == (0, H) and rstd.shape == (0,) and c.vals.shape == (0, k)
    dx, dw = K.rmsnorm_bwd(e, c, w, rstd)
    assert dx.shape == (0, H) and dw.shape == (H,) and float(dw.abs().max()) == 0.0
    y, mean, rstd, c = K.layernorm_fwd_compress_channel(e, w, None, 1e-5, plan, 4, 128)
    assert y.shape == (0, H) and mean.shape == (0,)
    assert K.act_bwd("silu", e, c).shape == (0, H)
    assert all(t.shape == (0, H) for t in K.hadamard_bwd(e, c, c))
    assert all(t.shape == (0, H) for t in K.gated_act_bwd("gelu", e, c, c, c))
    assert K.gated_act_fwd("silu", e, e, plan, plan, plan, 4, 128)[0].shape == (0, H)
    assert K.act_fwd_compress("gelu", e, plan, 4, 128)[0].shape == (0, H)
    assert K.hadamard_fwd_compress(e, e, plan, plan, 4, 128)[0].shape == (0, H)
    gw = K.gradw_gemm(torch.zeros(0, 16, dtype=torch.bfloat16, device="cuda"), c, out_dtype=torch.float32)
    assert gw.shape == (16, H) and float(gw.abs().max()) == 0.0
    p, sp = K.softmax_fwd(e, 0.01)
    assert p.shape == (0, H) and sp.cols.numel() == 0 and K.softmax_bwd(e, sp).shape == (0, H)


@pytest.mark.parametrize("act", ["silu", "gelu"])
def test_forward_activation_tables_match_the_framework_for_every_bf16_value(K, act):
    """with enough rows per workgroup the forward kernels look act(x) up in a table built from the same arithmetic
    (inputs outside it are computed): all 65 536 bf16 patterns again, through the one-pass gated forward, the
    activation forward with its save, and the gated backward's derivative table against the separate backward calls"""
    H = 4096
    pat = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16).view(-1, H)      # 16 rows
    gate = pat.repeat(512, 1).cuda()                                                                   # 8192 rows
    up = torch.ones_like(gate)
    plan = K.select_channels(torch.zeros(H, device="cuda"), 0)
    want = torch.nn.functional.silu(gate) if act == "silu" else torch.nn.functional.gelu(gate)

    def same(a, b):
        return bool(((torch.isnan(a) & torch.isnan(b)) | (a.view(torch.int16) == b.view(torch.int16))).all())

    h, c_a, c_u, c_g = K.gated_act_fwd(act, gate, up, plan, plan, plan, 4, 128)
    assert same(h, want)
    y, c_x = K.act_fwd_compress(act, gate, plan, 4, 128)
    assert same(y, want)
    assert torch.equal(c_x.stored, c_g.stored) and torch.equal(c_x.scales.view(torch.int16), c_g.scales.view(torch.int16))
    # finite inputs for the backward comparison (codes of a row holding inf / nan are not meaningful)
    fin = torch.nan_to_num(gate).clamp(-300, 300)             # 4 rows x 256 threads per workgroup: the tables are in use
    finp = K.select_channels(K.channel_absmax(fin), 20)
    g = torch.full_like(fin, 0.75)
    ones = torch.ones_like(fin)
    a = torch.nn.functional.silu(fin) if act == "silu" else torch.nn.functional.gelu(fin)
    ca, cu, cg = (K.compress_channel(t, finp, 4, 128) for t in (a, ones, fin))
    d_gate, d_up = K.gated_act_bwd(act, g, ca, cu, cg)
    d_a, d_u = K.hadamard_bwd(g, ca, cu)
    assert same(d_up, d_u) and same(d_gate, K.act_bwd(act, d_a, cg))
    few = slice(0, 16)                                         # one row per workgroup: no table
    cf = [K.compress_channel(t[few].contiguous(), finp, 4, 128) for t in (a, ones, fin)]
    dg_few, _ = K.gated_act_bwd(act, g[few].contiguous(), *cf)
    assert same(dg_few, d_gate[few])
