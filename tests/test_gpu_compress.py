"""GPU parity: the HIP compress / decompress kernels (through the C ABI) against the CPU oracle on identical
seeded inputs.  Codes, packed bytes, outlier indices / values and scales must be bit-exact; the reconstruction
is required to be bit-exact too (the stated bar is 1 bf16 ulp)."""
import numpy as np
import pytest
import torch

from conftest import bf16_ulp_diff, bits_equal, from_bits
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
    return x.bfloat16(), hot


# ------------------------------------------------------------------ calibration
@pytest.mark.parametrize("M,H,k", [(64, 512, 5), (300, 4096, 41), (33, 11008, 110), (16, 256, 0), (7, 64, 64)])
def test_absmax_and_selection(K, M, H, k):
    x, _ = make_x(M + H, M, H, max(k, 1), 25.0)
    amax = K.channel_absmax(x.cuda())
    assert torch.equal(amax.cpu(), O.hyc_channel_scores(x))
    plan = K.select_channels(amax, k)
    want = O.hyc_select_channels(O.hyc_channel_scores(x), k)
    assert torch.equal(plan.idx.cpu(), want)
    words = plan.plan.cpu().numpy().view(np.uint32)
    mask = np.zeros(H, dtype=bool); mask[want.numpy()] = True
    for c in range(H // 8):
        m8 = sum(int(mask[8 * c + j]) << j for j in range(8))
        assert (words[c] & 0xFF) == m8 and (words[c] >> 16) == int(mask[:8 * c].sum())


def test_selection_ties_go_to_lower_index(K):
    s = torch.tensor([3., 1., 3., 3., 0., 1., 3., 2.] * 8)
    plan = K.select_channels(s.cuda(), 10)
    assert torch.equal(plan.idx.cpu(), O.hyc_select_channels(s, 10))


@pytest.mark.parametrize("H,k", [(4096, 41), (512, 100), (20000, 7)])
def test_selection_of_general_scores(K, H, k):
    # fp32 scores with bits in their low half (the selection's two low radix passes run) and of both signs, with ties
    gen = torch.Generator().manual_seed(H + k)
    s = torch.randn(H, generator=gen)
    s[torch.randperm(H, generator=gen)[:H // 4]] = float(s[0])
    plan = K.select_channels(s.cuda(), k)
    assert torch.equal(plan.idx.cpu(), O.hyc_select_channels(s, k))


def test_absmax_accumulates(K):
    x1, _ = make_x(1, 40, 128, 2, 9.0)
    x2, _ = make_x(2, 24, 128, 2, 30.0)
    a = K.channel_absmax(x1.cuda())
    a = K.channel_absmax(x2.cuda(), a)
    assert torch.equal(a.cpu(), O.hyc_channel_scores(torch.cat([x1, x2])))


# ------------------------------------------------------------------ channel mode
CH_CASES = [
    (4, 128, 64, 4096, 41), (2, 64, 64, 4096, 41), (4, 128, 24, 11008, 110), (2, 64, 24, 11008, 110),
    (8, 128, 32, 4096, 41), (1, 64, 32, 4096, 41), (4, 32, 17, 512, 5), (4, 256, 17, 2048, 20),
    (8, 512, 9, 4096, 0), (2, 32, 5, 256, 3), (1, 32, 3, 256, 2), (8, 32, 1, 64, 1), (4, 64, 130, 1024, 10),
    (8, 128, 20, 16384, 164), (4, 128, 6, 32768, 328),
    # more rows than workgroups (rows are walked with the next one requested ahead), full and partial last wave
    (4, 128, 4133, 4096, 41), (2, 64, 4133, 4096, 41), (4, 128, 800, 11008, 110), (2, 64, 2100, 11008, 110),
    (8, 64, 900, 4096, 41),
    # more outlier channels than threads in a workgroup; several outliers per chunk
    (2, 32, 40, 1024, 200), (4, 32, 40, 512, 300), (4, 64, 40, 512, 300), (8, 128, 40, 1024, 700),
]


@pytest.mark.parametrize("rule", ["absmax", "range"])
@pytest.mark.parametrize("bits,group,M,H,k", CH_CASES)
def test_channel_roundtrip(K, bits, group, M, H, k, rule):
    x, _ = make_x(bits * 1000 + H + M, M, H, max(k, 1), 30.0)
    if M > 8:
        x[5] = x[5].abs()         # one-sided rows: where the two scale rules differ most
        x[6] = -x[6].abs()
    if M > 3:
        x[1, :group] = 0          # a constant (zero-scale) group
        x[2, group:2 * group] = 1.5
    idx = O.hyc_select_channels(O.hyc_channel_scores(x), k)
    xd = x.cuda()
    plan = K.select_channels(K.channel_absmax(xd), k, rule)
    assert torch.equal(plan.idx.cpu(), idx)
    c = K.compress_channel(xd, plan, bits, group)
    vals, stored, scales = O.hyc_compress(x, idx, bits, group, rule)
    assert bits_equal(c.scales.cpu(), scales)
    assert bits_equal(c.vals.cpu(), vals)
    assert c.stored.dtype == stored.dtype and torch.equal(c.stored.cpu(), stored)
    xh = K.decompress_channel(c).cpu()
    want = O.hyc_decompress(vals, stored, idx, scales, bits, group)
    assert bits_equal(xh, want)
    assert bits_equal(xh[:, idx.long()], x[:, idx.long()])


@pytest.mark.parametrize("rule", ["absmax", "range"])
@pytest.mark.parametrize("bits", [1, 2, 4, 8])
@pytest.mark.parametrize("group,fused", [(128, False), (32, False), (128, True)])
def test_group_scale_of_every_bf16_value(K, bits, group, fused, rule):
    """The kernels form the scale as bf16(d * fl(1 / levels)) where the bf16 tensor expression divides.  Every finite
    non-negative bf16 value d is made the range (and twice the abs-max) of one group: both signs of the extreme, both
    rules, all code widths, the standalone encoder (group 32: generic kernel, group 128: fast kernel) and the encoder
    inside the RMSNorm forward; scales and codes must equal the oracle's, which divides."""
    H = 1024
    pats = torch.arange(0, 0x7F80, dtype=torch.int32)                      # +0 ... largest finite, subnormals included
    per_row = H // group
    M = (pats.numel() + per_row - 1) // per_row
    d = torch.zeros(M * per_row, dtype=torch.int32)
    d[:pats.numel()] = pats
    ext = d.to(torch.int16).view(torch.bfloat16).reshape(M, per_row)
    gen = torch.Generator().manual_seed(bits * 10 + group)
    # the rest of a group: values between 0 and the extreme, so that the extreme is both the range and the abs-max
    x = (torch.rand(M, per_row, group, generator=gen) * ext.float()[..., None]).bfloat16()
    x = torch.minimum(x, ext[..., None])
    x[..., 0] = 0
    x[..., 3] = ext
    x[1::2] = -x[1::2]                                                      # odd rows: the extreme is the minimum
    if rule == "absmax":
        x = (x.float() * 0.5).bfloat16()                                    # 2 * max|x| runs over every bf16 value (exact halving
                                                                            # except in the lowest binade, which is covered as is)
    x = x.reshape(M, H).contiguous()
    idx = torch.tensor([], dtype=torch.int32)
    plan = K.select_channels(torch.zeros(H, device="cuda"), 0, rule)
    vals, stored, scales = O.hyc_compress(x, idx, bits, group, rule)
    if fused:
        if bits == 1:
            pytest.skip("1-bit codes take the generic forward kernel, covered by group 32")
        w = torch.ones(H, device="cuda")
        _, _, c = K.rmsnorm_fwd_compress_channel(x.cuda(), w, 1e-6, plan, bits, group)
    else:
        c = K.compress_channel(x.cuda(), plan, bits, group)
    assert bits_equal(c.scales.cpu(), scales)
    assert torch.equal(c.stored.cpu(), stored)


@pytest.mark.parametrize("bits,group", [(4, 64), (2, 64), (8, 128)])
def test_channel_special_values(K, bits, group):
    """A -0 in an outlier channel comes back as +0 (the reconstruction is a sum with a +0); a group that holds an
    inf has a non-finite scale and reconstructs as NaN everywhere, its outlier channels included."""
    M, H, k = 8, 1024, 10
    x, _ = make_x(77, M, H, k, 30.0)
    amax = O.hyc_channel_scores(x)
    idx = O.hyc_select_channels(amax, k)
    ch = int(idx[0])
    other = next(c for c in range(ch - ch % group, ch - ch % group + group) if c not in set(idx.tolist()))
    x[3, ch] = -0.0
    x[4, other] = float("inf")
    x[5, other] = float("-inf")
    plan = K.select_channels(amax.cuda(), k)
    assert torch.equal(plan.idx.cpu(), idx)
    c = K.compress_channel(x.cuda(), plan, bits, group)
    vals, stored, scales = O.hyc_compress(x, idx, bits, group)
    assert bits_equal(c.vals.cpu(), vals)
    # The reference zeroes outliers as x - x*mask, which turns a non-outlier inf into NaN before the scale is taken;
    # the kernel masks bits and keeps the inf.  Either way the group's scale is non-finite and the group decodes to NaN.
    rows = [r for r in range(M) if r not in (4, 5)]
    assert bits_equal(c.scales.cpu()[rows], scales[rows]) and torch.equal(c.stored.cpu()[rows], stored[rows])
    assert not bool(c.scales.cpu()[4, ch // group].float().isfinite())
    got = K.decompress_channel(c).cpu()
    want = O.hyc_decompress(vals, stored, idx, scales, bits, group)
    assert torch.equal(got.isnan(), want.isnan())
    assert bool(want[4, ch].isnan()) and bool(want[5, ch].isnan())
    ok = ~want.isnan()
    assert torch.equal(got.view(torch.int16)[ok], want.view(torch.int16)[ok])
    assert got[3, ch].view(torch.int16).item() == 0          # +0, not the stored -0


def test_channel_config1_shape(K):
    """BASELINE config 1: [4,512,4096], 41 channels x50, 1 % outliers, INT4, group 128."""
    for seed in (0, 1, 2):
        x, hot = make_x(seed, 2048, 4096, 41, 50.0)
        xd = x.cuda()
        plan = K.select_channels(K.channel_absmax(xd), 41)
        assert sorted(plan.idx.cpu().tolist()) == sorted(hot.tolist())
        c = K.compress_channel(xd, plan, 4, 128)
        vals, stored, scales = O.hyc_compress(x, plan.idx.cpu(), 4, 128)
        assert torch.equal(c.stored.cpu(), stored) and bits_equal(c.scales.cpu(), scales) and bits_equal(c.vals.cpu(), vals)
        assert bits_equal(K.decompress_channel(c).cpu(), O.hyc_decompress(vals, stored, plan.idx.cpu(), scales, 4, 128))


def test_empty_and_errors(K, hyc):
    x = torch.zeros(0, 512, dtype=torch.bfloat16, device="cuda")
    plan = K.select_channels(torch.zeros(512, device="cuda"), 5)
    c = K.compress_channel(x, plan, 4, 128)
    assert c.stored.shape == (0, 256) and K.decompress_channel(c).shape == (0, 512)
    y = torch.zeros(4, 520, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(NotImplementedError):
        K.compress_channel(y, plan, 4, 128)                    # 520 is not a multiple of 16
    with pytest.raises(NotImplementedError):
        K.compress_channel(torch.zeros(4, 512, dtype=torch.bfloat16, device="cuda"), plan, 4, 96)
    with pytest.raises(ValueError):
        K.compress_channel(torch.zeros(4, 512, dtype=torch.bfloat16), plan, 4, 128)   # CPU tensor: no fallback
    with pytest.raises(ValueError):
        K.compress_channel(torch.zeros(4, 512, dtype=torch.float32, device="cuda"), plan, 4, 128)


# ------------------------------------------------------------------ threshold mode (reference scheme)
def _coo_of(c, S):
    """CSR of a ThresholdCompressed -> the COO index matrix [3, nnz] the reference's to_sparse() gives"""
    rp = c.row_ptr.cpu().long()
    rows = torch.repeat_interleave(torch.arange(c.M), rp[1:] - rp[:-1])
    return torch.stack([rows // S, rows % S, c.cols.cpu().long()]), c.vals.cpu()


@pytest.mark.parametrize("H,ratio", [(4096, 0.45), (8192, 0.3), (2048, 0.999)])
def test_threshold_rows_with_more_outliers_than_a_wave_stages(K, H, ratio):
    """a low threshold keeps more than 1024 outlier elements per row: the first 1024 leave through the wave's staging
    row in LDS, the rest go to memory one by one; order and values must be the reference's either way"""
    B, S, bits = 2, 9, 4
    gen = torch.Generator().manual_seed(H)
    x = torch.randn(B, S, H, generator=gen).bfloat16()
    thr, L, R, scale = O.get_statistics(x, 0, ratio, 1.0, bits, "per-token", 0)
    coo, stored, _ = O.ref_compress(x, thr, scale, bits, 1.0, L, R)
    coo = coo.coalesce()
    c = K.compress_threshold(x.reshape(-1, H).cuda(), S, float(thr), scale.cuda(), bits)
    rp = c.row_ptr.cpu()
    assert int((rp[1:] - rp[:-1]).max()) > 1024
    idx, vals = _coo_of(c, S)
    assert torch.equal(idx, coo.indices())
    assert bits_equal(vals, coo.values())
    assert bits_equal(K.decompress_threshold(c).cpu().reshape(B, S, H), O.ref_decompress(coo, stored, bits, scale, L=L, R=R))


@pytest.mark.parametrize("bits", [1, 2, 4, 8])
@pytest.mark.parametrize("method", ["per-tensor", "per-channel", "per-token"])
@pytest.mark.parametrize("rank", [0, 2])
def test_threshold_roundtrip(K, bits, method, rank):
    B, S, H = 3, 40, 512
    gen = torch.Generator().manual_seed(bits * 10 + rank)
    x = torch.randn(B, S, H, generator=gen)
    x[..., torch.randperm(H, generator=gen)[:4]] *= 12
    x = x.bfloat16()
    torch.manual_seed(5)
    thr, L, R, scale = O.get_statistics(x, 0, 0.02, 1.0, bits, method, rank)
    coo, stored, _ = O.ref_compress(x, thr, scale, bits, 1.0, L, R)
    coo = coo.coalesce()
    c = K.compress_threshold(x.reshape(-1, H).cuda(), S, float(thr), scale.cuda(), bits,
                             L.cuda() if rank else None, R.cuda() if rank else None)
    idx, vals = _coo_of(c, S)
    assert torch.equal(idx, coo.indices())
    assert bits_equal(vals, coo.values())
    assert torch.equal(c.stored.cpu().reshape(stored.shape), stored)
    want = O.ref_decompress(coo, stored, bits, scale, L=L, R=R)
    got = K.decompress_threshold(c).cpu().reshape(B, S, H)
    assert bits_equal(got, want)
    cnt = K.outlier_counts(x.reshape(-1, H).cuda(), S, float(thr), 8, L.cuda() if rank else None, R.cuda() if rank else None)
    rp = c.row_ptr.cpu()
    assert torch.equal(cnt.cpu(), rp[1:] - rp[:-1])


def test_threshold_rank16_within_one_ulp(K):
    """rank > 2: the fp32 accumulation order of L@R is not fixed by the reference (library GEMM), so the
    base may differ in the last bf16 bit; everything downstream is compared through the reconstruction."""
    B, S, H = 2, 32, 256
    gen = torch.Generator().manual_seed(3)
    x = torch.randn(B, S, H, generator=gen).bfloat16()
    torch.manual_seed(6)
    thr, L, R, scale = O.get_statistics(x, 0, 0.02, 1.0, 8, "per-channel", 16)
    coo, stored, _ = O.ref_compress(x, thr, scale, 8, 1.0, L, R)
    want = O.ref_decompress(coo, stored, 8, scale, L=L, R=R)
    c = K.compress_threshold(x.reshape(-1, H).cuda(), S, float(thr), scale.cuda(), 8, L.cuda(), R.cuda())
    got = K.decompress_threshold(c).cpu().reshape(B, S, H)
    assert (got.float() - want.float()).abs().max() <= 2.5 * scale.float().max()
    frac_same = (bf16_ulp_diff(got, want) == 0).float().mean()
    assert frac_same > 0.9


def test_quantize_every_bf16_pattern(K):
    """all finite bf16 values as activations, one scale per token: pins the reciprocal shortcut of the kernel
    (x * fl(1/s) instead of x / s) and the IEEE fallback outside its range, bit for bit, for every bit width."""
    pat = np.arange(65536, dtype=np.uint32)
    pat[((pat >> 7) & 0xFF) == 0xFF] = 0                       # inf / nan -> 0
    x = from_bits(pat.astype(np.uint16)).reshape(1, 16, 4096)
    rng = np.random.default_rng(0)
    L, R = torch.zeros(16, 16).bfloat16(), torch.zeros(16, 4096).bfloat16()
    thr = torch.tensor(float("inf"))
    for trial in range(6):
        if trial == 0:
            sp = np.array([0x3F80, 0x3E1A, 0x3DCD, 0x4049, 0x3C03, 0x0080, 0x7F00, 0x0001, 0x0040, 0x1000, 0x6F00,
                           0x3F7F, 0x3F01, 0x4000, 0x007F, 0x0100], dtype=np.uint16)
        else:
            sp = rng.integers(0x0001, 0x7F7F, size=16).astype(np.uint16)
        scale = from_bits(sp).reshape(16, 1)
        for bits in (1, 2, 4, 8):
            _, stored, _ = O.ref_compress(x, thr, scale, bits, 1.0, L, R)
            c = K.compress_threshold(x.reshape(-1, 4096).cuda(), 16, float(thr), scale.cuda(), bits)
            assert c.cols.numel() == 0
            assert torch.equal(c.stored.cpu().reshape(stored.shape), stored), (trial, bits)


def test_golden_cases_on_gpu(K, golden_compress):
    """the reference's own outputs (tests/golden) reproduced by the HIP kernels"""
    gc = golden_compress
    n = int(gc["n_cases"])
    checked = 0
    for i in range(n):
        p = f"c{i}_"
        meta = gc[p + "meta"]
        bits, rank, shape = int(meta[0]), int(meta[1]), tuple(int(v) for v in meta[4:])
        x = from_bits(gc[p + "x"])
        if len(shape) == 4:
            x = O.head_to_hidden_shape(x)
        B, S, H = x.shape
        if H % (64 // bits) != 0:
            continue
        thr, scale = from_bits(gc[p + "thr"]), from_bits(gc[p + "scale"])
        L, R = from_bits(gc[p + "L"]), from_bits(gc[p + "R"])
        c = K.compress_threshold(x.reshape(-1, H).contiguous().cuda(), S, float(thr), scale.cuda(), bits,
                                 L.cuda() if rank else None, R.cuda() if rank else None)
        idx, vals = _coo_of(c, S)
        assert torch.equal(idx, from_bits(gc[p + "coo_idx"])), i
        assert bits_equal(vals, from_bits(gc[p + "coo_val"])), i
        stored = from_bits(gc[p + "stored"])
        if not torch.equal(c.stored.cpu().reshape(stored.shape), stored):
            # only where the reference computes 0/0 (a channel whose calibrated scale is 0): its NaN -> uint8 cast is
            # platform-defined, the kernels define q = 0; the oracle with define_nan=True states exactly that
            _, stored_d, _ = O.ref_compress(x, thr, scale, bits, 1.0, L, R, define_nan=True)
            assert (scale == 0).any(), i
            assert torch.equal(c.stored.cpu().reshape(stored_d.shape), stored_d), i
        got = K.decompress_threshold(c).cpu().reshape(B, S, H)
        want = from_bits(gc[p + "xhat"])
        if len(shape) == 4:
            want = O.head_to_hidden_shape(want)
        assert bits_equal(got, want), i
        checked += 1
    assert checked >= 40


# ------------------------------------------------------------------ the configurations at their full size
FULL_SIZE = [  # (name, M, H, bits, group, hot channels, gain)
    ("config 1: [4,512,4096], 41 channels x50, INT4 G128", 2048, 4096, 4, 128, 41, 50.0),
    ("config 3: [4,1024,4096], INT2 G64", 4096, 4096, 2, 64, 41, 30.0),
    ("config 4: [4,1024,11008], 110 channels x20, INT4 G128", 4096, 11008, 4, 128, 110, 20.0),
]


@pytest.mark.parametrize("rule", ["absmax", "range"])
@pytest.mark.parametrize("name,M,H,bits,group,n_hot,gain", FULL_SIZE)
def test_full_size_configurations(K, name, M, H, bits, group, n_hot, gain, rule):
    """At the configurations' own sizes: the channel choice equals the oracle's; rows are independent, so the packed
    bytes, scales, outlier values and the reconstruction of a seeded sample of 96 rows must equal, bit for bit, the
    oracle run on those rows alone; and over ALL rows the properties the scheme guarantees hold: outlier channels
    come back exactly, every other element is within half a quantisation step (one bf16 ulp of slack) of the
    original unless its code sits on the clamp, and the scale of each group is bf16(bf16(max - min) / levels) under the
    range rule, bf16(bf16(2 max|x|) / levels) under the abs-max rule."""
    x, hot = make_x(len(name), M, H, n_hot, gain)
    k = K.num_outlier_channels(H, 0.01)
    xd = x.cuda()
    plan = K.select_channels(K.channel_absmax(xd), k, rule)
    idx = O.hyc_select_channels(O.hyc_channel_scores(x), k)
    assert torch.equal(plan.idx.cpu(), idx)
    assert set(hot.tolist()) <= set(idx.tolist()) or n_hot > k
    c = K.compress_channel(xd, plan, bits, group)
    xh = K.decompress_channel(c)
    rows = torch.randperm(M, generator=torch.Generator().manual_seed(M + H))[:96].sort().values
    vals, stored, scales = O.hyc_compress(x[rows], idx, bits, group, rule)
    assert torch.equal(c.stored.cpu()[rows].view(torch.uint8), stored.view(torch.uint8))
    assert bits_equal(c.scales.cpu()[rows], scales) and bits_equal(c.vals.cpu()[rows], vals)
    assert bits_equal(xh.cpu()[rows], O.hyc_decompress(vals, stored, idx, scales, bits, group))
    # whole-tensor properties, evaluated on the device in fp32
    xf, hf = xd.float(), xh.float()
    keep = torch.ones(H, dtype=torch.bool, device="cuda")
    keep[plan.idx.long()] = False
    assert torch.equal(xd[:, ~keep], xh[:, ~keep])
    inl = torch.where(keep, xf, torch.zeros((), device="cuda")).view(M, H // group, group)
    span = ((inl.amax(-1) - inl.amin(-1)) if rule == "range" else 2 * inl.abs().amax(-1)).bfloat16().float()
    levels = float(2 ** bits - 1)
    assert bits_equal((span / levels).bfloat16().cpu(), c.scales.cpu())
    s = c.scales.float().repeat_interleave(group, dim=1)
    err = (hf - xf).abs()
    off = float(2 ** (bits - 1))
    clamped = (xf / s.clamp_min(1e-30)).abs() >= off - 0.5              # the code sits on (or next to) a clamp bound
    slack = hf.abs() * 2.0 ** -7 + 1e-30                                # one bf16 rounding of the product
    bad = keep[None, :] & ~clamped & (err > 0.5 * s + slack)
    assert int(bad.sum()) == 0
