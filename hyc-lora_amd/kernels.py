"""Host-side launchers: torch tensors in, torch tensors out, every computation done by the HIP library.

torch is used for device memory and the current stream only.  Nothing here computes on the CPU and
nothing falls back to torch ops for the hot path: inputs that are not CUDA tensors raise.
"""
import ctypes
from dataclasses import dataclass
from typing import Optional

import torch

from . import _abi
from ._abi import HycDesc, check

BF16 = torch.bfloat16


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream():
    """handle of torch's current stream on the current device (the kernels are launched on it)"""
    if _raw_stream is not None:                    # no Stream object is built: 0.5 us instead of 5 per launch
        return ctypes.c_void_p(_raw_stream(torch.cuda.current_device()))
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _p(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _need(t, dtype, name):
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise ValueError("%s must be a CUDA (ROCm) tensor: the hot path runs on the GPU only" % name)
    if t.dtype != dtype:
        raise ValueError("%s must be %s, got %s" % (name, dtype, t.dtype))
    if not t.is_contiguous():
        raise ValueError("%s must be contiguous" % name)
    return t


def _need_vec(t, dtype, n, name):
    """a contiguous device vector of exactly n elements (the kernels index it without further checks)"""
    _need(t, dtype, name)
    if t.numel() != n:
        raise ValueError("%s must hold %d elements, got %d" % (name, n, t.numel()))
    return t


def _need_weight(w, H):
    if not isinstance(w, torch.Tensor) or not w.is_cuda or not w.is_contiguous() or w.numel() != H:
        raise ValueError("weight must be a contiguous CUDA tensor of %d elements" % H)
    return w


def threshold_value(t):
    """Python float of a threshold.  A device tensor costs one host round trip the first time; the float is then kept
    on the tensor object together with the tensor's version counter, so the frozen threshold of a calibrated module
    (the same 0-d tensor call after call) is read back once, not at every step, and an in-place update of the tensor
    (`copy_`, `mul_`, a restored state) is seen.  The read-back is a synchronisation: the calibration calls of a module
    must run outside a stream capture."""
    if not isinstance(t, torch.Tensor):
        return float(t)
    cached = getattr(t, "_hyc_float", None)
    version = t._version
    if cached is None or cached[0] != version:
        cached = (version, float(t))
        try:
            t._hyc_float = cached
        except AttributeError:
            pass
    return cached[1]


class KeptBudget:
    """Room for the sparse side data (kept softmax probabilities, element outliers) of one calibrated site, so that its
    steady-state calls never wait for the GPU.

    The reference reads the number of kept entries back on every call (`to_sparse()`, compress_function.py:153, :269)
    before it can allocate them.  Here a call that has a budget allocates `capacity(rows)` entries - 1.25 x the largest
    kept fraction seen so far, plus a little - cuts the row offsets off at that capacity on the device (hyc_csr_offsets)
    and leaves the true total in a device word.  Entries past the capacity are dropped, which must not go unnoticed: the
    total travels to pinned host memory behind the kernels, and the next call of the site that finds it arrived checks
    it (`poll`), raises if entries were dropped and grows the budget.  `sync_check()` does the same at once.
    """
    MARGIN = 1.25

    def __init__(self):
        self.per_row = -1.0        # largest kept entries per row seen (negative: nothing seen yet)
        self._pending = []         # (event, pinned int64 scalar, capacity, rows) of calls not checked yet
        self._spare = []           # pinned scalars to use again

    @property
    def ready(self):
        return self.per_row >= 0.0

    def observe(self, nnz, rows):
        self.per_row = max(self.per_row, nnz / max(rows, 1))

    def capacity(self, rows):
        return int(self.per_row * self.MARGIN * rows) + rows // 8 + 1024

    def watch(self, total, capacity, rows):
        """keep an eye on `total` (int64 device scalar of a call that was given `capacity`)"""
        if torch.cuda.is_current_stream_capturing():
            return                                  # a captured call is checked by whoever replays it (SparseRows.total)
        host = self._spare.pop() if self._spare else torch.empty((), dtype=torch.int64, pin_memory=True)
        host.copy_(total, non_blocking=True)
        done = torch.cuda.Event()
        done.record()
        self._pending.append((done, host, capacity, rows))

    def _check(self, host, capacity, rows):
        n = int(host)
        self._spare.append(host)
        self.observe(n, rows)
        if n > capacity:
            raise RuntimeError("a compressed activation kept %d sparse entries but its buffers were sized for %d "
                               "(1.25 x the largest share seen before): the entries beyond were dropped and the "
                               "gradients computed from that call are not exact.  The budget has been raised; "
                               "repeat the step." % (n, capacity))

    def poll(self):
        """check the calls whose totals have arrived; never waits (and asks nothing of the runtime during a capture)"""
        if torch.cuda.is_current_stream_capturing():
            return
        while self._pending and self._pending[0][0].query():
            _, host, capacity, rows = self._pending.pop(0)
            self._check(host, capacity, rows)

    def sync_check(self):
        """wait for every watched call and check it"""
        while self._pending:
            done, host, capacity, rows = self._pending.pop(0)
            done.synchronize()
            self._check(host, capacity, rows)


def kept_budget(threshold):
    """The KeptBudget that travels with a threshold tensor (created on first use; None for a plain number).  A site that
    is still calibrating measures a fresh threshold tensor on every call, so each of its calls finds a new budget and
    sizes its buffers exactly; the frozen threshold of a calibrated site is the same tensor call after call, so its
    first steady-state call reads the total back once and the later ones do not."""
    if not isinstance(threshold, torch.Tensor):
        return None
    budget = getattr(threshold, "_hyc_budget", None)
    if budget is None:
        budget = KeptBudget()
        try:
            threshold._hyc_budget = budget
        except AttributeError:
            return None
    return budget


def _csr_offsets(lib, counts, rows, budget):
    """(row_ptr, nnz to allocate, total) from per-row counts.  Without a budget, or with one that has seen nothing yet,
    the total is read back (one host round trip) and the buffers are exact; otherwise nothing waits."""
    dev = counts.device
    row_ptr = torch.empty(rows + 1, dtype=torch.int32, device=dev)
    total = torch.empty((), dtype=torch.int64, device=dev)
    if budget is not None and budget.ready:
        budget.poll()
        cap = budget.capacity(rows)
        check(lib.hyc_csr_offsets(_p(counts), rows, cap, _p(row_ptr), _p(total), _stream()))
        budget.watch(total, cap, rows)
        return row_ptr, cap, total
    check(lib.hyc_csr_offsets(_p(counts), rows, -1, _p(row_ptr), _p(total), _stream()))
    nnz = int(total.item())
    if budget is not None:
        budget.observe(nnz, rows)
    return row_ptr, nnz, total


def num_outlier_channels(H, ratio):
    """k = floor(ratio*H + 1/2)"""
    import math
    return int(math.floor(ratio * H + 0.5))


# ----------------------------------------------------------------------------------------------------
# channel mode
# ----------------------------------------------------------------------------------------------------
SCALE_RULES = {"range": _abi.SCALE_RANGE, "absmax": _abi.SCALE_ABSMAX}
DEFAULT_SCALE_RULE = "absmax"


@dataclass
class ChannelPlan:
    """the static part of one activation site: its outlier-channel set and the rule its group scales follow
    ("absmax": 2 max|x| / (2^bits - 1), the reference's formula over the interval made symmetric about zero, so that no
    element ends up more than half a step away; "range": the reference's (max - min) / (2^bits - 1) as it stands,
    which has no zero point and clips groups that are not centred on 0)"""
    H: int
    k: int
    idx: torch.Tensor    # int32 [k], ascending
    plan: torch.Tensor   # int32 [H/8] (bit pattern of the uint32 lookup words)
    scale_rule: str = DEFAULT_SCALE_RULE


def kth_value(x, k):
    """the k-th smallest (1-based) of all elements of x (bf16 or fp32) as a 0-d fp32 tensor; the value
    `torch.kthvalue(x.flatten().float(), k).values` gives, without a sort and without a host round trip"""
    if x.dtype not in (BF16, torch.float32):
        raise ValueError("x must be bfloat16 or float32, got %s" % x.dtype)
    if not x.is_cuda:
        raise ValueError("x must live on the GPU")
    x = x.contiguous()
    lib = _abi.load()
    out = torch.empty((), dtype=torch.float32, device=x.device)
    ws = torch.empty(lib.hyc_kth_value_workspace_bytes() // 4, dtype=torch.int32, device=x.device)
    code = _abi.DTYPE_BF16 if x.dtype == BF16 else _abi.DTYPE_F32
    check(lib.hyc_kth_value(_p(x), code, x.numel(), int(k), _p(out), _p(ws), _stream()))
    return out


def channel_absmax(x2d, amax=None):
    """running per-channel max |x| (fp32 [H]); pass the previous result to accumulate"""
    if isinstance(x2d, torch.Tensor) and x2d.is_cuda and not x2d.is_contiguous():
        x2d = x2d.contiguous()                     # calibration only (twice per site): a copy is acceptable
    _need(x2d, BF16, "x")
    M, H = x2d.shape
    if amax is None:
        amax = torch.zeros(H, dtype=torch.float32, device=x2d.device)
    _need_vec(amax, torch.float32, H, "amax")
    check(_abi.load().hyc_channel_absmax(_p(x2d), M, H, _p(amax), _stream()))
    return amax


def select_channels(amax, k, scale_rule=DEFAULT_SCALE_RULE):
    if scale_rule not in SCALE_RULES:
        raise ValueError("scale_rule must be 'absmax' or 'range', got %r" % (scale_rule,))
    _need(amax, torch.float32, "amax")
    H = amax.numel()
    if H % 8 or not 0 <= k <= H:
        raise ValueError("select_channels: H=%d must be a multiple of 8 and 0 <= k=%d <= H" % (H, k))
    idx = torch.empty(max(k, 1), dtype=torch.int32, device=amax.device)[:k]
    plan = torch.empty(H // 8, dtype=torch.int32, device=amax.device)
    check(_abi.load().hyc_select_channels(_p(amax), H, k, _p(idx), _p(plan), _stream()))
    return ChannelPlan(H, k, idx, plan, scale_rule)


def _check_plan(plan, device=None):
    """the kernels index plan.plan [H/8] and plan.idx [k] without further checks, so they must be int32 device
    tensors of exactly those sizes, on the device of the activation they are used with"""
    for name, t, n in (("plan.plan", plan.plan, plan.H // 8), ("plan.idx", plan.idx, plan.k)):
        if not isinstance(t, torch.Tensor) or not t.is_cuda:
            raise ValueError("%s must be a CUDA (ROCm) tensor; after loading a checkpoint on the host, move the "
                             "calibration state to the GPU (load_calibration_state does)" % name)
        if t.dtype != torch.int32 or not t.is_contiguous() or t.numel() != n:
            raise ValueError("%s must be a contiguous int32 tensor of %d elements" % (name, n))
        if device is not None:
            want = torch.device(device)
            index = want.index if want.index is not None else torch.cuda.current_device()
            if t.device.type != want.type or t.device.index != index:
                raise ValueError("%s lives on %s, the activation on %s" % (name, t.device, device))
    if plan.scale_rule not in SCALE_RULES:
        raise ValueError("scale_rule must be 'absmax' or 'range', got %r" % (plan.scale_rule,))


def channel_desc(plan: ChannelPlan, bits, group, device=None):
    _check_plan(plan, device)
    d = HycDesc()
    d.mode, d.bits, d.group, d.k = _abi.MODE_CHANNEL, bits, group, plan.k
    d.chan_plan = plan.plan.data_ptr()
    d.chan_idx = plan.idx.data_ptr() if plan.k else None
    d.scale_rule = SCALE_RULES[plan.scale_rule]
    return d


def dense_desc(bits=4):
    d = HycDesc()
    d.mode, d.bits = _abi.MODE_DENSE, bits
    return d


@dataclass
class ChannelCompressed:
    """a [M,H] bf16 activation held as codes + outlier channels + group scales"""
    stored: torch.Tensor   # uint8 [M, H*bits/8] (int8 [M,H] for 8 bits)
    vals: torch.Tensor     # bf16 [M, k]
    scales: torch.Tensor   # bf16 [M, H/group]
    plan: ChannelPlan
    bits: int
    group: int
    M: int
    H: int

    def desc(self):
        return channel_desc(self.plan, self.bits, self.group, self.stored.device)

    def nbytes(self):
        return self.stored.numel() * self.stored.element_size() + 2 * self.vals.numel() + 2 * self.scales.numel()


def alloc_channel(M, H, plan, bits, group, device):
    if plan.H != H:
        raise ValueError("the outlier-channel plan was made for %d channels, the activation has %d" % (plan.H, H))
    _check_plan(plan, torch.device(device) if not isinstance(device, torch.device) else device)
    stored = torch.empty((M, H * bits // 8), dtype=torch.int8 if bits == 8 else torch.uint8, device=device)
    vals = torch.empty((M, plan.k), dtype=BF16, device=device)
    scales = torch.empty((M, H // group), dtype=BF16, device=device)
    return ChannelCompressed(stored, vals, scales, plan, bits, group, M, H)


def _need_rows(t, name):
    """a bf16 [M, H] matrix whose rows are contiguous; the rows themselves may be further apart (a column slice)"""
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise ValueError("%s must be a CUDA (ROCm) tensor: the hot path runs on the GPU only" % name)
    if t.dtype != BF16 or t.dim() != 2 or (t.shape[1] > 1 and t.stride(1) != 1):
        raise ValueError("%s must be a bfloat16 matrix with contiguous rows" % name)
    return t


def compress_channel(x2d, plan, bits, group):
    _need_rows(x2d, "x")
    M, H = x2d.shape
    lib = _abi.load()
    check(lib.hyc_check_shape(H, bits, group, _abi.MODE_CHANNEL))
    out = alloc_channel(M, H, plan, bits, group, x2d.device)
    d = out.desc()
    pitch = x2d.stride(0) if M > 1 else H
    check(lib.hyc_compress_rows(_p(x2d), pitch, M, H, ctypes.byref(d), _p(out.stored), _p(out.vals), _p(out.scales), None,
                                _stream()))
    return out


def decompress_channel(c: ChannelCompressed):
    xhat = torch.empty((c.M, c.H), dtype=BF16, device=c.stored.device)
    d = c.desc()
    check(_abi.load().hyc_decompress(_p(c.stored), _p(c.vals), _p(c.scales), c.M, c.H, ctypes.byref(d), _p(xhat), _stream()))
    return xhat


# ----------------------------------------------------------------------------------------------------
# threshold mode (the scheme of the reference snapshot)
# ----------------------------------------------------------------------------------------------------
def scale_strides(scale, S, H):
    """(stride_token, stride_channel) of a per-tensor [] / per-channel [1,H] / per-token [S,1] scale"""
    n = scale.numel()
    if n == 1:
        return 0, 0
    if scale.dim() >= 2 and scale.shape[-1] == H and n == H:
        return 0, 1
    if scale.dim() >= 2 and scale.shape[-1] == 1 and n == S:
        return 1, 0
    raise ValueError("scale of shape %s is neither per-tensor, per-channel [1,%d] nor per-token [%d,1]"
                     % (tuple(scale.shape), H, S))


@dataclass
class ThresholdCompressed:
    stored: torch.Tensor               # uint8 [M, H*bits/8] / int8 [M,H]
    row_ptr: torch.Tensor              # int32 [M+1]
    cols: torch.Tensor                 # int32 [nnz]
    vals: torch.Tensor                 # bf16 [nnz]
    threshold: float
    scale: torch.Tensor
    L: Optional[torch.Tensor]
    R: Optional[torch.Tensor]
    bits: int
    M: int
    H: int
    S: int

    def desc(self):
        return threshold_desc(self.threshold, self.scale, self.bits, self.S, self.H, self.L, self.R,
                              self.row_ptr, self.cols, self.vals)


def threshold_desc(threshold, scale, bits, S, H, L=None, R=None, row_ptr=None, cols=None, vals=None):
    d = HycDesc()
    d.mode, d.bits = _abi.MODE_THRESHOLD, bits
    d.threshold = float(threshold)
    d.scale = scale.data_ptr()
    d.scale_stride_token, d.scale_stride_channel = scale_strides(scale, S, H)
    d.S = S
    rank = 0 if L is None else L.shape[-1]
    d.rank = rank
    if rank:
        d.L, d.R = L.data_ptr(), R.data_ptr()
    if row_ptr is not None:
        d.csr_row_ptr = row_ptr.data_ptr()
        d.csr_cols = cols.data_ptr() if cols.numel() else None
        d.csr_vals = vals.data_ptr() if vals.numel() else None
    return d


def fit_rows(L, S):
    """pad with zero rows / cut L [S', r] to S rows (the reference's pad_cut_L); L is tiny"""
    have = L.shape[0]
    if have == S:
        return L.contiguous()
    if have > S:
        return L[:S].contiguous()
    out = torch.zeros((S, L.shape[1]), dtype=L.dtype, device=L.device)
    out[:have] = L
    return out


def compress_threshold(x2d, S, threshold, scale, bits, L=None, R=None, budget=None):
    """codes + CSR outliers of x [M,H] (row m is sequence position m mod S).  One host read-back
    (the outlier total) sizes the CSR arrays, as `.to_sparse()` does in the reference; with a KeptBudget that has seen
    a call they are sized ahead of time and nothing waits."""
    _need(x2d, BF16, "x")
    _need(scale, BF16, "scale")
    M, H = x2d.shape
    lib = _abi.load()
    check(lib.hyc_check_shape(H, bits, 0, _abi.MODE_THRESHOLD))
    dev = x2d.device
    if L is not None:
        L = fit_rows(_need(L, BF16, "L"), S)
        _need(R, BF16, "R")
    stored = torch.empty((M, H * bits // 8), dtype=torch.int8 if bits == 8 else torch.uint8, device=dev)
    counts = torch.empty(M, dtype=torch.int32, device=dev)
    d = threshold_desc(threshold, scale, bits, S, H, L, R)
    check(lib.hyc_compress(_p(x2d), M, H, ctypes.byref(d), _p(stored), None, None, _p(counts), _stream()))
    row_ptr, nnz, _ = _csr_offsets(lib, counts, M, budget)
    cols = torch.empty(nnz, dtype=torch.int32, device=dev)
    vals = torch.empty(nnz, dtype=BF16, device=dev)
    check(lib.hyc_ref_outlier_fill(_p(x2d), M, H, ctypes.byref(d), _p(row_ptr), _p(cols) if nnz else None,
                                   _p(vals) if nnz else None, _stream()))
    return ThresholdCompressed(stored, row_ptr, cols, vals, float(threshold), scale, L, R, bits, M, H, S)


def outlier_counts(x2d, S, threshold, bits=8, L=None, R=None):
    _need(x2d, BF16, "x")
    M, H = x2d.shape
    counts = torch.empty(M, dtype=torch.int32, device=x2d.device)
    one = torch.ones(1, dtype=BF16, device=x2d.device)
    if L is not None:
        L = fit_rows(L, S)
    d = threshold_desc(threshold, one, bits, S, H, L, R)
    check(_abi.load().hyc_ref_outlier_count(_p(x2d), M, H, ctypes.byref(d), _p(counts), _stream()))
    return counts


def decompress_threshold(c: ThresholdCompressed):
    xhat = torch.empty((c.M, c.H), dtype=BF16, device=c.stored.device)
    d = c.desc()
    check(_abi.load().hyc_decompress(_p(c.stored), None, None, c.M, c.H, ctypes.byref(d), _p(xhat), _stream()))
    return xhat


# ----------------------------------------------------------------------------------------------------
# fused operators
# ----------------------------------------------------------------------------------------------------
def _wdtype(w):
    if w.dtype == torch.float32:
        return _abi.DTYPE_F32
    if w.dtype == BF16:
        return _abi.DTYPE_BF16
    raise ValueError("RMSNorm weight must be bf16 or fp32, got %s" % w.dtype)


def rmsnorm_fwd_compress_channel(x2d, w, eps, plan, bits, group):
    """-> (y bf16 [M,H], rstd fp32 [M], ChannelCompressed of x)"""
    _need(x2d, BF16, "x")
    M, H = x2d.shape
    _need_weight(w, H)
    lib = _abi.load()
    check(lib.hyc_check_shape(H, bits, group, _abi.MODE_CHANNEL))
    y = torch.empty_like(x2d)
    rstd = torch.empty(M, dtype=torch.float32, device=x2d.device)
    c = alloc_channel(M, H, plan, bits, group, x2d.device)
    d = c.desc()
    check(lib.hyc_rmsnorm_fwd_compress(_p(x2d), _p(w), _wdtype(w), float(eps), M, H, ctypes.byref(d), _p(y), _p(rstd),
                                       _p(c.stored), _p(c.vals), _p(c.scales), None, _stream()))
    return y, rstd, c


def rmsnorm_fwd_compress_threshold(x2d, w, eps, S, threshold, scale, bits, L=None, R=None, budget=None):
    """-> (y, rstd, ThresholdCompressed of x)"""
    _need(x2d, BF16, "x")
    _need(scale, BF16, "scale")
    M, H = x2d.shape
    _need_weight(w, H)
    lib = _abi.load()
    dev = x2d.device
    if L is not None:
        L = fit_rows(_need(L, BF16, "L"), S)
        _need(R, BF16, "R")
    y = torch.empty_like(x2d)
    rstd = torch.empty(M, dtype=torch.float32, device=dev)
    stored = torch.empty((M, H * bits // 8), dtype=torch.int8 if bits == 8 else torch.uint8, device=dev)
    counts = torch.empty(M, dtype=torch.int32, device=dev)
    d = threshold_desc(threshold, scale, bits, S, H, L, R)
    check(lib.hyc_rmsnorm_fwd_compress(_p(x2d), _p(w), _wdtype(w), float(eps), M, H, ctypes.byref(d), _p(y), _p(rstd),
                                       _p(stored), None, None, _p(counts), _stream()))
    row_ptr, nnz, _ = _csr_offsets(lib, counts, M, budget)
    cols = torch.empty(nnz, dtype=torch.int32, device=dev)
    vals = torch.empty(nnz, dtype=BF16, device=dev)
    check(lib.hyc_ref_outlier_fill(_p(x2d), M, H, ctypes.byref(d), _p(row_ptr), _p(cols) if nnz else None,
                                   _p(vals) if nnz else None, _stream()))
    return y, rstd, ThresholdCompressed(stored, row_ptr, cols, vals, float(threshold), scale, L, R, bits, M, H, S)


def layernorm_fwd_supported(H, bits):
    """rows the one-pass LayerNorm forward covers"""
    return bits in (1, 2, 4, 8) and H % (64 // bits) == 0 and H * bits // 64 <= 1024


def _need_bias(bias, w, H):
    if bias is None:
        return None
    if not bias.is_cuda or not bias.is_contiguous() or bias.numel() != H or bias.dtype != w.dtype:
        raise ValueError("bias must be a contiguous CUDA tensor of %d elements in the weight's dtype" % H)
    return bias


def layernorm_fwd_compress_channel(x2d, w, bias, eps, plan, bits, group):
    """-> (y bf16 [M,H], mean fp32 [M], rstd fp32 [M], ChannelCompressed of x), one pass over x"""
    _need(x2d, BF16, "x")
    M, H = x2d.shape
    _need_weight(w, H)
    _need_bias(bias, w, H)
    lib = _abi.load()
    check(lib.hyc_check_shape(H, bits, group, _abi.MODE_CHANNEL))
    y = torch.empty_like(x2d)
    mean = torch.empty(M, dtype=torch.float32, device=x2d.device)
    rstd = torch.empty(M, dtype=torch.float32, device=x2d.device)
    c = alloc_channel(M, H, plan, bits, group, x2d.device)
    d = c.desc()
    check(lib.hyc_layernorm_fwd_compress(_p(x2d), _p(w), _p(bias), _wdtype(w), float(eps), M, H, ctypes.byref(d), _p(y),
                                         _p(mean), _p(rstd), _p(c.stored), _p(c.vals), _p(c.scales), None, _stream()))
    return y, mean, rstd, c


def layernorm_fwd_compress_threshold(x2d, w, bias, eps, S, threshold, scale, bits, L=None, R=None, budget=None):
    """-> (y, mean, rstd, ThresholdCompressed of x)"""
    _need(x2d, BF16, "x")
    _need(scale, BF16, "scale")
    M, H = x2d.shape
    _need_weight(w, H)
    _need_bias(bias, w, H)
    lib = _abi.load()
    dev = x2d.device
    if L is not None:
        L = fit_rows(_need(L, BF16, "L"), S)
        _need(R, BF16, "R")
    y = torch.empty_like(x2d)
    mean = torch.empty(M, dtype=torch.float32, device=dev)
    rstd = torch.empty(M, dtype=torch.float32, device=dev)
    stored = torch.empty((M, H * bits // 8), dtype=torch.int8 if bits == 8 else torch.uint8, device=dev)
    counts = torch.empty(M, dtype=torch.int32, device=dev)
    d = threshold_desc(threshold, scale, bits, S, H, L, R)
    check(lib.hyc_layernorm_fwd_compress(_p(x2d), _p(w), _p(bias), _wdtype(w), float(eps), M, H, ctypes.byref(d), _p(y),
                                         _p(mean), _p(rstd), _p(stored), None, None, _p(counts), _stream()))
    row_ptr, nnz, _ = _csr_offsets(lib, counts, M, budget)
    cols = torch.empty(nnz, dtype=torch.int32, device=dev)
    vals = torch.empty(nnz, dtype=BF16, device=dev)
    check(lib.hyc_ref_outlier_fill(_p(x2d), M, H, ctypes.byref(d), _p(row_ptr), _p(cols) if nnz else None,
                                   _p(vals) if nnz else None, _stream()))
    return y, mean, rstd, ThresholdCompressed(stored, row_ptr, cols, vals, float(threshold), scale, L, R, bits, M, H, S)


def _source(c, M, H):
    """(stored, vals, scales, desc) of a ChannelCompressed, or of a dense bf16 x_hat, that holds an [M, H] activation"""
    if isinstance(c, (ChannelCompressed, ThresholdCompressed)) and (c.M, c.H) != (M, H):
        raise ValueError("the saved activation is [%d, %d], the gradient is [%d, %d]" % (c.M, c.H, M, H))
    if isinstance(c, ChannelCompressed):
        return c.stored, c.vals, c.scales, c.desc()
    if isinstance(c, ThresholdCompressed):
        c = decompress_threshold(c)
    _need(c, BF16, "x_hat")
    if c.numel() != M * H or c.shape[-1] != H:
        raise ValueError("the saved activation is %s, the gradient is [%d, %d]" % (tuple(c.shape), M, H))
    return c, None, None, dense_desc()


def rmsnorm_bwd(dy2d, src, w, rstd, c2_quirk=True):
    """-> (dx bf16 [M,H], dw in w's dtype [H]); src is a ChannelCompressed, ThresholdCompressed or dense x_hat"""
    _need(dy2d, BF16, "dy")
    M, H = dy2d.shape
    _need_weight(w, H)
    _need_vec(rstd, torch.float32, M, "rstd")
    lib = _abi.load()
    stored, vals, scales, d = _source(src, M, H)
    P = lib.hyc_rmsnorm_bwd_partials(M, H)
    partials = torch.empty((max(P, 1), H), dtype=torch.float32, device=dy2d.device)
    dx = torch.empty_like(dy2d)
    dw = torch.empty(H, dtype=w.dtype, device=dy2d.device)
    check(lib.hyc_rmsnorm_bwd(_p(dy2d), _p(stored), _p(vals), _p(scales), _p(w), _wdtype(w), _p(rstd), M, H,
                              ctypes.byref(d), 1 if c2_quirk else 0, _p(dx), _p(partials), _p(dw), _stream()))
    return dx, dw


def layernorm_bwd(dy2d, src, w, mean, rstd):
    """-> (dx bf16 [M,H], dw in w's dtype [H]) with xn = (x_hat - mean) * rstd; db = dy.sum(0) is the caller's"""
    _need(dy2d, BF16, "dy")
    M, H = dy2d.shape
    _need_weight(w, H)
    _need_vec(mean, torch.float32, M, "mean")
    _need_vec(rstd, torch.float32, M, "rstd")
    lib = _abi.load()
    stored, vals, scales, d = _source(src, M, H)
    P = lib.hyc_rmsnorm_bwd_partials(M, H)
    partials = torch.empty((max(P, 1), H), dtype=torch.float32, device=dy2d.device)
    dx = torch.empty_like(dy2d)
    dw = torch.empty(H, dtype=w.dtype, device=dy2d.device)
    check(lib.hyc_layernorm_bwd(_p(dy2d), _p(stored), _p(vals), _p(scales), _p(w), _wdtype(w), _p(mean), _p(rstd), M, H,
                                ctypes.byref(d), _p(dx), _p(partials), _p(dw), _stream()))
    return dx, dw


def rmsnorm_bwd_partial(dy2d, src, w, rstd, c2_quirk=True):
    """-> (dx bf16 [M,H], fp32 partial rows [P,H] whose column sum is dw); the caller does the last reduction"""
    _need(dy2d, BF16, "dy")
    M, H = dy2d.shape
    _need_weight(w, H)
    _need_vec(rstd, torch.float32, M, "rstd")
    lib = _abi.load()
    stored, vals, scales, d = _source(src, M, H)
    P = lib.hyc_rmsnorm_bwd_partials(M, H)
    partials = torch.empty((max(P, 1), H), dtype=torch.float32, device=dy2d.device)
    dx = torch.empty_like(dy2d)
    check(lib.hyc_rmsnorm_bwd(_p(dy2d), _p(stored), _p(vals), _p(scales), _p(w), _wdtype(w), _p(rstd), M, H,
                              ctypes.byref(d), 1 if c2_quirk else 0, _p(dx), _p(partials), None, _stream()))
    return dx, partials[:lib.hyc_rmsnorm_bwd_partial_rows(M, H, ctypes.byref(d))]


def act_bwd(act, g2d, src):
    """act in {'silu', 'gelu'} -> dx bf16 [M,H]"""
    _need(g2d, BF16, "grad_output")
    M, H = g2d.shape
    stored, vals, scales, d = _source(src, M, H)
    dx = torch.empty_like(g2d)
    code = {"silu": _abi.ACT_SILU, "gelu": _abi.ACT_GELU_TANH}[act]
    check(_abi.load().hyc_act_bwd(code, _p(g2d), _p(stored), _p(vals), _p(scales), M, H, ctypes.byref(d), _p(dx), _stream()))
    return dx


def hadamard_bwd(g2d, src1, src2):
    """-> (g * x2_hat, x1_hat * g)"""
    _need(g2d, BF16, "grad_output")
    M, H = g2d.shape
    s1, v1, c1, d1 = _source(src1, M, H)
    s2, v2, c2, d2 = _source(src2, M, H)
    dx1, dx2 = torch.empty_like(g2d), torch.empty_like(g2d)
    check(_abi.load().hyc_hadamard_bwd(_p(g2d), _p(s1), _p(v1), _p(c1), ctypes.byref(d1), _p(s2), _p(v2), _p(c2),
                                       ctypes.byref(d2), M, H, _p(dx1), _p(dx2), _stream()))
    return dx1, dx2


def gated_act_bwd(act, g2d, src_act, src_up, src_gate):
    """backward of act(gate) * up in one pass -> (d_gate, d_up); the three sources are ChannelCompressed"""
    _need(g2d, BF16, "grad_output")
    M, H = g2d.shape
    sa, va, ca, da = _source(src_act, M, H)
    su, vu, cu, du = _source(src_up, M, H)
    sg, vg, cg, dg = _source(src_gate, M, H)
    d_gate, d_up = torch.empty_like(g2d), torch.empty_like(g2d)
    code = {"silu": _abi.ACT_SILU, "gelu": _abi.ACT_GELU_TANH}[act]
    check(_abi.load().hyc_gated_act_bwd(code, _p(g2d), _p(sa), _p(va), _p(ca), ctypes.byref(da), _p(su), _p(vu), _p(cu),
                                        ctypes.byref(du), _p(sg), _p(vg), _p(cg), ctypes.byref(dg), M, H, _p(d_gate),
                                        _p(d_up), _stream()))
    return d_gate, d_up


def _row_kernel_fits(H, bits, group, widths):
    return bits in widths and group in (64, 128) and H % (64 // bits) == 0 and H * bits // 64 <= 1024


def act_fwd_compress_supported(H, bits, group):
    """shapes the one-pass activation forward covers"""
    return _row_kernel_fits(H, bits, group, (2, 4, 8))


def hadamard_fwd_compress_supported(H, bits1, group1, bits2, group2):
    """shapes the one-pass product forward covers (two operands of 2-bit codes: at most 512 chunks per segment)"""
    return (bits1 == bits2 and group1 == group2 and _row_kernel_fits(H, bits1, group1, (2, 4, 8)) and
            (bits1 != 2 or H * bits1 // 64 <= 512))


def act_fwd_compress(act, x2d, plan, bits, group):
    """y = act(x) (F.silu / F.gelu values) and the compressed x from one read of x -> (y, ChannelCompressed)"""
    _need_rows(x2d, "x")
    M, H = x2d.shape
    c = alloc_channel(M, H, plan, bits, group, x2d.device)
    d = c.desc()
    y = torch.empty((M, H), dtype=BF16, device=x2d.device)
    code = {"silu": _abi.ACT_SILU, "gelu": _abi.ACT_GELU_TANH}[act]
    check(_abi.load().hyc_act_fwd_compress(code, _p(x2d), x2d.stride(0) if M > 1 else H, M, H, ctypes.byref(d), _p(y),
                                           _p(c.stored), _p(c.vals), _p(c.scales), _stream()))
    return y, c


def hadamard_fwd_compress(a2d, b2d, plan_a, plan_b, bits, group):
    """y = a * b and both operands compressed, each read once -> (y, c_a, c_b)"""
    _need_rows(a2d, "x1")
    _need_rows(b2d, "x2")
    if a2d.shape != b2d.shape:
        raise ValueError("x1 %s and x2 %s differ in shape" % (tuple(a2d.shape), tuple(b2d.shape)))
    M, H = a2d.shape
    ca = alloc_channel(M, H, plan_a, bits, group, a2d.device)
    cb = alloc_channel(M, H, plan_b, bits, group, a2d.device)
    da, db = ca.desc(), cb.desc()
    y = torch.empty((M, H), dtype=BF16, device=a2d.device)
    check(_abi.load().hyc_hadamard_fwd_compress(_p(a2d), a2d.stride(0) if M > 1 else H, _p(b2d), b2d.stride(0) if M > 1 else H,
                                                M, H, ctypes.byref(da), ctypes.byref(db), _p(y), _p(ca.stored), _p(ca.vals),
                                                _p(ca.scales), _p(cb.stored), _p(cb.vals), _p(cb.scales), _stream()))
    return y, ca, cb


def gated_act_fwd_supported(H, bits, group):
    """shapes the one-pass forward covers (the rest takes the activation, three compress calls and a product)"""
    if bits not in (2, 4, 8) or group not in (64, 128) or H % (64 // bits) != 0:
        return False
    chunks, most, lpg = H * bits // 64, 512 if bits == 2 else 768, group // 8
    # one workgroup per row, or 2 to 4 workgroups (whole scale groups each) for rows of up to 1024 chunks
    return chunks <= most or (chunks <= 1024 and any(chunks % n == 0 and (chunks // n) % lpg == 0 and
                                                     -(-(chunks // n) // 64) * 64 <= most for n in (2, 3, 4)))


def gated_act_fwd(act, gate2d, up2d, plan_act, plan_up, plan_gate, bits, group):
    """h = act(gate) * up and the compressed act(gate), up, gate in one pass -> (h, c_act, c_up, c_gate).
    gate and up are bf16 [M, H] matrices with contiguous rows (column slices of one projection output are fine);
    the plans are the outlier-channel sets of the three sites."""
    _need_rows(gate2d, "gate")
    _need_rows(up2d, "up")
    if gate2d.shape != up2d.shape:
        raise ValueError("gate %s and up %s differ in shape" % (tuple(gate2d.shape), tuple(up2d.shape)))
    M, H = gate2d.shape
    dev = gate2d.device
    outs = [alloc_channel(M, H, p, bits, group, dev) for p in (plan_act, plan_up, plan_gate)]
    descs = [o.desc() for o in outs]
    h = torch.empty((M, H), dtype=BF16, device=dev)
    code = {"silu": _abi.ACT_SILU, "gelu": _abi.ACT_GELU_TANH}[act]
    flat = []
    for o in outs:
        flat += [_p(o.stored), _p(o.vals), _p(o.scales)]
    check(_abi.load().hyc_gated_act_fwd(code, _p(gate2d), gate2d.stride(0) if M > 1 else H, _p(up2d),
                                        up2d.stride(0) if M > 1 else H, M, H, ctypes.byref(descs[0]), ctypes.byref(descs[1]),
                                        ctypes.byref(descs[2]), _p(h), *flat, _stream()))
    return (h,) + tuple(outs)


# ----------------------------------------------------------------------------------------------------
# weight gradient
# ----------------------------------------------------------------------------------------------------
STAGED_GRADW_MIN_TILES = 96


def gradw_staged_by_default(N_out, H):
    """whether dW [N_out, H] from a channel-compressed activation restores x_hat first.  Every 256 output features
    decode the same activation tile again (about a fifth on top of the dense product's time), against one pass that
    writes x_hat and its second read.  Measured at 4096 and 16 384 tokens, H = 4096 and 11008, N_out = 256 ... 4096:
    the staged route wins from 96 output tiles of 256 x 256 on (N_out >= 1536 at H = 4096, >= 768 at H = 11008)."""
    return -(-N_out // 256) * (H // 256) >= STAGED_GRADW_MIN_TILES


def gradw_gemm(dy2d, src, out_dtype=BF16, alpha=1.0, out=None, beta=0.0, staged=None):
    """dW [N_out, H] = alpha * dy^T @ x_hat (+ beta * out); src as for rmsnorm_bwd.

    A compressed src is decoded inside the GEMM, or (`staged`; None = by `gradw_staged_by_default`, never for the
    few output features LoRA training has) restored once into a transient matrix for the same kernel's dense form."""
    _need_rows(dy2d, "grad_output")                # rows may be a column slice of a wider matrix (pitch = stride(0))
    M, N_out = dy2d.shape
    H = src.H if isinstance(src, (ChannelCompressed, ThresholdCompressed)) else src.shape[-1]
    if staged is None:
        staged = gradw_staged_by_default(N_out, H)
    if staged and isinstance(src, ChannelCompressed):
        src = decompress_channel(src)
    stored, vals, scales, d = _source(src, M, H)
    lib = _abi.load()
    if out is None:
        out = torch.empty((N_out, H), dtype=out_dtype, device=dy2d.device)
    elif (not out.is_cuda or not out.is_contiguous() or tuple(out.shape) != (N_out, H)
          or out.dtype not in (BF16, torch.float32)):
        raise ValueError("out must be a contiguous bf16 or fp32 [%d, %d] CUDA tensor" % (N_out, H))
    ws_bytes = lib.hyc_gradw_workspace_bytes(M, N_out, H)
    ws = torch.empty(ws_bytes // 4, dtype=torch.float32, device=dy2d.device) if ws_bytes else None
    code = _abi.DTYPE_F32 if out.dtype == torch.float32 else _abi.DTYPE_BF16
    check(lib.hyc_gradw_gemm(_p(dy2d), dy2d.stride(0) if M > 1 else N_out, _p(stored), _p(vals), _p(scales), M, N_out, H, ctypes.byref(d),
                             float(alpha), float(beta), _p(out), code, _p(ws), _stream()))
    return out


# ----------------------------------------------------------------------------------------------------
# softmax
# ----------------------------------------------------------------------------------------------------
@dataclass
class SparseRows:
    """probabilities above the threshold, CSR over the flattened leading dims"""
    row_ptr: torch.Tensor   # int32 [rows+1]
    cols: torch.Tensor      # int32 [nnz] (or the capacity a KeptBudget provided: row_ptr says what is in use)
    vals: torch.Tensor      # bf16 [nnz]
    shape: tuple
    total: Optional[torch.Tensor] = None   # int64 0-d on the device: the entries above the threshold (> cols.numel(): some were dropped)

    @property
    def rows(self):
        return self.row_ptr.numel() - 1


def _csr_from_counts(lib, y2d, threshold, counts, budget=None):
    rows, N = y2d.shape
    dev = y2d.device
    row_ptr, nnz, total = _csr_offsets(lib, counts, rows, budget)
    cols = torch.empty(nnz, dtype=torch.int32, device=dev)
    vals = torch.empty(nnz, dtype=BF16, device=dev)
    check(lib.hyc_softmax_fill(_p(y2d), rows, N, float(threshold), _p(row_ptr), _p(cols) if nnz else None,
                               _p(vals) if nnz else None, _stream()))
    return row_ptr, cols, vals, total


def softmax_fwd(x, threshold=None, causal_period=None, inplace=False, budget=None):
    """y = softmax(x, -1) bf16; with a threshold also the kept entries (y > bf16(threshold)) as SparseRows.
    budget: the site's KeptBudget (see there): once it has seen a call, the kept entries are sized ahead of time and the
    call returns without waiting for the GPU.
    causal_period = S applies the causal mask of S query positions inside the kernel (row r is position r % S).
    inplace: y overwrites x (rows of at most 4096 entries: a row is held in registers before anything is written)."""
    _need(x, BF16, "x")
    N = x.shape[-1]
    x2 = x.reshape(-1, N)
    rows = x2.shape[0]
    lib = _abi.load()
    if inplace and N > 4096:
        raise ValueError("in-place softmax needs rows of at most 4096 entries")
    y = x2 if inplace else torch.empty_like(x2)
    counts = None if threshold is None else torch.empty(rows, dtype=torch.int32, device=x.device)
    thr = 0.0 if threshold is None else float(threshold)
    if causal_period is None:
        check(lib.hyc_softmax_fwd(_p(x2), rows, N, thr, _p(y), _p(counts), _stream()))
    else:
        check(lib.hyc_softmax_causal_fwd(_p(x2), rows, N, int(causal_period), thr, _p(y), _p(counts), _stream()))
    if threshold is None:
        return y.reshape(x.shape), None
    row_ptr, cols, vals, total = _csr_from_counts(lib, y, threshold, counts, budget)
    return y.reshape(x.shape), SparseRows(row_ptr, cols, vals, tuple(x.shape), total)


def softmax_sparsify(y, threshold, budget=None):
    """kept entries of already computed probabilities (budget: as for softmax_fwd)"""
    _need(y, BF16, "y")
    N = y.shape[-1]
    y2 = y.reshape(-1, N)
    lib = _abi.load()
    counts = torch.empty(y2.shape[0], dtype=torch.int32, device=y.device)
    check(lib.hyc_softmax_fwd(None, y2.shape[0], N, float(threshold), _p(y2), _p(counts), _stream()))
    row_ptr, cols, vals, total = _csr_from_counts(lib, y2, threshold, counts, budget)
    return SparseRows(row_ptr, cols, vals, tuple(y.shape), total)


def softmax_bwd(g, sp: SparseRows, inplace=False):
    """dx = (g - sum(g * p_hat)) * p_hat; with inplace, dx overwrites g"""
    _need(g, BF16, "grad_output")
    N = g.shape[-1]
    g2 = g.reshape(-1, N)
    if sp.rows != g2.shape[0] or sp.shape[-1] != N:
        raise ValueError("the kept probabilities are %s, the gradient is %s" % (tuple(sp.shape), tuple(g.shape)))
    dx = g2 if inplace else torch.empty_like(g2)
    check(_abi.load().hyc_softmax_bwd(_p(g2), g2.shape[0], N, _p(sp.row_ptr), _p(sp.cols) if sp.cols.numel() else None,
                                      _p(sp.vals) if sp.vals.numel() else None, _p(dx), _stream()))
    return dx.reshape(g.shape)


def softmax_dense(sp: SparseRows):
    N = sp.shape[-1]
    out = torch.empty((sp.rows, N), dtype=BF16, device=sp.row_ptr.device)
    check(_abi.load().hyc_softmax_dense(sp.rows, N, _p(sp.row_ptr), _p(sp.cols) if sp.cols.numel() else None,
                                        _p(sp.vals) if sp.vals.numel() else None, _p(out), _stream()))
    return out.reshape(sp.shape)


def sparse_rows_to_coo(sp: SparseRows):
    """the sparse COO tensor `.to_sparse()` gives for the pruned probabilities (int64 indices, row-major)"""
    counts = (sp.row_ptr[1:] - sp.row_ptr[:-1]).long()
    rows = torch.repeat_interleave(torch.arange(sp.rows, device=counts.device), counts)
    lead = []
    for dim in reversed(sp.shape[:-1]):
        lead.append(rows % dim)
        rows = rows // dim
    idx = torch.stack(list(reversed(lead)) + [sp.cols.long()])
    return torch.sparse_coo_tensor(idx, sp.vals, sp.shape, is_coalesced=True)


def coo_to_sparse_rows(coo):
    coo = coo.coalesce()
    shape = tuple(coo.shape)
    idx = coo.indices()
    rows = torch.zeros_like(idx[0])
    for i, dim in enumerate(shape[:-1]):
        rows = rows * dim + idx[i]
    n_rows = 1
    for dim in shape[:-1]:
        n_rows *= dim
    row_ptr = torch.zeros(n_rows + 1, dtype=torch.int32, device=idx.device)
    if rows.numel():
        torch.cumsum(torch.bincount(rows, minlength=n_rows), 0, out=row_ptr[1:])
    return SparseRows(row_ptr, idx[-1].to(torch.int32).contiguous(), coo.values().to(BF16).contiguous(), shape)


def softmax_sparse_coo(y, threshold):
    return sparse_rows_to_coo(softmax_sparsify(y, threshold))


def sparse_coo_to_dense(coo):
    return softmax_dense(coo_to_sparse_rows(coo))


def softmax_prune(y, threshold):
    """y * (y > threshold) as a dense tensor (the reference's prune_softmax; not used by the softmax operator)"""
    return softmax_dense(softmax_sparsify(y, threshold))


# ----------------------------------------------------------------------------------------------------
# low-rank base
# ----------------------------------------------------------------------------------------------------
def low_rank_update(l, r, x, subtract, out=None):
    """out = bf16(x -/+ l @ r), x [B,S,H] (or [S,H]); in place when out is x"""
    _need(x, BF16, "x")
    _need(l, BF16, "l")
    _need(r, BF16, "r")
    S, H = x.shape[-2], x.shape[-1]
    M = x.numel() // H
    if l.shape[0] != S or r.shape[0] != l.shape[1] or r.shape[1] != H:
        raise ValueError("Incompatible dimensions")
    if out is None:
        out = torch.empty_like(x)
    elif _need(out, BF16, "out").shape != x.shape:
        raise ValueError("out must have x's shape")
    check(_abi.load().hyc_low_rank_update(_p(l), _p(r), _p(x), _p(out), M, S, H, l.shape[1], 1 if subtract else 0, _stream()))
    return out


# ----------------------------------------------------------------------------------------------------
# NF4 frozen base weights
# ----------------------------------------------------------------------------------------------------
@dataclass
class NF4Weight:
    """a frozen [out, in] bf16 weight held as 4-bit level indices + one fp32 abs-max per 64 consecutive weights"""
    packed: torch.Tensor   # uint8 [out*in/2]
    absmax: torch.Tensor   # fp32 [out*in/64]
    shape: tuple

    def nbytes(self):
        return self.packed.numel() + 4 * self.absmax.numel()


def nf4_quantize(w):
    _need(w, BF16, "w")
    n = w.numel()
    if n % 64:
        raise ValueError("NF4 blocks hold 64 weights: %d is not a multiple of 64" % n)
    packed = torch.empty(n // 2, dtype=torch.uint8, device=w.device)
    absmax = torch.empty(n // 64, dtype=torch.float32, device=w.device)
    check(_abi.load().hyc_nf4_quantize(_p(w), n, _p(packed), _p(absmax), _stream()))
    return NF4Weight(packed, absmax, tuple(w.shape))


def nf4_dequantize(q: NF4Weight, out=None):
    n = q.packed.numel() * 2
    if out is None:
        out = torch.empty(q.shape, dtype=BF16, device=q.packed.device)
    elif _need(out, BF16, "out").numel() != n:
        raise ValueError("out must hold %d weights" % n)
    check(_abi.load().hyc_nf4_dequantize(_p(q.packed), _p(q.absmax), n, _p(out), _stream()))
    return out


# ----------------------------------------------------------------------------------------------------
# rotary embedding + attention layout
# ----------------------------------------------------------------------------------------------------
def _need_tables(cos, sin, S, hd):
    if (cos is None) != (sin is None):
        raise ValueError("cos and sin go together")
    if cos is not None:
        _need_vec(cos, BF16, S * hd, "cos")
        _need_vec(sin, BF16, S * hd, "sin")


def rope_to_heads(x, heads, cos=None, sin=None, want_rows=False):
    """x bf16 [B, S, heads*hd] -> rotated [B, heads, S, hd] contiguous (and, with want_rows, also [B, S, heads*hd]);
    cos / sin bf16 [S, hd]; without them only the layout changes.  x may be a column slice of a wider [B, S, *]
    tensor (tokens a fixed pitch apart)."""
    if not isinstance(x, torch.Tensor) or not x.is_cuda or x.dtype != BF16 or x.dim() != 3:
        raise ValueError("x must be a bfloat16 [B, S, H] tensor on the GPU")
    B, S, H = x.shape
    pitch = x.stride(1) if S > 1 else H
    if x.stride(2) != 1 or (B > 1 and x.stride(0) != S * pitch):
        raise ValueError("x must have contiguous channels and evenly spaced tokens")
    if heads <= 0 or H % heads:
        raise ValueError("%d channels do not split into %d heads" % (H, heads))
    hd = H // heads
    _need_tables(cos, sin, S, hd)
    out_heads = torch.empty((B, heads, S, hd), dtype=BF16, device=x.device)
    out_rows = torch.empty((B, S, H), dtype=BF16, device=x.device) if want_rows else None
    check(_abi.load().hyc_rope_to_heads(_p(x), pitch, _p(cos), _p(sin), B, S, heads, hd, _p(out_heads), _p(out_rows),
                                        _stream()))
    return (out_heads, out_rows) if want_rows else out_heads


def rope_from_heads(g, cos=None, sin=None):
    """gradient bf16 [B, heads, S, hd] -> [B, S, heads*hd] through the transposed rotation"""
    _need(g, BF16, "g")
    B, heads, S, hd = g.shape
    _need_tables(cos, sin, S, hd)
    out = torch.empty((B, S, heads * hd), dtype=BF16, device=g.device)
    check(_abi.load().hyc_rope_from_heads(_p(g), _p(cos), _p(sin), B, S, heads, hd, _p(out), _stream()))
    return out


# ----------------------------------------------------------------------------------------------------
# seeded dropout
# ----------------------------------------------------------------------------------------------------
def dropout(x, p, seed, backward=False):
    """forward: keep ? x / (1 - p) : 0; backward: keep ? x : 0; keep is a pure function of (seed, element index)"""
    _need(x, BF16, "x")
    out = torch.empty_like(x)
    check(_abi.load().hyc_dropout(_p(x), _p(out), x.numel(), float(p), int(seed) & 0xFFFFFFFFFFFFFFFF,
                                  1 if backward else 0, _stream()))
    return out
