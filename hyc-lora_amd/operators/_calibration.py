"""Calibration protocol shared by every operator module (reference: the block after Function.apply in each
module, e.g. operators/efficient_silu.py:86-111 or operators/efficient_rmsnorm.py:312-337).

Reference scheme ("ref" mode): `iteration` counts the calls; the first two calls compute fresh statistics
(threshold, L, scale, R), compress with them, and fold them into the running mean
`static = (iteration*static + fresh) / (iteration+1)`; from the third call on the stored values are used.
`static_value` keeps the reference's order [threshold, L, scale, R].  Like in the reference these are plain
Python attributes, not buffers; `calibration_state` / `load_calibration_state` carry them across a restart.

Channel scheme ("hyc" mode): the state is the running per-channel abs-max (elementwise max over the first two
calls) and the outlier-channel plan selected from it; frozen from the third call on.
"""
import torch

from .. import kernels as K
from .compress_function import pad_cut_L

MODES = ("ref", "hyc")


def running_mean(previous, fresh, iteration):
    """mean over the calibration calls so far: `fresh` on the first call, (iteration*previous + fresh)/(iteration+1) after"""
    if previous is None:
        return fresh
    return (iteration * previous + fresh) / (iteration + 1)


def fold_statistics(static_value, iteration, outlier, L, scale, R):
    """one step of the running mean over the calibration calls; returns the new list"""
    fresh = [outlier, L, scale, R]
    out = list(static_value)
    for slot in range(4):
        new = fresh[slot]
        if out[slot] is None:
            out[slot] = new
        else:
            if slot == 1:
                new = pad_cut_L(new, out[slot])
            out[slot] = (iteration * out[slot] + new) / (iteration + 1)
    return out


class CompressionSite:
    """per-activation state: the reference's (iteration, static_value) pair plus the channel-mode plan"""

    def __init__(self, outlier_ratio, sub_outlier_ratio, sub_outlier_bit, sub_outlier_quantize_method, rank,
                 mode="ref", group_size=128, scale_rule=K.DEFAULT_SCALE_RULE):
        if mode not in MODES:
            raise ValueError("mode must be 'ref' or 'hyc', got %r" % (mode,))
        if scale_rule not in K.SCALE_RULES:
            raise ValueError("scale_rule must be 'absmax' or 'range', got %r" % (scale_rule,))
        self.outlier_ratio = outlier_ratio
        self.sub_outlier_ratio = sub_outlier_ratio
        self.sub_outlier_bit = sub_outlier_bit
        self.sub_outlier_quantize_method = sub_outlier_quantize_method
        self.rank = rank
        self.mode = mode
        self.group_size = group_size
        self.scale_rule = scale_rule   # hyc mode: how the (token, group) scales are formed, see kernels.ChannelPlan
        self.amax = None     # hyc mode: running channel abs-max (fp32 [H])
        self.plan = None     # hyc mode: ChannelPlan

    # -- channel mode ---------------------------------------------------------------------------------
    def channel_plan(self, x2d, iteration):
        """the plan to compress this call with; calibrates during the first two calls"""
        if iteration < 2 or self.plan is None:
            self.amax = K.channel_absmax(x2d, self.amax)
            k = K.num_outlier_channels(x2d.shape[-1], self.outlier_ratio)
            self.plan = K.select_channels(self.amax, k, self.scale_rule)
        return self.plan


def as_rows(x):
    """[..., H] -> contiguous [M, H] view plus the tokens-per-batch-element S the static scale is indexed by"""
    H = x.shape[-1]
    S = x.shape[-2] if x.dim() >= 2 else 1
    return x.contiguous().reshape(-1, H), S


# ---- persistence ------------------------------------------------------------------------------------------
# The reference keeps `iteration` / `static_value` as plain attributes (efficient_rmsnorm.py:293-294), so a resumed
# run calibrates again on whatever two batches come first.  These two functions carry the state across a restart
# without touching `state_dict()` (checkpoints stay loadable by code that knows nothing about it).
def _site_state(site):
    if site.plan is None:
        return None
    return {"amax": site.amax, "H": site.plan.H, "k": site.plan.k, "idx": site.plan.idx, "plan": site.plan.plan,
            "scale_rule": site.plan.scale_rule}


def calibration_state(model):
    """{qualified module name: state} for every memory-efficient module below `model` (tensors stay where they are;
    the result can be handed to torch.save)"""
    out = {}
    for name, mod in model.named_modules():
        if not hasattr(mod, "iteration") or not any("static_value" in k or isinstance(v, CompressionSite)
                                                    for k, v in vars(mod).items()):
            continue
        entry = {"iteration": int(mod.iteration)}
        for key, val in vars(mod).items():
            if "static_value" in key:
                entry[key] = list(val) if isinstance(val, (list, tuple)) else val
            elif isinstance(val, CompressionSite):
                entry[key] = _site_state(val)
        out[name] = entry
    return out


def load_calibration_state(model, state, strict=True, device=None):
    """inverse of calibration_state.  Every tensor of the state is moved to `device`; by default that is the device
    of the module's parameters or, for the modules that have none (activations, products, GEMMs), the current GPU:
    the kernels read the outlier-channel plans and static scales through raw device pointers, so a state that was
    loaded with map_location="cpu" must not stay on the host.  Returns the names in `state` that matched no module."""
    modules = dict(model.named_modules())
    unknown = []
    for name, entry in state.items():
        mod = modules.get(name)
        if mod is None or not hasattr(mod, "iteration"):
            unknown.append(name)
            continue
        target = device
        if target is None:
            param = next(mod.parameters(), None)
            if param is not None and param.is_cuda:
                target = param.device
            elif torch.cuda.is_available():
                target = torch.device("cuda", torch.cuda.current_device())
        if target is None:
            raise ValueError("load_calibration_state: module %s has no GPU parameters and no GPU is available; "
                             "pass device=" % name)

        def place(t):
            return t.to(target) if isinstance(t, torch.Tensor) else t

        for key, val in entry.items():
            if key == "iteration":
                mod.iteration = int(val)
            elif "static_value" in key:
                setattr(mod, key, [place(v) for v in val] if isinstance(val, (list, tuple)) else place(val))
            else:
                site = getattr(mod, key)
                if val is None:
                    site.amax, site.plan = None, None
                else:
                    site.amax = place(val["amax"])
                    # states written before the scale rule existed used the range rule
                    site.plan = K.ChannelPlan(val["H"], val["k"], place(val["idx"]).to(torch.int32).contiguous(),
                                              place(val["plan"]).to(torch.int32).contiguous(),
                                              val.get("scale_rule", "range"))
                    # a site that is still calibrating plans again on its next call: with the rule it was saved with
                    site.scale_rule = site.plan.scale_rule
    if strict and unknown:
        raise KeyError("no memory-efficient module named %s" % ", ".join(unknown))
    return unknown
