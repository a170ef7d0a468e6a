"""x -/+ L @ R in one pass.  Reference: operators/fused_compression.py:80-99 (low_rank_extraction, in place) and
:184-210 (low_rank_addition, returns a new tensor)."""
from .. import kernels as K


def low_rank_extraction(l, r, x):
    """x[b] -= l @ r, in place; l [s, r], r [r, d], x [b, s, d] bf16"""
    assert l.shape[1] == r.shape[0], "Incompatible dimensions"
    assert l.is_contiguous(), "Matrix A must be contiguous"
    assert r.is_contiguous(), "Matrix B must be contiguous"
    K.low_rank_update(l, r, x, subtract=True, out=x)
    return x


def low_rank_addition(l, r, x):
    """o[b] = x[b] + l @ r"""
    assert l.shape[1] == r.shape[0], "Incompatible dimensions"
    assert l.is_contiguous(), "Matrix A must be contiguous"
    assert r.is_contiguous(), "Matrix B must be contiguous"
    return K.low_rank_update(l, r, x, subtract=False)
