"""torchsso.utils.inv / torchsso.utils.cholesky on the HIP engine.

Stand in for the reference's CuPy/cuSOLVER calls: inv = potrf + potrs against
the identity (torchsso/utils/inv_cupy.py:27-34,114-128), cholesky =
cupy.linalg.cholesky transposed (torchsso/utils/cholesky_cupy.py:9-14).
"""
from torchsso import _ops


def inv(m):
    """Inverse of a symmetric positive definite matrix (new tensor)."""
    outs, _ = _ops.damped_inverse_batched([m.detach().contiguous()])
    return outs[0]


def cholesky(m, upper=True):
    """U (upper=True) with m = U^T U, or its transpose L with m = L L^T."""
    outs, _ = _ops.cholesky_upper_batched([m.detach().contiguous()])
    u = outs[0]
    return u if upper else u.t().contiguous()
