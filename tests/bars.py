"""The bar a softmax gradient is held to in the GPU tests (shared by several test files)."""
import torch

TOL = {torch.bfloat16: 2e-3, torch.float16: 1e-3}  # north_star: |err| against an fp32 computation


def assert_grad(dx, auto, dtype, what=None, absolute=False, y=None, g=None, scale=None):
    """A gradient against fp32 autograd of the unfused path from x.  At every BASELINE shape
    (`absolute`) the bar is north_star's absolute one.  In general it is that bar plus what
    storing the probabilities and the result in the 16-bit type costs: the kernels (like the
    reference's) work from the probabilities y as they were stored, each off by up to half a
    unit in the last place, relative -- dx_j = scale * y_j * (g_j - sum_k g_k y_k) inherits that
    through y_j (half a unit of |dx_j|) and through the sum (at most half a unit of
    |scale| * y_j * max|g|) -- and the result is rounded to the type once more (half a unit of
    |dx_j|).  The allowance is one unit of |dx_j| + |scale| * y_j * max|g| per element."""
    err = (dx.float() - auto.float()).abs()
    if absolute:
        assert err.max().item() <= TOL[dtype], (what, err.max().item())
        return
    ulp = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11
    size = auto.float().abs()
    if y is not None:
        size = size + abs(1.0 if scale is None else scale) * y.float() * g.float().abs().amax(-1, keepdim=True)
    ok = err <= TOL[dtype] + ulp * size
    assert ok.all(), (what, err.max().item(), (err - ulp * size).max().item())
