"""Batch-norm kernels (csrc/batchnorm.hip) through the C-ABI wrappers and the
``cxgnncomp.BatchNorm1d`` module against the float64 oracle (oracle/pyref.py,
pinned to torch's batch_norm on the CPU).  Tolerance: 1e-4 relative / 2e-5 absolute on the
normalised values and 1e-4 of the largest |dx|, both widened per column by what one fp32
rounding of the column mean is worth in units of the standard deviation (|mean| * 2^-22 /
std: no fp32 batch norm can do better on a column whose mean is far from zero);
statistics 1e-5 relative to the column's standard deviation."""
import numpy as np
import pytest
import torch

from conftest import announce
from oracle import pyref

pytestmark = pytest.mark.gpu

SHAPES = [(1000, 256), (4097, 64), (169343, 256), (3, 8), (2, 1), (513, 7), (70001, 47), (257, 1500), (100, 1028)]


def _data(n, c, seed=0):
    g = torch.Generator().manual_seed(seed)
    scale = torch.rand(c, generator=g) * 20 + 0.05
    shift = torch.randn(c, generator=g) * 100         # means far from zero: one-pass sums of squares would cancel
    x = torch.randn(n, c, generator=g) * scale + shift
    dy = torch.randn(n, c, generator=g)
    gamma = torch.rand(c, generator=g) + 0.5
    beta = torch.randn(c, generator=g)
    return x, dy, gamma, beta


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("relu", [False, True])
@pytest.mark.parametrize("affine", [True, False])
def test_batchnorm_kernels_against_oracle(shape, relu, affine):
    from cxgnncomp_backend import _ops
    n, c = shape
    x, dy, gamma, beta = _data(n, c)
    if not affine:
        gamma = beta = None
    eps = 1e-5
    announce("batchnorm n=%d c=%d relu=%s affine=%s" % (n, c, relu, affine))
    xc, dyc = x.cuda(), dy.cuda()
    gc = gamma.cuda() if affine else None
    bc = beta.cuda() if affine else None
    mean, invstd, var_unbiased = _ops.batchnorm_stats(xc, eps)
    y = _ops.batchnorm_apply(xc, mean, invstd, gc, bc, relu)
    dx, dgamma, dbeta = _ops.batchnorm_bwd(xc, dyc, mean, invstd, gc, bc, relu)
    torch.cuda.synchronize()
    ry, rmean, rvar, rvar_unbiased = pyref.batchnorm_fwd(x.numpy(), None if gamma is None else gamma.numpy(),
                                                         None if beta is None else beta.numpy(), eps, relu)
    std = np.sqrt(rvar + eps)
    assert np.all(np.abs(mean.cpu().numpy() - rmean) <= 1e-5 * std + 1e-6 * np.abs(rmean))
    assert np.allclose(1.0 / invstd.cpu().numpy().astype(np.float64), std, rtol=2e-5)
    assert np.allclose(var_unbiased.cpu().numpy(), rvar_unbiased, rtol=4e-5, atol=1e-9)
    g_abs = np.ones(c) if gamma is None else np.abs(gamma.numpy())
    col_tol = 2e-5 + 2.0 ** -22 * np.abs(rmean) / std * g_abs          # rounding of the fp32 mean, in output units
    assert np.all(np.abs(y.cpu().numpy() - ry) <= col_tol + 1e-4 * np.abs(ry))
    active = None
    if relu:
        # forward values within rounding of zero may fall on either side of the ReLU: the oracle
        # takes the side the kernels took there, and everywhere else the sides must agree
        ry_lin = pyref.batchnorm_fwd(x.numpy(), None if gamma is None else gamma.numpy(),
                                     None if beta is None else beta.numpy(), eps, False)[0]
        active = y.cpu().numpy() > 0
        clear = np.abs(ry_lin) > 4 * (col_tol + 1e-4 * np.abs(ry_lin))
        assert np.array_equal(active[clear], (ry_lin > 0)[clear])
    rdx, rdgamma, rdbeta = pyref.batchnorm_bwd(x.numpy(), dy.numpy(), None if gamma is None else gamma.numpy(),
                                               None if beta is None else beta.numpy(), eps, relu, active)
    mean_err = 2.0 ** -22 * np.abs(rmean) / std                          # error of xhat from the fp32 mean
    scale_dx = np.abs(rdx).max(axis=0) + 1e-30
    assert np.all(np.abs(dx.cpu().numpy() - rdx) <= (1e-4 + 4 * mean_err) * scale_dx + 1e-6)
    sum_scale = np.sqrt(n)
    assert np.all(np.abs(dgamma.cpu().numpy() - rdgamma) <= 1e-4 * np.abs(rdgamma) + (2e-5 + mean_err) * sum_scale * 4)
    assert np.allclose(dbeta.cpu().numpy(), rdbeta, rtol=1e-4, atol=2e-5 * sum_scale)
    # reproducible bit for bit
    m2, i2, v2 = _ops.batchnorm_stats(xc, eps)
    dx2, dg2, db2 = _ops.batchnorm_bwd(xc, dyc, mean, invstd, gc, bc, relu)
    assert torch.equal(mean, m2) and torch.equal(invstd, i2) and torch.equal(dx, dx2) and torch.equal(dgamma, dg2)


@pytest.mark.parametrize("relu", [False, True])
def test_batchnorm_module_matches_torch_module(relu):
    """Same parameters, buffers and state dict as torch.nn.BatchNorm1d; training step,
    running statistics, evaluation mode and the fallbacks."""
    import cxgnncomp
    torch.manual_seed(0)
    n, c = 5000, 96
    x = (torch.randn(n, c) * 3 + 7).cuda()
    ours = cxgnncomp.BatchNorm1d(c).cuda()
    ref = torch.nn.BatchNorm1d(c).cuda()
    with torch.no_grad():
        ours.weight.uniform_(0.5, 1.5)
        ours.bias.normal_()
    ref.load_state_dict(ours.state_dict())
    announce("BatchNorm1d module relu=%s" % relu)
    for step in range(3):
        xa = (x + step).clone().requires_grad_(True)
        xb = (x + step).clone().requires_grad_(True)
        ya = ours(xa, relu=relu)
        yb = ref(xb)
        if relu:
            yb = torch.relu(yb)
        g = torch.randn_like(ya)
        ya.backward(g)
        yb.backward(g)
        assert torch.allclose(ya, yb, rtol=1e-4, atol=2e-5)
        assert torch.allclose(xa.grad, xb.grad, rtol=1e-3, atol=1e-5 * float(xb.grad.abs().max()) + 1e-7)
    assert torch.allclose(ours.weight.grad, ref.weight.grad, rtol=1e-3, atol=1e-3)
    assert torch.allclose(ours.bias.grad, ref.bias.grad, rtol=1e-3, atol=1e-3)
    assert torch.allclose(ours.running_mean, ref.running_mean, rtol=1e-5, atol=1e-6)
    assert torch.allclose(ours.running_var, ref.running_var, rtol=1e-4)
    assert int(ours.num_batches_tracked) == int(ref.num_batches_tracked) == 3
    ours.eval()
    ref.eval()
    with torch.no_grad():
        ya = ours(x, relu=relu)
        yb = torch.relu(ref(x)) if relu else ref(x)
    assert torch.allclose(ya, yb, rtol=1e-4, atol=2e-5)
    ours.train()
    with pytest.raises(ValueError):
        ours(x[:1])
    # inputs the kernels do not take go through torch's path
    x3 = torch.randn(4, c, 5).cuda()
    assert torch.allclose(ours(x3), torch.nn.functional.batch_norm(x3, None, None, ours.weight, ours.bias, True),
                          rtol=1e-4, atol=1e-5)
    assert ours.state_dict().keys() == ref.state_dict().keys()


@pytest.mark.parametrize("shape", SHAPES + [(0, 12)])
def test_column_sum_against_float64(shape):
    from cxgnncomp_backend import _ops
    n, c = shape
    g = torch.Generator().manual_seed(1)
    x = torch.randn(n, c, generator=g) * 3 + 0.5
    announce("column_sum n=%d c=%d" % (n, c))
    xc = x.cuda()
    got = _ops.column_sum(xc)
    want = x.double().sum(dim=0).numpy()
    scale = np.sqrt(max(n, 1)) * 3
    assert np.all(np.abs(got.cpu().numpy() - want) <= 1e-4 * np.abs(want) + 1e-5 * scale)
    assert torch.equal(got, _ops.column_sum(xc))
