"""The CPU component hooks (`trigrad_amd.barycentric`, `interpolate3_scalar`,
`interpolate3_vector`), modelled on reference tests/test_components.py: random
inputs in the same ranges (seeded here), backward checked against derivatives.

The reference gradchecks a float64 build; this build is float32, so the analytic
backward is compared (a) bit for bit with the oracle's float32 restatement of
util.h and (b) with float64 autograd of the textbook formula at float32 accuracy.
"""
import numpy as np
import pytest
import torch

import trigrad_amd

RNG = np.random.default_rng(2024)


def uniform(shape, lo=-5, hi=5):
    return torch.from_numpy(RNG.uniform(lo, hi, size=shape).astype(np.float32))


CASES_I = [(uniform(3, 0, 1), [uniform(1) for _ in range(3)], uniform(3, 0.2, 5)) for _ in range(40)]
CASES_V = [(uniform(3, 0, 1), [uniform(3) for _ in range(3)], uniform(3, 0.2, 5)) for _ in range(40)]
CASES_B = [[uniform(2) for _ in range(4)] for _ in range(40)]


def _rel(a, b, tol):
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    scale = max(1.0, float(np.abs(b).max()))
    assert np.abs(a - b).max() <= tol * scale, (a, b)


@pytest.mark.parametrize("bary,values,w", CASES_I)
def test_interpolate3_scalar(bary, values, w, oracle):
    bary = (bary / bary.sum()).clone().requires_grad_()
    a, b, c = (v.clone().requires_grad_() for v in values)
    w = w.clone().requires_grad_()
    out = trigrad_amd.interpolate3_scalar(bary, a, b, c, w)
    g = torch.tensor([1.7])
    out.backward(g)
    bn, wn = bary.detach().numpy(), w.detach().numpy()
    assert out.item() == oracle.interpolate3_scalar(bn, a.item(), b.item(), c.item(), wn)
    gb, gv, gw = oracle.interpolate3_scalar_backward(np.float32(1.7), bn, a.item(), b.item(), c.item(), wn)
    np.testing.assert_array_equal(bary.grad.numpy(), gb)
    np.testing.assert_array_equal(np.array([a.grad.item(), b.grad.item(), c.grad.item()], np.float32), gv)
    np.testing.assert_array_equal(w.grad.numpy(), gw)
    b64, w64 = bary.detach().double().requires_grad_(), w.detach().double().requires_grad_()
    v64 = torch.stack([a, b, c]).detach().double().reshape(3).requires_grad_()
    ref = (b64 * w64 * v64).sum() / (b64 * w64).sum()
    ref.backward(torch.tensor(1.7, dtype=torch.float64))
    _rel(out.item(), ref.item(), 1e-5)
    _rel(bary.grad, b64.grad, 2e-4)
    _rel(w.grad, w64.grad, 2e-4)
    _rel([a.grad.item(), b.grad.item(), c.grad.item()], v64.grad, 2e-5)


@pytest.mark.parametrize("bary,values,w", CASES_V)
def test_interpolate3_vector(bary, values, w, oracle):
    bary = (bary / bary.sum()).clone().requires_grad_()
    a, b, c = (v.clone().requires_grad_() for v in values)
    w = w.clone().requires_grad_()
    out = trigrad_amd.interpolate3_vector(bary, a, b, c, w)
    g = torch.tensor([0.3, -1.1, 2.0])
    out.backward(g)
    args = [t.detach().numpy() for t in (bary, a, b, c, w)]
    np.testing.assert_array_equal(out.detach().numpy(), oracle.interpolate3_vector(*args))
    want = oracle.interpolate3_vector_backward(g.numpy(), *args)
    for got, w_ in zip((bary.grad, a.grad, b.grad, c.grad, w.grad), want):
        np.testing.assert_array_equal(got.numpy(), w_)
    d = [t.detach().double().requires_grad_() for t in (bary, a, b, c, w)]
    ref = (d[0][0] * d[4][0] * d[1] + d[0][1] * d[4][1] * d[2] + d[0][2] * d[4][2] * d[3]) / (d[0] * d[4]).sum()
    (ref * g.double()).sum().backward()
    _rel(out.detach(), ref.detach(), 1e-5)
    for got, t in zip((bary.grad, a.grad, b.grad, c.grad, w.grad), d):
        _rel(got, t.grad, 3e-4)


@pytest.mark.parametrize("points", CASES_B)
def test_barycentric(points, oracle):
    pts = [p.clone().requires_grad_() for p in points]
    out = trigrad_amd.barycentric(*pts)
    g = torch.tensor([0.5, -0.25, 1.5])
    out.backward(g)
    args = [p.detach().numpy() for p in pts]
    np.testing.assert_array_equal(out.detach().numpy(), oracle.barycentric(*args))
    want = oracle.barycentric_backward(g.numpy(), *args)
    for got, w_ in zip((p.grad for p in pts), want):
        np.testing.assert_array_equal(got.numpy(), w_)
    d = [p.detach().double().requires_grad_() for p in points]

    def area(u, v, x):
        return (v[0] - u[0]) * (x[1] - u[1]) - (v[1] - u[1]) * (x[0] - u[0])
    lam = torch.stack([area(d[1], d[2], d[3]), area(d[2], d[0], d[3]), area(d[0], d[1], d[3])]) / area(d[0], d[1], d[2])
    (lam * g.double()).sum().backward()
    if abs(area(d[0], d[1], d[2]).item()) > 0.5:  # well-conditioned triangles only at float32
        _rel(out.detach(), lam.detach(), 1e-4)
        for got, t in zip((p.grad for p in pts), d):
            _rel(got, t.grad, 1e-3)
    assert abs(out.sum().item() - 1.0) < 1e-3 * max(1.0, float(out.abs().max()))


def test_component_argument_checks():
    with pytest.raises(ValueError, match="p0 must be of shape"):
        trigrad_amd.barycentric(torch.zeros(3), torch.zeros(2), torch.zeros(2), torch.zeros(2))
    with pytest.raises(TypeError, match="bary must be of type torch.float32"):
        trigrad_amd.interpolate3_vector(torch.zeros(3, dtype=torch.float64), *[torch.zeros(3)] * 4)
