"""CPU component hooks as autograd Functions: `barycentric`, `interpolate3_scalar`,
`interpolate3_vector` with the reference's signatures and checks
(src/trigrad/tests_wrapper.py:10-87); the arithmetic runs in libtrigrad_hip.so's
host-side entry points (tg_barycentric*, tg_interpolate3_*)."""
import ctypes as C

import torch
from torch.autograd import Function

from . import _C, _lib
from .util import create_check

check_tensor = create_check("cpu", lambda: _C.precision)


def _f(t):
    t = t.detach().contiguous()
    return t, C.c_void_p(t.data_ptr())


def _out(n):
    t = torch.empty((n,), dtype=_C.precision)
    return t, C.c_void_p(t.data_ptr())


def _load():
    return _lib.load(64 if _C.precision == torch.float64 else 32)


class Barycentric(Function):
    @staticmethod
    def forward(ctx, p0, p1, q0, q1):
        for t, name in ((p0, "p0"), (p1, "p1"), (q0, "q0"), (q1, "q1")):
            check_tensor(t, name, 2)
        ctx.save_for_backward(p0, p1, q0, q1)
        keep = [_f(t) for t in (p0, p1, q0, q1)]
        out, po = _out(3)
        _load().tg_barycentric(*[p for _, p in keep], po)
        return out

    @staticmethod
    def backward(ctx, grad_bary):
        keep = [_f(t) for t in (grad_bary, *ctx.saved_tensors)]
        grads, pg = _out(8)
        _load().tg_barycentric_backward(*[p for _, p in keep], pg)
        g = grads.view(4, 2)
        return g[0].clone(), g[1].clone(), g[2].clone(), g[3].clone()


def barycentric(p0, p1, q0, q1):
    return Barycentric.apply(p0, p1, q0, q1)


class Interpolate3Scalar(Function):
    @staticmethod
    def forward(ctx, bary, a, b, c, w):
        check_tensor(bary, "bary", 3)
        check_tensor(a, "a", 1)
        check_tensor(b, "b", 1)
        check_tensor(c, "c", 1)
        check_tensor(w, "w", 3)
        ctx.save_for_backward(bary, a, b, c, w)
        kb, kw = _f(bary), _f(w)
        val = _load().tg_interpolate3_scalar(kb[1], float(a), float(b), float(c), kw[1])
        return torch.tensor([val], dtype=_C.precision)

    @staticmethod
    def backward(ctx, grad_out):
        bary, a, b, c, w = ctx.saved_tensors
        kb, kw = _f(bary), _f(w)
        gb, pgb = _out(3)
        gv, pgv = _out(3)
        gw, pgw = _out(3)
        _load().tg_interpolate3_scalar_backward(float(grad_out), kb[1], float(a), float(b), float(c), kw[1], pgb, pgv, pgw)
        return gb, gv[0:1].clone(), gv[1:2].clone(), gv[2:3].clone(), gw


def interpolate3_scalar(bary, a, b, c, w):
    return Interpolate3Scalar.apply(bary, a, b, c, w)


class Interpolate3Vector(Function):
    @staticmethod
    def forward(ctx, bary, a, b, c, w):
        for t, name in ((bary, "bary"), (a, "a"), (b, "b"), (c, "c"), (w, "w")):
            check_tensor(t, name, 3)
        ctx.save_for_backward(bary, a, b, c, w)
        keep = [_f(t) for t in (bary, a, b, c, w)]
        out, po = _out(3)
        _load().tg_interpolate3_vector(*[p for _, p in keep], po)
        return out

    @staticmethod
    def backward(ctx, grad_out):
        keep = [_f(t) for t in (grad_out, *ctx.saved_tensors)]
        outs = [_out(3) for _ in range(5)]
        _load().tg_interpolate3_vector_backward(*[p for _, p in keep], *[p for _, p in outs])
        return tuple(t for t, _ in outs)  # grad_bary, grad_a, grad_b, grad_c, grad_w


def interpolate3_vector(bary, a, b, c, w):
    return Interpolate3Vector.apply(bary, a, b, c, w)
