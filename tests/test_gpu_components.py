"""The six host-side component hooks of libtrigrad_hip.so (reference src/trigrad/tests.cu:43-76: barycentric,
interpolate3_scalar, interpolate3_vector and their backward functions) as the GPU box loads the library: the same
comparisons as tests/test_components.py, run there so that the record of that run covers them, plus a direct call of
every hook through the C ABI against the oracle, bit for bit."""
import ctypes as C

import numpy as np
import pytest

import test_components as T

pytestmark = pytest.mark.gpu


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


def test_component_hooks_of_the_loaded_library(cuda, oracle):
    from trigrad_amd import _lib
    lib = _lib.load(32)
    rng = np.random.default_rng(77)
    f = np.float32
    for _ in range(25):
        bary = rng.uniform(0, 1, 3).astype(f)
        bary /= bary.sum()
        w = rng.uniform(0.2, 5, 3).astype(f)
        a3, b3, c3 = (rng.uniform(-5, 5, 3).astype(f) for _ in range(3))
        a, b, c = (f(x) for x in rng.uniform(-5, 5, 3))
        pts = [rng.uniform(-5, 5, 2).astype(f) for _ in range(4)]
        g3, g1 = rng.uniform(-2, 2, 3).astype(f), f(rng.uniform(-2, 2))

        out3 = np.zeros(3, f)
        lib.tg_barycentric(_p(pts[0]), _p(pts[1]), _p(pts[2]), _p(pts[3]), _p(out3))
        np.testing.assert_array_equal(out3, oracle.barycentric(*pts))
        grads = np.zeros((4, 2), f)
        lib.tg_barycentric_backward(_p(g3), _p(pts[0]), _p(pts[1]), _p(pts[2]), _p(pts[3]), _p(grads))
        np.testing.assert_array_equal(grads, oracle.barycentric_backward(g3, *pts))

        assert f(lib.tg_interpolate3_scalar(_p(bary), a, b, c, _p(w))) == oracle.interpolate3_scalar(bary, a, b, c, w)
        gb, gv, gw = (np.zeros(3, f) for _ in range(3))
        lib.tg_interpolate3_scalar_backward(g1, _p(bary), a, b, c, _p(w), _p(gb), _p(gv), _p(gw))
        for got, want in zip((gb, gv, gw), oracle.interpolate3_scalar_backward(g1, bary, a, b, c, w)):
            np.testing.assert_array_equal(got, want)

        lib.tg_interpolate3_vector(_p(bary), _p(a3), _p(b3), _p(c3), _p(w), _p(out3))
        np.testing.assert_array_equal(out3, oracle.interpolate3_vector(bary, a3, b3, c3, w))
        outs = [np.zeros(3, f) for _ in range(5)]
        lib.tg_interpolate3_vector_backward(_p(g3), _p(bary), _p(a3), _p(b3), _p(c3), _p(w), *(_p(o) for o in outs))
        for got, want in zip(outs, oracle.interpolate3_vector_backward(g3, bary, a3, b3, c3, w)):
            np.testing.assert_array_equal(got, want)


@pytest.mark.parametrize("case", range(8))
def test_component_functions_on_the_gpu_box(case, cuda, oracle):
    T.test_interpolate3_scalar(*T.CASES_I[case], oracle)
    T.test_interpolate3_vector(*T.CASES_V[case], oracle)
    T.test_barycentric(T.CASES_B[case], oracle)
