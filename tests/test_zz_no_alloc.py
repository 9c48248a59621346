"""he_rescale_static (the entry point that allocates nothing: its scratch is part of the library's device image)
against he_rescale (caller-provided workspace) through the C-ABI: bit-identical limbs on two calls in a row, the
second on a smaller input, so that whatever the first call left in the shared scratch must not matter."""
import numpy as np
import pytest

from gpu_util import DeviceArray, make_pair, rand_limbs

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def capi():
    from lancelot_amd import capi as c
    c.lib()
    return c


def _both(capi, ctx, p, rng, n_polys, L):
    lib, h = capi.lib(), ctx.he_handle()
    ct = rand_limbs(p, rng, range(L), n_polys=n_polys)
    din = DeviceArray(capi, host=ct)
    want = DeviceArray(capi, shape=(n_polys, L - 1, p.n))
    got = DeviceArray(capi, shape=(n_polys, L - 1, p.n))
    ws = DeviceArray(capi, shape=(n_polys, p.n))
    capi.check(lib.he_rescale(h, din.ptr, want.ptr, n_polys, L, ws.ptr, None))
    capi.check(lib.he_rescale_static(h, din.ptr, got.ptr, n_polys, L, None))
    return ct, want.numpy(), got.numpy()


def test_rescale_static_equals_rescale_twice(oracle, capi):
    cahel, parms, ctx, p = make_pair(oracle, 13, [60, 40, 50, 45, 30, 59, 60, 60], 2)
    rng = np.random.default_rng(77)
    # first call: four polynomials (the most the scratch holds), six limbs
    ct, want, got = _both(capi, ctx, p, rng, 4, 6)
    assert (got == want).all()
    assert (want == p.rescale(ct)).all()
    # second call right after it, smaller: two polynomials, three limbs; the scratch still holds the first call's words
    ct, want, got = _both(capi, ctx, p, rng, 2, 3)
    assert (got == want).all()
    assert (want == p.rescale(ct)).all()


def test_rescale_static_rejects_what_does_not_fit(oracle, capi):
    cahel, parms, ctx, p = make_pair(oracle, 12, [50, 50, 50, 50], 1)
    lib, h = capi.lib(), ctx.he_handle()
    din = DeviceArray(capi, shape=(5, 3, p.n))
    dout = DeviceArray(capi, shape=(5, 2, p.n))
    assert lib.he_rescale_static(h, din.ptr, dout.ptr, 5, 3, None) == -2      # HE_E_UNSUPPORTED: more than 4 polynomials
    assert lib.he_rescale_static(h, din.ptr, dout.ptr, 0, 3, None) == -1
    assert lib.he_rescale_static(h, din.ptr, dout.ptr, 2, 1, None) == -1      # nothing to drop at L = 1
