"""The committed vectors of tests/golden/ckks_n512.npz (written by tests/golden/make_vectors.py with the CPU checker):
the checker must still reproduce them (CPU), and the HIP path must reproduce them through the C-ABI (GPU)."""
import os

import numpy as np
import pytest

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ckks_n512.npz")


@pytest.fixture(scope="module")
def vec():
    d = np.load(GOLDEN)
    return {k: d[k] for k in d.files}


def test_fixture_parameters(vec, oracle):
    n = 1 << int(vec["logn"])
    moduli = [int(q) for q in vec["moduli"]]
    assert moduli == oracle.coeff_modulus_create(n, [50, 40, 45, 50, 50, 49])
    for q in moduli:
        assert oracle.is_prime(q) and q % (2 * n) == 1


def test_oracle_reproduces_golden_vectors(vec, oracle):
    p = oracle.Params(int(vec["logn"]), [int(q) for q in vec["moduli"]], int(vec["size_p"]))
    c, ct, ct2, evk, elt = vec["c"], vec["ct"], vec["ct2"], list(vec["evk"]), int(vec["galois_elt"])
    assert (p.ntt_fwd(c.copy()) == vec["ntt_fwd"]).all()
    assert (p.ntt_inv(c.copy()) == vec["ntt_inv"]).all()
    assert (p.ntt_inv(vec["ntt_fwd"].copy()) == c).all()
    assert (p.tensor(ct, ct2) == vec["tensor"]).all() and (p.square(ct) == vec["square"]).all()
    assert (p.galois_ntt(c, elt) == vec["galois"]).all()
    y = p.modup(c)
    assert (y == vec["modup"]).all()
    cx = p.inner_prod(y, evk)
    assert (cx == vec["inner"]).all()
    assert (np.stack([p.moddown(cx[b]) for b in range(2)]) == vec["moddown"]).all()
    ks = p.key_switch(c, evk)
    assert (np.stack([p.add(ct[b], ks[b]) for b in range(2)]) == vec["keyswitch"]).all()
    assert (p.rescale(ct) == vec["rescale"]).all()


@pytest.mark.gpu
def test_hip_path_reproduces_golden_vectors(vec, oracle):
    from gpu_util import DeviceArray, make_pair
    from lancelot_amd import capi
    lib = capi.lib()
    cahel, parms, ctx, p = make_pair(oracle, int(vec["logn"]), [50, 40, 45, 50, 50, 49], int(vec["size_p"]))
    assert [int(q) for q in vec["moduli"]] == p.moduli
    h, L, K, n = ctx.he_handle(), p.size_q, p.size_p, p.n
    c, ct, ct2, elt = vec["c"], vec["ct"], vec["ct2"], int(vec["galois_elt"])

    d = DeviceArray(capi, host=c)
    capi.check(lib.he_ntt_forward(h, d.ptr, 1, L, L, 0, L, 0, None))
    assert (d.numpy() == vec["ntt_fwd"]).all()
    capi.check(lib.he_ntt_inverse(h, d.ptr, 1, L, L, 0, L, 0, None))
    assert (d.numpy() == c).all()
    d = DeviceArray(capi, host=c)
    capi.check(lib.he_ntt_inverse(h, d.ptr, 1, L, L, 0, L, 0, None))
    assert (d.numpy() == vec["ntt_inv"]).all()

    da, db = DeviceArray(capi, host=ct), DeviceArray(capi, host=ct2)
    out3 = DeviceArray(capi, shape=(3, L, n))
    capi.check(lib.he_tensor(h, da.ptr, db.ptr, out3.ptr, L, None))
    assert (out3.numpy() == vec["tensor"]).all()
    capi.check(lib.he_tensor_square(h, da.ptr, out3.ptr, L, None))
    assert (out3.numpy() == vec["square"]).all()
    out2 = DeviceArray(capi, shape=(2, L, n))
    capi.check(lib.he_add(h, da.ptr, db.ptr, out2.ptr, 2, L, 0, None))
    assert (out2.numpy() == vec["add"]).all()
    capi.check(lib.he_sub(h, da.ptr, db.ptr, out2.ptr, 2, L, 0, None))
    assert (out2.numpy() == vec["sub"]).all()

    dc, dg = DeviceArray(capi, host=c), DeviceArray(capi, shape=(L, n))
    capi.check(lib.he_galois_ntt(h, dc.ptr, dg.ptr, L, elt, None))
    assert (dg.numpy() == vec["galois"]).all()

    beta = L // K
    dy = DeviceArray(capi, shape=(beta, L + K, n))
    ws = DeviceArray(capi, shape=(2 * L, n))
    capi.check(lib.he_modup(h, L, dc.ptr, dy.ptr, ws.ptr, None))
    assert (dy.numpy() == vec["modup"]).all()
    dev_evk = [DeviceArray(capi, host=k) for k in vec["evk"]]
    ptrs = capi.evk_array([k.ptr for k in dev_evk])
    dcx = DeviceArray(capi, shape=(2, L + K, n))
    capi.check(lib.he_ks_inner_product(h, L, dy.ptr, ptrs, dcx.ptr, 0, 0, None))
    assert (dcx.numpy() == vec["inner"]).all()
    dout = DeviceArray(capi, shape=(2, L, n))
    capi.check(lib.he_moddown(h, L, dcx.ptr, dout.ptr, 2, 0, ws.ptr, None))
    assert (dout.numpy() == vec["moddown"]).all()

    kws = DeviceArray(capi, shape=(lib.he_keyswitch_workspace_words(h, L),))
    for key, e in (("keyswitch", 0), ("keyswitch_galois", elt)):
        dct = DeviceArray(capi, host=ct)
        capi.check(lib.he_keyswitch(h, L, dc.ptr, ptrs, dct.ptr, e, kws.ptr, None))
        assert (dct.numpy() == vec[key]).all(), key

    dres = DeviceArray(capi, shape=(2, L - 1, n))
    rws = DeviceArray(capi, shape=(2, n))
    capi.check(lib.he_rescale(h, da.ptr, dres.ptr, 2, L, rws.ptr, None))
    assert (dres.numpy() == vec["rescale"]).all()
