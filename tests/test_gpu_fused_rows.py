"""Base conversion fused with the rows pass of the forward transform (bconv_rows_fp_kernel, and bconv_rows_mx_kernel at
N = 2^16: every prime below 2^50, N >= 2^12) against the oracle, through the C-ABI entry points that use it: he_modup (with the copy of a digit's own
limbs), he_moddown (1 to 6 polynomials, overwriting and adding), he_keyswitch, he_keyswitch_rescale (the merged
ModDown + rescale prologue) and its batch form; every degree from 2^12 to 2^16, full and partial last digits, and
the same calls with the fusion switched off by the environment."""
import numpy as np
import pytest

from gpu_util import DeviceArray, make_pair, rand_limbs

pytestmark = pytest.mark.gpu

CASES = [  # logn, bits, size_p, levels
    (12, [50, 49, 48, 50, 47, 50, 50, 50], 2, (6, 5, 2)),
    (13, [45, 50, 49, 50, 50, 40, 50, 50, 50], 3, (6, 4)),
    (14, [50, 49, 48, 50, 50, 50], 2, (4, 3)),
    (15, [50, 50, 49, 50, 48], 1, (4, 2)),
    (16, [50] * 16, 8, (8, 3)),
    (16, [50, 49, 50, 50, 50, 50], 2, (4,)),
    (16, [50, 49, 50, 48, 50, 50, 47, 50, 50, 50, 49, 50], 3, (7, 5)),   # 7 and 9, 5 and 7 output limbs: groups of four with a rest
]


@pytest.fixture(scope="module")
def capi():
    from lancelot_amd import capi as c
    c.lib()
    return c


def _evk(p, rng, capi):
    dnum = p.size_q // p.size_p
    host = [rand_limbs(p, rng, range(p.size_qp), n_polys=2) for _ in range(dnum)]
    dev = [DeviceArray(capi, host=k) for k in host]
    return host, dev, capi.evk_array([d.ptr for d in dev])


@pytest.mark.parametrize("no_fused", ["0", "1", "vector_units"])
@pytest.mark.parametrize("logn,bits,size_p,levels", CASES)
def test_entry_points_with_fused_conversion(oracle, capi, monkeypatch, logn, bits, size_p, levels, no_fused):
    if no_fused == "vector_units":
        # N = 2^16 forms the conversion's products on the int8 matrix cores; this leg keeps them on the FP64 vector units
        if logn != 16:
            pytest.skip("the matrix-core kernel serves N = 2^16 only")
        monkeypatch.setenv("CAHEL_HIP_NO_MATRIX_BCONV", "1")
    else:
        monkeypatch.setenv("CAHEL_HIP_NO_FUSED_BCONV", no_fused)
    cahel, parms, ctx, p = make_pair(oracle, logn, bits, size_p)
    rng = np.random.default_rng(100 + logn)
    lib, h = capi.lib(), ctx.he_handle()
    K, n = p.size_p, p.n
    host_evk, dev_evk, ptrs = _evk(p, rng, capi)
    for L in levels:
        beta = -(-L // K)
        tables = [p.table_index(L, t) for t in range(L + K)]
        # ModUp (the digits' own limbs are copied by the same launch)
        c = rand_limbs(p, rng, range(L))
        c[0, :4] = [0, 1, p.moduli[0] - 1, p.moduli[0] - 2]          # edge residues
        dc = DeviceArray(capi, host=c)
        dy = DeviceArray(capi, shape=(beta, L + K, n))
        ws = DeviceArray(capi, shape=(2 * L, n))
        capi.check(lib.he_modup(h, L, dc.ptr, dy.ptr, ws.ptr, None))
        assert (dy.numpy() == p.modup(c)).all(), ("modup", L)
        # the largest and smallest sums of the conversion: every coefficient of every limb q - 1 (then 1) in
        # coefficient form, which is what the conversion sees after the inverse transform
        for fill in ("max", "one"):
            coeff = np.stack([np.full(n, (p.moduli[t] - 1) if fill == "max" else 1, dtype=np.uint64) for t in range(L)])
            cc = p.ntt_fwd(coeff.copy(), list(range(L)))
            capi.check(lib.he_memcpy_h2d(dc.ptr, np.ascontiguousarray(cc).ctypes.data, cc.nbytes, None))
            capi.check(lib.he_modup(h, L, dc.ptr, dy.ptr, ws.ptr, None))
            assert (dy.numpy() == p.modup(cc)).all(), ("modup", fill, L)
        # ModDown of 1, 2, 3 and 6 polynomials, overwriting and adding
        for n_polys in (1, 2, 3, 6):
            cx = np.stack([rand_limbs(p, rng, tables) for _ in range(n_polys)])
            md = np.stack([p.moddown(cx[b]) for b in range(n_polys)])
            wsd = DeviceArray(capi, shape=(n_polys, L, n))
            dcx, dout = DeviceArray(capi, host=cx), DeviceArray(capi, shape=(n_polys, L, n))
            capi.check(lib.he_moddown(h, L, dcx.ptr, dout.ptr, n_polys, 0, wsd.ptr, None))
            assert (dout.numpy() == md).all(), ("moddown", L, n_polys)
            base = rand_limbs(p, rng, range(L), n_polys=n_polys)
            dcx, dacc = DeviceArray(capi, host=cx), DeviceArray(capi, host=base)
            capi.check(lib.he_moddown(h, L, dcx.ptr, dacc.ptr, n_polys, 1, wsd.ptr, None))
            assert (dacc.numpy() == np.stack([p.add(base[b], md[b]) for b in range(n_polys)])).all(), ("moddown+", L, n_polys)
        # key switch, and key switch + rescale, with and without a Galois element
        kws = DeviceArray(capi, shape=(lib.he_keyswitch_workspace_words(h, L),))
        for elt in (0, 5):
            c = rand_limbs(p, rng, range(L))
            ct = rand_limbs(p, rng, range(L), n_polys=2)
            ks = p.key_switch(p.galois_ntt(c, elt) if elt else c, host_evk)
            want = np.stack([p.add(ct[b], ks[b]) for b in range(2)])
            dc, dct = DeviceArray(capi, host=c), DeviceArray(capi, host=ct)
            capi.check(lib.he_keyswitch(h, L, dc.ptr, ptrs, dct.ptr, elt, kws.ptr, None))
            assert (dct.numpy() == want).all(), ("keyswitch", L, elt)
            if L >= 2:
                dct, dout = DeviceArray(capi, host=ct), DeviceArray(capi, shape=(2, L - 1, n))
                capi.check(lib.he_keyswitch_rescale(h, L, dc.ptr, ptrs, dct.ptr, dout.ptr, elt, kws.ptr, None))
                assert (dout.numpy() == p.rescale(want)).all(), ("keyswitch_rescale", L, elt)
        # the batch form over three inputs (separate kernels for the inner product, same conversions)
        if L >= 2:
            items = 4 if logn == 16 else 3   # (four items: the merged ModDown + rescale then takes the matrix-core kernel at N = 2^16)
            c3 = rand_limbs(p, rng, range(L), n_polys=items)
            ct3 = np.stack([rand_limbs(p, rng, range(L), n_polys=2) for _ in range(items)])
            bws = DeviceArray(capi, shape=(lib.he_keyswitch_batch_workspace_words(h, L, items),))
            dc3, dct3 = DeviceArray(capi, host=c3), DeviceArray(capi, host=ct3)
            dout3 = DeviceArray(capi, shape=(items, 2, L - 1, n))
            capi.check(lib.he_keyswitch_rescale_batch(h, L, items, dc3.ptr, L, ptrs, dct3.ptr, dout3.ptr, 0, bws.ptr, None))
            got = dout3.numpy()
            for k in range(items):
                ks = p.key_switch(c3[k], host_evk)
                assert (got[k] == p.rescale(np.stack([p.add(ct3[k][b], ks[b]) for b in range(2)]))).all(), ("batch", L, k)


@pytest.mark.parametrize("no_fused", ["0", "1"])
@pytest.mark.parametrize("logn,bits,size_p,levels", CASES + [(11, [45, 40, 40, 50], 1, (3, 2)), (12, [60, 40, 50, 45, 30, 59, 60, 60], 2, (6, 3))])
def test_multiply_relin_rescale_entry_point(oracle, capi, monkeypatch, logn, bits, size_p, levels, no_fused):
    """he_multiply_relin_rescale (tensor product formed inside the key switch's first pass when every prime is below
    2^50; tensor kernel + key switch otherwise or when switched off) against the oracle's tensor, relinearize and
    rescale; a product of two ciphertexts and a square."""
    monkeypatch.setenv("CAHEL_HIP_NO_FUSED_TENSOR", no_fused)
    cahel, parms, ctx, p = make_pair(oracle, logn, bits, size_p)
    rng = np.random.default_rng(200 + logn)
    lib, h = capi.lib(), ctx.he_handle()
    n = p.n
    host_evk, dev_evk, ptrs = _evk(p, rng, capi)
    for L in levels:
        if L < 2:
            continue
        a = rand_limbs(p, rng, range(L), n_polys=2)
        b = rand_limbs(p, rng, range(L), n_polys=2)
        a[0, 0, :3] = [0, p.moduli[0] - 1, 1]
        b[1, 0, :3] = [p.moduli[0] - 1, p.moduli[0] - 1, 0]
        da, db = DeviceArray(capi, host=a), DeviceArray(capi, host=b)
        ws = DeviceArray(capi, shape=(lib.he_multiply_relin_rescale_workspace_words(h, L),))
        dout = DeviceArray(capi, shape=(2, L - 1, n))
        capi.check(lib.he_multiply_relin_rescale(h, L, da.ptr, db.ptr, ptrs, dout.ptr, ws.ptr, None))
        t3 = p.tensor(a, b)
        ks = p.key_switch(t3[2], host_evk)
        want = p.rescale(np.stack([p.add(t3[k], ks[k]) for k in range(2)]))
        assert (dout.numpy() == want).all(), ("product", L)
        assert (da.numpy() == a).all() and (db.numpy() == b).all()
        capi.check(lib.he_multiply_relin_rescale(h, L, da.ptr, da.ptr, ptrs, dout.ptr, ws.ptr, None))
        t3 = p.tensor(a, a)
        ks = p.key_switch(t3[2], host_evk)
        want = p.rescale(np.stack([p.add(t3[k], ks[k]) for k in range(2)]))
        assert (dout.numpy() == want).all(), ("square", L)
    assert lib.he_multiply_relin_rescale(h, 1, da.ptr, db.ptr, ptrs, dout.ptr, ws.ptr, None) == -1


@pytest.mark.parametrize("logn,bits,size_p,L,items", [(13, [45, 50, 49, 50, 50, 40, 50, 50, 50], 3, 6, 3),
                                                       (12, [60, 40, 50, 45, 30, 59, 60, 60], 2, 5, 4),
                                                       (16, [50, 49, 50, 50, 50, 50], 2, 4, 2),
                                                       (12, [50, 49, 48, 50, 47, 50, 50, 50], 2, 5, 9),
                                                       (12, [50, 49, 48, 50, 47, 50, 50, 50], 2, 6, 7)])
@pytest.mark.parametrize("inner", ["fused", "fp_kernel"])
def test_multiply_relin_rescale_batch_equals_single_calls(oracle, capi, monkeypatch, logn, bits, size_p, L, items, inner):
    """The batch entry point against the oracle item by item.  With every prime below 2^50 its inner product runs
    inside the blocks pass of ModUp's forward transform, the items of one tile next to each other on one XCD
    ("fused"); switched off, it is the FP64 kernel that shares key words among up to 8 items (groups of 2, 4 and 8,
    full and partial); with larger primes (the second parameter set) the integer kernel."""
    monkeypatch.setenv("CAHEL_HIP_NO_BATCH_FUSED_KS", "0" if inner == "fused" else "1")
    cahel, parms, ctx, p = make_pair(oracle, logn, bits, size_p)
    rng = np.random.default_rng(300 + logn)
    lib, h = capi.lib(), ctx.he_handle()
    n = p.n
    host_evk, dev_evk, ptrs = _evk(p, rng, capi)
    a = np.stack([rand_limbs(p, rng, range(L), n_polys=2) for _ in range(items)])
    b = np.stack([rand_limbs(p, rng, range(L), n_polys=2) for _ in range(items)])
    da, db = DeviceArray(capi, host=a), DeviceArray(capi, host=b)
    ws = DeviceArray(capi, shape=(lib.he_multiply_relin_rescale_batch_workspace_words(h, L, items),))
    dout = DeviceArray(capi, shape=(items, 2, L - 1, n))
    capi.check(lib.he_multiply_relin_rescale_batch(h, L, items, da.ptr, db.ptr, ptrs, dout.ptr, ws.ptr, None))
    got = dout.numpy()
    for k in range(items):
        t3 = p.tensor(a[k], b[k])
        ks = p.key_switch(t3[2], host_evk)
        assert (got[k] == p.rescale(np.stack([p.add(t3[j], ks[j]) for j in range(2)]))).all(), k
    # squares of every item
    capi.check(lib.he_multiply_relin_rescale_batch(h, L, items, da.ptr, da.ptr, ptrs, dout.ptr, ws.ptr, None))
    got = dout.numpy()
    for k in range(items):
        t3 = p.tensor(a[k], a[k])
        ks = p.key_switch(t3[2], host_evk)
        assert (got[k] == p.rescale(np.stack([p.add(t3[j], ks[j]) for j in range(2)]))).all(), ("square", k)
