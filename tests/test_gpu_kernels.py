"""Parity of every HIP kernel against the CPU oracle, called through the C-ABI of libcahel_hip.so.

Bit-exact: every integer stage must reproduce the oracle's limbs word for word on the same seeded inputs.
"""
import ctypes as C

import numpy as np
import pytest

from gpu_util import DeviceArray, make_pair, rand_limbs

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def capi():
    from lancelot_amd import capi as c
    c.lib()
    return c


@pytest.fixture(scope="module")
def small(oracle):
    # N = 4096, 6 Q limbs (mixed widths) + 2 special: three digits of two limbs
    return make_pair(oracle, 12, [60, 40, 50, 45, 30, 59, 60, 60], 2)


@pytest.fixture(scope="module")
def full(oracle):
    # benchmark shape: N = 2^16, 24 Q limbs + 8 special limbs of 50 bits (beta = 3)
    return make_pair(oracle, 16, [50] * 32, 8)


def test_tables_match_oracle(small):
    cahel, parms, ctx, p = small
    psi, ipsi = ctx.psi_table(), ctx.ipsi_table()
    assert (psi[:, :, 0] == p.tw).all() and (psi[:, :, 1] == p.twq).all()
    assert (ipsi[:, :, 0] == p.itw).all() and (ipsi[:, :, 1] == p.itwq).all()
    for L in range(1, p.size_q + 1):
        lt, got = p.level(L), ctx.level_tables(L)
        assert got["beta"] == lt.beta
        assert got["part_hat_inv"][0::2] == [int(v) for v in lt.hatinv]
        assert got["digit_mats"] == [int(v) for v in lt.mats]
        assert got["digit_mat_off"] == [int(v) for v in lt.mat_off]
        assert got["qlast_inv"][0::2] == [int(v) for v in lt.qlast_inv]
        for w, wq, q in zip(got["part_hat_inv"][0::2], got["part_hat_inv"][1::2], p.moduli):
            assert wq == (w << 64) // q


# [60, 50, 35, 59]: a prime above 2^50 keeps the launch on the integer back end; [50, 49, 35, 50]: all below
# 2^50, the FP64 back end
@pytest.mark.parametrize("one_pass", ["default", "off", "forced"])
@pytest.mark.parametrize("bits", [[60, 50, 35, 59], [50, 49, 35, 50]])
@pytest.mark.parametrize("logn", [9, 10, 11, 12, 13, 14, 15, 16, 17])
def test_ntt_all_sizes(oracle, capi, monkeypatch, logn, bits, one_pass):
    """Forward and inverse against the oracle at every degree; up to N = 2^14 with all primes below 2^50 the plain
    transform can be one kernel with the limb resident in LDS (by default where it is the faster form: N <= 2^12, or
    many limbs), and is rows pass + blocks pass otherwise."""
    if one_pass != "default" and (logn > 14 or bits[0] == 60):
        pytest.skip("the switches only change N <= 2^14 on the FP64 back end")
    monkeypatch.setenv("CAHEL_HIP_NO_ONE_PASS", "1" if one_pass == "off" else "0")
    monkeypatch.setenv("CAHEL_HIP_FORCE_ONE_PASS", "1" if one_pass == "forced" else "0")
    cahel, parms, ctx, p = make_pair(oracle, logn, bits, 1)
    rng = np.random.default_rng(logn)
    h = ctx.he_handle()
    x = rand_limbs(p, rng, range(4), n_polys=2)
    x[0, 0, :8] = 0
    x[0, 1, :] = p.moduli[1] - 1          # a whole limb of q - 1: the largest lazy values
    x[1, 2, :] = 1
    d = DeviceArray(capi, host=x)
    capi.check(capi.lib().he_ntt_forward(h, d.ptr, 2, 4, 4, 0, 4, 0, None))
    want = np.stack([p.ntt_fwd(x[i].copy()) for i in range(2)])
    got = d.numpy()
    assert (got == want).all()
    capi.check(capi.lib().he_ntt_inverse(h, d.ptr, 2, 4, 4, 0, 4, 0, None))
    assert (d.numpy() == x).all()
    # inverse of arbitrary canonical data (not an NTT image of anything special) against the oracle
    d2 = DeviceArray(capi, host=x)
    capi.check(capi.lib().he_ntt_inverse(h, d2.ptr, 2, 4, 4, 0, 4, 0, None))
    assert (d2.numpy() == np.stack([p.ntt_inv(x[i].copy()) for i in range(2)])).all()


def test_ntt_limb_maps(small, capi):
    """Partial limb ranges, the Ql u P table map and poly strides larger than the transformed range."""
    cahel, parms, ctx, p = small
    rng = np.random.default_rng(1)
    h = ctx.he_handle()
    L, K, Q = 4, p.size_p, p.size_q
    tidx = [p.table_index(L, t) for t in range(L + K)]
    x = rand_limbs(p, rng, tidx, n_polys=3)
    d = DeviceArray(capi, host=x)
    capi.check(capi.lib().he_ntt_forward(h, d.ptr, 3, L + K, L + K, 0, L, Q, None))
    want = np.stack([p.ntt_fwd(x[i].copy(), tidx) for i in range(3)])
    assert (d.numpy() == want).all()
    # only the special limbs, in place inside the wider buffer (what ModDown does)
    capi.check(capi.lib().he_ntt_inverse(h, d.at(L * p.n), 3, L + K, K, Q, K, 0, None))
    got = d.numpy()
    assert (got[:, :L] == want[:, :L]).all() and (got[:, L:] == x[:, L:]).all()
    # a single limb in the middle of Q
    y = rand_limbs(p, rng, [3])
    dy = DeviceArray(capi, host=y)
    capi.check(capi.lib().he_ntt_forward(h, dy.ptr, 1, 1, 1, 3, 1, 0, None))
    assert (dy.numpy() == p.ntt_fwd(y.copy(), [3])).all()


def test_ntt_benchmark_shape(full, capi):
    """N = 2^16, 24 limbs, 2 polynomials: forward vs oracle, inverse round trip."""
    cahel, parms, ctx, p = full
    rng = np.random.default_rng(2)
    x = rand_limbs(p, rng, range(24), n_polys=2)
    d = DeviceArray(capi, host=x)
    h = ctx.he_handle()
    capi.check(capi.lib().he_ntt_forward(h, d.ptr, 2, 24, 24, 0, 24, 0, None))
    assert (d.numpy() == np.stack([p.ntt_fwd(x[i].copy()) for i in range(2)])).all()
    capi.check(capi.lib().he_ntt_inverse(h, d.ptr, 2, 24, 24, 0, 24, 0, None))
    assert (d.numpy() == x).all()


def test_integer_and_fp64_back_ends_agree(oracle, capi, monkeypatch):
    """The same 50-bit parameter set with the FP64 back end and, forced by the environment, the integer one."""
    results = []
    for no_fp in ("0", "1"):
        monkeypatch.setenv("CAHEL_HIP_NO_FP64", no_fp)
        cahel, parms, ctx, p = make_pair(oracle, 13, [50, 50, 49, 50, 50, 50], 2)
        rng = np.random.default_rng(11)
        lib, h = capi.lib(), ctx.he_handle()
        L = 4
        c = rand_limbs(p, rng, range(L))
        ct = rand_limbs(p, rng, range(L), n_polys=2)
        host_evk, dev_evk, ptrs = _evk(p, rng, capi)
        dc, dct = DeviceArray(capi, host=c), DeviceArray(capi, host=ct)
        ws = DeviceArray(capi, shape=(lib.he_keyswitch_workspace_words(h, L),))
        capi.check(lib.he_keyswitch(h, L, dc.ptr, ptrs, dct.ptr, 5, ws.ptr, None))
        ks = p.key_switch(p.galois_ntt(c, 5), host_evk)
        want = np.stack([p.add(ct[b], ks[b]) for b in range(2)])
        got = dct.numpy()
        assert (got == want).all(), no_fp
        dres = DeviceArray(capi, shape=(2, L - 1, p.n))
        rws = DeviceArray(capi, shape=(2, p.n))
        capi.check(lib.he_rescale(h, dct.ptr, dres.ptr, 2, L, rws.ptr, None))
        assert (dres.numpy() == p.rescale(want)).all(), no_fp
        results.append(dres.numpy())
    assert (results[0] == results[1]).all()


@pytest.mark.parametrize("logn,bits,size_p,L", [(13, [60, 40, 40, 60], 1, 3), (13, [60, 40, 40, 60], 1, 2),
                                                 (12, [60, 45, 50, 52, 44, 60, 49, 58], 2, 5)])
def test_mixed_back_end_agrees_with_the_integer_one(oracle, capi, monkeypatch, logn, bits, size_p, L):
    """Chains that mix primes below and above 2^50 (Lancelot's [60, 40, 40, 60]): by default every workgroup follows
    its own limb's prime, with CAHEL_HIP_NO_MIXED=1 the whole launch takes the integer kernels.  Key switch, key
    switch + rescale, plain rescale and the public transforms (with the limb maps of the key level) against the
    oracle, both ways."""
    for no_mixed in ("0", "1"):
        monkeypatch.setenv("CAHEL_HIP_NO_MIXED", no_mixed)
        cahel, parms, ctx, p = make_pair(oracle, logn, bits, size_p)
        rng = np.random.default_rng(17)
        lib, h = capi.lib(), ctx.he_handle()
        host_evk, dev_evk, ptrs = _evk(p, rng, capi)
        ws = DeviceArray(capi, shape=(lib.he_keyswitch_workspace_words(h, L),))
        c, ct = rand_limbs(p, rng, range(L)), rand_limbs(p, rng, range(L), n_polys=2)
        dc, dct = DeviceArray(capi, host=c), DeviceArray(capi, host=ct)
        capi.check(lib.he_keyswitch(h, L, dc.ptr, ptrs, dct.ptr, 5, ws.ptr, None))
        ks = p.key_switch(p.galois_ntt(c, 5), host_evk)
        want = np.stack([p.add(ct[b], ks[b]) for b in range(2)])
        assert (dct.numpy() == want).all(), no_mixed
        if L >= 2:
            dres = DeviceArray(capi, shape=(2, L - 1, p.n))
            rws = DeviceArray(capi, shape=(2, p.n))
            capi.check(lib.he_rescale(h, dct.ptr, dres.ptr, 2, L, rws.ptr, None))
            assert (dres.numpy() == p.rescale(want)).all(), no_mixed
            dct2 = DeviceArray(capi, host=ct)
            capi.check(lib.he_keyswitch_rescale(h, L, dc.ptr, ptrs, dct2.ptr, dres.ptr, 0, ws.ptr, None))
            ks0 = p.key_switch(c, host_evk)
            assert (dres.numpy() == p.rescale(np.stack([p.add(ct[b], ks0[b]) for b in range(2)]))).all(), no_mixed
        # forward and inverse transforms over all of Q u P (two polynomials), in place
        full = rand_limbs(p, rng, range(p.size_qp), n_polys=2)
        dfull = DeviceArray(capi, host=full)
        capi.check(lib.he_ntt_forward(h, dfull.ptr, 2, p.size_qp, p.size_qp, 0, p.size_qp, 0, None))
        assert (dfull.numpy() == np.stack([p.ntt_fwd(full[b].copy(), list(range(p.size_qp))) for b in range(2)])).all(), no_mixed
        capi.check(lib.he_ntt_inverse(h, dfull.ptr, 2, p.size_qp, p.size_qp, 0, p.size_qp, 0, None))
        assert (dfull.numpy() == full).all(), no_mixed


@pytest.mark.parametrize("logn,bits,size_p,L", [(13, [50, 50, 49, 50, 50, 50], 2, 4), (13, [50, 50, 49, 50, 50, 50], 2, 3),
                                                 (14, [50, 49, 48, 50, 47, 50, 50, 50, 50], 3, 5),
                                                 (11, [45, 40, 40, 50], 1, 3), (9, [40, 40, 45, 45], 2, 2)])
def test_fused_and_separate_key_switch_agree(oracle, capi, monkeypatch, logn, bits, size_p, L):
    """he_keyswitch with the inner product inside the forward NTT (the default for primes below 2^50) and, forced
    by the environment, with the separate kernels: both equal the oracle, with and without a Galois element, with a
    partial last digit (L = 3 over two special primes, L = 5 over three), and at the smallest degree."""
    for no_fuse in ("0", "1"):
        monkeypatch.setenv("CAHEL_HIP_NO_FUSED_KS", no_fuse)
        cahel, parms, ctx, p = make_pair(oracle, logn, bits, size_p)
        rng = np.random.default_rng(12)
        lib, h = capi.lib(), ctx.he_handle()
        host_evk, dev_evk, ptrs = _evk(p, rng, capi)
        ws = DeviceArray(capi, shape=(lib.he_keyswitch_workspace_words(h, L),))
        for elt in (0, 5):
            c = rand_limbs(p, rng, range(L))
            ct = rand_limbs(p, rng, range(L), n_polys=2)
            dc, dct = DeviceArray(capi, host=c), DeviceArray(capi, host=ct)
            capi.check(lib.he_keyswitch(h, L, dc.ptr, ptrs, dct.ptr, elt, ws.ptr, None))
            ks = p.key_switch(p.galois_ntt(c, elt) if elt else c, host_evk)
            want = np.stack([p.add(ct[b], ks[b]) for b in range(2)])
            assert (dct.numpy() == want).all(), (no_fuse, elt)


@pytest.mark.parametrize("logn,bits,size_p,L", [(13, [50, 50, 49, 50, 50, 50], 2, 4), (13, [50, 50, 49, 50, 50, 50], 2, 3),
                                                 (12, [60, 40, 50, 45, 30, 59, 60, 60], 2, 6), (11, [45, 40, 40, 50], 1, 3),
                                                 (11, [45, 40, 40, 50], 1, 2), (9, [40, 40, 45, 45], 2, 2)])
def test_keyswitch_rescale_equals_the_two_steps(oracle, capi, logn, bits, size_p, L):
    """he_keyswitch_rescale (ModDown's and the rescale's forward transforms merged) against the oracle's key switch
    followed by its rescale, on both arithmetic back ends, with and without a Galois element."""
    cahel, parms, ctx, p = make_pair(oracle, logn, bits, size_p)
    rng = np.random.default_rng(13)
    lib, h = capi.lib(), ctx.he_handle()
    host_evk, dev_evk, ptrs = _evk(p, rng, capi)
    ws = DeviceArray(capi, shape=(lib.he_keyswitch_workspace_words(h, L),))
    for elt in (0, 2 * p.n - 1):
        c = rand_limbs(p, rng, range(L))
        ct = rand_limbs(p, rng, range(L), n_polys=2)
        dc, dct = DeviceArray(capi, host=c), DeviceArray(capi, host=ct)
        dout = DeviceArray(capi, shape=(2, L - 1, p.n))
        capi.check(lib.he_keyswitch_rescale(h, L, dc.ptr, ptrs, dct.ptr, dout.ptr, elt, ws.ptr, None))
        ks = p.key_switch(p.galois_ntt(c, elt) if elt else c, host_evk)
        want = p.rescale(np.stack([p.add(ct[b], ks[b]) for b in range(2)]))
        assert (dout.numpy() == want).all(), elt
        assert (dct.numpy() == ct).all()                 # the input ciphertext is only read
    assert lib.he_keyswitch_rescale(h, 1, dc.ptr, ptrs, dct.ptr, dout.ptr, 0, ws.ptr, None) == -1


@pytest.mark.parametrize("logn,bits,size_p,L", [(13, [50, 50, 49, 50, 50, 50], 2, 4), (12, [60, 40, 50, 45, 30, 59, 60, 60], 2, 5),
                                                 (14, [50, 49, 48, 50, 47, 50, 50, 50, 50], 3, 5)])
def test_moddown_on_one_to_six_polynomials(oracle, capi, logn, bits, size_p, L):
    """he_moddown on 1 to 4 polynomials (one conversion launch) and on 6 (three ciphertexts as items of two),
    overwriting and adding, against the oracle on both arithmetic back ends."""
    cahel, parms, ctx, p = make_pair(oracle, logn, bits, size_p)
    rng = np.random.default_rng(31)
    lib, h = capi.lib(), ctx.he_handle()
    K, n = p.size_p, p.n
    tables = [p.table_index(L, t) for t in range(L + K)]
    for n_polys in (1, 2, 3, 4, 6):
        ws = DeviceArray(capi, shape=(n_polys, L, n))
        cx = np.stack([rand_limbs(p, rng, tables) for _ in range(n_polys)])
        md = np.stack([p.moddown(cx[b]) for b in range(n_polys)])
        dcx, dout = DeviceArray(capi, host=cx), DeviceArray(capi, shape=(n_polys, L, n))
        capi.check(lib.he_moddown(h, L, dcx.ptr, dout.ptr, n_polys, 0, ws.ptr, None))
        assert (dout.numpy() == md).all(), n_polys
        base = rand_limbs(p, rng, range(L), n_polys=n_polys)
        dcx, dacc = DeviceArray(capi, host=cx), DeviceArray(capi, host=base)
        capi.check(lib.he_moddown(h, L, dcx.ptr, dacc.ptr, n_polys, 1, ws.ptr, None))
        assert (dacc.numpy() == np.stack([p.add(base[b], md[b]) for b in range(n_polys)])).all(), n_polys


@pytest.mark.parametrize("logn,bits,size_p,L", [(13, [50, 50, 49, 50, 50, 50], 2, 4), (12, [60, 40, 50, 45, 30, 59, 60, 60], 2, 5),
                                                 (11, [45, 40, 40, 50], 1, 2)])
def test_rotate_entry_point(oracle, capi, logn, bits, size_p, L):
    """he_rotate = (sigma(c0), 0) + KeySwitch(sigma(c1)) against the oracle, both back ends."""
    cahel, parms, ctx, p = make_pair(oracle, logn, bits, size_p)
    rng = np.random.default_rng(14)
    lib, h = capi.lib(), ctx.he_handle()
    host_evk, dev_evk, ptrs = _evk(p, rng, capi)
    ws = DeviceArray(capi, shape=(lib.he_keyswitch_workspace_words(h, L),))
    for elt in (5, 2 * p.n - 1):
        ct = rand_limbs(p, rng, range(L), n_polys=2)
        din, dout = DeviceArray(capi, host=ct), DeviceArray(capi, shape=(2, L, p.n))
        capi.check(lib.he_rotate(h, L, din.ptr, ptrs, dout.ptr, elt, ws.ptr, None))
        ks = p.key_switch(p.galois_ntt(ct[1], elt), host_evk)
        want = np.stack([p.add(p.galois_ntt(ct[0], elt), ks[0]), ks[1]])
        assert (dout.numpy() == want).all(), elt
        assert (din.numpy() == ct).all()
    assert lib.he_rotate(h, L, din.ptr, ptrs, din.ptr, 5, ws.ptr, None) == -1      # in place


@pytest.mark.parametrize("logn,bits,size_p,L,n_steps", [(11, [45, 40, 40, 50], 1, 3, 25), (12, [60, 40, 50, 45, 30, 59, 60, 60], 2, 5, 4),
                                                         (11, [50, 50, 49, 50, 50, 50], 2, 4, 3), (9, [40, 40, 45, 45], 2, 2, 1)])
def test_hoisted_rotations_entry_point(oracle, capi, logn, bits, size_p, L, n_steps):
    """he_hoisted_rotations (every step in one launch, or in several when steps * digits exceeds 64) against the
    oracle's hoisting; two random keys alternate between the steps."""
    cahel, parms, ctx, p = make_pair(oracle, logn, bits, size_p)
    rng = np.random.default_rng(15)
    lib, h = capi.lib(), ctx.he_handle()
    beta = -(-L // size_p)
    keys = [_evk(p, rng, capi) for _ in range(2)]
    elts = [pow(5, k + 1, 2 * p.n) for k in range(n_steps - 1)] + [2 * p.n - 1]
    flat = capi.evk_array([keys[i % 2][1][d].ptr for i in range(n_steps) for d in range(beta)])
    d_elts = (C.c_uint32 * n_steps)(*elts)
    ws = DeviceArray(capi, shape=(lib.he_keyswitch_workspace_words(h, L),))
    ct = rand_limbs(p, rng, range(L), n_polys=2)
    din, dout = DeviceArray(capi, host=ct), DeviceArray(capi, shape=(2, L, p.n))
    capi.check(lib.he_hoisted_rotations(h, L, din.ptr, flat, d_elts, n_steps, dout.ptr, ws.ptr, None))
    want = p.hoisting(ct, elts, [keys[i % 2][0] for i in range(n_steps)])
    assert (dout.numpy() == want).all()
    assert (din.numpy() == ct).all()
    assert lib.he_hoisted_rotations(h, L, din.ptr, flat, d_elts, n_steps, din.ptr, ws.ptr, None) == -1   # in place
    assert lib.he_hoisted_rotations(h, L, din.ptr, flat, d_elts, 0, dout.ptr, ws.ptr, None) == -1
    d_elts[0] = 4
    assert lib.he_hoisted_rotations(h, L, din.ptr, flat, d_elts, n_steps, dout.ptr, ws.ptr, None) == -1   # even element


@pytest.mark.parametrize("no_local", ["0", "1"])
@pytest.mark.parametrize("logn,bits,size_p,L,items", [(11, [60, 40, 40, 60], 1, 2, 9), (12, [50, 50, 49, 50, 50, 50], 2, 4, 3),
                                                       (9, [45, 40, 40, 50], 1, 2, 2)])
def test_hoisted_rotations_with_block_local_steps(oracle, capi, monkeypatch, logn, bits, size_p, L, items, no_local):
    """Steps that are multiples of N / 512 (Galois elements 1 modulo 2^(log N - 7)) permute the NTT order inside
    aligned blocks of 256 words; the batch kernel then gathers from a copy of the block in LDS.  Against the oracle
    item by item, with that path on and switched off, for groups of 8 + 1, 2 + 1 and 2 items."""
    monkeypatch.setenv("CAHEL_HIP_NO_LOCAL_HOIST", no_local)
    cahel, parms, ctx, p = make_pair(oracle, logn, bits, size_p)
    rng = np.random.default_rng(17)
    lib, h = capi.lib(), ctx.he_handle()
    beta = -(-L // size_p)
    keys = [_evk(p, rng, capi) for _ in range(2)]
    unit = max(1, p.n // 512)
    steps = [unit * k for k in (1, 2, 3, 5)]
    elts = [pow(5, s, 2 * p.n) for s in steps]
    assert all((e - 1) % (1 << max(logn - 7, 2)) == 0 for e in elts)
    n_steps = len(elts)
    flat = capi.evk_array([keys[i % 2][1][d].ptr for i in range(n_steps) for d in range(beta)])
    d_elts = (C.c_uint32 * n_steps)(*elts)
    wsb = DeviceArray(capi, shape=(lib.he_keyswitch_batch_workspace_words(h, L, items),))
    cts = np.stack([rand_limbs(p, rng, range(L), n_polys=2) for _ in range(items)])
    din, dout = DeviceArray(capi, host=cts), DeviceArray(capi, shape=(items, 2, L, p.n))
    for add_input in (0, 1):
        capi.check(lib.he_hoisted_rotations_batch(h, L, items, din.ptr, flat, d_elts, n_steps, add_input, dout.ptr, wsb.ptr, None))
        got = dout.numpy()
        for k in range(items):
            want = p.hoisting(cts[k], elts, [keys[i % 2][0] for i in range(n_steps)])
            if add_input:
                want = np.stack([p.add(want[b], cts[k][b]) for b in range(2)])
            assert (got[k] == want).all(), (add_input, k)


@pytest.mark.parametrize("local", [False, True])
@pytest.mark.parametrize("bits,L", [([60, 60, 60, 60, 60], 4), ([50, 49, 50, 50, 50], 4), ([60, 40, 60, 40, 60], 4)])
def test_hoisted_rotations_largest_residues(oracle, capi, bits, L, local):
    """Every residue of the inputs and of the keys is q - 1 and the launch has the most products it accepts (16 steps x
    4 digits = 64 per output word): the lazy sums of the hoisting kernel (three 64-bit words relieved every 8 terms for
    the 60-bit primes, the exact FP64 pair for those below 2^50) and its final 128-bit reduction at their bounds.
    5 items: a group of 4 and a remainder.  Against the oracle, item by item."""
    logn, size_p, items, n_steps = 11, 1, 5, 16
    cahel, parms, ctx, p = make_pair(oracle, logn, bits, size_p)
    lib, h = capi.lib(), ctx.he_handle()
    beta = -(-L // size_p)
    assert n_steps * beta == 64
    top = lambda tidx, n_polys: np.stack([np.stack([np.full(p.n, p.moduli[t] - 1, dtype=np.uint64) for t in tidx])] * n_polys)
    host_key = [top(range(p.size_qp), 2) for _ in range(beta)]
    dev_key = [DeviceArray(capi, host=k) for k in host_key]
    unit = p.n // 512
    steps = [unit * (k + 1) for k in range(n_steps)] if local else [k + 1 for k in range(n_steps)]
    elts = [pow(5, s, 2 * p.n) for s in steps]
    flat = capi.evk_array([dev_key[d].ptr for _ in range(n_steps) for d in range(beta)])
    d_elts = (C.c_uint32 * n_steps)(*elts)
    wsb = DeviceArray(capi, shape=(lib.he_keyswitch_batch_workspace_words(h, L, items),))
    ct = top(range(L), 2)
    cts = np.stack([ct] * items)
    din, dout = DeviceArray(capi, host=cts), DeviceArray(capi, shape=(items, 2, L, p.n))
    capi.check(lib.he_hoisted_rotations_batch(h, L, items, din.ptr, flat, d_elts, n_steps, 1, dout.ptr, wsb.ptr, None))
    want = p.hoisting(ct, elts, [host_key] * n_steps)
    want = np.stack([p.add(want[b], ct[b]) for b in range(2)])
    got = dout.numpy()
    for k in range(items):
        assert (got[k] == want).all(), k


@pytest.mark.parametrize("logn,bits,size_p,L,items", [(11, [45, 40, 40, 50], 1, 3, 5), (11, [60, 40, 40, 60], 1, 2, 3),
                                                       (12, [60, 40, 50, 45, 30, 59, 60, 60], 2, 5, 2),
                                                       (11, [50, 50, 49, 50, 50, 50], 2, 4, 3),
                                                       (13, [50, 50, 49, 50, 50, 50], 2, 4, 3),
                                                       (13, [50, 50, 49, 50, 50, 50], 2, 3, 2)])
def test_batched_entry_points_equal_separate_calls(oracle, capi, logn, bits, size_p, L, items):
    """he_keyswitch_rescale_batch, he_hoisted_rotations_batch and he_pair_square_sum over several inputs against
    one call per input (which the other tests pin to the oracle), on both arithmetic back ends."""
    cahel, parms, ctx, p = make_pair(oracle, logn, bits, size_p)
    rng = np.random.default_rng(16)
    lib, h = capi.lib(), ctx.he_handle()
    beta = -(-L // size_p)
    keys = [_evk(p, rng, capi) for _ in range(2)]
    ws1 = DeviceArray(capi, shape=(lib.he_keyswitch_workspace_words(h, L),))
    wsb = DeviceArray(capi, shape=(lib.he_keyswitch_batch_workspace_words(h, L, items),))
    assert wsb.numpy().size == items * ws1.numpy().size

    # relinearise + rescale of dense size-3 ciphertexts: c = third polynomial, stride 3 L limbs
    ct3 = np.stack([rand_limbs(p, rng, range(L), n_polys=3) for _ in range(items)])
    ct2 = np.ascontiguousarray(ct3[:, :2])
    d3, d2 = DeviceArray(capi, host=ct3), DeviceArray(capi, host=ct2)
    dout = DeviceArray(capi, shape=(items, 2, L - 1, p.n))
    c_ptr = d3.ptr + 2 * L * p.n * 8
    capi.check(lib.he_keyswitch_rescale_batch(h, L, items, c_ptr, 3 * L, keys[0][2], d2.ptr, dout.ptr, 0, wsb.ptr, None))
    got = dout.numpy()
    for k in range(items):
        dc, dct = DeviceArray(capi, host=ct3[k, 2]), DeviceArray(capi, host=ct2[k])
        one = DeviceArray(capi, shape=(2, L - 1, p.n))
        capi.check(lib.he_keyswitch_rescale(h, L, dc.ptr, keys[0][2], dct.ptr, one.ptr, 0, ws1.ptr, None))
        assert (got[k] == one.numpy()).all(), k
    assert lib.he_keyswitch_rescale_batch(h, L, 2, c_ptr, 3 * L, keys[0][2], d2.ptr, dout.ptr, 5, wsb.ptr, None) == -1
    assert lib.he_keyswitch_rescale_batch(h, L, items, c_ptr, L - 1, keys[0][2], d2.ptr, dout.ptr, 0, wsb.ptr, None) == -1

    # hoisted rotations, with and without the input added
    n_steps = 3
    elts = [5, 25, 2 * p.n - 1]
    flat = capi.evk_array([keys[i % 2][1][d].ptr for i in range(n_steps) for d in range(beta)])
    d_elts = (C.c_uint32 * n_steps)(*elts)
    hout = DeviceArray(capi, shape=(items, 2, L, p.n))
    for add_input in (0, 1):
        capi.check(lib.he_hoisted_rotations_batch(h, L, items, d2.ptr, flat, d_elts, n_steps, add_input, hout.ptr,
                                                  wsb.ptr, None))
        got = hout.numpy()
        for k in range(items):
            din, one = DeviceArray(capi, host=ct2[k]), DeviceArray(capi, shape=(2, L, p.n))
            capi.check(lib.he_hoisted_rotations(h, L, din.ptr, flat, d_elts, n_steps, one.ptr, ws1.ptr, None))
            want = one.numpy()
            if add_input:
                want = np.stack([p.add(want[b], ct2[k, b]) for b in range(2)])
            assert (got[k] == want).all(), (add_input, k)
    assert (d2.numpy() == ct2).all()

    # sum over chunks of (a - b)^2 from a device table of ciphertext pointers
    chunks = 2
    cts = [DeviceArray(capi, host=rand_limbs(p, rng, range(L), n_polys=2)) for _ in range(4)]
    pairs = [(0, 1), (2, 3), (1, 3), (3, 0), (2, 2)][:items]
    table = np.array([[cts[a].ptr, cts[b].ptr] * chunks for a, b in pairs], dtype=np.uint64)     # both chunks the same pair
    table[0, 2:] = [cts[2].ptr, cts[0].ptr]                                                         # but for item 0
    dtab = DeviceArray(capi, host=table)
    sq01, sq2 = DeviceArray(capi, shape=(len(pairs), 2, L, p.n)), DeviceArray(capi, shape=(len(pairs), 1, L, p.n))
    capi.check(lib.he_pair_square_sum(h, L, len(pairs), chunks, dtab.ptr, sq01.ptr, sq2.ptr, None))
    got = np.concatenate([sq01.numpy(), sq2.numpy()], axis=1)
    host = [c.numpy() for c in cts]
    def square(a, b):
        d = np.stack([p.sub(host[a][i], host[b][i]) for i in range(2)])
        return p.tensor(d, d)
    for k, (a, b) in enumerate(pairs):
        second = square(2, 0) if k == 0 else square(a, b)
        want = np.stack([p.add(x, y) for x, y in zip(square(a, b), second)])
        assert (got[k] == want).all(), k
    assert lib.he_pair_square_sum(h, L, 0, chunks, dtab.ptr, sq01.ptr, sq2.ptr, None) == -1


@pytest.mark.parametrize("seed", range(10))
def test_random_parameter_sets(oracle, capi, seed):
    """Seeded random shapes: degree, number and size of the primes (which decides the arithmetic back end per
    launch), special primes, digits, level, Galois elements.  Key switch, key switch + rescale, rotation and
    hoisted rotations against the oracle, limb for limb."""
    rng = np.random.default_rng(1000 + seed)
    logn = int(rng.integers(9, 14))
    size_p = int(rng.integers(1, 4))
    dnum = int(rng.integers(1, 5))
    size_q = size_p * dnum
    style = int(rng.integers(0, 3))          # all below 2^50, all above, mixed
    lo, hi = ((30, 50), (51, 60), (30, 60))[style]
    bits = [int(b) for b in rng.integers(lo, hi + 1, size_q + size_p)]
    for b in set(bits):                      # at most four primes per bit size keeps the prime search short
        while bits.count(b) > 4:
            bits[bits.index(b)] = b - 1 if b > 31 else b + 1
    L = int(rng.integers(1, size_q + 1))
    cahel, parms, ctx, p = make_pair(oracle, logn, bits, size_p)
    lib, h = capi.lib(), ctx.he_handle()
    beta = -(-L // size_p)
    keys = [_evk(p, rng, capi) for _ in range(2)]
    ws = DeviceArray(capi, shape=(lib.he_keyswitch_workspace_words(h, L),))
    elt = int(2 * rng.integers(0, p.n) + 1)
    tag = (logn, bits, size_p, L, elt)

    c, ct = rand_limbs(p, rng, range(L)), rand_limbs(p, rng, range(L), n_polys=2)
    dc, dct = DeviceArray(capi, host=c), DeviceArray(capi, host=ct)
    capi.check(lib.he_keyswitch(h, L, dc.ptr, keys[0][2], dct.ptr, elt, ws.ptr, None))
    ks = p.key_switch(p.galois_ntt(c, elt), keys[0][0])
    summed = np.stack([p.add(ct[b], ks[b]) for b in range(2)])
    assert (dct.numpy() == summed).all(), tag

    if L >= 2:
        dct = DeviceArray(capi, host=ct)
        dout = DeviceArray(capi, shape=(2, L - 1, p.n))
        capi.check(lib.he_keyswitch_rescale(h, L, dc.ptr, keys[0][2], dct.ptr, dout.ptr, elt, ws.ptr, None))
        assert (dout.numpy() == p.rescale(summed)).all(), tag

    dout = DeviceArray(capi, shape=(2, L, p.n))
    dct = DeviceArray(capi, host=ct)
    capi.check(lib.he_rotate(h, L, dct.ptr, keys[1][2], dout.ptr, elt, ws.ptr, None))
    ks = p.key_switch(p.galois_ntt(ct[1], elt), keys[1][0])
    assert (dout.numpy() == np.stack([p.add(p.galois_ntt(ct[0], elt), ks[0]), ks[1]])).all(), tag

    elts = [elt, int(2 * rng.integers(0, p.n) + 1), 2 * p.n - 1]
    flat = capi.evk_array([keys[i % 2][1][d].ptr for i in range(3) for d in range(beta)])
    capi.check(lib.he_hoisted_rotations(h, L, dct.ptr, flat, (C.c_uint32 * 3)(*elts), 3, dout.ptr, ws.ptr, None))
    assert (dout.numpy() == p.hoisting(ct, elts, [keys[i % 2][0] for i in range(3)])).all(), tag


def test_ntt_rejects_bad_arguments(small, capi):
    cahel, parms, ctx, p = small
    d = DeviceArray(capi, shape=(1, p.n))
    lib, h = capi.lib(), ctx.he_handle()
    assert lib.he_ntt_forward(h, d.ptr, 1, 1, 1, p.size_qp, 1, 0, None) == -1      # table out of range
    assert lib.he_ntt_forward(h, d.ptr, 1, 1, 2, 0, 2, 0, None) == -1              # limbs > stride
    assert lib.he_ntt_forward(h, None, 1, 1, 1, 0, 1, 0, None) == -1
    with pytest.raises(RuntimeError):
        capi.check(-1)


def test_elementwise(small, capi):
    cahel, parms, ctx, p = small
    rng = np.random.default_rng(3)
    lib, h = capi.lib(), ctx.he_handle()
    limbs = p.size_qp
    a, b, c = (rand_limbs(p, rng, range(limbs), n_polys=2) for _ in range(3))
    a[0, :, 0], b[0, :, 0] = 0, [q - 1 for q in p.moduli]
    da, db, dc, do = (DeviceArray(capi, host=v) for v in (a, b, c, a))
    flat = lambda f, *xs: np.stack([f(*(x[i] for x in xs)) for i in range(2)])
    capi.check(lib.he_add(h, da.ptr, db.ptr, do.ptr, 2, limbs, 0, None))
    assert (do.numpy() == flat(p.add, a, b)).all()
    capi.check(lib.he_sub(h, da.ptr, db.ptr, do.ptr, 2, limbs, 0, None))
    assert (do.numpy() == flat(p.sub, a, b)).all()
    capi.check(lib.he_negate(h, da.ptr, do.ptr, 2, limbs, 0, None))
    assert (do.numpy() == flat(p.negate, a)).all()
    capi.check(lib.he_multiply(h, da.ptr, db.ptr, do.ptr, 2, limbs, 0, None))
    assert (do.numpy() == flat(p.mul, a, b)).all()
    capi.check(lib.he_multiply_add(h, da.ptr, db.ptr, dc.ptr, do.ptr, 2, limbs, 0, 0, None))
    assert (do.numpy() == flat(p.mul_add, a, b, c)).all()
    capi.check(lib.he_multiply_add(h, da.ptr, db.ptr, dc.ptr, do.ptr, 2, limbs, 0, 1, None))
    assert (do.numpy() == flat(lambda x, y, z: p.mul_add(x, y, z, True), a, b, c)).all()
    # in place (out aliases a)
    capi.check(lib.he_add(h, da.ptr, db.ptr, da.ptr, 2, limbs, 0, None))
    assert (da.numpy() == flat(p.add, a, b)).all()


def test_tensor_and_square(small, capi):
    cahel, parms, ctx, p = small
    rng = np.random.default_rng(4)
    lib, h = capi.lib(), ctx.he_handle()
    for L in (6, 3, 1):
        a, b = (rand_limbs(p, rng, range(L), n_polys=2) for _ in range(2))
        a[:, :, 0] = [q - 1 for q in p.moduli[:L]]
        b[:, :, 0] = [q - 1 for q in p.moduli[:L]]
        da, db = DeviceArray(capi, host=a), DeviceArray(capi, host=b)
        do = DeviceArray(capi, shape=(3, L, p.n))
        capi.check(lib.he_tensor(h, da.ptr, db.ptr, do.ptr, L, None))
        assert (do.numpy() == p.tensor(a, b)).all()
        capi.check(lib.he_tensor_square(h, da.ptr, do.ptr, L, None))
        assert (do.numpy() == p.square(a)).all()
        # in place on a 3-poly buffer whose first two polys hold the operand
        buf = np.zeros((3, L, p.n), dtype=np.uint64)
        buf[:2] = a
        dbuf = DeviceArray(capi, host=buf)
        capi.check(lib.he_tensor(h, dbuf.ptr, db.ptr, dbuf.ptr, L, None))
        assert (dbuf.numpy() == p.tensor(a, b)).all()


@pytest.mark.parametrize("s1,s2", [(2, 3), (3, 2), (3, 3), (2, 2), (1, 2), (4, 2), (3, 5), (5, 5), (16, 16), (1, 9)])
def test_tensor_mxn(small, capi, s1, s2):
    """he_tensor_mxn against the oracle for operand sizes up to 3 x 3 (operands in registers) and beyond (the
    general kernel, up to 16 x 16: sixteen products of the largest residues in one 128-bit sum), out of place and
    into the first operand's buffer, with edge residues; sizes beyond 16 are refused."""
    cahel, parms, ctx, p = small
    rng = np.random.default_rng(70 + 10 * s1 + s2)
    L = 5
    a = rand_limbs(p, rng, range(L), n_polys=s1)
    b = rand_limbs(p, rng, range(L), n_polys=s2)
    for i in range(L):
        a[:, i, 0] = p.moduli[i] - 1
        b[:, i, 0] = p.moduli[i] - 1
        b[:, i, 1] = 0
    want = p.tensor_mxn(a, b)
    lib, h = capi.lib(), ctx.he_handle()
    da, db = DeviceArray(capi, host=a), DeviceArray(capi, host=b)
    dout = DeviceArray(capi, shape=want.shape)
    capi.check(lib.he_tensor_mxn(h, da.ptr, s1, db.ptr, s2, dout.ptr, L, None))
    assert (dout.numpy() == want).all()
    # in place: the first operand sits at the start of a buffer with room for the result
    big = np.zeros(want.shape, dtype=np.uint64)
    big[:s1] = a
    dbig = DeviceArray(capi, host=big)
    capi.check(lib.he_tensor_mxn(h, dbig.ptr, s1, db.ptr, s2, dbig.ptr, L, None))
    assert (dbig.numpy() == want).all()
    assert lib.he_tensor_mxn(h, da.ptr, 17, db.ptr, s2, dout.ptr, L, None) == -2
    assert lib.he_tensor_mxn(h, da.ptr, 0, db.ptr, s2, dout.ptr, L, None) == -1


@pytest.mark.parametrize("step", [1, -1, 7, 0, 1000])
def test_galois(small, capi, oracle, step):
    cahel, parms, ctx, p = small
    rng = np.random.default_rng(5)
    elt = oracle.galois_elt_from_step(step, p.n)
    assert cahel.get_elts_from_steps([step], p.n) == [elt]
    a = rand_limbs(p, rng, range(p.size_qp))
    da, do = DeviceArray(capi, host=a), DeviceArray(capi, shape=a.shape)
    capi.check(capi.lib().he_galois_ntt(ctx.he_handle(), da.ptr, do.ptr, p.size_qp, elt, None))
    assert (do.numpy() == p.galois_ntt(a, elt)).all()
    assert capi.lib().he_galois_ntt(ctx.he_handle(), da.ptr, do.ptr, 1, 4, None) == -1      # even element
    assert capi.lib().he_galois_ntt(ctx.he_handle(), da.ptr, da.ptr, 1, elt, None) == -1    # in place


@pytest.mark.parametrize("L", [6, 5, 2])
def test_rescale(small, capi, L):
    cahel, parms, ctx, p = small
    rng = np.random.default_rng(6 + L)
    ct = rand_limbs(p, rng, range(L), n_polys=3)
    din = DeviceArray(capi, host=ct)
    dout = DeviceArray(capi, shape=(3, L - 1, p.n))
    ws = DeviceArray(capi, shape=(3, p.n))
    capi.check(capi.lib().he_rescale(ctx.he_handle(), din.ptr, dout.ptr, 3, L, ws.ptr, None))
    assert (dout.numpy() == p.rescale(ct)).all()
    assert (din.numpy() == ct).all()                      # the input is left untouched
    assert capi.lib().he_rescale(ctx.he_handle(), din.ptr, dout.ptr, 3, 1, ws.ptr, None) == -1


def _evk(p, rng, capi):
    dnum = p.size_q // p.size_p
    host = [rand_limbs(p, rng, range(p.size_qp), n_polys=2) for _ in range(dnum)]
    dev = [DeviceArray(capi, host=k) for k in host]
    return host, dev, capi.evk_array([d.ptr for d in dev])


@pytest.mark.parametrize("bits", [[60] * 9, [50] * 9, [60, 40] * 4 + [60]])
def test_inner_product_largest_residues(oracle, capi, bits):
    """he_ks_inner_product with every digit word and every key word equal to q - 1 (8 digits of one limb each): the
    128-bit sums of the integer kernel and their reduction, and the FP64 kernel's, at their bounds; plain and
    accumulating onto a result that is q - 1 everywhere."""
    cahel, parms, ctx, p = make_pair(oracle, 11, bits, 1)
    lib, h = capi.lib(), ctx.he_handle()
    L, K, n = 8, 1, p.n
    tidx = [p.table_index(L, t) for t in range(L + K)]
    row = np.stack([np.full(n, p.moduli[t] - 1, dtype=np.uint64) for t in tidx])
    y = np.stack([row] * L)
    host_evk = [np.stack([np.stack([np.full(n, p.moduli[t] - 1, dtype=np.uint64) for t in range(p.size_qp)])] * 2) for _ in range(L)]
    dev_evk = [DeviceArray(capi, host=k) for k in host_evk]
    ptrs = capi.evk_array([d.ptr for d in dev_evk])
    dy = DeviceArray(capi, host=y)
    dcx = DeviceArray(capi, host=np.stack([row, row]))
    cx = p.inner_prod(y, host_evk)
    capi.check(lib.he_ks_inner_product(h, L, dy.ptr, ptrs, dcx.ptr, 0, 1, None))
    assert (dcx.numpy() == np.stack([p._add_tidx(row, cx[b], tidx) for b in range(2)])).all()
    capi.check(lib.he_ks_inner_product(h, L, dy.ptr, ptrs, dcx.ptr, 0, 0, None))
    assert (dcx.numpy() == cx).all()
    assert (cx == (L % np.array([p.moduli[t] for t in tidx], dtype=np.uint64))[None, :, None]).all()   # 8 x (q - 1)^2 = 8 mod q


@pytest.mark.parametrize("L", [6, 5, 4, 3, 1])
def test_modup_inner_moddown(small, capi, L):
    cahel, parms, ctx, p = small
    rng = np.random.default_rng(10 + L)
    lib, h = capi.lib(), ctx.he_handle()
    K, n = p.size_p, p.n
    beta = -(-L // K)
    c = rand_limbs(p, rng, range(L))
    dc = DeviceArray(capi, host=c)
    dy = DeviceArray(capi, shape=(beta, L + K, n))
    ws = DeviceArray(capi, shape=(2 * L, n))
    capi.check(lib.he_modup(h, L, dc.ptr, dy.ptr, ws.ptr, None))
    y = p.modup(c)
    assert (dy.numpy() == y).all()
    host_evk, dev_evk, ptrs = _evk(p, rng, capi)
    dcx = DeviceArray(capi, shape=(2, L + K, n))
    capi.check(lib.he_ks_inner_product(h, L, dy.ptr, ptrs, dcx.ptr, 0, 0, None))
    cx = p.inner_prod(y, host_evk)
    assert (dcx.numpy() == cx).all()
    # accumulate + automorphism on load (the hoisting form)
    elt = 25
    capi.check(lib.he_ks_inner_product(h, L, dy.ptr, ptrs, dcx.ptr, elt, 1, None))
    tidx = [p.table_index(L, t) for t in range(L + K)]
    cx2 = p.inner_prod(p.galois_ntt(y, elt), host_evk)
    acc = np.stack([p._add_tidx(cx[b], cx2[b], tidx) for b in range(2)])
    assert (dcx.numpy() == acc).all()
    # ModDown: plain and accumulating
    dcx = DeviceArray(capi, host=cx)
    dout = DeviceArray(capi, shape=(2, L, n))
    capi.check(lib.he_moddown(h, L, dcx.ptr, dout.ptr, 2, 0, ws.ptr, None))
    md = np.stack([p.moddown(cx[0]), p.moddown(cx[1])])
    assert (dout.numpy() == md).all()
    base = rand_limbs(p, rng, range(L), n_polys=2)
    dcx, dacc = DeviceArray(capi, host=cx), DeviceArray(capi, host=base)
    capi.check(lib.he_moddown(h, L, dcx.ptr, dacc.ptr, 2, 1, ws.ptr, None))
    assert (dacc.numpy() == np.stack([p.add(base[b], md[b]) for b in range(2)])).all()


@pytest.mark.parametrize("L,elt", [(6, 0), (5, 0), (6, 5), (3, 125)])
def test_keyswitch(small, capi, L, elt):
    cahel, parms, ctx, p = small
    rng = np.random.default_rng(20 + L)
    lib, h = capi.lib(), ctx.he_handle()
    c = rand_limbs(p, rng, range(L))
    ct = rand_limbs(p, rng, range(L), n_polys=2)
    host_evk, dev_evk, ptrs = _evk(p, rng, capi)
    words = lib.he_keyswitch_workspace_words(h, L)
    beta = -(-L // p.size_p)
    assert words == (beta + 2) * (L + p.size_p) * p.n + 2 * L * p.n + 2 * p.n
    dc, dct = DeviceArray(capi, host=c), DeviceArray(capi, host=ct)
    ws = DeviceArray(capi, shape=(words,))
    capi.check(lib.he_keyswitch(h, L, dc.ptr, ptrs, dct.ptr, elt, ws.ptr, None))
    src = p.galois_ntt(c, elt) if elt else c
    ks = p.key_switch(src, host_evk)
    assert (dct.numpy() == np.stack([p.add(ct[b], ks[b]) for b in range(2)])).all()
    assert (dc.numpy() == c).all()


def test_tensor_and_square_benchmark_shape(full, capi):
    """he_tensor and he_tensor_square at N = 2^16, L = 24 limbs of 50 bits (the exact-FP64 kernels), edge residues
    included, against the oracle; out of place and into the first operand's buffer."""
    cahel, parms, ctx, p = full
    rng = np.random.default_rng(33)
    lib, h = capi.lib(), ctx.he_handle()
    L = 24
    a = rand_limbs(p, rng, range(L), n_polys=2)
    b = rand_limbs(p, rng, range(L), n_polys=2)
    for i in range(L):
        a[:, i, 0] = p.moduli[i] - 1
        b[:, i, 0] = p.moduli[i] - 1
        a[:, i, 1] = 0
        b[0, i, 2], b[1, i, 2] = 1, p.moduli[i] - 1
    da, db = DeviceArray(capi, host=a), DeviceArray(capi, host=b)
    dout = DeviceArray(capi, shape=(3, L, p.n))
    capi.check(lib.he_tensor(h, da.ptr, db.ptr, dout.ptr, L, None))
    want = p.tensor(a, b)
    assert (dout.numpy() == want).all()
    capi.check(lib.he_tensor_square(h, da.ptr, dout.ptr, L, None))
    assert (dout.numpy() == p.square(a)).all()
    big = np.zeros((3, L, p.n), dtype=np.uint64)
    big[:2] = a
    dbig = DeviceArray(capi, host=big)
    capi.check(lib.he_tensor(h, dbig.ptr, db.ptr, dbig.ptr, L, None))
    assert (dbig.numpy() == want).all()


def test_keyswitch_benchmark_shape(full, capi):
    """Key switch at N = 2^16, L = 24, K = 8, beta = 3 against the oracle."""
    cahel, parms, ctx, p = full
    rng = np.random.default_rng(30)
    lib, h = capi.lib(), ctx.he_handle()
    L = 24
    c = rand_limbs(p, rng, range(L))
    ct = rand_limbs(p, rng, range(L), n_polys=2)
    host_evk, dev_evk, ptrs = _evk(p, rng, capi)
    dc, dct = DeviceArray(capi, host=c), DeviceArray(capi, host=ct)
    ws = DeviceArray(capi, shape=(lib.he_keyswitch_workspace_words(h, L),))
    capi.check(lib.he_keyswitch(h, L, dc.ptr, ptrs, dct.ptr, 0, ws.ptr, None))
    ks = p.key_switch(c, host_evk)
    assert (dct.numpy() == np.stack([p.add(ct[b], ks[b]) for b in range(2)])).all()


@pytest.mark.parametrize("no_fp", ["0", "1"])
def test_rows_pass_on_registers_at_benchmark_shape(oracle, capi, monkeypatch, no_fp):
    """N = 2^16 with enough limbs for full tiles: the rows pass keeps its outer half on registers.  Both back ends
    (FP64, and the integer one forced by the environment) against the oracle: plain forward and inverse transforms,
    the rescale (prologue that broadcasts the last limb) and key switch + rescale (prologue of the merged ModDown +
    rescale, inverse transform with a scaling epilogue)."""
    monkeypatch.setenv("CAHEL_HIP_NO_FP64", no_fp)
    cahel, parms, ctx, p = make_pair(oracle, 16, [50] * 32, 8)
    rng = np.random.default_rng(33)
    lib, h = capi.lib(), ctx.he_handle()
    L = 24
    x = rand_limbs(p, rng, range(L), n_polys=2)
    x[0, 1, :] = p.moduli[1] - 1                               # a whole limb of q - 1: the largest lazy values
    d = DeviceArray(capi, host=x)
    capi.check(lib.he_ntt_forward(h, d.ptr, 2, L, L, 0, L, 0, None))
    assert (d.numpy() == np.stack([p.ntt_fwd(x[i].copy()) for i in range(2)])).all()
    d = DeviceArray(capi, host=x)
    capi.check(lib.he_ntt_inverse(h, d.ptr, 2, L, L, 0, L, 0, None))
    assert (d.numpy() == np.stack([p.ntt_inv(x[i].copy()) for i in range(2)])).all()
    dres = DeviceArray(capi, shape=(2, L - 1, p.n))
    rws = DeviceArray(capi, shape=(2, p.n))
    capi.check(lib.he_rescale(h, DeviceArray(capi, host=x).ptr, dres.ptr, 2, L, rws.ptr, None))
    assert (dres.numpy() == p.rescale(x)).all()
    c = rand_limbs(p, rng, range(L))
    host_evk, dev_evk, ptrs = _evk(p, rng, capi)
    dc, dct = DeviceArray(capi, host=c), DeviceArray(capi, host=x)
    ws = DeviceArray(capi, shape=(lib.he_keyswitch_workspace_words(h, L),))
    capi.check(lib.he_keyswitch_rescale(h, L, dc.ptr, ptrs, dct.ptr, dres.ptr, 0, ws.ptr, None))
    ks = p.key_switch(c, host_evk)
    assert (dres.numpy() == p.rescale(np.stack([p.add(x[b], ks[b]) for b in range(2)]))).all()
    # the same at L = 8: launches of fewer than 16 limbs take quarter tiles (256 rows x 4 columns, 64 threads)
    L = 8
    x = rand_limbs(p, rng, range(L), n_polys=2)
    d = DeviceArray(capi, host=x)
    capi.check(lib.he_ntt_forward(h, d.ptr, 2, L, L, 0, L, 0, None))
    assert (d.numpy() == np.stack([p.ntt_fwd(x[i].copy(), list(range(L))) for i in range(2)])).all()
    d = DeviceArray(capi, host=x)
    capi.check(lib.he_ntt_inverse(h, d.ptr, 2, L, L, 0, L, 0, None))
    assert (d.numpy() == np.stack([p.ntt_inv(x[i].copy(), list(range(L))) for i in range(2)])).all()
    dres = DeviceArray(capi, shape=(2, L - 1, p.n))
    capi.check(lib.he_rescale(h, DeviceArray(capi, host=x).ptr, dres.ptr, 2, L, rws.ptr, None))
    assert (dres.numpy() == p.rescale(x)).all()
    c = rand_limbs(p, rng, range(L))
    dc, dct = DeviceArray(capi, host=c), DeviceArray(capi, host=x)
    ws = DeviceArray(capi, shape=(lib.he_keyswitch_workspace_words(h, L),))
    capi.check(lib.he_keyswitch_rescale(h, L, dc.ptr, ptrs, dct.ptr, dres.ptr, 0, ws.ptr, None))
    ks = p.key_switch(c, host_evk)
    assert (dres.numpy() == p.rescale(np.stack([p.add(x[b], ks[b]) for b in range(2)]))).all()


def test_samplers(small, capi, oracle):
    cahel, parms, ctx, p = small
    lib, h = capi.lib(), ctx.he_handle()
    key = oracle.chacha_key(77)
    kp = key.ctypes.data_as(C.POINTER(C.c_uint32))
    limbs = p.size_qp
    out = DeviceArray(capi, shape=(limbs, p.n))
    cdt = oracle.gauss_cdt()
    dcdt = DeviceArray(capi, host=cdt)
    for kind, fn in ((0, p.sample_ternary), (1, p.sample_error), (2, p.sample_uniform)):
        capi.check(lib.he_sample(h, kind, kp, 5, out.ptr, limbs, 0, limbs, 0, None, 0, None))
        assert (out.numpy() == fn(key, 5, limbs)).all(), kind
    capi.check(lib.he_sample(h, 3, kp, 9, out.ptr, limbs, 0, limbs, 0, dcdt.ptr, len(cdt), None))
    assert (out.numpy() == p.sample_gauss(key, 9, limbs, cdt)).all()
    assert lib.he_sample(h, 3, kp, 9, out.ptr, limbs, 0, limbs, 0, None, 0, None) == -1


def test_decompose_real(small, capi, oracle):
    cahel, parms, ctx, p = small
    rng = np.random.default_rng(40)
    coeffs = np.round(rng.uniform(-2.0 ** 62, 2.0 ** 62, p.n))
    coeffs[:4] = [0.0, -0.0, 1.0, -1.0]
    dco = DeviceArray(capi, host=coeffs)
    out = DeviceArray(capi, shape=(p.size_q, p.n))
    capi.check(capi.lib().he_decompose_real(ctx.he_handle(), dco.ptr, out.ptr, p.size_q, 0, None))
    want = np.empty((p.size_q, p.n), dtype=np.uint64)
    oracle.lib().orc_decompose_coeffs(C.byref(p.c), coeffs.ctypes.data_as(C.POINTER(C.c_double)),
                                      want.ctypes.data_as(oracle.u64p), C.c_uint32(p.size_q))
    assert (out.numpy() == want).all()


# ---- CKKS encode / decode on the device ----

@pytest.mark.parametrize("slots,complex_values", [(None, False), (None, True), (64, True), (2, False)])
def test_ckks_encode_decode(small, capi, oracle, slots, complex_values):
    """he_ckks_encode / he_ckks_decode against the oracle's encoder: coefficients within one unit (the FP64
    transforms differ in operation order only), decoded values to 2^-20, full and sparse slot counts."""
    cahel, parms, ctx, p = small
    lib, h = capi.lib(), ctx.he_handle()
    ss = slots or p.n // 2
    rng = np.random.default_rng(50 + ss)
    count = ss if ss < 8 else ss - 3                      # ragged: the tail is zero padded
    z = rng.uniform(-1, 1, count) + (1j * rng.uniform(-1, 1, count) if complex_values else 0)
    scale, limbs = 2.0 ** 40, p.size_q
    o_enc = oracle.Encoder(p)
    re = DeviceArray(capi, host=np.ascontiguousarray(np.real(z), dtype=np.float64))
    im = DeviceArray(capi, host=np.ascontiguousarray(np.imag(z), dtype=np.float64)) if complex_values else None
    ws = DeviceArray(capi, shape=(lib.he_ckks_workspace_words(h, limbs),))
    out = DeviceArray(capi, shape=(limbs, p.n))
    capi.check(lib.he_ckks_encode(h, re.ptr, im.ptr if im else None, count, ss, scale, limbs, out.ptr, ws.ptr, None))
    got = out.numpy()
    want = o_enc.encode(z, scale, limbs, ss)
    coeff_got = p.ntt_inv(got.copy()).astype(np.int64)
    coeff_want = p.ntt_inv(want.copy()).astype(np.int64)
    q0 = p.moduli[0]
    diff = (coeff_got[0] - coeff_want[0]) % q0
    diff = np.minimum(diff, q0 - diff)
    assert diff.max() <= 1
    max_coeff = ws.numpy().view(np.float64)[0]
    centred = np.where(coeff_got[0] > q0 // 2, coeff_got[0] - q0, coeff_got[0])
    assert max_coeff == np.abs(centred).max()
    # decode what was encoded
    dec = DeviceArray(capi, shape=(2 * ss,), dtype=np.float64)
    capi.check(lib.he_ckks_decode(h, out.ptr, limbs, ss, scale, dec.ptr, ws.ptr, None))
    v = dec.numpy().reshape(ss, 2)
    got_z = v[:, 0] + 1j * v[:, 1]
    want_z = o_enc.decode(got, scale, ss)
    assert np.max(np.abs(got_z - want_z)) < 2.0 ** -20
    full = np.zeros(ss, dtype=np.complex128)
    full[:count] = z
    assert np.max(np.abs(got_z - full)) < 2.0 ** -20


def test_ckks_decode_large_values(small, capi, oracle):
    """Composition over several limbs: random residues, i.e. coefficients spread over (-Q/2, Q/2)."""
    cahel, parms, ctx, p = small
    lib, h = capi.lib(), ctx.he_handle()
    limbs, ss = p.size_q, p.n // 2
    rng = np.random.default_rng(60)
    plain = rand_limbs(p, rng, list(range(limbs)))
    scale = float(np.prod([float(q) for q in p.moduli[:limbs]])) / 2.0 ** 20
    d_plain = DeviceArray(capi, host=plain)
    ws = DeviceArray(capi, shape=(lib.he_ckks_workspace_words(h, limbs),))
    dec = DeviceArray(capi, shape=(2 * ss,), dtype=np.float64)
    capi.check(lib.he_ckks_decode(h, d_plain.ptr, limbs, ss, scale, dec.ptr, ws.ptr, None))
    v = dec.numpy().reshape(ss, 2)
    want = oracle.Encoder(p).decode(plain, scale, ss)
    got = v[:, 0] + 1j * v[:, 1]
    assert np.max(np.abs(got - want)) < 2.0 ** -20 * np.max(np.abs(want))


def test_ckks_encode_bad_arguments(small, capi):
    cahel, parms, ctx, p = small
    lib, h = capi.lib(), ctx.he_handle()
    buf = DeviceArray(capi, shape=(lib.he_ckks_workspace_words(h, p.size_q),))
    out = DeviceArray(capi, shape=(p.size_q, p.n))
    for slots, count in ((3, 2), (p.n, 4), (8, 9), (1, 1)):
        assert lib.he_ckks_encode(h, buf.ptr, None, count, slots, 2.0 ** 30, p.size_q, out.ptr, buf.ptr, None) == -1
    assert lib.he_ckks_decode(h, out.ptr, p.size_q + 1, 8, 2.0 ** 30, buf.ptr, buf.ptr, None) == -1


def test_issue_rate_probe(capi):
    """he_probe_issue_rate: every kind returns a rate, an unknown kind and empty launches are refused, and the
    ordering that the design notes rely on holds (a 32-bit addition issues faster than an FP64 multiply-add or a
    32-bit multiply; the FP64 matrix instruction interleaved with FP64 vector multiply-adds does not reach the sum
    of the two alone).  The probes live in a library of their own, beside the engine's."""
    lib, r = capi.probe_lib(), C.c_double()
    assert lib.he_probe_issue_rate(6, 256, 10, C.byref(r), None) == -1
    assert lib.he_probe_issue_rate(0, 0, 10, C.byref(r), None) == -1
    assert lib.he_probe_issue_rate(0, 256, 0, C.byref(r), None) == -1
    assert lib.he_probe_issue_rate(0, 256, 10, None, None) == -1
    rate = []
    for kind in range(6):
        capi.check(lib.he_probe_issue_rate(kind, 1024, 500, C.byref(r), None))
        rate.append(r.value)
    assert all(v > 5e12 for v in rate), rate
    fma, mad, mul, add, mfma, both = rate
    assert add > 1.5 * fma and add > 1.5 * mad and add > 1.5 * mul, rate
    assert both < 0.75 * (fma + mfma), rate


def test_sampler_refuses_a_misaligned_output(small, capi):
    """The sampler stores 16 bytes at a time: an output pointer that is only 8-byte aligned is refused."""
    cahel, parms, ctx, p = small
    lib, h = capi.lib(), ctx.he_handle()
    buf = DeviceArray(capi, shape=(2 * p.n + 2,))
    key = (C.c_uint32 * 8)(*range(8))
    assert lib.he_sample(h, 0, key, 7, buf.ptr + 8, 2, 0, 2, 0, None, 0, None) == -1
    capi.check(lib.he_sample(h, 0, key, 7, buf.ptr + 16, 2, 0, 2, 0, None, 0, None))
