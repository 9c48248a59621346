"""Full-size configurations on the GPU.

C1 (N = 2^14, 4 + 1 primes of 50 bits): HMult + relinearise + rescale through pyCAHEL is compared with the oracle limb
for limb, keys and ciphertexts included.  At the benchmark shape (N = 2^16, L = 24, K = 8) the C-ABI entry points
that `bench.py` times (one product per call, a batch, a rotation) are compared with the oracle limb for limb on
random residues; the scheme-level checks there and on Lancelot's [60, 40, 40, 60] chain are properties that do not
depend on the size: commutativity of the product (bit-exact), decryption of a size-3 ciphertext against its
relinearisation, rotation = roll of the slots, rotate-and-sum = sum of all slots, and the encrypted Krum distances
against the float64 closed form.
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

REL = 2.0 ** -20


def _context(logn, bits, size_p, steps=(), seed=2025, sec="none"):
    import lancelot_amd  # noqa: F401
    import pyCAHEL as cahel
    n = 1 << logn
    mods = cahel.coeff_modulus_create(n, list(bits))
    parms = cahel.params(cahel.scheme_type.ckks)
    parms.set_poly_modulus_degree(n)
    parms.set_coeff_modulus(mods)
    parms.set_special_modulus_size(size_p)
    if steps:
        parms.set_galois_elts(cahel.get_elts_from_steps(list(steps), n))
    ctx = cahel.context(parms, True, getattr(cahel.sec_level_type, sec))
    ctx.set_seed(seed)
    return cahel, parms, ctx, mods


def test_c1_hmult_relin_rescale_bit_exact(oracle):
    """Config C1: N = 2^14, Q = 4 x 50 bits, P = 1 x 50 bits, scale 2^40, 8192 slots."""
    O = oracle
    logn, bits = 14, [50] * 5
    cahel, parms, ctx, mods = _context(logn, bits, 1)
    p = O.Params(logn, [m.value() for m in mods], 1)
    ks = O.KeySet(p, seed=2025)
    sk = cahel.secret_key(parms)
    sk.gen_secretkey(ctx)
    ks.gen_secret()
    pk = cahel.public_key(ctx)
    sk.gen_publickey(ctx, pk)
    o_pk = ks.gen_public()
    rlk = cahel.relin_key(ctx)
    sk.gen_relinkey(ctx, rlk)
    o_rlk = ks.gen_relin()
    enc = cahel.ckks_encoder(ctx)
    rng = np.random.default_rng(2025)
    x, y = rng.uniform(-1, 1, p.n // 2), rng.uniform(-1, 1, p.n // 2)
    px, py = enc.encode(ctx, x, 2.0 ** 40), enc.encode(ctx, y, 2.0 ** 40)
    cx = pk.encrypt_asymmetric(ctx, px)
    o_cx = ks.encrypt_asymmetric(o_pk, px.to_numpy())
    cy = pk.encrypt_asymmetric(ctx, py)
    o_cy = ks.encrypt_asymmetric(o_pk, py.to_numpy())
    assert (cx.to_numpy() == o_cx).all() and (cy.to_numpy() == o_cy).all()
    cahel.multiply_and_relin_inplace(ctx, cx, cy, rlk)
    cahel.rescale_to_next_inplace(ctx, cx)
    want = p.rescale(p.relinearize(p.tensor(o_cx, o_cy), o_rlk))
    assert (cx.to_numpy() == want).all()
    pt = sk.decrypt(ctx, cx)
    assert (pt.to_numpy() == ks.decrypt(want, O.gauss_cdt())).all()
    got = np.array(enc.decode(ctx, pt))
    # 2^30 of scale left.  The reference's rescale floors (src/rns.cu:507-570: no rounding offset), which leaves a mean
    # of 1/2 on every coefficient of both polynomials; through c1 * s that is (1/2) (1 + X + ... + X^(N-1)) s, whose
    # value in the slot nearest to X = 1 is about N / pi * sqrt(2 N / 3) / scale = 5e-4 here for a typical secret
    # (measured with this seed: 9.8e-5 in slot 0, 1.3e-6 in the median slot)
    assert np.max(np.abs(got - x * y)) < 3e-4
    assert np.median(np.abs(got - x * y)) < 5e-6


@pytest.mark.parametrize("inner", ["fused", "fp_kernel"])
def test_c2_benchmark_shape_entry_points_bit_exact(oracle, monkeypatch, inner):
    """N = 2^16, L = 24, K = 8 (dnum = 3), 50-bit primes, random residues: he_multiply_relin_rescale, its batch form
    (8 products, as `bench.py` issues them: the fused conversion kernel then forms all 24 or 23 output limbs of a
    unit in one workgroup, where one product per call takes 5 or 6; with the inner product inside the blocks pass and
    as the FP64 kernel of its own) and he_rotate
    against the oracle's tensor / relinearise / rescale and apply_galois, every limb."""
    from gpu_util import DeviceArray, make_pair, rand_limbs
    from lancelot_amd import capi
    monkeypatch.setenv("CAHEL_HIP_NO_BATCH_FUSED_KS", "0" if inner == "fused" else "1")
    cahel, parms, ctx, p = make_pair(oracle, 16, [50] * 32, 8)
    lib, h = capi.lib(), ctx.he_handle()
    rng = np.random.default_rng(4242)
    n, L, K = p.n, 24, 8
    host_evk = [rand_limbs(p, rng, range(L + K), n_polys=2) for _ in range(L // K)]
    dev_evk = [DeviceArray(capi, host=k) for k in host_evk]
    ptrs = capi.evk_array([d.ptr for d in dev_evk])
    items = 8
    a = np.stack([rand_limbs(p, rng, range(L), n_polys=2) for _ in range(items)])
    b = np.stack([rand_limbs(p, rng, range(L), n_polys=2) for _ in range(items)])
    want = [p.rescale(p.relinearize(p.tensor(a[k], b[k]), host_evk)) for k in range(items)]
    da, db = DeviceArray(capi, host=a), DeviceArray(capi, host=b)
    # one product per call (items 0 and 2, the second a square)
    ws = DeviceArray(capi, shape=(lib.he_multiply_relin_rescale_workspace_words(h, L),))
    out = DeviceArray(capi, shape=(2, L - 1, n))
    capi.check(lib.he_multiply_relin_rescale(h, L, da.ptr, db.ptr, ptrs, out.ptr, ws.ptr, None))
    assert (out.numpy() == want[0]).all()
    last = da.ptr + 8 * (items - 1) * 2 * L * n
    capi.check(lib.he_multiply_relin_rescale(h, L, last, last, ptrs, out.ptr, ws.ptr, None))
    assert (out.numpy() == p.rescale(p.relinearize(p.tensor(a[items - 1], a[items - 1]), host_evk))).all()
    # the batch
    bws = DeviceArray(capi, shape=(lib.he_multiply_relin_rescale_batch_workspace_words(h, L, items),))
    bout = DeviceArray(capi, shape=(items, 2, L - 1, n))
    capi.check(lib.he_multiply_relin_rescale_batch(h, L, items, da.ptr, db.ptr, ptrs, bout.ptr, bws.ptr, None))
    got = bout.numpy()
    for k in range(items):
        assert (got[k] == want[k]).all(), k
    # a rotation (the key plays the Galois key of the element)
    elt = pow(5, 7, 2 * n)
    rws = DeviceArray(capi, shape=(lib.he_keyswitch_workspace_words(h, L),))
    rout = DeviceArray(capi, shape=(2, L, n))
    capi.check(lib.he_rotate(h, L, da.ptr, ptrs, rout.ptr, elt, rws.ptr, None))
    assert (rout.numpy() == p.apply_galois(a[0], elt, host_evk)).all()
    assert (da.numpy() == a).all() and (db.numpy() == b).all()


@pytest.fixture(scope="module")
def bench_world():
    """The benchmark shape: N = 2^16, 24 + 8 primes of 50 bits, keys for the 15 power-of-two steps."""
    steps = [1 << k for k in range(15)]
    cahel, parms, ctx, _ = _context(16, [50] * 32, 8, steps, sec="tc128")
    sk = cahel.secret_key(parms)
    sk.gen_secretkey(ctx)
    pk = cahel.public_key(ctx)
    sk.gen_publickey(ctx, pk)
    rlk = cahel.relin_key(ctx)
    sk.gen_relinkey(ctx, rlk)
    glk = cahel.galois_key(ctx)
    sk.create_galois_keys(ctx, glk)
    enc = cahel.ckks_encoder(ctx)
    rng = np.random.default_rng(2025)
    n = 1 << 16
    x, y = rng.uniform(-1, 1, n // 2), rng.uniform(-1, 1, n // 2)
    cx = pk.encrypt_asymmetric(ctx, enc.encode(ctx, x, 2.0 ** 40))
    cy = pk.encrypt_asymmetric(ctx, enc.encode(ctx, y, 2.0 ** 40))
    return dict(cahel=cahel, ctx=ctx, sk=sk, pk=pk, rlk=rlk, glk=glk, enc=enc, x=x, y=y, cx=cx, cy=cy, steps=steps)


def _decode(w, ct):
    return np.array(w["enc"].decode(w["ctx"], w["sk"].decrypt(w["ctx"], ct)))


def test_c3_hmult_properties(bench_world):
    w = bench_world
    c, ctx = w["cahel"], w["ctx"]
    xy, yx = c.ciphertext(ctx), c.ciphertext(ctx)
    c.multiply(ctx, w["cx"], w["cy"], xy)
    c.multiply(ctx, w["cy"], w["cx"], yx)
    assert xy.size() == 3 and (xy.to_numpy() == yx.to_numpy()).all()        # the tensor product commutes exactly
    three = _decode(w, xy)                                                    # size-3 decryption: c0 + c1 s + c2 s^2
    c.relinearize_inplace(ctx, xy, w["rlk"])
    c.relinearize_inplace(ctx, yx, w["rlk"])
    assert xy.size() == 2 and (xy.to_numpy() == yx.to_numpy()).all()
    two = _decode(w, xy)
    assert np.max(np.abs(two - three)) < 2.0 ** -20 * max(1.0, np.max(np.abs(three)))   # key-switch noise only
    # scale 2^80 before the rescale.  The uncorrected base conversion of the encryption's ModDown leaves an error
    # in [0, K) on every coefficient of c1; times the ternary secret that is a random walk over the coefficient
    # index, i.e. a low-frequency error of a few 10^-5 in the first slots and about 10^-8 elsewhere.
    assert np.max(np.abs(three - w["x"] * w["y"])) < 2e-4
    assert np.median(np.abs(three - w["x"] * w["y"])) < 1e-7
    c.rescale_to_next_inplace(ctx, xy)
    assert xy.chain_index() == 2
    got = _decode(w, xy)
    # about 2^30 of scale left; the floor-style rescale's bias in the slots nearest to X = 1 is about
    # N / pi * sqrt(2 N / 3) / scale = 4e-3 at this degree (measured 3.1e-3 in slot 0, 5.1e-6 in the median slot)
    assert np.max(np.abs(got - w["x"] * w["y"])) < 5e-3
    assert np.median(np.abs(got - w["x"] * w["y"])) < 2e-5
    # the same product through the fused call
    fused = c.ciphertext(ctx)
    c.multiply(ctx, w["cx"], w["cy"], fused)
    c.relinearize_inplace(ctx, fused, w["rlk"])
    c.rescale_to_next_inplace(ctx, fused)
    assert (fused.to_numpy() == xy.to_numpy()).all()


def test_c3_fused_and_separate_kernels_agree(monkeypatch):
    """At N = 2^16, L = 24, K = 8 the key switch with the inner product inside the blocks pass of ModUp's transform
    and with the separate kernels (he_modup + he_ks_inner_product, which the small-size tests pin to the oracle one
    by one) must give the same limbs."""
    from lancelot_amd import capi
    outs = []
    for no_fuse in ("0", "1"):
        monkeypatch.setenv("CAHEL_HIP_NO_FUSED_KS", no_fuse)
        cahel, parms, ctx, mods = _context(16, [50] * 32, 8)
        lib, h = capi.lib(), ctx.he_handle()
        n, L, qp = 1 << 16, 24, 32
        rng = np.random.default_rng(77)
        q = np.array([m.value() for m in mods], dtype=np.uint64)
        rand = lambda limbs, polys: (rng.integers(0, 1 << 62, (polys, len(limbs), n), dtype=np.uint64)
                                     % q[list(limbs)][None, :, None])
        evk = [rand(range(qp), 2) for _ in range(3)]
        c, ct = rand(range(L), 1)[0], rand(range(L), 2)
        import ctypes as C
        def dev(a):
            ptr = C.c_void_p()
            capi.check(lib.he_malloc(C.byref(ptr), a.nbytes))
            capi.check(lib.he_memcpy_h2d(ptr.value, np.ascontiguousarray(a).ctypes.data, a.nbytes, None))
            return ptr.value
        d_evk = [dev(k) for k in evk]
        d_c, d_ct = dev(c), dev(ct)
        ws = C.c_void_p()
        capi.check(lib.he_malloc(C.byref(ws), 8 * lib.he_keyswitch_workspace_words(h, L)))
        capi.check(lib.he_keyswitch(h, L, d_c, capi.evk_array(d_evk), d_ct, 0, ws.value, None))
        out = np.empty_like(ct)
        capi.check(lib.he_memcpy_d2h(out.ctypes.data, d_ct, out.nbytes, None))
        for ptr in d_evk + [d_c, d_ct, ws.value]:
            lib.he_free(ptr)
        outs.append(out)
    assert (outs[0] == outs[1]).all()


def test_c4_rotations(bench_world):
    w = bench_world
    c, ctx = w["cahel"], w["ctx"]
    base = _decode(w, w["cx"])
    for step in (1, 64, 16384):
        rot = c.ciphertext(ctx)
        c.rotate_vector(ctx, w["cx"], step, w["glk"], rot)
        err = np.abs(_decode(w, rot) - np.roll(base, -step))      # key-switch noise at scale 2^40, K = 8
        assert np.max(err) < 1e-3 and np.median(err) < 1e-6
    acc = c.ciphertext(ctx)
    c.add(ctx, w["cx"], w["cx"], acc)
    c.sub_inplace(ctx, acc, w["cx"])                     # acc = cx, as a fresh object
    tmp = c.ciphertext(ctx)
    for step in w["steps"]:
        c.rotate_vector(ctx, acc, step, w["glk"], tmp)
        c.add_inplace(ctx, acc, tmp)
    total = _decode(w, acc)
    want = float(np.sum(w["x"]))
    assert np.max(np.abs(total - want)) < 1e-5 * max(1.0, abs(want))       # measured 3.7e-6
    # hoisted rotations of one ciphertext: sum of the rotated copies
    hoisted = c.hoisting(ctx, w["cx"], w["glk"], [1, 2, 4])
    ref = sum(np.roll(base, -s) for s in (1, 2, 4))
    assert np.max(np.abs(_decode(w, hoisted) - ref)) < 1e-3 and np.median(np.abs(_decode(w, hoisted) - ref)) < 1e-6


def test_c5_krum_round_full_shape():
    """10 clients x 62,006 parameters at N = 2^16 with Lancelot's chain [60, 40, 40, 60], one special prime."""
    from lancelot_amd import krum
    rng = np.random.default_rng(2025)
    updates = [rng.normal(0.0, 0.01, 62006).astype(np.float32) for _ in range(10)]
    for k in (8, 9):
        updates[k] = updates[k] * 10
    chosen, dist, timings = krum.gpu_krum(updates, krum.KrumConfig(seed=2025))
    want = krum.plain_distance_matrix(updates)
    off = ~np.eye(10, dtype=bool)
    # 2^40 / q_last - 1 = 3.6e-6 from set_scale(2^40) after the rescale by q_last = 1099507695617, plus about 2e-6 of
    # encryption, key-switch and rotation noise relative to the smallest distances
    assert np.max(np.abs(dist[off] - want[off]) / want[off]) < 2e-5
    assert chosen == krum.krum_select(want) and chosen not in (8, 9)
    assert timings["total"] > 0


@pytest.mark.parametrize("switch", ["", "CAHEL_HIP_NO_XCD_CONTIG", "CAHEL_HIP_NO_XCD_MAP"])
def test_hoisted_rotations_batch_workgroup_orders(oracle, monkeypatch, switch):
    """N = 2^15, Lancelot's chain, 5 ciphertexts, steps 4, 8, 12 and 20 (multiples of N / 8192 but not of N / 512: the
    automorphisms stay inside aligned stretches of 4,096 words, so the launch gathers from memory and takes the workgroup
    order in which an XCD walks through such a stretch): against the oracle's hoisting item by item, with that order,
    with the plain XCD-aware one and with the plain one."""
    import ctypes as C
    from gpu_util import DeviceArray, make_pair, rand_limbs
    from lancelot_amd import capi
    if switch:
        monkeypatch.setenv(switch, "1")
    cahel, parms, ctx, p = make_pair(oracle, 15, [60, 40, 40, 60], 1)
    lib, h = capi.lib(), ctx.he_handle()
    rng = np.random.default_rng(31)
    L, items, steps = 2, 5, [4, 8, 12, 20]
    beta = L
    elts = [pow(5, s, 2 * p.n) for s in steps]
    assert all((e - 1) % 16 == 0 and (e - 1) % 256 != 0 for e in elts)
    host_keys = [[rand_limbs(p, rng, range(p.size_qp), n_polys=2) for _ in range(beta)] for _ in range(2)]
    dev_keys = [[DeviceArray(capi, host=k) for k in ks] for ks in host_keys]
    flat = capi.evk_array([dev_keys[i % 2][d].ptr for i in range(len(steps)) for d in range(beta)])
    d_elts = (C.c_uint32 * len(steps))(*elts)
    wsb = DeviceArray(capi, shape=(lib.he_keyswitch_batch_workspace_words(h, L, items),))
    cts = np.stack([rand_limbs(p, rng, range(L), n_polys=2) for _ in range(items)])
    din, dout = DeviceArray(capi, host=cts), DeviceArray(capi, shape=(items, 2, L, p.n))
    capi.check(lib.he_hoisted_rotations_batch(h, L, items, din.ptr, flat, d_elts, len(steps), 1, dout.ptr, wsb.ptr, None))
    got = dout.numpy()
    for k in range(items):
        want = p.hoisting(cts[k], elts, [host_keys[i % 2] for i in range(len(steps))])
        want = np.stack([p.add(want[b], cts[k][b]) for b in range(2)])
        assert (got[k] == want).all(), k


@pytest.mark.parametrize("kind", ["gather", "block_local"])
def test_hoisted_rotations_benchmark_shape(oracle, kind):
    """he_hoisted_rotations and he_hoisted_rotations_batch (3 ciphertexts, with and without the input added) at
    N = 2^16, L = 24, K = 8 (three digits): a step set that gathers from memory (1, 2, 3, 5) and one whose automorphisms
    stay inside 256-word blocks (multiples of N / 512 = 128), two random keys alternating between the steps, every limb
    against the oracle's hoisting (src/evaluate.cu:2412-2629)."""
    import ctypes as C
    from gpu_util import DeviceArray, make_pair, rand_limbs
    from lancelot_amd import capi
    cahel, parms, ctx, p = make_pair(oracle, 16, [50] * 32, 8)
    lib, h = capi.lib(), ctx.he_handle()
    rng = np.random.default_rng(1816)
    L, K, items = 24, 8, 3
    beta = L // K
    steps = [1, 2, 3, 5] if kind == "gather" else [128 * k for k in (1, 2, 3, 5)]
    elts = [pow(5, s, 2 * p.n) for s in steps]
    assert all(((e - 1) % 512 == 0) == (kind == "block_local") for e in elts)
    host_keys = [[rand_limbs(p, rng, range(L + K), n_polys=2) for _ in range(beta)] for _ in range(2)]
    dev_keys = [[DeviceArray(capi, host=k) for k in ks] for ks in host_keys]
    flat = capi.evk_array([dev_keys[i % 2][d].ptr for i in range(len(steps)) for d in range(beta)])
    d_elts = (C.c_uint32 * len(steps))(*elts)
    cts = np.stack([rand_limbs(p, rng, range(L), n_polys=2) for _ in range(items)])
    want = [p.hoisting(cts[k], elts, [host_keys[i % 2] for i in range(len(steps))]) for k in range(items)]
    din = DeviceArray(capi, host=cts)
    ws = DeviceArray(capi, shape=(lib.he_keyswitch_workspace_words(h, L),))
    out = DeviceArray(capi, shape=(2, L, p.n))
    capi.check(lib.he_hoisted_rotations(h, L, din.at(2 * L * p.n), flat, d_elts, len(steps), out.ptr, ws.ptr, None))
    assert (out.numpy() == want[1]).all()
    wsb = DeviceArray(capi, shape=(lib.he_keyswitch_batch_workspace_words(h, L, items),))
    dout = DeviceArray(capi, shape=(items, 2, L, p.n))
    for add_input in (0, 1):
        capi.check(lib.he_hoisted_rotations_batch(h, L, items, din.ptr, flat, d_elts, len(steps), add_input, dout.ptr,
                                                  wsb.ptr, None))
        got = dout.numpy()
        for k in range(items):
            w = want[k] if not add_input else np.stack([p.add(want[k][b], cts[k][b]) for b in range(2)])
            assert (got[k] == w).all(), (add_input, k)
    assert (din.numpy() == cts).all()


def _centred_distance(a, b, q):
    d = (a.astype(np.int64) - b.astype(np.int64)) % q
    return np.minimum(d, q - d)


@pytest.mark.parametrize("bits,size_p,slots", [([50] * 32, 8, 32768), ([50] * 32, 8, 256),
                                               ([60, 40, 40, 60], 1, 32768), ([60, 40, 40, 60], 1, 16384),
                                               ([60, 40, 40, 60], 1, 8192), ([60, 40, 40, 60], 1, 4096),
                                               ([60, 40, 40, 60], 1, 256)])
def test_encoder_at_full_degree(oracle, bits, size_p, slots):
    """he_ckks_encode / he_ckks_decode and their batch forms (he_ckks_encode_batch, he_decrypt_decode_batch) at
    N = 2^16 with all 32,768 slots (the special FFT then has 4 stages wider than a workgroup's LDS tile, which one
    kernel runs with 16 values per thread), with 16,384, 8,192 and 4,096 slots (3, 2 and 1 such stages: the other
    instances of that kernel) and with a sparse slot count that fits the tile, on 24 limbs (the general Garner composition) and on Lancelot's 3 limbs (the one templated on
    the limb count): encoded coefficients within one unit of the oracle's encoder, decoded values within 2^-20 of its
    decoder and of the message (src/ckks.cu:104-209, 292-465)."""
    import ctypes as C
    from gpu_util import DeviceArray, make_pair
    from lancelot_amd import capi
    cahel, parms, ctx, p = make_pair(oracle, 16, bits, size_p)
    lib, h = capi.lib(), ctx.he_handle()
    limbs, n, items = p.size_q, p.n, 3
    count = slots - 5
    scale = 2.0 ** 40
    rng = np.random.default_rng(slots + limbs)
    z = rng.uniform(-1, 1, (items, count)) + 1j * rng.uniform(-1, 1, (items, count))
    o_enc = oracle.Encoder(p)
    want = [o_enc.encode(z[k], scale, limbs, slots) for k in range(items)]
    want_coeff = [p.ntt_inv(w.copy()) for w in want]
    re = DeviceArray(capi, host=np.ascontiguousarray(z.real))
    im = DeviceArray(capi, host=np.ascontiguousarray(z.imag))
    ws = DeviceArray(capi, shape=(lib.he_ckks_workspace_words(h, limbs),))
    out = DeviceArray(capi, shape=(limbs, n))
    capi.check(lib.he_ckks_encode(h, re.ptr, im.ptr, count, slots, scale, limbs, out.ptr, ws.ptr, None))
    got = out.numpy()
    got_coeff = p.ntt_inv(got.copy())
    for i in range(limbs):
        assert _centred_distance(got_coeff[i], want_coeff[0][i], p.moduli[i]).max() <= 1, i
    q0 = p.moduli[0]
    centred = np.where(got_coeff[0] > q0 // 2, got_coeff[0].astype(np.int64) - q0, got_coeff[0].astype(np.int64))
    assert ws.numpy().view(np.float64)[0] == np.abs(centred).max()
    dec = DeviceArray(capi, shape=(2 * slots,), dtype=np.float64)
    capi.check(lib.he_ckks_decode(h, out.ptr, limbs, slots, scale, dec.ptr, ws.ptr, None))
    v = dec.numpy().reshape(slots, 2)
    got_z = v[:, 0] + 1j * v[:, 1]
    padded = np.zeros((items, slots), dtype=np.complex128)
    padded[:, :count] = z
    assert np.max(np.abs(got_z - o_enc.decode(got, scale, slots))) < REL
    assert np.max(np.abs(got_z - padded[0])) < REL
    # the batch forms: three messages into polynomial 0 of three ciphertexts, whose polynomial 1 is zero, so that
    # decryption returns the plaintext whatever the key
    wsb = DeviceArray(capi, shape=(lib.he_ckks_encode_batch_workspace_words(h, items),))
    cts = DeviceArray(capi, host=np.zeros((items, 2, limbs, n), dtype=np.uint64))
    capi.check(lib.he_ckks_encode_batch(h, re.ptr, im.ptr, count, slots, scale, limbs, items, count, cts.ptr,
                                        2 * limbs, wsb.ptr, None))
    got_cts = cts.numpy()
    assert (got_cts[0, 0] == got).all()                       # the batch's first item equals the single call
    assert not got_cts[:, 1].any()
    for k in range(items):
        coeff = p.ntt_inv(got_cts[k, 0].copy())
        for i in range(limbs):
            assert _centred_distance(coeff[i], want_coeff[k][i], p.moduli[i]).max() <= 1, (k, i)
    table = np.array([cts.at(k * 2 * limbs * n) for k in range(items)], dtype=np.uint64)
    d_table = DeviceArray(capi, host=table)
    sk = DeviceArray(capi, host=np.ones((limbs, n), dtype=np.uint64))
    take = min(slots, 300)
    dws = DeviceArray(capi, shape=(lib.he_decrypt_decode_batch_workspace_words(h, limbs, slots, items),))
    dout = DeviceArray(capi, shape=(items, take, 2), dtype=np.float64)
    capi.check(lib.he_decrypt_decode_batch(h, d_table.ptr, items, limbs, sk.ptr, None, slots, scale, take, dout.ptr,
                                           dws.ptr, None))
    vals = dout.numpy()
    for k in range(items):
        got_k = vals[k, :, 0] + 1j * vals[k, :, 1]
        assert np.max(np.abs(got_k - o_enc.decode(got_cts[k, 0], scale, slots)[:take])) < REL, k
        assert np.max(np.abs(got_k - padded[k, :take])) < REL, k


def test_c5_pair_distances_against_the_oracle():
    """C5 at its real shape (N = 2^16, chain [60, 40, 40, 60], one special prime, 2 chunks per client): for three of the
    pairs, the ciphertext that pair_square_distances returns against the oracle's sub -> square -> add -> relinearise
    -> rescale -> hoisted rounds on the same ciphertexts and the same seeded keys, every limb
    (lancelot-main-GPU/utils/byzantine_fl.py:173-321)."""
    from lancelot_amd import krum
    from oracle import ckks_oracle as O
    rng = np.random.default_rng(2025)
    updates = [rng.normal(0.0, 0.01, 62006).astype(np.float32) for _ in range(4)]
    updates[3] = updates[3] * 10
    cfg = krum.KrumConfig(seed=77, reproducible=True)
    state = krum.gpu_init(cfg)
    c, ctx = state.cahel, state.context
    n = 1 << cfg.log_n
    mods = O.coeff_modulus_create(n, list(cfg.modulus_bits))
    p = O.Params(cfg.log_n, mods, cfg.special_modulus_size)
    ks = O.KeySet(p, seed=cfg.seed)
    ks.gen_secret()
    ks.gen_public()
    o_rlk = ks.gen_relin()
    rounds = krum.rotate_sum_plan(cfg.log_n - 1, cfg)
    steps = sorted({s for r in rounds for s in r})
    elts = list(c.get_elts_from_steps(steps, n))
    o_glk = {e: ks.gen_galois(e) for e in elts}
    for d in range(state.rlk.digit_count()):
        assert (state.rlk.digit_to_numpy(d) == o_rlk[d]).all()
    assert state.glk.key_count() == len(elts)
    for i in (0, len(elts) // 2, len(elts) - 1):
        for d in range(state.rlk.digit_count()):
            assert (state.glk.key(i).digit_to_numpy(d) == o_glk[elts[i]][d]).all()
    cts = krum.encrypt_updates(state, krum.split_updates(updates, state.slots))
    assert len(cts[0]) == 2
    pairs = [(0, 1), (1, 3), (2, 3)]
    got = c.pair_square_distances(ctx, cts, pairs, state.rlk, state.glk, rounds, cfg.scale, 0)
    c._synchronize()
    host = [[ct.to_numpy() for ct in row] for row in cts]
    for (i, j), ct in zip(pairs, got):
        acc = None
        for a, b in zip(host[i], host[j]):
            sq = p.square(np.stack([p.sub(b[k], a[k]) for k in range(2)]))
            acc = sq if acc is None else np.stack([p.add(acc[k], sq[k]) for k in range(3)])
        r = p.rescale(p.relinearize(acc, o_rlk))
        for rnd in rounds:
            es = [elts[steps.index(s)] for s in rnd]
            hs = p.hoisting(r, es, [o_glk[e] for e in es])
            r = np.stack([p.add(r[k], hs[k]) for k in range(2)])
        assert (ct.to_numpy() == r).all(), (i, j)
    # and the decrypted distances, which are what the round reports
    values = state.sk.decrypt_decode_many(ctx, got, state.slots, 1)[:, 0]
    want = krum.plain_distance_matrix(updates)
    for (i, j), v in zip(pairs, values):
        assert abs(v - want[i, j]) / want[i, j] < 2e-5


@pytest.mark.parametrize("bits,size_p,L", [([50, 49, 50, 50, 50, 50], 2, 4), ([50, 49, 50, 50, 50, 50], 2, 3),
                                            ([60, 40, 40, 60], 1, 3)])
@pytest.mark.parametrize("no_fuse", ["0", "1"])
def test_largest_degree_entry_points_bit_exact(oracle, monkeypatch, bits, size_p, L, no_fuse):
    """N = 2^17, the largest degree of the reference's parameter tables (include/util/hestdparms.h): the rows pass has
    512 rows there (a register block of five stages), the base conversions run as kernels of their own.  he_keyswitch,
    he_keyswitch_rescale, he_multiply_relin_rescale, he_rotate and he_hoisted_rotations against the oracle, every
    limb, on the FP64 and the mixed back end, with the inner product inside the forward transform and as a kernel of
    its own, with a partial last digit."""
    import ctypes as C
    from gpu_util import DeviceArray, make_pair, rand_limbs
    from lancelot_amd import capi
    monkeypatch.setenv("CAHEL_HIP_NO_FUSED_KS", no_fuse)
    cahel, parms, ctx, p = make_pair(oracle, 17, bits, size_p)
    lib, h = capi.lib(), ctx.he_handle()
    rng = np.random.default_rng(1700 + L)
    n = p.n
    beta = -(-L // size_p)
    host_evk = [rand_limbs(p, rng, range(p.size_qp), n_polys=2) for _ in range(p.size_q // size_p)]
    dev_evk = [DeviceArray(capi, host=k) for k in host_evk]
    ptrs = capi.evk_array([d.ptr for d in dev_evk])
    a, b = rand_limbs(p, rng, range(L), n_polys=2), rand_limbs(p, rng, range(L), n_polys=2)
    da, db = DeviceArray(capi, host=a), DeviceArray(capi, host=b)
    ws = DeviceArray(capi, shape=(lib.he_multiply_relin_rescale_workspace_words(h, L),))
    # key switch of b[1] onto a, with and without the rescale
    ks = p.key_switch(b[1], host_evk[:beta])
    want_ks = np.stack([p.add(a[k], ks[k]) for k in range(2)])
    dct = DeviceArray(capi, host=a)
    capi.check(lib.he_keyswitch(h, L, db.at(L * n), ptrs, dct.ptr, 0, ws.ptr, None))
    assert (dct.numpy() == want_ks).all()
    out = DeviceArray(capi, shape=(2, L - 1, n))
    capi.check(lib.he_keyswitch_rescale(h, L, db.at(L * n), ptrs, da.ptr, out.ptr, 0, ws.ptr, None))
    assert (out.numpy() == p.rescale(want_ks)).all()
    # the whole product
    capi.check(lib.he_multiply_relin_rescale(h, L, da.ptr, db.ptr, ptrs, out.ptr, ws.ptr, None))
    assert (out.numpy() == p.rescale(p.relinearize(p.tensor(a, b), host_evk[:beta]))).all()
    # a rotation and a hoisted sum of three
    elt = pow(5, 3, 2 * n)
    rot = DeviceArray(capi, shape=(2, L, n))
    capi.check(lib.he_rotate(h, L, da.ptr, ptrs, rot.ptr, elt, ws.ptr, None))
    assert (rot.numpy() == p.apply_galois(a, elt, host_evk[:beta])).all()
    steps = [1, 256, 777]
    elts = [pow(5, s, 2 * n) for s in steps]
    flat = capi.evk_array([dev_evk[d].ptr for _ in steps for d in range(beta)])
    d_elts = (C.c_uint32 * len(steps))(*elts)
    capi.check(lib.he_hoisted_rotations(h, L, da.ptr, flat, d_elts, len(steps), rot.ptr, ws.ptr, None))
    assert (rot.numpy() == p.hoisting(a, elts, [host_evk[:beta]] * len(steps))).all()
    assert (da.numpy() == a).all() and (db.numpy() == b).all()


def test_largest_degree_scheme_flow(oracle):
    """N = 2^17 through pyCAHEL: keys, encryption of 65,536 slots, multiply + relinearize_inplace + rescale, a rotation
    and the decryption against the oracle limb for limb (same seeded randomness), decoded slots against the plain
    product."""
    O = oracle
    from gpu_util import make_pair
    logn, bits = 17, [50, 40, 40, 50, 50]
    cahel, parms, ctx, p = make_pair(O, logn, bits, 1, seed=17)
    # (make_pair builds the context without Galois elements: one of its own here)
    parms.set_galois_elts(cahel.get_elts_from_steps([5], p.n))
    ctx = cahel.context(parms, True, cahel.sec_level_type.tc128)
    ctx.set_seed(17)
    ks = O.KeySet(p, seed=17)
    sk = cahel.secret_key(parms)
    sk.gen_secretkey(ctx)
    ks.gen_secret()
    pk = cahel.public_key(ctx)
    sk.gen_publickey(ctx, pk)
    o_pk = ks.gen_public()
    rlk = cahel.relin_key(ctx)
    sk.gen_relinkey(ctx, rlk)
    o_rlk = ks.gen_relin()
    glk = cahel.galois_key(ctx)
    sk.create_galois_keys(ctx, glk)
    elt = cahel.get_elts_from_steps([5], p.n)[0]
    o_glk = ks.gen_galois(elt)
    enc = cahel.ckks_encoder(ctx)
    assert enc.slot_count() == 65536
    rng = np.random.default_rng(17)
    x, y = rng.uniform(-1, 1, p.n // 2), rng.uniform(-1, 1, p.n // 2)
    px, py = enc.encode(ctx, x, 2.0 ** 40), enc.encode(ctx, y, 2.0 ** 40)
    cx, cy = pk.encrypt_asymmetric(ctx, px), pk.encrypt_asymmetric(ctx, py)
    o_cx = ks.encrypt_asymmetric(o_pk, px.to_numpy())
    o_cy = ks.encrypt_asymmetric(o_pk, py.to_numpy())
    assert (cx.to_numpy() == o_cx).all() and (cy.to_numpy() == o_cy).all()
    prod = cahel.ciphertext(ctx)
    cahel.multiply(ctx, cx, cy, prod)
    cahel.relinearize_inplace(ctx, prod, rlk)
    cahel.rescale_to_next_inplace(ctx, prod)
    want = p.rescale(p.relinearize(p.tensor(o_cx, o_cy), o_rlk))
    assert (prod.to_numpy() == want).all()
    rot = cahel.ciphertext(ctx)
    cahel.rotate_vector(ctx, prod, 5, glk, rot)
    assert (rot.to_numpy() == p.apply_galois(want, elt, o_glk)).all()
    pt = sk.decrypt(ctx, rot)
    assert (pt.to_numpy() == ks.decrypt(p.apply_galois(want, elt, o_glk), O.gauss_cdt())).all()
    got = np.array(enc.decode(ctx, pt))
    err = np.abs(got - np.roll(x * y, -5))
    assert np.median(err) < 1e-4 and np.max(err) < 2e-2      # 2^30 of scale left; the floor-rescale bias in the first slots


@pytest.mark.parametrize("logn,bits", [(16, [60, 40, 40, 60]), (15, [60, 40, 40, 60]), (16, [50, 45, 50, 49, 50]),
                                       (15, [45, 40, 60])])
@pytest.mark.parametrize("variant", ["default", "two_rows_passes", "integer", "integer_two_rows_passes", "no_mixed"])
def test_single_limb_digits_small_launches(oracle, monkeypatch, logn, bits, variant):
    """One special prime (K = 1, Lancelot's chain): ModUp and ModDown reduce a single source limb into every other
    prime, and a launch of a few limbs runs the source's inverse rows pass inside the forward rows pass
    (CAHEL_HIP_NO_SOURCE_INTT=1 keeps the two passes apart).  he_modup, he_moddown (overwriting and adding), he_keyswitch
    with and without a Galois element and he_rotate against the oracle, limb for limb, on the mixed, FP64 and integer
    back ends (and with CAHEL_HIP_NO_MIXED=1, where the chain [45, 40, 60] transforms its sources in FP64 and their
    targets on the integer back end), at every level of the chain (src/rns.cu:610-782 ModUp / ModDown,
    src/evaluate.cu:1622-1760 key switch)."""
    import ctypes as C
    from gpu_util import DeviceArray, make_pair, rand_limbs
    from lancelot_amd import capi
    monkeypatch.setenv("CAHEL_HIP_NO_SOURCE_INTT", "1" if variant.endswith("two_rows_passes") else "0")
    monkeypatch.setenv("CAHEL_HIP_NO_FP64", "1" if variant.startswith("integer") else "0")
    monkeypatch.setenv("CAHEL_HIP_NO_MIXED", "1" if variant == "no_mixed" else "0")
    cahel, parms, ctx, p = make_pair(oracle, logn, bits, 1)
    lib, h = capi.lib(), ctx.he_handle()
    rng = np.random.default_rng(logn + len(bits))
    K, n = 1, p.n
    host_evk = [rand_limbs(p, rng, range(p.size_qp), n_polys=2) for _ in range(p.size_q)]
    dev_evk = [DeviceArray(capi, host=k) for k in host_evk]
    for L in range(p.size_q, 0, -1):
        ptrs = capi.evk_array([dev_evk[d].ptr for d in range(L)])
        tables = [p.table_index(L, t) for t in range(L + K)]
        c = rand_limbs(p, rng, range(L))
        c[:, :4] = np.array(p.moduli[:L], dtype=np.uint64)[:, None] - 1       # largest residues
        dc = DeviceArray(capi, host=c)
        dy = DeviceArray(capi, shape=(L, L + K, n))
        ws = DeviceArray(capi, shape=(2 * L, n))
        capi.check(lib.he_modup(h, L, dc.ptr, dy.ptr, ws.ptr, None))
        assert (dy.numpy() == p.modup(c)).all(), L
        assert (dc.numpy() == c).all()
        cx = np.stack([rand_limbs(p, rng, tables) for _ in range(2)])
        md = np.stack([p.moddown(cx[b]) for b in range(2)])
        dcx, dout = DeviceArray(capi, host=cx), DeviceArray(capi, shape=(2, L, n))
        capi.check(lib.he_moddown(h, L, dcx.ptr, dout.ptr, 2, 0, ws.ptr, None))
        assert (dout.numpy() == md).all(), L
        base = rand_limbs(p, rng, range(L), n_polys=2)
        dcx, dacc = DeviceArray(capi, host=cx), DeviceArray(capi, host=base)
        capi.check(lib.he_moddown(h, L, dcx.ptr, dacc.ptr, 2, 1, ws.ptr, None))
        assert (dacc.numpy() == np.stack([p.add(base[b], md[b]) for b in range(2)])).all(), L
        kws = DeviceArray(capi, shape=(lib.he_keyswitch_workspace_words(h, L),))
        ct = rand_limbs(p, rng, range(L), n_polys=2)
        for elt in (0, 5):
            dct = DeviceArray(capi, host=ct)
            capi.check(lib.he_keyswitch(h, L, dc.ptr, ptrs, dct.ptr, elt, kws.ptr, None))
            ks = p.key_switch(p.galois_ntt(c, elt) if elt else c, host_evk)
            assert (dct.numpy() == np.stack([p.add(ct[b], ks[b]) for b in range(2)])).all(), (L, elt)
        dct, drot = DeviceArray(capi, host=ct), DeviceArray(capi, shape=(2, L, n))
        elt = pow(5, 3, 2 * n)
        capi.check(lib.he_rotate(h, L, dct.ptr, ptrs, drot.ptr, elt, kws.ptr, None))
        ks = p.key_switch(p.galois_ntt(ct[1], elt), host_evk)
        assert (drot.numpy() == np.stack([p.add(p.galois_ntt(ct[0], elt), ks[0]), ks[1]])).all(), L
