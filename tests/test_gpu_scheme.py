"""pyCAHEL-level parity on the GPU: keys, encryption, evaluator and decryption against the CPU oracle.

Product and oracle draw the same seeded ChaCha20 streams in the same order, so every key and ciphertext limb
must agree word for word (integer stages: bit-exact).  Decoded slots are compared with the oracle's decode
to 2^-20 relative (encode/decode use FP64 transforms whose operation order differs), and with the plaintext
truth to the scheme's own precision.
"""
import numpy as np
import pytest

from gpu_util import make_pair

pytestmark = pytest.mark.gpu

REL = 2.0 ** -20
SEED = 2025


def rel_err(a, b):
    return float(np.max(np.abs(np.asarray(a) - np.asarray(b))) / max(1.0, float(np.max(np.abs(b)))))


@pytest.fixture(scope="module")
def world(oracle):
    """N = 2^12, 6 Q limbs + 2 special (3 digits), Galois keys for steps 1, 2, 3, -1, 4 and conjugation."""
    O = oracle
    import lancelot_amd  # noqa: F401
    import pyCAHEL as cahel
    logn, n = 12, 4096
    bits = [50, 40, 40, 40, 40, 40, 50, 50]
    steps = [1, 2, 3, -1, 0, 4]
    mods = cahel.coeff_modulus_create(n, bits)
    parms = cahel.params(cahel.scheme_type.ckks)
    parms.set_poly_modulus_degree(n)
    parms.set_coeff_modulus(mods)
    parms.set_special_modulus_size(2)
    elts = cahel.get_elts_from_steps(steps, n)
    parms.set_galois_elts(elts)
    ctx = cahel.context(parms, True, cahel.sec_level_type.none)
    ctx.set_seed(SEED)
    p = O.Params(logn, [m.value() for m in mods], 2)
    ks = O.KeySet(p, seed=SEED)
    sk = cahel.secret_key(parms)
    sk.gen_secretkey(ctx)
    o_sk = ks.gen_secret()
    pk = cahel.public_key(ctx)
    sk.gen_publickey(ctx, pk)
    o_pk = ks.gen_public()
    rlk = cahel.relin_key(ctx)
    sk.gen_relinkey(ctx, rlk)
    o_rlk = ks.gen_relin()
    glk = cahel.galois_key(ctx)
    sk.create_galois_keys(ctx, glk)
    o_glk = [ks.gen_galois(e) for e in elts]
    enc = cahel.ckks_encoder(ctx)
    return dict(cahel=cahel, parms=parms, ctx=ctx, p=p, ks=ks, sk=sk, o_sk=o_sk, pk=pk, o_pk=o_pk, rlk=rlk,
                o_rlk=o_rlk, glk=glk, o_glk=o_glk, enc=enc, o_enc=O.Encoder(p), elts=elts, steps=steps, O=O)


def test_keys_match_oracle(world):
    w = world
    assert (w["sk"].to_numpy(w["ctx"]) == w["o_sk"]).all()
    assert (w["pk"].to_numpy() == w["o_pk"]).all()
    assert w["rlk"].digit_count() == 3
    for d in range(3):
        assert (w["rlk"].digit_to_numpy(d) == w["o_rlk"][d]).all()
    assert w["glk"].key_count() == len(w["elts"])
    for i in range(len(w["elts"])):
        for d in range(3):
            assert (w["glk"].key(i).digit_to_numpy(d) == w["o_glk"][i][d]).all()


def _encrypt_both(w, values, scale=2.0 ** 40):
    pt = w["enc"].encode(w["ctx"], values, scale)
    o_pt = w["o_enc"].encode(values, scale, w["p"].size_q)
    ct = w["pk"].encrypt_asymmetric(w["ctx"], pt)
    o_ct = w["ks"].encrypt_asymmetric(w["o_pk"], pt.to_numpy())   # same plaintext limbs on both sides
    return pt, o_pt, ct, o_ct


def _encrypt_product_only(w, values, scale=2.0 ** 40):
    """Encrypts on the GPU only and advances the oracle's stream counter by the three streams it used."""
    ct = w["pk"].encrypt_asymmetric(w["ctx"], w["enc"].encode(w["ctx"], values, scale))
    w["ks"].stream += 3
    return ct


def test_encode_matches_oracle(world):
    w = world
    rng = np.random.default_rng(1)
    z = rng.uniform(-1, 1, w["p"].n // 2)
    pt = w["enc"].encode(w["ctx"], z, 2.0 ** 40)
    o_pt = w["o_enc"].encode(z, 2.0 ** 40, w["p"].size_q)
    # rounding of the FP64 transform may differ by one unit in a coefficient; compare decoded values
    got = np.array(w["enc"].decode(w["ctx"], pt))
    assert rel_err(got, w["o_enc"].decode(o_pt, 2.0 ** 40).real) < REL
    assert rel_err(got, z) < REL
    coeff_diff = w["p"].ntt_inv(pt.to_numpy().copy())[0].astype(np.int64) - w["p"].ntt_inv(o_pt.copy())[0].astype(np.int64)
    assert np.max(np.abs(coeff_diff)) <= 1


def test_encrypt_multiply_relin_rescale_bit_exact(world):
    w = world
    c, ctx, p = w["cahel"], w["ctx"], w["p"]
    rng = np.random.default_rng(2)
    x, y = rng.uniform(-1, 1, p.n // 2), rng.uniform(-1, 1, p.n // 2)
    _, _, cx, o_cx = _encrypt_both(w, x)
    _, _, cy, o_cy = _encrypt_both(w, y)
    assert (cx.to_numpy() == o_cx).all() and (cy.to_numpy() == o_cy).all()
    prod = c.ciphertext(ctx)
    c.multiply(ctx, cx, cy, prod)
    o_t = p.tensor(o_cx, o_cy)
    assert prod.size() == 3 and (prod.to_numpy() == o_t).all()
    c.relinearize_inplace(ctx, prod, w["rlk"])
    o_r = p.relinearize(o_t, w["o_rlk"])
    assert prod.size() == 2 and (prod.to_numpy() == o_r).all()
    c.rescale_to_next_inplace(ctx, prod)
    o_s = p.rescale(o_r)
    assert prod.chain_index() == 2 and (prod.to_numpy() == o_s).all()
    assert prod.scale() == (2.0 ** 80) / p.moduli[p.size_q - 1]
    # decrypt (with the seeded flooding noise) and decode
    pt = w["sk"].decrypt(ctx, prod)
    o_pt = w["ks"].decrypt(o_s, w["O"].gauss_cdt())
    assert (pt.to_numpy() == o_pt).all()
    got = np.array(w["enc"].decode(ctx, pt))
    want = w["o_enc"].decode(o_pt, prod.scale()).real
    assert rel_err(got, want) < REL
    assert np.max(np.abs(got - x * y)) < 1e-5          # cahel-main/unittest/evaluator.cu:419-472 bound
    # relinearise + rescale in one call: the same limbs
    both = c.ciphertext(ctx)
    c.multiply(ctx, cx, cy, both)
    c.relinearize_rescale_inplace(ctx, both, w["rlk"])
    assert both.size() == 2 and both.chain_index() == 2 and both.scale() == prod.scale()
    assert (both.to_numpy() == o_s).all()
    # square, multiply_and_relin_inplace
    sq = c.ciphertext(ctx)
    c.square(ctx, cx, sq)
    assert (sq.to_numpy() == p.square(o_cx)).all()
    c.multiply_and_relin_inplace(ctx, cx, cy, w["rlk"])
    assert (cx.to_numpy() == o_r).all()


def test_deferred_relinearisation_is_invisible(world):
    """relinearize_inplace defers its key switch so that a rescale_to_next right after it does both in one device call
    (the reference's callers run the two back to back, lancelot-main-GPU/utils/byzantine_fl.py:254-256).  Whatever is
    done with the ciphertext between or instead of the two calls, the limbs are the oracle's: rescale at once, a read in
    between, a copy, an addition, a rescale into another object, a key that is dropped before the switch has run, and a
    destination that still had a switch pending."""
    w = world
    c, ctx, p = w["cahel"], w["ctx"], w["p"]
    rng = np.random.default_rng(33)
    x, y = rng.uniform(-1, 1, p.n // 2), rng.uniform(-1, 1, p.n // 2)
    _, _, cx, o_cx = _encrypt_both(w, x)
    _, _, cy, o_cy = _encrypt_both(w, y)
    o_t = p.tensor(o_cx, o_cy)
    o_r = p.relinearize(o_t, w["o_rlk"])
    o_s = p.rescale(o_r)

    def product():
        prod = c.ciphertext(ctx)
        c.multiply(ctx, cx, cy, prod)
        c.relinearize_inplace(ctx, prod, w["rlk"])
        assert prod.size() == 2 and prod._has_pending_key_switch()
        return prod

    a = product()                                   # the reference's sequence, nothing in between
    c.rescale_to_next_inplace(ctx, a)
    assert not a._has_pending_key_switch() and a.chain_index() == 2 and (a.to_numpy() == o_s).all()
    b = product()                                   # a read in between
    assert (b.to_numpy() == o_r).all() and not b._has_pending_key_switch()
    c.rescale_to_next_inplace(ctx, b)
    assert (b.to_numpy() == o_s).all()
    d = product()                                   # a copy, then the original goes on
    e = d.copy()
    assert (e.to_numpy() == o_r).all() and not e._has_pending_key_switch()
    c.rescale_to_next_inplace(ctx, d)
    assert (d.to_numpy() == o_s).all()
    f = product()                                   # an addition
    c.add_inplace(ctx, f, e)
    assert (f.to_numpy() == np.stack([p.add(o_r[k], o_r[k]) for k in range(2)])).all()
    g, h = product(), c.ciphertext(ctx)             # rescale into another object; the source is still the relinearised product
    c.rescale_to_next(ctx, g, h)
    assert (h.to_numpy() == o_s).all() and h.chain_index() == 2 and g.chain_index() == 1
    assert (g.to_numpy() == o_r).all()
    with pytest.raises(ValueError, match="destination_size must be 3"):
        c.relinearize_inplace(ctx, product(), w["rlk"])
    # a second key, dropped while its switch is pending
    rlk2 = c.relin_key(ctx)
    w["sk"].gen_relinkey(ctx, rlk2)
    o_rlk2 = w["ks"].gen_relin()
    i = c.ciphertext(ctx)
    c.multiply(ctx, cx, cy, i)
    c.relinearize_inplace(ctx, i, rlk2)
    del rlk2
    c._trim_pool()
    junk = [c.ciphertext(ctx) for _ in range(3)]
    for ct in junk:
        c.multiply(ctx, cy, cy, ct)                 # allocations that would reuse the key's blocks had they been freed
    c.rescale_to_next_inplace(ctx, i)
    assert (i.to_numpy() == p.rescale(p.relinearize(o_t, o_rlk2))).all()
    # a destination with a switch pending is overwritten as a whole
    j = product()
    c.multiply(ctx, cx, cy, j)
    assert j.size() == 3 and not j._has_pending_key_switch() and (j.to_numpy() == o_t).all()
    k = product()
    c.sub(ctx, cx, cy, k)
    assert (k.to_numpy() == np.stack([p.sub(o_cx[b], o_cy[b]) for b in range(2)])).all()
    # a copy of a key owns plain blocks: the switch runs at once, same limbs
    m = c.ciphertext(ctx)
    c.multiply(ctx, cx, cy, m)
    c.relinearize_inplace(ctx, m, w["rlk"].copy())
    assert not m._has_pending_key_switch()
    c.rescale_to_next_inplace(ctx, m)
    assert (m.to_numpy() == o_s).all()


def test_add_sub_negate_plain_ops(world):
    w = world
    c, ctx, p = w["cahel"], w["ctx"], w["p"]
    rng = np.random.default_rng(3)
    x, y = rng.uniform(-1, 1, p.n // 2), rng.uniform(-1, 1, p.n // 2)
    pt_x, _, cx, o_cx = _encrypt_both(w, x)
    pt_y, _, cy, o_cy = _encrypt_both(w, y)
    out = c.ciphertext(ctx)
    both = lambda f: np.stack([f(o_cx[i], o_cy[i]) for i in range(2)])
    c.add(ctx, cx, cy, out)
    assert (out.to_numpy() == both(p.add)).all()
    c.sub(ctx, cx, cy, out)
    assert (out.to_numpy() == both(p.sub)).all()
    # sub with destination aliasing the second operand (include/evaluate.h:52-61)
    alias = cy.copy()
    c.sub(ctx, cx, alias, alias)
    assert (alias.to_numpy() == both(p.sub)).all()
    c.negate(ctx, cx, out)
    assert (out.to_numpy() == np.stack([p.negate(o_cx[i]) for i in range(2)])).all()
    c.add_many(ctx, [cx, cy, cx], out)
    assert (out.to_numpy() == np.stack([p.add(p.add(o_cx[i], o_cy[i]), o_cx[i]) for i in range(2)])).all()
    c.add_plain(ctx, cx, pt_y, out)
    assert (out.to_numpy() == np.stack([p.add(o_cx[0], pt_y.to_numpy()), o_cx[1]])).all()
    c.sub_plain(ctx, cx, pt_y, out)
    assert (out.to_numpy() == np.stack([p.sub(o_cx[0], pt_y.to_numpy()), o_cx[1]])).all()
    c.multiply_plain(ctx, cx, pt_y, out)
    assert (out.to_numpy() == np.stack([p.mul(o_cx[i], pt_y.to_numpy()) for i in range(2)])).all()
    assert out.scale() == 2.0 ** 80
    # size-3 accumulation used by the lazy relinearisation of the Krum protocol
    s1, s2 = c.ciphertext(ctx), c.ciphertext(ctx)
    c.square(ctx, cx, s1)
    c.square(ctx, cy, s2)
    c.add_inplace(ctx, s1, s2)
    o3 = np.stack([p.add(p.square(o_cx)[i], p.square(o_cy)[i]) for i in range(3)])
    assert (s1.to_numpy() == o3).all()


@pytest.mark.parametrize("step", [1, 3, -1])
def test_rotate_bit_exact(world, step):
    w = world
    c, ctx, p = w["cahel"], w["ctx"], w["p"]
    rng = np.random.default_rng(4)
    z = rng.uniform(-1, 1, p.n // 2)
    _, _, ct, o_ct = _encrypt_both(w, z)
    out = c.ciphertext(ctx)
    c.rotate_vector(ctx, ct, step, w["glk"], out)
    idx = w["steps"].index(step)
    o_out = p.apply_galois(o_ct, w["elts"][idx], w["o_glk"][idx])
    assert (out.to_numpy() == o_out).all()
    w["sk"].set_noise_flooding(False)
    got = np.array(w["enc"].decode(ctx, w["sk"].decrypt(ctx, out)))
    w["sk"].set_noise_flooding(True)
    assert np.max(np.abs(got - np.roll(z, -step))) < 1e-6


def test_rotate_after_rescale_and_conjugate(world):
    """Key switching at a lower level (L = 5: digits of 2, 2 and 1 limbs) and the conjugation key."""
    w = world
    c, ctx, p = w["cahel"], w["ctx"], w["p"]
    rng = np.random.default_rng(5)
    z = rng.uniform(-1, 1, p.n // 2)
    _, _, ct, o_ct = _encrypt_both(w, z)
    c.mod_switch_to_next_inplace(ctx, ct)
    o_ct = np.ascontiguousarray(o_ct[:, :5])
    assert ct.chain_index() == 2 and (ct.to_numpy() == o_ct).all()
    c.rotate_vector_inplace(ctx, ct, 2, w["glk"])
    idx = w["steps"].index(2)
    assert (ct.to_numpy() == p.apply_galois(o_ct, w["elts"][idx], w["o_glk"][idx])).all()
    conj = c.ciphertext(ctx)
    c.complex_conjugate(ctx, ct, w["glk"], conj)
    ci = w["steps"].index(0)
    assert (conj.to_numpy() == p.apply_galois(ct.to_numpy(), w["elts"][ci], w["o_glk"][ci])).all()


def test_rotate_naf_fallback(world):
    """No key for step 5: the rotation is split into the signed powers of two 1 + 4 (src/evaluate.cu:2395-2408)."""
    w = world
    c, ctx, p = w["cahel"], w["ctx"], w["p"]
    assert c._naf(5) == [1, 4] and c._naf(-3) == [1, -4] and c._naf(127) == [-1, 128] and c._naf(0) == []
    rng = np.random.default_rng(8)
    z = rng.uniform(-1, 1, p.n // 2)
    _, _, ct, o_ct = _encrypt_both(w, z)
    out = c.ciphertext(ctx)
    c.rotate_vector(ctx, ct, 5, w["glk"], out)
    for s in (1, 4):
        i = w["steps"].index(s)
        o_ct = p.apply_galois(o_ct, w["elts"][i], w["o_glk"][i])
    assert (out.to_numpy() == o_ct).all()


def test_rotate_missing_power_of_two_raises(world):
    w = world
    c, ctx = w["cahel"], w["ctx"]
    ct = _encrypt_product_only(w, np.zeros(w["p"].n // 2))
    with pytest.raises(ValueError, match="Galois key not present"):
        c.rotate_vector_inplace(ctx, ct, 64, w["glk"])


def test_hoisting_bit_exact(world):
    w = world
    c, ctx, p = w["cahel"], w["ctx"], w["p"]
    rng = np.random.default_rng(6)
    z = rng.uniform(-1, 1, p.n // 2)
    _, _, ct, o_ct = _encrypt_both(w, z)
    assert (ct.to_numpy() == o_ct).all()
    steps = [1, 2, 3]
    out = c.hoisting(ctx, ct, w["glk"], steps)
    idxs = [w["steps"].index(s) for s in steps]
    o_out = p.hoisting(o_ct, [w["elts"][i] for i in idxs], [w["o_glk"][i] for i in idxs])
    assert (out.to_numpy() == o_out).all()
    w["sk"].set_noise_flooding(False)
    got = np.array(w["enc"].decode(ctx, w["sk"].decrypt(ctx, out)))
    w["sk"].set_noise_flooding(True)
    assert np.max(np.abs(got - sum(np.roll(z, -s) for s in steps))) < 1e-6
    with pytest.raises(RuntimeError, match="Galois key not present in hoisting"):
        c.hoisting(ctx, ct, w["glk"], [7])


def test_encrypt_symmetric_bit_exact_and_round_trip(world):
    """secret_key.encrypt_symmetric (src/secretkey.cu:517-560 over encrypt_zero_symmetric :451-515, NTT branch) at
    the first data level: (-(a s + e) + m, a) with e and a drawn from the next two seeded streams, limb for limb
    against the oracle's samplers and arithmetic; decrypts back to the message."""
    w = world
    c, ctx, p, ks = w["cahel"], w["ctx"], w["p"], w["ks"]
    rng = np.random.default_rng(17)
    z = rng.uniform(-1, 1, p.n // 2)
    pt = w["enc"].encode(ctx, z, 2.0 ** 40)
    ct = w["sk"].encrypt_symmetric(ctx, pt, False)
    L = p.size_q
    e = p.ntt_fwd(p.sample_error(ks.key, ks._next(), L))
    a = p.sample_uniform(ks.key, ks._next(), L)
    c0 = p.add(p.mul_add(a, np.ascontiguousarray(w["o_sk"][:L]), e, negate=True), pt.to_numpy())
    got = ct.to_numpy()
    assert ct.size() == 2 and ct.chain_index() == 1 and ct.scale() == 2.0 ** 40
    assert (got[1] == a).all() and (got[0] == c0).all()
    w["sk"].set_noise_flooding(False)
    try:
        back = np.array(w["enc"].decode(ctx, w["sk"].decrypt(ctx, ct)))
    finally:
        w["sk"].set_noise_flooding(True)
    assert rel_err(back, z) < REL


def test_multiply_with_size_three_operands(world):
    """multiply / square of ciphertexts that were not relinearised (size 3): the general tensor product of
    src/evaluate.cu:474-488, 531-545.  Limbs against the oracle, and the size-5 results decrypt (c0 + c1 s + ... +
    c4 s^4) to the product of the slots; a size-5 operand squares to 9 polynomials.  As in the reference, operands of
    different sizes are refused
    (src/evaluate.cu:369-370)."""
    w = world
    c, ctx, p = w["cahel"], w["ctx"], w["p"]
    rng = np.random.default_rng(21)
    x, y, z, v = (rng.uniform(-1, 1, p.n // 2) for _ in range(4))
    scale = 2.0 ** 25
    _, _, cx, o_cx = _encrypt_both(w, x, scale)
    _, _, cy, o_cy = _encrypt_both(w, y, scale)
    _, _, cz, o_cz = _encrypt_both(w, z, scale)
    _, _, cv, o_cv = _encrypt_both(w, v, scale)
    xy, zv = c.ciphertext(ctx), c.ciphertext(ctx)
    c.multiply(ctx, cx, cy, xy)
    c.multiply(ctx, cz, cv, zv)
    o_xy, o_zv = p.tensor(o_cx, o_cy), p.tensor(o_cz, o_cv)
    same_scale = _encrypt_product_only(w, z, scale * scale)
    with pytest.raises(ValueError, match="poly number mismatch"):
        c.multiply_inplace(ctx, xy, same_scale)
    prod = c.ciphertext(ctx)
    c.multiply(ctx, xy, zv, prod)
    assert prod.size() == 5 and (prod.to_numpy() == p.tensor_mxn(o_xy, o_zv)).all()
    assert prod.scale() == scale ** 4
    w["sk"].set_noise_flooding(False)
    try:
        got = np.array(w["enc"].decode(ctx, w["sk"].decrypt(ctx, prod)))
        assert np.max(np.abs(got - x * y * z * v)) < 1e-3
        # squaring a size-3 ciphertext in place
        c.square_inplace(ctx, xy)
        assert xy.size() == 5 and (xy.to_numpy() == p.tensor_mxn(o_xy, o_xy)).all()
        got = np.array(w["enc"].decode(ctx, w["sk"].decrypt(ctx, xy)))
        assert np.max(np.abs(got - (x * y) ** 2)) < 1e-3
        # and once more: 5 x 5 polynomials take the general kernel (operands read in place), 9 come back
        o_xy2 = p.tensor_mxn(o_xy, o_xy)
        c.square_inplace(ctx, xy)
        assert xy.size() == 9 and (xy.to_numpy() == p.tensor_mxn(o_xy2, o_xy2)).all()
        got = np.array(w["enc"].decode(ctx, w["sk"].decrypt(ctx, xy)))
        assert np.max(np.abs(got - (x * y) ** 4)) < 1e-2
    finally:
        w["sk"].set_noise_flooding(True)


def test_error_behaviour(world):
    w = world
    c, ctx, p = w["cahel"], w["ctx"], w["p"]
    z = np.ones(p.n // 2)
    a = _encrypt_product_only(w, z)
    b = _encrypt_product_only(w, z, 2.0 ** 30)
    with pytest.raises(ValueError, match="scale mismatch"):
        c.add_inplace(ctx, a, b)
    with pytest.raises(ValueError, match="destination_size must be 3"):
        c.relinearize_inplace(ctx, a, w["rlk"])
    lower = a.copy()
    c.mod_switch_to_inplace(ctx, lower, 3)
    assert lower.chain_index() == 3 and lower.coeff_modulus_size() == 4
    with pytest.raises(ValueError, match="parameter mismatch"):
        c.add_inplace(ctx, a, lower)
    with pytest.raises(ValueError, match="cannot switch to higher level modulus"):
        c.mod_switch_to_inplace(ctx, lower, 1)
    with pytest.raises(RuntimeError, match="unsupported scheme"):
        c.rotate_rows_inplace(ctx, a, 1, w["glk"])
    with pytest.raises(RuntimeError, match="unsupported scheme"):
        c.multiply_many(ctx, [a, a], w["rlk"], a)
    last = a.copy()
    c.mod_switch_to_inplace(ctx, last, 6)
    with pytest.raises(ValueError, match="end of modulus switching chain reached"):
        c.rescale_to_next_inplace(ctx, last)
    sq = a.copy()
    c.square_inplace(ctx, sq)
    with pytest.raises(ValueError, match="ciphertext size must be 2"):
        c.hoisting(ctx, sq, w["glk"], [1])
    with pytest.raises(ValueError, match="values_size is too large"):
        w["enc"].encode(ctx, np.zeros(p.n), 2.0 ** 40)


def test_lancelot_smoke_script_flow(oracle):
    """The sequence of lancelot-main-GPU/ckks.py:1-57 with its parameters, checked against the closed form."""
    import lancelot_amd  # noqa: F401
    import pyCAHEL as cahel
    n = 2 ** 13
    scale = 2.0 ** 40
    params = cahel.params(cahel.scheme_type.ckks)
    params.set_poly_modulus_degree(n)
    params.set_coeff_modulus(cahel.coeff_modulus_create(n, [60, 40, 40, 60]))
    params.set_special_modulus_size(1)
    params.set_galois_elts(cahel.get_elts_from_steps([-2], n))
    context = cahel.context(params, True, cahel.sec_level_type.tc128)
    sk = cahel.secret_key(params)
    sk.gen_secretkey(context)
    pk = cahel.public_key(context)
    sk.gen_publickey(context, pk)
    rlk = cahel.relin_key(context)
    sk.gen_relinkey(context, rlk)
    glk = cahel.galois_key(context)
    sk.create_galois_keys(context, glk)
    encoder = cahel.ckks_encoder(context)
    slot_count = encoder.slot_count()
    msg = [1.0, 2.0, 3.0, 4.0] + [0.0] * (slot_count - 4)
    ct = pk.encrypt_asymmetric(context, encoder.encode(context, msg, scale))
    cahel.square_inplace(context, ct)
    cahel.relinearize_inplace(context, ct, rlk)
    cahel.rescale_to_next_inplace(context, ct)
    pt_2 = encoder.encode_to(context, [2.0] * slot_count, 2, scale)
    ct.set_scale(scale)
    cahel.multiply_plain_inplace(context, ct, pt_2)
    cahel.rescale_to_next_inplace(context, ct)
    cahel.add_inplace(context, ct, ct)
    cahel.rotate_vector_inplace(context, ct, -2, glk)
    result = encoder.decode(context, sk.decrypt(context, ct))
    want = np.roll(4.0 * np.array(msg) ** 2, 2)
    assert np.max(np.abs(np.array(result) - want)) < 1e-3
    assert ["%.1f" % abs(v) for v in result[:6]] == ["0.0", "0.0", "4.0", "16.0", "36.0", "64.0"]


def test_encrypted_krum_small(oracle):
    """Encrypted Krum distances on 4 clients x 5000 parameters (2 chunks at N = 2^13) against float64."""
    from lancelot_amd import krum
    rng = np.random.default_rng(7)
    updates = [rng.normal(0, 0.01, 5000).astype(np.float32) for _ in range(4)]
    updates[3] = updates[3] * 10
    cfg = krum.KrumConfig(log_n=13, modulus_bits=(60, 40, 40, 60), special_modulus_size=1, seed=11, reproducible=True)
    chosen, dist, timings = krum.gpu_krum(updates, cfg)
    want = krum.plain_distance_matrix(updates)
    # the budget is dominated by the driver's set_scale(2^40) after the rescale (byzantine_fl.py:256): the true scale
    # is 2^80 / q_last, so every distance carries the relative offset 2^40 / q_last - 1 (a few 1e-6 for a 40-bit
    # prime); encryption and key-switch noise add about 1e-6 more
    assert rel_err(dist, want) < 2e-5
    assert chosen == krum.krum_select(want) and chosen != 3
    # pair by pair over the lanes instead of all pairs at once: the same ciphertexts, so the same values up to the
    # flooding noise of the decryptions
    cfg_pairs = krum.KrumConfig(log_n=13, modulus_bits=(60, 40, 40, 60), special_modulus_size=1, seed=11,
                                reproducible=True, batched=False)
    chosen1, dist1, _ = krum.gpu_krum(updates, cfg_pairs)
    assert chosen1 == chosen and rel_err(dist1, dist) < 1e-6
    # the slot sum as doublings only, and as the reference's split (hoisting(1..15), then doublings)
    for variant in (dict(hoisting=False), dict(hoisting_radix=0), dict(hoisting=False, batched=False)):
        plain = krum.KrumConfig(log_n=13, modulus_bits=(60, 40, 40, 60), special_modulus_size=1, seed=11, **variant)
        chosen2, dist2, _ = krum.gpu_krum(updates, plain)
        assert chosen2 == chosen and rel_err(dist2, want) < 2e-5
    assert {"encode", "encrypt", "evaluate", "decrypt", "total"} <= set(timings)
    # the pairs are spread over streams by default; on the null stream alone the ciphertexts are the same, and the
    # decryptions differ only by which flooding-noise sample each of them drew (the threads share one counter)
    serial = krum.KrumConfig(log_n=13, modulus_bits=(60, 40, 40, 60), special_modulus_size=1, seed=11, lanes=0, reproducible=True, batched=False)
    chosen3, dist3, _ = krum.gpu_krum(updates, serial)
    assert chosen3 == chosen and rel_err(dist3, dist1) < 1e-6


def test_batched_pair_distances_equal_the_pairwise_ciphertexts(oracle):
    """pair_square_distances (every stage one launch for all pairs) against sub / square / add / relinearise +
    rescale / hoisting per pair: the same limbs."""
    from lancelot_amd import krum
    rng = np.random.default_rng(9)
    updates = [rng.normal(0, 0.01, 3000).astype(np.float32) for _ in range(3)]
    cfg = krum.KrumConfig(log_n=12, modulus_bits=(60, 40, 40, 60), special_modulus_size=1, seed=13, reproducible=True,
                          hoisting_radix=8, lanes=0, sec_level="none")
    state = krum.gpu_init(cfg)
    cts = krum.encrypt_updates(state, krum.split_updates(updates, state.slots))
    assert len(cts[0]) == 2
    pairs = [(0, 1), (0, 2), (1, 2), (2, 0)]
    rounds = krum.rotate_sum_plan(11, cfg)
    assert [len(r) for r in rounds] == [3, 7, 7, 7]   # the short round first, block-local rounds last
    c = state.cahel
    batch = c.pair_square_distances(state.context, cts, pairs, state.rlk, state.glk, rounds, cfg.scale)
    c._synchronize()
    for (i, j), got in zip(pairs, batch):
        want = krum.pair_distance(state, cts[i], cts[j])
        assert got.chain_index() == want.chain_index() and got.scale() == want.scale()
        assert (got.to_numpy() == want.to_numpy()).all(), (i, j)
    # the slot sum one level further down
    state.config.sum_drop_levels = 1
    low = c.pair_square_distances(state.context, cts, pairs[:2], state.rlk, state.glk, rounds, cfg.scale, 1)
    for (i, j), got in zip(pairs, low):
        want = krum.pair_distance(state, cts[i], cts[j])
        assert got.chain_index() == want.chain_index() == batch[0].chain_index() + 1
        assert (got.to_numpy() == want.to_numpy()).all(), (i, j)
    decoded = state.sk.decrypt_decode_many(state.context, low, state.slots, 1)[:, 0]
    plain = krum.plain_distance_matrix(updates)
    assert abs(decoded[0] - plain[0, 1]) < 1e-3 * plain[0, 1] and abs(decoded[1] - plain[0, 2]) < 1e-3 * plain[0, 2]
    with pytest.raises(ValueError, match="end of modulus switching chain"):
        c.pair_square_distances(state.context, cts, pairs[:1], state.rlk, state.glk, rounds, cfg.scale, 2)
    state.config.sum_drop_levels = 0
    assert c.pair_square_distances(state.context, cts, [], state.rlk, state.glk, rounds, 0.0) == []
    with pytest.raises(ValueError, match="pair out of range"):
        c.pair_square_distances(state.context, cts, [(0, 3)], state.rlk, state.glk, rounds, 0.0)
    with pytest.raises(RuntimeError, match="Galois key not present"):
        c.pair_square_distances(state.context, cts, pairs, state.rlk, state.glk, [[9]], 0.0)


def test_encode_encrypt_many_equals_one_by_one(oracle):
    """ckks_encoder.encode_encrypt_many against encode + encrypt_asymmetric item by item on a context with the same
    seed: the same ciphertexts (item k draws the stream ids that the k-th single encryption draws)."""
    from lancelot_amd import krum
    rng = np.random.default_rng(22)
    updates = [rng.normal(0, 0.01, 9000).astype(np.float32) for _ in range(3)]     # 3 chunks of 4096 slots, the last ragged
    base = dict(log_n=13, modulus_bits=(60, 40, 40, 60), special_modulus_size=1, seed=14)
    many = krum.gpu_init(krum.KrumConfig(batched=True, **base))
    single = krum.gpu_init(krum.KrumConfig(batched=False, reproducible=True, **base))
    cts_many = krum.encrypt_updates(many, krum.split_updates(updates, many.slots))
    cts_single = krum.encrypt_updates(single, krum.split_updates(updates, single.slots))
    assert len(cts_many) == 3 and len(cts_many[0]) == 3
    for a_row, b_row in zip(cts_many, cts_single):
        for a, b in zip(a_row, b_row):
            assert a.chain_index() == b.chain_index() and a.scale() == b.scale()
            assert (a.to_numpy() == b.to_numpy()).all()
    # a matrix that is not the one of split_updates, and the argument checks
    c, ctx = many.cahel, many.context
    cts = many.encoder.encode_encrypt_many(ctx, many.pk, np.ones((2, 100)), 2.0 ** 40)
    got = many.sk.decrypt_decode_many(ctx, cts, many.slots, 101)
    assert np.max(np.abs(got[:, :100] - 1.0)) < 1e-6 and np.max(np.abs(got[:, 100])) < 1e-6
    with pytest.raises(ValueError, match="two-dimensional"):
        many.encoder.encode_encrypt_many(ctx, many.pk, np.ones(8), 2.0 ** 40)
    with pytest.raises(ValueError, match="too large"):
        many.encoder.encode_encrypt_many(ctx, many.pk, np.full((1, 8), 1e30), 2.0 ** 40)


def test_decrypt_decode_many_equals_one_by_one(world):
    """secret_key.decrypt_decode_many against decrypt + decode_array per ciphertext: identical without the flooding
    noise, within its size with it (the batch draws the stream ids that the single calls would)."""
    w = world
    c, ctx = w["cahel"], w["ctx"]
    rng = np.random.default_rng(21)
    slots = w["p"].n // 2
    cts = [_encrypt_both(w, rng.uniform(-1, 1, slots))[2] for _ in range(5)]
    c.rotate_vector_inplace(ctx, cts[3], 1, w["glk"])
    w["sk"].set_noise_flooding(False)
    one = np.stack([w["enc"].decode_array(ctx, w["sk"].decrypt(ctx, ct), 7) for ct in cts])
    many = w["sk"].decrypt_decode_many(ctx, cts, slots, 7)
    assert many.shape == (5, 7) and (many == one).all()
    w["sk"].set_noise_flooding(True)
    noisy = w["sk"].decrypt_decode_many(ctx, cts, slots, 7)
    assert 0 < np.max(np.abs(noisy - one)) < 1e-6
    assert w["sk"].decrypt_decode_many(ctx, [], slots, 1).shape == (0, 1)
    with pytest.raises(ValueError, match="slot count out of range"):
        w["sk"].decrypt_decode_many(ctx, cts, slots, slots + 1)
    other = c.ciphertext(ctx)
    c.multiply(ctx, cts[0], cts[1], other)          # size 3
    with pytest.raises(ValueError, match="encrypted is not valid"):
        w["sk"].decrypt_decode_many(ctx, [cts[0], other], slots, 1)


def test_encrypted_krum_aggregate_small(oracle):
    """Distances, decrypt-sort-mask and the masked sum: the aggregate is the chosen client's update."""
    from lancelot_amd import krum
    rng = np.random.default_rng(8)
    updates = [rng.normal(0, 0.01, 5000).astype(np.float32) for _ in range(4)]
    updates[1] = updates[1] * 10
    cfg = krum.KrumConfig(log_n=13, modulus_bits=(60, 40, 40, 60), special_modulus_size=1, seed=12)
    chosen, weights, timings = krum.gpu_krum_aggregate(updates, cfg)
    want = krum.krum_select(krum.plain_distance_matrix(updates))
    assert chosen == want and chosen != 1
    assert weights.shape == (5000,)
    assert np.max(np.abs(weights - updates[chosen].astype(np.float64))) < 1e-5
    assert {"mask", "mask_multiply", "evaluate", "total"} <= set(timings)
