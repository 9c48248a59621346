"""End-to-end checks of the oracle's CKKS composition (encoder, keys, key switching).

Pinned by scheme invariants rather than by vectors (the reference's randomness comes from
/dev/urandom and cannot be reproduced): the canonical embedding m(zeta^(5^j)) = scale * z_j for the
encoder (src/ckks.cu:104-209), Dec(relin(ct)) = Dec(ct) up to key-switch noise, Dec(rot(ct, k)) =
roll(Dec(ct), -k) with generator 5 (include/galois.cuh:11), hoisting = sum of single rotations
(src/evaluate.cu:2412-2629), and the reference's own acceptance bound for multiply+relinearize
|error| < 1e-5 (unittest/evaluator.cu:419-472).
"""
import numpy as np
import pytest


@pytest.fixture(scope="module")
def ctx(oracle):
    O = oracle
    n, logn = 1 << 11, 11
    mods = O.coeff_modulus_create(n, [50, 40, 40, 40, 40, 40, 50, 50])
    p = O.Params(logn, mods, 2)     # 6 Q limbs (3 digits of 2), 2 special; dnum = size_q / size_p
                                    # must be exact (include/secretkey.h:141-144)
    ks = O.KeySet(p, seed=2025)
    ks.gen_secret()
    pk = ks.gen_public()
    rlk = ks.gen_relin()
    enc = O.Encoder(p)
    return O, p, ks, pk, rlk, enc


def test_encoder_canonical_embedding(oracle):
    O = oracle
    logn, n = 7, 128
    p = O.Params(logn, O.get_primes(n, 50, 2), 1)
    enc = O.Encoder(p)
    rng = np.random.default_rng(1)
    z = rng.uniform(-1, 1, n // 2) + 1j * rng.uniform(-1, 1, n // 2)
    scale = 2.0 ** 30
    coeffs = enc.encode_coeffs(z, scale)
    zeta = np.exp(1j * np.pi / n)
    for j in range(n // 2):
        x = zeta ** pow(5, j, 2 * n)
        val = np.polyval(coeffs[::-1], x)
        assert abs(val / scale - z[j]) < 1e-6
    # real input gives a real polynomial whose conjugate slots hold conj(z): coefficients are real by construction
    pt = enc.encode(z, scale, 1)
    back = enc.decode(pt, scale)
    assert np.max(np.abs(back - z)) < 1e-6


def test_encoder_sparse_and_constants(oracle):
    O = oracle
    logn, n = 7, 128
    p = O.Params(logn, O.get_primes(n, 50, 2), 1)
    enc = O.Encoder(p)
    scale = 2.0 ** 30
    # a constant vector encodes to the constant polynomial
    c = enc.encode_coeffs([0.5] * (n // 2), scale)
    assert c[0] == round(0.5 * scale) and not c[1:].any()
    # 4 sparse slots: the message repeats with period 4 over the full slot vector
    z = np.array([1.0, -2.0, 0.25, 3.0])
    pt = enc.encode(z, scale, 1, sparse_slots=4)
    full = enc.decode(pt, scale)
    assert np.max(np.abs(full.real - np.tile(z, n // 8))) < 1e-6
    assert np.max(np.abs(enc.decode(pt, scale, sparse_slots=4).real - z)) < 1e-6


def test_encrypt_decrypt_roundtrip(ctx):
    O, p, ks, pk, rlk, enc = ctx
    rng = np.random.default_rng(2)
    z = rng.uniform(-1, 1, p.n // 2)
    scale = 2.0 ** 40
    ct = ks.encrypt_asymmetric(pk, enc.encode(z, scale, p.size_q))
    got = enc.decode(ks.decrypt(ct), scale).real
    assert np.max(np.abs(got - z)) < 1e-7
    noisy = enc.decode(ks.decrypt(ct, O.gauss_cdt()), scale).real
    assert np.max(np.abs(noisy - z)) < 1e-6


def test_multiply_relin_rescale(ctx):
    O, p, ks, pk, rlk, enc = ctx
    rng = np.random.default_rng(3)
    x, y = rng.uniform(-1, 1, p.n // 2), rng.uniform(-1, 1, p.n // 2)
    scale = 2.0 ** 40
    cx = ks.encrypt_asymmetric(pk, enc.encode(x, scale, p.size_q))
    cy = ks.encrypt_asymmetric(pk, enc.encode(y, scale, p.size_q))
    t3 = p.tensor(cx, cy)
    want3 = enc.decode(ks.decrypt(t3), scale * scale).real
    assert np.max(np.abs(want3 - x * y)) < 1e-6
    ct = p.relinearize(t3, rlk)
    got = enc.decode(ks.decrypt(ct), scale * scale).real
    assert np.max(np.abs(got - x * y)) < 1e-5          # unittest/evaluator.cu:419-472 bound
    assert np.max(np.abs(got - want3)) < 1e-6          # key switching only adds small noise
    rs = p.rescale(ct)
    got = enc.decode(ks.decrypt(rs), scale * scale / p.moduli[p.size_q - 1]).real
    assert np.max(np.abs(got - x * y)) < 1e-5
    # square = tensor with itself
    sq = p.relinearize(p.square(cx), rlk)
    assert np.max(np.abs(enc.decode(ks.decrypt(sq), scale * scale).real - x * x)) < 1e-5


def test_key_switch_at_lower_levels(ctx):
    """Relinearisation after dropping limbs exercises partial digits (L = 5, 3) and fewer digits."""
    O, p, ks, pk, rlk, enc = ctx
    rng = np.random.default_rng(4)
    x = rng.uniform(-1, 1, p.n // 2)
    scale = 2.0 ** 30
    c = ks.encrypt_asymmetric(pk, enc.encode(x, scale, p.size_q))
    for L in (5, 4, 3, 2):
        cl = np.ascontiguousarray(c[:, :L])
        got = enc.decode(ks.decrypt(p.relinearize(p.square(cl), rlk)), scale * scale).real
        assert np.max(np.abs(got - x * x)) < 1e-4, L


@pytest.mark.parametrize("step", [1, 5, -3, 0])
def test_rotation(ctx, step):
    O, p, ks, pk, rlk, enc = ctx
    rng = np.random.default_rng(5)
    slots = p.n // 2
    z = rng.uniform(-1, 1, slots) + 1j * rng.uniform(-1, 1, slots)
    scale = 2.0 ** 40
    ct = ks.encrypt_asymmetric(pk, enc.encode(z, scale, p.size_q))
    g = O.galois_elt_from_step(step, p.n)
    glk = ks.gen_galois(g)
    got = enc.decode(ks.decrypt(p.apply_galois(ct, g, glk)), scale)
    want = np.conj(z) if step == 0 else np.roll(z, -step)
    assert np.max(np.abs(got - want)) < 1e-6


def test_hoisting_is_sum_of_rotations(ctx):
    O, p, ks, pk, rlk, enc = ctx
    rng = np.random.default_rng(6)
    slots = p.n // 2
    z = rng.uniform(-1, 1, slots)
    scale = 2.0 ** 40
    ct = ks.encrypt_asymmetric(pk, enc.encode(z, scale, p.size_q))
    steps = [1, 2, 3]
    elts = [O.galois_elt_from_step(s, p.n) for s in steps]
    glks = [ks.gen_galois(g) for g in elts]
    got = enc.decode(ks.decrypt(p.hoisting(ct, elts, glks)), scale).real
    want = sum(np.roll(z, -s) for s in steps)
    assert np.max(np.abs(got - want)) < 1e-6


def test_sampler_distributions(oracle):
    O = oracle
    n = 1 << 12
    p = O.Params(12, O.get_primes(n, 50, 3), 1)
    key = O.chacha_key(1)
    t = p.sample_ternary(key, 0, 3)
    q = np.array(p.moduli[:3], dtype=np.uint64)[:, None]
    signed = np.where(t > q // 2, t.astype(np.int64) - q.astype(np.int64), t.astype(np.int64))
    assert (signed[0] == signed[1]).all() and (signed[0] == signed[2]).all()      # same value on every limb
    assert set(np.unique(signed[0])) == {-1, 0, 1}
    counts = np.bincount(signed[0] + 1) / n
    assert np.all(np.abs(counts - 1 / 3) < 0.03)
    e = p.sample_error(key, 1, 2)
    es = np.where(e > q[:2] // 2, e.astype(np.int64) - q[:2].astype(np.int64), e.astype(np.int64))
    assert (es[0] == es[1]).all() and abs(es[0].mean()) < 0.2 and abs(es[0].std() - np.sqrt(10.5)) < 0.2
    assert np.abs(es[0]).max() <= 21
    u = p.sample_uniform(key, 2, 3)
    assert (u < q).all() and not (u[0] == u[1]).all()
    assert abs(float(u[0].mean()) / p.moduli[0] - 0.5) < 0.03
    g = p.sample_gauss(key, 3, 1, O.gauss_cdt())
    gs = np.where(g > q[:1] // 2, g.astype(np.int64) - q[:1].astype(np.int64), g.astype(np.int64))
    assert abs(gs.mean()) < 0.4 and abs(gs.std() - O.FLOODING_SIGMA) < 0.3
    # different streams differ, same stream repeats
    assert (p.sample_ternary(key, 0, 1) == t[:1]).all() and not (p.sample_ternary(key, 9, 1) == t[:1]).all()
