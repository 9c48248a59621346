"""save / load of plaintexts, ciphertexts and keys in the reference's byte layout (cahel-main/include/plaintext.h
:109-200, include/ciphertext.h:174-290, include/secretkey.h:53-59, 212-256, 354-398).

No file written by the reference exists in its tree, so the layout is pinned field by field against the documented
order with `struct`, the identifiers against BLAKE2b from Python's hashlib, and the payload by round trips: a
record that is loaded back must give the same limbs and must keep working (decrypt, relinearise, rotate)."""
import hashlib
import struct

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

SEED = 77


def _world(bits=(50, 40, 40, 40, 50, 50), special=2, n=4096):
    import lancelot_amd  # noqa: F401
    import pyCAHEL as cahel
    mods = cahel.coeff_modulus_create(n, list(bits))
    parms = cahel.params(cahel.scheme_type.ckks)
    parms.set_poly_modulus_degree(n)
    parms.set_coeff_modulus(mods)
    parms.set_special_modulus_size(special)
    parms.set_galois_elts(cahel.get_elts_from_steps([1, -2, 0], n))
    ctx = cahel.context(parms, True, cahel.sec_level_type.none)
    ctx.set_seed(SEED)
    sk = cahel.secret_key(parms)
    sk.gen_secretkey(ctx)
    sk.set_noise_flooding(False)
    pk = cahel.public_key(ctx)
    sk.gen_publickey(ctx, pk)
    rlk = cahel.relin_key(ctx)
    sk.gen_relinkey(ctx, rlk)
    glk = cahel.galois_key(ctx)
    sk.create_galois_keys(ctx, glk)
    return dict(cahel=cahel, parms=parms, ctx=ctx, sk=sk, pk=pk, rlk=rlk, glk=glk, enc=cahel.ckks_encoder(ctx),
                vals=[m.value() for m in mods], n=n, special=special)


@pytest.fixture(scope="module")
def world():
    return _world()


def _expected_id(w, limbs):
    words = [3, w["n"], w["special"]] + w["vals"] + w["vals"][:limbs] + [0]
    return struct.unpack("<4Q", hashlib.blake2b(struct.pack("<%dQ" % len(words), *words), digest_size=32).digest())


def test_chain_identifiers(world):
    """Chain index 0 hashes every modulus; data level c the first size_q - c + 1 (src/context.cu:352-401)."""
    w, ctx = world, world["ctx"]
    size_q = ctx.size_q()
    assert ctx.parms_id_at(0) == _expected_id(w, size_q + ctx.size_p()) == w["parms"].parms_id()
    for c in range(1, size_q + 1):
        assert ctx.parms_id_at(c) == _expected_id(w, size_q - c + 1)


def test_ciphertext_record_layout_and_round_trip(world, tmp_path):
    w, c, ctx = world, world["cahel"], world["ctx"]
    rng = np.random.default_rng(1)
    x = rng.uniform(-1, 1, w["enc"].slot_count())
    ct = w["pk"].encrypt_asymmetric(ctx, w["enc"].encode(ctx, x, 2.0 ** 40))
    c.mod_switch_to_next_inplace(ctx, ct)                      # chain index 2: a level below the first
    blob = ct.to_bytes()
    limbs, n = ct.coeff_modulus_size(), w["n"]
    words = 2 * limbs * n
    assert len(blob) == 32 + 1 + 4 * 8 + 8 + 8 + 8 * words + 64
    assert struct.unpack_from("<4Q", blob, 0) == ctx.parms_id_at(2) == ct.parms_id()
    ntt, chain, size, degree, nlimbs, scale, count = struct.unpack_from("<BQQQQdQ", blob, 32)
    assert (ntt, chain, size, degree, nlimbs, scale, count) == (1, 2, 2, n, limbs, 2.0 ** 40, words)
    data = np.frombuffer(blob, dtype="<u8", count=words, offset=32 + 1 + 48)
    assert (data.reshape(2, limbs, n) == ct.to_numpy()).all()
    assert blob[-64:] == bytes(64)
    back = c.ciphertext(ctx)
    back.from_bytes(ctx, blob)
    assert (back.to_numpy() == ct.to_numpy()).all()
    assert (back.chain_index(), back.size(), back.scale(), back.parms_id()) == (2, 2, 2.0 ** 40, ct.parms_id())
    assert back.to_bytes() == blob
    got = w["enc"].decode(ctx, w["sk"].decrypt(ctx, back))
    assert np.max(np.abs(np.asarray(got).real[:len(x)] - x)) < 1e-6
    # through a file, and a size-3 ciphertext
    c.mod_switch_to_next_inplace(ctx, ct)
    prod = c.ciphertext(ctx)
    c.multiply(ctx, ct, ct, prod)
    path = str(tmp_path / "ct.bin")
    prod.save(path)
    again = c.ciphertext(ctx)
    again.load(ctx, path)
    assert again.size() == 3 and (again.to_numpy() == prod.to_numpy()).all() and again.scale() == prod.scale()


def test_plaintext_record_layout_and_round_trip(world):
    w, c, ctx = world, world["cahel"], world["ctx"]
    x = np.linspace(-1, 1, w["enc"].slot_count())
    pt = w["enc"].encode(ctx, x, 2.0 ** 30)
    blob = pt.to_bytes()
    limbs, n = ctx.size_q(), w["n"]
    assert len(blob) == 32 + 3 * 8 + 8 + 8 + 8 * limbs * n
    assert struct.unpack_from("<4Q", blob, 0) == ctx.parms_id_at(1)
    assert struct.unpack_from("<QQQdQ", blob, 32) == (limbs, 1, n, 2.0 ** 30, limbs * n)
    assert (np.frombuffer(blob, dtype="<u8", offset=32 + 40).reshape(limbs, n) == pt.to_numpy()).all()
    back = c.plaintext(ctx)
    back.from_bytes(ctx, blob)
    assert (back.to_numpy() == pt.to_numpy()).all() and back.scale() == 2.0 ** 30 and back.chain_index() == 1
    assert np.max(np.abs(np.asarray(w["enc"].decode(ctx, back)).real[:len(x)] - x)) < 1e-6


def test_keys_survive_a_round_trip(world):
    """Loaded keys are the same limbs and do the same work: encryption under the loaded public key decrypts, and
    relinearisation / rotation with the loaded keys give the ciphertext the original keys give, word for word."""
    w, c, ctx = world, world["cahel"], world["ctx"]
    pk2, rlk2, glk2 = c.public_key(ctx), c.relin_key(ctx), c.galois_key(ctx)
    pk_blob, rlk_blob, glk_blob = w["pk"].to_bytes(), w["rlk"].to_bytes(), w["glk"].to_bytes()
    pk2.from_bytes(ctx, pk_blob)
    rlk2.from_bytes(ctx, rlk_blob)
    glk2.from_bytes(ctx, glk_blob)
    assert (pk2.to_numpy() == w["pk"].to_numpy()).all()
    # headers: identifier of the key level, generated flag, count, then the nested records
    dnum = ctx.size_q() // ctx.size_p()
    assert struct.unpack_from("<4Q", rlk_blob, 0) == ctx.parms_id_at(0)
    assert struct.unpack_from("<BQ", rlk_blob, 32) == (1, dnum)
    qp = ctx.size_q() + ctx.size_p()
    assert struct.unpack_from("<4Q", rlk_blob, 41) == ctx.parms_id_at(0)          # first nested public-key record
    assert struct.unpack_from("<BQQQQ", rlk_blob, 41 + 32) == (1, 0, 2, w["n"], qp)
    assert len(rlk_blob) == 41 + dnum * len(pk_blob)
    assert struct.unpack_from("<BQ", glk_blob, 32) == (1, len(ctx.galois_elts()))
    assert len(glk_blob) == 41 + len(ctx.galois_elts()) * len(rlk_blob)
    assert rlk2.digit_count() == dnum and glk2.key_count() == len(ctx.galois_elts())
    for d in range(dnum):
        assert (rlk2.digit_to_numpy(d) == w["rlk"].digit_to_numpy(d)).all()
        assert (glk2.key(1).digit_to_numpy(d) == w["glk"].key(1).digit_to_numpy(d)).all()
    assert rlk2.to_bytes() == rlk_blob and glk2.to_bytes() == glk_blob
    rng = np.random.default_rng(2)
    x = rng.uniform(-1, 1, w["enc"].slot_count())
    ct = pk2.encrypt_asymmetric(ctx, w["enc"].encode(ctx, x, 2.0 ** 40))
    got = np.asarray(w["enc"].decode(ctx, w["sk"].decrypt(ctx, ct))).real
    assert np.max(np.abs(got[:len(x)] - x)) < 1e-6
    outs = []
    for rlk, glk in ((w["rlk"], w["glk"]), (rlk2, glk2)):
        prod = c.ciphertext(ctx)
        c.multiply(ctx, ct, ct, prod)
        c.relinearize_inplace(ctx, prod, rlk)
        c.rescale_to_next_inplace(ctx, prod)
        rot = c.ciphertext(ctx)
        c.rotate_vector(ctx, prod, -2, glk, rot)
        outs.append((prod.to_numpy(), rot.to_numpy()))
    assert (outs[0][0] == outs[1][0]).all() and (outs[0][1] == outs[1][1]).all()


def test_load_rejects_what_does_not_fit(world):
    """Truncated input is an I/O error (RuntimeError, as the reference's "I/O error"); a record of another parameter
    set, another degree or with a wrong word count is refused before anything reaches the device tables."""
    w, c, ctx = world, world["cahel"], world["ctx"]
    ct = w["pk"].encrypt_asymmetric(ctx, w["enc"].encode(ctx, [0.5, -0.25], 2.0 ** 40))
    blob = ct.to_bytes()
    keep = ct.to_numpy().copy()
    for cut in (0, 10, 40, 100, len(blob) - 65, len(blob) - 1):
        with pytest.raises(RuntimeError, match="I/O error"):
            ct.from_bytes(ctx, blob[:cut])
    assert (ct.to_numpy() == keep).all()                      # a failed load leaves the object as it was
    other = _world(bits=(50, 41, 40, 40, 50, 50))             # same shape, one other prime
    foreign = other["pk"].encrypt_asymmetric(other["ctx"], other["enc"].encode(other["ctx"], [1.0, 0.5], 2.0 ** 40))
    with pytest.raises(ValueError, match="parms_id"):
        ct.from_bytes(ctx, foreign.to_bytes())
    with pytest.raises(ValueError, match="parms_id"):
        c.relin_key(ctx).from_bytes(ctx, other["rlk"].to_bytes())
    with pytest.raises(ValueError, match="parms_id"):
        c.galois_key(ctx).from_bytes(ctx, other["glk"].to_bytes())
    small = _world(n=2048)
    with pytest.raises(ValueError, match="poly_modulus_degree"):
        ct.from_bytes(ctx, small["pk"].encrypt_asymmetric(small["ctx"], small["enc"].encode(small["ctx"], [1.0, 0.5], 2.0 ** 40)).to_bytes())
    bad = bytearray(blob)
    struct.pack_into("<Q", bad, 32 + 1, 9)                     # chain index beyond the chain
    with pytest.raises(ValueError, match="chain index"):
        ct.from_bytes(ctx, bytes(bad))
    bad = bytearray(blob)
    struct.pack_into("<Q", bad, 32 + 1 + 8, 4)                 # four polynomials
    with pytest.raises(ValueError, match="size"):
        ct.from_bytes(ctx, bytes(bad))
    bad = bytearray(blob)
    struct.pack_into("<Q", bad, 32 + 1 + 40, 17)               # word count that contradicts the header
    with pytest.raises(ValueError, match="data size"):
        ct.from_bytes(ctx, bytes(bad))
    with pytest.raises(ValueError, match="key-level"):
        c.public_key(ctx).from_bytes(ctx, blob)                # a data-level ciphertext is not a public key
    with pytest.raises(RuntimeError, match="I/O error"):
        ct.load(ctx, "/nonexistent/dir/ct.bin")
