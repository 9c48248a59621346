"""CPU-only checks of the product: the C-ABI library loads and exports every declared symbol, and the host
number theory agrees with the reference's known answers and with the oracle.  No GPU calls."""
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def cahel():
    import lancelot_amd  # noqa: F401
    import pyCAHEL
    return pyCAHEL


def test_library_exports_every_declared_symbol():
    from lancelot_amd import capi
    header = open(os.path.join(ROOT, "include", "cahel_hip.h")).read()
    declared = set(re.findall(r"\b(he_[a-z0-9_]+)\s*\(", header))
    declared -= {"he_context", "he_stream", "he_event"}
    assert len(declared) >= 35
    lib = capi.lib()
    for name in sorted(declared):
        assert hasattr(lib, name), name
    assert declared == set(capi.SIGNATURES), declared ^ set(capi.SIGNATURES)
    assert lib.he_error_string(0) == b"success" and lib.he_error_string(-3).startswith(b"tables of this level")
    # the measurement library is a shared object of its own: its names are not part of the engine's interface
    probe_header = open(os.path.join(ROOT, "include", "cahel_probe.h")).read()
    probes = set(re.findall(r"\b(he_probe_[a-z0-9_]+)\s*\(", probe_header))
    assert probes == set(capi.PROBE_SIGNATURES) and not probes & declared
    for name in sorted(probes):
        assert hasattr(capi.probe_lib(), name) and not hasattr(lib, name), name


def test_pycahel_exports_the_reference_names(cahel):
    # cahel-main/python/src/binding.cu:8-156
    names = """scheme_type mul_tech_type sec_level_type modulus coeff_modulus_create params context secret_key
    public_key relin_key galois_key get_elts_from_steps ckks_encoder plaintext ciphertext negate negate_inplace add
    add_inplace add_plain add_plain_inplace add_many sub sub_inplace sub_plain sub_plain_inplace multiply
    multiply_inplace multiply_and_relin_inplace multiply_plain multiply_plain_inplace multiply_many square
    square_inplace exponentiate exponentiate_inplace relinearize relinearize_inplace mod_switch_to
    mod_switch_to_inplace mod_switch_to_next mod_switch_to_next_inplace rescale_to_next rescale_to_next_inplace
    apply_galois apply_galois_inplace rotate_rows rotate_rows_inplace rotate_columns rotate_columns_inplace
    rotate_vector rotate_vector_inplace hoisting hoisting_inplace complex_conjugate complex_conjugate_inplace""".split()
    for name in names:
        assert hasattr(cahel, name), name
    for cls, methods in {"params": ["set_mul_tech", "set_poly_modulus_degree", "set_special_modulus_size",
                                    "set_galois_elts", "set_coeff_modulus"],
                         "secret_key": ["gen_secretkey", "gen_publickey", "gen_relinkey", "create_galois_keys",
                                        "encrypt_symmetric", "decrypt"],
                         "public_key": ["encrypt_asymmetric"],
                         "ckks_encoder": ["slot_count", "encode", "encode_to", "decode"],
                         "ciphertext": ["set_scale"]}.items():
        for m in methods:
            assert hasattr(getattr(cahel, cls), m), (cls, m)
    assert cahel.scheme_type.ckks != cahel.scheme_type.bfv and int(cahel.sec_level_type.tc128) == 128


def test_host_number_theory_known_answers(cahel, oracle):
    # cahel-main/unittest/util/numth.cu:197-216, :112-150; src/util/globals.cu:77-101
    assert cahel._minimal_primitive_root(2, 11) == 10 and cahel._minimal_primitive_root(4, 29) == 12
    assert cahel._minimal_primitive_root(8, 1234565441) == 249725733
    assert cahel._get_primes(16384, 48, 3) == [0xfffffffd8001, 0xfffffffa0001, 0xfffffff00001]
    assert cahel._get_primes(8192, 44, 3) == [0xfffffffc001, 0xffffff6c001, 0xfffffebc001]
    for v in (0, 1, -1, 2, -2, 3, -3, 127, -127, 123, -123):
        parts = cahel._naf(v)
        assert sum(parts) == v
        assert len(parts) == {0: 0, 1: 1, 2: 1, 3: 2, 127: 2}.get(abs(v), len(parts))
    for n, bits in ((8192, [60, 40, 40, 60]), (65536, [50] * 32), (4096, [30, 30, 36])):
        assert [m.value() for m in cahel.coeff_modulus_create(n, bits)] == oracle.coeff_modulus_create(n, bits)
    for q in oracle.get_primes(65536, 50, 3):
        assert cahel._minimal_primitive_root(131072, q) == oracle.minimal_primitive_root(131072, q)


def test_galois_elements(cahel, oracle):
    n = 65536
    steps = [0, 1, 2, 15, -1, -7, 16384]
    assert cahel.get_elts_from_steps(steps, n) == [oracle.galois_elt_from_step(s, n) for s in steps]
    with pytest.raises(ValueError, match="step count too large"):
        cahel.get_elts_from_steps([n // 2], n)


def test_parameter_errors(cahel):
    with pytest.raises(ValueError):
        cahel.modulus(1)
    with pytest.raises(ValueError):
        cahel.modulus(1 << 61)
    with pytest.raises(ValueError, match="bit_sizes is invalid"):
        cahel.coeff_modulus_create(8192, [61])
    with pytest.raises(ValueError, match="poly_modulus_degree is invalid"):
        cahel.coeff_modulus_create(1000, [40])
    p = cahel.params(cahel.scheme_type.ckks)
    with pytest.raises(ValueError, match="only supported for BFV"):
        p.set_mul_tech(cahel.mul_tech_type.hps)
    none = cahel.params(cahel.scheme_type.none)
    with pytest.raises(RuntimeError):
        none.set_poly_modulus_degree(4096)
    # parameter validation happens before any device work
    p.set_poly_modulus_degree(8192)
    p.set_coeff_modulus(cahel.coeff_modulus_create(8192, [60, 60, 60, 60]))
    with pytest.raises(ValueError, match="insecure"):
        cahel.context(p, True, cahel.sec_level_type.tc128)
    p.set_coeff_modulus(cahel.coeff_modulus_create(8192, [40, 40, 40, 40, 40]))
    p.set_special_modulus_size(2)
    with pytest.raises(ValueError, match="multiple of the special modulus size"):
        cahel.context(p, True, cahel.sec_level_type.none)
    bfv = cahel.params(cahel.scheme_type.bfv)
    bfv.set_poly_modulus_degree(8192)
    bfv.set_coeff_modulus(cahel.coeff_modulus_create(8192, [40, 40]))
    with pytest.raises(ValueError, match="implements CKKS"):
        cahel.context(bfv, True, cahel.sec_level_type.none)


def test_krum_host_logic():
    import numpy as np
    from lancelot_amd import krum
    rng = np.random.default_rng(0)
    ups = [rng.normal(0, 0.01, 1000) for _ in range(5)]
    ups[4] = ups[4] * 10
    chunks = krum.split_updates(ups, 256)
    assert len(chunks) == 5 and len(chunks[0]) == 4 and all(len(c) == 256 for c in chunks[0])
    assert np.allclose(np.concatenate(chunks[2])[:1000], ups[2]) and not np.concatenate(chunks[2])[1000:].any()
    d = krum.plain_distance_matrix(ups)
    assert d.shape == (5, 5) and np.allclose(d, d.T) and abs(d[0, 1] - np.sum((ups[0] - ups[1]) ** 2)) < 1e-12
    assert krum.krum_select(d) != 4
    with pytest.raises(ValueError):
        krum.split_updates([np.zeros(3), np.zeros(4)], 2)


@pytest.mark.parametrize("log_slots", [1, 3, 4, 5, 8, 12, 15])
def test_rotate_sum_plan_adds_every_slot_once(log_slots):
    """Whatever the split into hoisted rounds and single rotations, acc += sum_k rot(acc, s_k) over the rounds must
    leave every slot holding each input slot exactly once."""
    from lancelot_amd import krum
    n = 1 << log_slots
    for cfg in (krum.KrumConfig(), krum.KrumConfig(hoisting_radix=0), krum.KrumConfig(hoisting=False),
                krum.KrumConfig(hoisting_radix=4), krum.KrumConfig(hoisting_radix=32)):
        cover = np.zeros(n, dtype=np.int64)
        cover[0] = 1
        for steps in krum.rotate_sum_plan(log_slots, cfg):
            assert all(0 < s < n for s in steps)
            cover = cover + sum(np.roll(cover, s) for s in steps)
        assert (cover == 1).all(), (log_slots, cfg)
    assert krum.rotate_sum_plan(15, krum.KrumConfig(hoisting_radix=0))[0] == list(range(1, 16))   # the reference's split


def test_package_without_native_module_only_imports_for_the_build(tmp_path):
    """A tree that has not been built yet: `import lancelot_amd` must fail loudly, but the build module must still
    be reachable (python -m lancelot_amd.build, and the LANCELOT_AMD_BUILD=1 import that build() does)."""
    import shutil
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    pkg = tmp_path / "lancelot_amd"
    pkg.mkdir()
    for name in ("__init__.py", "build.py", "capi.py", "krum.py"):
        shutil.copy(os.path.join(root, "lancelot_amd", name), pkg / name)
    env = dict(os.environ, PYTHONPATH=str(tmp_path))
    run = lambda code, **extra: subprocess.run([sys.executable, "-c", code], cwd=tmp_path, env=dict(env, **extra),
                                               capture_output=True, text=True)
    plain = run("import lancelot_amd")
    assert plain.returncode != 0 and "native module is missing" in plain.stderr
    building = run("from lancelot_amd import build; print(build.LIB)", LANCELOT_AMD_BUILD="1")
    assert building.returncode == 0 and "libcahel_hip.so" in building.stdout
    as_module = subprocess.run([sys.executable, "-m", "lancelot_amd.build", "--help"], cwd=tmp_path, env=env,
                               capture_output=True, text=True)
    assert as_module.returncode == 0 and "libcahel_hip.so" in as_module.stdout


def test_blake2b_known_answers(cahel):
    """The hash behind the parameter identifiers: RFC 7693 appendix A ("abc", 64-byte digest) and Python's own
    BLAKE2b over lengths around the 128-byte block boundary, for several digest sizes."""
    import hashlib
    rfc = ("ba80a53f981c4d0d6a2797b69f12f6e94c212f14685ac4b74b12bb6fdbffa2d1"
           "7d87c5392aab792dc252d5de4533cc9518d38aa8dbf1925ab92386edd4009923")
    assert cahel._blake2b(b"abc", 64).hex() == rfc
    for n in (0, 1, 3, 64, 127, 128, 129, 255, 256, 257, 1000):
        data = bytes((7 * i + 3) & 255 for i in range(n))
        for size in (1, 20, 32, 64):
            assert cahel._blake2b(data, size) == hashlib.blake2b(data, digest_size=size).digest(), (n, size)
    with pytest.raises(ValueError):
        cahel._blake2b(b"", 65)


def test_parms_id_hashes_the_reference_words(cahel):
    """parms_id = BLAKE2b-256 over the 64-bit words (scheme, degree, special modulus count, key moduli, coefficient
    moduli, plain modulus = 0), include/util/encryptionparams.h:337-379; it changes with every one of them."""
    import hashlib
    import struct

    def make(n, bits, special, scheme=None):
        p = cahel.params(scheme or cahel.scheme_type.ckks)
        p.set_poly_modulus_degree(n)
        mods = cahel.coeff_modulus_create(n, bits)
        p.set_coeff_modulus(mods)
        p.set_special_modulus_size(special)
        return p, [m.value() for m in mods]

    p, vals = make(8192, [60, 40, 40, 60], 1)
    words = [3, 8192, 1] + vals + vals + [0]
    digest = hashlib.blake2b(struct.pack("<%dQ" % len(words), *words), digest_size=32).digest()
    assert p.parms_id() == struct.unpack("<4Q", digest)
    others = [make(4096, [60, 40, 40, 60], 1)[0], make(8192, [60, 40, 40, 60], 2)[0], make(8192, [60, 40, 41, 60], 1)[0],
              make(8192, [60, 40, 40, 60], 1, cahel.scheme_type.bfv)[0]]
    ids = {p.parms_id()} | {o.parms_id() for o in others}
    assert len(ids) == 5


def test_params_record_layout_and_round_trip(cahel):
    """EncryptionParameters.save: scheme u8 | degree u64 | count u64 | moduli | plain modulus 0
    (include/util/encryptionparams.h:381-409, src/modulus.cu:134-155); load gives the same parameters and
    identifier back, refuses a bad scheme byte or modulus, and reports truncation as an I/O error."""
    import struct
    p = cahel.params(cahel.scheme_type.ckks)
    p.set_poly_modulus_degree(4096)
    mods = [m.value() for m in cahel.coeff_modulus_create(4096, [50, 40, 50])]
    p.set_coeff_modulus([cahel.modulus(v) for v in mods])
    blob = p.to_bytes()
    assert blob == struct.pack("<BQQ", 3, 4096, 3) + struct.pack("<3Q", *mods) + struct.pack("<Q", 0)
    q = cahel.params(cahel.scheme_type.bfv)
    q.from_bytes(blob)
    assert (q.poly_modulus_degree(), q.coeff_modulus(), q.parms_id()) == (4096, mods, p.parms_id())
    with pytest.raises(RuntimeError, match="I/O error"):
        q.from_bytes(blob[:-3])
    with pytest.raises(ValueError):
        q.from_bytes(bytes([7]) + blob[1:])                                   # no such scheme
    with pytest.raises(ValueError):
        q.from_bytes(blob[:17] + struct.pack("<Q", 1) + blob[25:])            # modulus 1
    assert (q.poly_modulus_degree(), q.coeff_modulus()) == (4096, mods)       # failed loads change nothing


def test_bench_refuses_more_than_one_gpu():
    """bench.py measures one GPU; with --gpus above 1 it says so and exits with an error, before touching a GPU."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       timeout=120)
    assert r.returncode != 0
    assert "one GPU" in (r.stdout + r.stderr)
