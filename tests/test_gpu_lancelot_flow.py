"""The call sequence of lancelot-main-GPU/utils/byzantine_fl.py with its own parameters (GPU_init :434-468: N = 2^16,
moduli [60, 40, 40, 60], one special prime, scale 2^40, Galois keys for the steps 1..15 and 2^4..2^14), replayed from
the list of calls it makes: Python-list encode, encrypt_asymmetric, mod_switch_to_inplace, sub, square_inplace,
add_inplace onto a squared zero (lazy relinearisation), relinearize_inplace, rescale_to_next_inplace, set_scale,
hoisting(context, ct, glk, [1..15]) + add_inplace, rotate_vector by 2^4..2^14 + add_inplace (:175-320); then the
sum / decrypt / decode of the distances (:327-350) and the ciphertext-by-ciphertext multiply of a mask with the
weights, accumulated at size 3 and decrypted unrelinearised (:372-428).  Checked against float64."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

N_SLOT, LOG_N_SLOT = 32768, 15


@pytest.fixture(scope="module")
def setup():
    import lancelot_amd  # noqa: F401
    import pyCAHEL as cahel
    log_n = LOG_N_SLOT + 1
    n = 2 ** log_n
    galois_steps = [i for i in range(1, 16)] + [2 ** i for i in range(4, log_n - 1)]
    params = cahel.params(cahel.scheme_type.ckks)
    params.set_poly_modulus_degree(n)
    params.set_coeff_modulus(cahel.coeff_modulus_create(n, [60, 40, 40, 60]))
    params.set_special_modulus_size(1)
    params.set_galois_elts(cahel.get_elts_from_steps(galois_steps, n))
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
    assert encoder.slot_count() == N_SLOT
    return cahel, context, pk, sk, glk, rlk, encoder, 2.0 ** 40


def pair_distance(cahel, context, pk, glk, rlk, encoder, scale, msg1, msg2):
    """One encrypted squared distance the way GPU_compute_pair_distance drives the library (lazy relinearisation,
    hoisted first sixteen rotations)."""
    zero = [0.0] * N_SLOT
    acc = pk.encrypt_asymmetric(context, encoder.encode(context, zero, scale))
    cahel.square_inplace(context, acc)
    tmp = cahel.ciphertext(context)
    for x1, x2 in zip(msg1, msg2):
        ct1 = pk.encrypt_asymmetric(context, encoder.encode(context, x1, scale))
        ct2 = pk.encrypt_asymmetric(context, encoder.encode(context, x2, scale))
        cahel.sub(context, ct2, ct1, tmp)
        cahel.square_inplace(context, tmp)
        cahel.add_inplace(context, acc, tmp)
    cahel.relinearize_inplace(context, acc, rlk)
    cahel.rescale_to_next_inplace(context, acc)
    acc.set_scale(scale)
    hoisted = cahel.hoisting(context, acc, glk, [1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15])
    cahel.add_inplace(context, acc, hoisted)
    rot = cahel.ciphertext(context)
    for idx in range(4, LOG_N_SLOT):
        cahel.rotate_vector(context, acc, int(2 ** idx), glk, rot)
        cahel.add_inplace(context, acc, rot)
    return acc


def test_byzantine_fl_call_sequence(setup):
    cahel, context, pk, sk, glk, rlk, encoder, scale = setup
    rng = np.random.default_rng(7)
    clients, words = 3, 2
    # client k: `words` chunks of N_SLOT values as Python lists (what multi_vectorization_cipher hands over)
    vectors = [[list(rng.normal(0.0, 0.01, N_SLOT) * (10.0 if k == 2 else 1.0)) for _ in range(words)] for k in range(clients)]
    plain = np.array(vectors, dtype=np.float64)

    # distance matrix (GPU_computing_distance_cipher): ciphertext [i][j] for i < j, mirrored
    dist = [[None] * clients for _ in range(clients)]
    for i in range(clients):
        for j in range(i + 1, clients):
            dist[i][j] = dist[j][i] = pair_distance(cahel, context, pk, glk, rlk, encoder, scale, vectors[i], vectors[j])
    want = np.array([[np.sum((plain[i] - plain[j]) ** 2) for j in range(clients)] for i in range(clients)])
    for i in range(clients):
        for j in range(i + 1, clients):
            assert dist[i][j].chain_index() == 2 and dist[i][j].size() == 2
            got = encoder.decode(context, sk.decrypt(context, dist[i][j]))
            # every slot holds the sum; the tolerance is the one of the full-shape Krum round
            assert abs(got[0] - want[i][j]) / want[i][j] < 2e-5, (i, j, got[0], want[i][j])
            assert abs(got[12345] - want[i][j]) / want[i][j] < 2e-5

    # GPU_decrypt_sort_mask: per client the sum of its distances, decrypted; argsort picks the client
    sums = []
    for i in range(clients):
        tmp = pk.encrypt_asymmetric(context, encoder.encode(context, [0.0] * N_SLOT, scale))
        cahel.mod_switch_to_inplace(context, tmp, 2)
        for j in range(clients):
            if j != i:
                cahel.add_inplace(context, tmp, dist[i][j])
        sums.append(encoder.decode(context, sk.decrypt(context, tmp))[0])
    order = np.argsort(sums)
    assert list(order) == list(np.argsort(want.sum(axis=1)))
    one = pk.encrypt_asymmetric(context, encoder.encode(context, [1.0] * N_SLOT, scale))
    zero = pk.encrypt_asymmetric(context, encoder.encode(context, [0.0] * N_SLOT, scale))
    mask_row = [one if k == order[0] else zero for k in range(clients)]

    # GPU_mul_mask_weight: sum over the clients of mask x weights, ciphertext by ciphertext, kept at size 3
    pt_zero = encoder.encode(context, [0.0] * N_SLOT, scale)
    tmp = cahel.ciphertext(context)
    for w in range(words):
        acc = pk.encrypt_asymmetric(context, pt_zero)
        cahel.square_inplace(context, acc)
        for k in range(clients):
            ct2 = pk.encrypt_asymmetric(context, encoder.encode(context, vectors[k][w], scale))
            cahel.multiply(context, ct2, mask_row[k], tmp)
            cahel.add_inplace(context, acc, tmp)
        assert acc.size() == 3
        got = np.array(encoder.decode(context, sk.decrypt(context, acc)))
        assert np.max(np.abs(got - plain[order[0]][w])) < 1e-5      # ciphertext x ciphertext noise at scale 2^80
