"""Pins every integer stage of the oracle against Python big-integer closed forms.

The reference's tests hold no vectors for these stages (cahel-main/unittest/ has no NTT, ModUp,
ModDown, key-switch or rescale test), so each stage is pinned by what the mathematics fixes:
  NTT      out[bitrev(i)] = sum_j a_j psi^((2i+1) j)   (evaluation at the odd powers of psi; Appendix
           of src/util/ntt.cu:46-56 + src/ntt/ntt_1d.cu:38-73), inverse = identity round trip,
           negacyclic convolution theorem against schoolbook multiplication
  ModUp    sum_i [x_i (Q_d/q_i)^-1]_{q_i} (Q_d/q_i) mod m_t, no overflow correction
           (src/rns_bconv.cu:587-623) and the invariant lift = x + u Q_d, 0 <= u < digit size
  inner    sum_d y_d evk_d mod m_t (src/eval_key_switch.cu:50-74)
  ModDown  (cx_j - NTT(delta)_j) P^-1 (src/rns_bconv.cu:965-1053) and P * out = in - delta
  rescale  (c_j - [c_last]_{q_j}) q_last^-1, floor style (src/rns.cu:544-570)
  Galois   NTT(a(X^g)) = permute(NTT(a)) (include/galois.cuh:45-57)
"""
import math
import random

import numpy as np
import pytest


@pytest.fixture(scope="module")
def small(oracle):
    """N = 64, 5 Q limbs of mixed widths + 2 special limbs: digits of size 2, 2, 1."""
    n = 64
    qs = oracle.get_primes(n, 31, 2) + oracle.get_primes(n, 45, 2) + oracle.get_primes(n, 60, 1)
    ps = oracle.get_primes(n, 59, 2)
    return oracle.Params(6, qs + ps, 2)


def rand_poly(p, rng, tidx):
    return np.array([[rng.randrange(p.moduli[t]) for _ in range(p.n)] for t in tidx], dtype=np.uint64)


def ntt_closed_form(a, q, psi, logn):
    n = 1 << logn
    out = [0] * n
    for i in range(n):
        w = pow(psi, 2 * i + 1, q)
        acc, x = 0, 1
        for j in range(n):
            acc += a[j] * x
            x = x * w % q
        r = 0
        for b in range(logn):
            r |= ((i >> b) & 1) << (logn - 1 - b)
        out[r] = acc % q
    return out


def test_tables(small, oracle):
    p = small
    for i, q in enumerate(p.moduli):
        psi = p.psi[i]
        assert pow(psi, p.n, q) == q - 1
        for k in (0, 1, 2, 3, 17, p.n - 1):
            r = oracle.bit_reverse(k, p.logn)
            assert int(p.tw[i][r]) == pow(psi, k, q)
            if k:
                assert int(p.itw[i][r]) == pow(psi, -k, q) * pow(2, -1, q) % q
            assert int(p.twq[i][r]) == (int(p.tw[i][r]) << 64) // q
            assert int(p.itwq[i][r]) == (int(p.itw[i][r]) << 64) // q


@pytest.mark.parametrize("logn", [3, 6, 8])
def test_ntt_closed_form(oracle, logn):
    n = 1 << logn
    rng = random.Random(logn)
    mods = oracle.get_primes(n, 50, 1) + oracle.get_primes(n, 60, 1) + oracle.get_primes(n, 20, 1)
    p = oracle.Params(logn, mods, 1)
    a = rand_poly(p, rng, range(3))
    got = p.ntt_fwd(a.copy())
    for i, q in enumerate(mods):
        assert [int(v) for v in got[i]] == ntt_closed_form([int(v) for v in a[i]], q, p.psi[i], logn)
    assert (p.ntt_inv(got.copy()) == a).all()


def test_ntt_edge_values_and_limb_table_map(small):
    p = small
    # all coefficients q-1, all zero, a single one; table map: data limb i -> table tidx[i]
    tidx = [6, 0, 5]
    a = np.array([[p.moduli[t] - 1] * p.n for t in tidx], dtype=np.uint64)
    f = p.ntt_fwd(a.copy(), tidx)
    for row, t in zip(f, tidx):
        q = p.moduli[t]
        assert [int(v) for v in row] == ntt_closed_form([q - 1] * p.n, q, p.psi[t], p.logn)
    assert (p.ntt_inv(f.copy(), tidx) == a).all()
    z = np.zeros((1, p.n), dtype=np.uint64)
    assert not p.ntt_fwd(z.copy()).any()
    one = z.copy()
    one[0, 0] = 1
    assert (p.ntt_fwd(one) == 1).all()


def test_negacyclic_convolution(small):
    p, rng = small, random.Random(1)
    n, q = p.n, p.moduli[4]
    a = [rng.randrange(q) for _ in range(n)]
    b = [rng.randrange(q) for _ in range(n)]
    ref = [0] * n
    for i in range(n):
        for j in range(n):
            k = i + j
            if k < n:
                ref[k] = (ref[k] + a[i] * b[j]) % q
            else:
                ref[k - n] = (ref[k - n] - a[i] * b[j]) % q
    A = np.zeros((5, n), dtype=np.uint64)
    B = np.zeros((5, n), dtype=np.uint64)
    A[4], B[4] = a, b
    prod = p.mul(p.ntt_fwd(A.copy()), p.ntt_fwd(B.copy()))
    assert [int(v) for v in p.ntt_inv(prod)[4]] == ref


def test_ntt_independent_radix2_at_4096(oracle):
    """Independent textbook recursion (decimation in time over Python integers) at N = 4096."""
    logn, n = 12, 4096
    q = oracle.get_primes(n, 50, 1)[0]
    p = oracle.Params(logn, [q, oracle.get_primes(n, 49, 1)[0]], 1)
    rng = random.Random(3)
    a = [rng.randrange(q) for _ in range(n)]
    psi = p.psi[0]
    tw = [a[j] * pow(psi, j, q) % q for j in range(n)]       # negacyclic -> cyclic
    w = psi * psi % q

    def fft(x, root):
        m = len(x)
        if m == 1:
            return x
        e, o = fft(x[0::2], root * root % q), fft(x[1::2], root * root % q)
        out, t = [0] * m, 1
        for k in range(m // 2):
            v = t * o[k] % q
            out[k], out[k + m // 2] = (e[k] + v) % q, (e[k] - v) % q
            t = t * root % q
        return out

    nat = fft(tw, w)                                         # nat[i] = a(psi^(2i+1))
    got = p.ntt_fwd(np.array([a, [0] * n], dtype=np.uint64))[0]
    rev = oracle.bitrev_perm(logn)
    assert [int(v) for v in got] == [nat[int(rev[i])] for i in range(n)]


def _digits(p, L):
    alpha = p.size_p
    return [(s, min(alpha, L - s)) for s in range(0, L, alpha)]


@pytest.mark.parametrize("L", [5, 4, 3, 2, 1])
def test_modup_bigint(small, L):
    p, rng = small, random.Random(10 + L)
    K = p.size_p
    x = rand_poly(p, rng, range(L))                     # coefficient form
    c = p.ntt_fwd(x.copy())
    y = p.modup(c)
    assert y.shape == (len(_digits(p, L)), L + K, p.n)
    for d, (s, sz) in enumerate(_digits(p, L)):
        part = p.moduli[s:s + sz]
        Qd = math.prod(part)
        tidx = [p.table_index(L, t) for t in range(L + K)]
        coef = p.ntt_inv(y[d].copy(), tidx)
        for j in range(p.n):
            xt = [int(x[s + i][j]) * pow((Qd // qi) % qi, -1, qi) % qi for i, qi in enumerate(part)]
            lifted = sum(v * (Qd // qi) for v, qi in zip(xt, part))
            exact = lifted % Qd
            assert (lifted - exact) % Qd == 0 and 0 <= (lifted - exact) // Qd < sz
            for t in range(L + K):
                m = p.moduli[tidx[t]]
                if s <= t < s + sz:
                    assert int(y[d][t][j]) == int(c[t][j])          # own limbs untouched, NTT form
                else:
                    assert int(coef[t][j]) == lifted % m


@pytest.mark.parametrize("L", [5, 3, 1])
def test_inner_product_bigint(small, L):
    p, rng = small, random.Random(20 + L)
    K, QP = p.size_p, p.size_qp
    beta = len(_digits(p, L))
    tidx = [p.table_index(L, t) for t in range(L + K)]
    y = np.stack([rand_poly(p, rng, tidx) for _ in range(beta)])
    evk = [np.stack([rand_poly(p, rng, range(QP)), rand_poly(p, rng, range(QP))]) for _ in range(beta)]
    out = p.inner_prod(y, evk)
    for b in range(2):
        for t in range(L + K):
            m = p.moduli[tidx[t]]
            for j in range(0, p.n, 7):
                want = sum(int(y[d][t][j]) * int(evk[d][b][tidx[t]][j]) for d in range(beta)) % m
                assert int(out[b][t][j]) == want


@pytest.mark.parametrize("L", [5, 2, 1])
def test_moddown_bigint(small, L):
    p, rng = small, random.Random(30 + L)
    K = p.size_p
    tidx = [p.table_index(L, t) for t in range(L + K)]
    xc = rand_poly(p, rng, tidx)                       # coefficient form over Ql u P
    cx = p.ntt_fwd(xc.copy(), tidx)
    out = p.ntt_inv(p.moddown(cx))
    ps = p.moduli[p.size_q:]
    P = math.prod(ps)
    for j in range(p.n):
        zt = [int(xc[L + k][j]) * pow((P // pk) % pk, -1, pk) % pk for k, pk in enumerate(ps)]
        delta = sum(z * (P // pk) for z, pk in zip(zt, ps))
        assert delta % P == _crt([int(xc[L + k][j]) for k in range(K)], ps) and delta // P < K
        for i in range(L):
            q = p.moduli[i]
            assert int(out[i][j]) == (int(xc[i][j]) - delta) * pow(P, -1, q) % q
            assert int(out[i][j]) * P % q == (int(xc[i][j]) - delta) % q


def _crt(res, mods):
    M = math.prod(mods)
    return sum(r * (M // m) * pow(M // m, -1, m) for r, m in zip(res, mods)) % M


@pytest.mark.parametrize("L", [5, 2])
def test_rescale_bigint(small, L):
    p, rng = small, random.Random(40 + L)
    xc = np.stack([rand_poly(p, rng, range(L)) for _ in range(2)])
    ct = np.stack([p.ntt_fwd(v.copy()) for v in xc])
    out = p.rescale(ct)
    assert out.shape == (2, L - 1, p.n)
    ql = p.moduli[L - 1]
    for pi in range(2):
        coef = p.ntt_inv(out[pi].copy())
        for i in range(L - 1):
            q = p.moduli[i]
            for j in range(p.n):
                want = (int(xc[pi][i][j]) - int(xc[pi][L - 1][j]) % q) * pow(ql, -1, q) % q
                assert int(coef[i][j]) == want


def test_rescale_divides_exactly(small):
    """On an integer polynomial v < Q the output is floor-style (v - [v]_{q_last}) / q_last."""
    p, rng = small, random.Random(5)
    L = 3
    Q = math.prod(p.moduli[:L])
    vals = [rng.randrange(Q) for _ in range(p.n)]
    xc = np.array([[v % p.moduli[i] for v in vals] for i in range(L)], dtype=np.uint64)
    out = p.ntt_inv(p.rescale(p.ntt_fwd(xc.copy())[None])[0])
    ql = p.moduli[L - 1]
    for j, v in enumerate(vals):
        want = (v - v % ql) // ql
        assert [int(out[i][j]) for i in range(L - 1)] == [want % p.moduli[i] for i in range(L - 1)]


def test_tensor_and_square_bigint(small):
    p, rng = small, random.Random(6)
    L = 4
    a = np.stack([rand_poly(p, rng, range(L)) for _ in range(2)])
    b = np.stack([rand_poly(p, rng, range(L)) for _ in range(2)])
    # edge values: both operands q-1 so that (a0+a1)(b0+b1) is as large as it gets
    for i in range(L):
        a[:, i, 0] = p.moduli[i] - 1
        b[:, i, 0] = p.moduli[i] - 1
    t, s = p.tensor(a, b), p.square(a)
    for i in range(L):
        q = p.moduli[i]
        for j in range(p.n):
            a0, a1, b0, b1 = (int(v) for v in (a[0][i][j], a[1][i][j], b[0][i][j], b[1][i][j]))
            assert [int(t[k][i][j]) for k in range(3)] == [a0 * b0 % q, (a0 * b1 + a1 * b0) % q, a1 * b1 % q]
            assert [int(s[k][i][j]) for k in range(3)] == [a0 * a0 % q, 2 * a0 * a1 % q, a1 * a1 % q]


@pytest.mark.parametrize("s1,s2", [(2, 2), (2, 3), (3, 2), (3, 3), (1, 3), (4, 2), (5, 5), (16, 16)])
def test_tensor_mxn_is_the_convolution_of_the_operands(small, s1, s2):
    """orc_tensor_mxn against Python integers: polynomial j of the product is the sum of ct1_a ct2_b over a + b = j
    (the ciphertexts multiplied as polynomials in the secret key), coefficient by coefficient and limb by limb, with
    both operands at q - 1 in one position so that the 128-bit sum is as large as it gets; the 2 x 2 case must equal
    the dedicated 2 x 2 routine, and squaring a size-2 operand the squaring routine."""
    p, rng = small, random.Random(60 + 10 * s1 + s2)
    L = 4
    a = np.stack([rand_poly(p, rng, range(L)) for _ in range(s1)])
    b = np.stack([rand_poly(p, rng, range(L)) for _ in range(s2)])
    for i in range(L):
        a[:, i, 0] = p.moduli[i] - 1
        b[:, i, 0] = p.moduli[i] - 1
        a[:, i, 1] = 0
    t = p.tensor_mxn(a, b)
    assert t.shape == (s1 + s2 - 1, L, p.n)
    for i in range(L):
        q = p.moduli[i]
        for j in range(0, p.n, 7):
            av = [int(a[k][i][j]) for k in range(s1)]
            bv = [int(b[k][i][j]) for k in range(s2)]
            want = [sum(av[x] * bv[k - x] for x in range(s1) if 0 <= k - x < s2) % q for k in range(s1 + s2 - 1)]
            assert [int(t[k][i][j]) for k in range(s1 + s2 - 1)] == want
    if (s1, s2) == (2, 2):
        assert (t == p.tensor(a, b)).all()
        assert (p.tensor_mxn(a, a) == p.square(a)).all()


def test_elementwise_bigint(small):
    p, rng = small, random.Random(8)
    a, b, c = (rand_poly(p, rng, range(5)) for _ in range(3))
    a[:, 0], b[:, 0] = 0, [q - 1 for q in p.moduli[:5]]
    for i in range(5):
        q = p.moduli[i]
        ai, bi, ci = ([int(v) for v in x[i]] for x in (a, b, c))
        assert [int(v) for v in p.add(a, b)[i]] == [(x + y) % q for x, y in zip(ai, bi)]
        assert [int(v) for v in p.sub(a, b)[i]] == [(x - y) % q for x, y in zip(ai, bi)]
        assert [int(v) for v in p.mul(a, b)[i]] == [x * y % q for x, y in zip(ai, bi)]
        assert [int(v) for v in p.negate(a)[i]] == [-x % q for x in ai]
        assert [int(v) for v in p.mul_add(a, b, c)[i]] == [(x * y + z) % q for x, y, z in zip(ai, bi, ci)]
        assert [int(v) for v in p.mul_add(a, b, c, True)[i]] == [-(x * y + z) % q for x, y, z in zip(ai, bi, ci)]


@pytest.mark.parametrize("step", [1, 3, -2, 0, 15])
def test_galois_permutation_is_the_automorphism(small, oracle, step):
    p, rng = small, random.Random(50)
    n = p.n
    g = oracle.galois_elt_from_step(step, n)
    a = rand_poly(p, rng, range(3))
    sig = np.zeros_like(a)
    for i in range(3):
        q = p.moduli[i]
        for j in range(n):
            k = j * g % (2 * n)
            if k < n:
                sig[i][k] = a[i][j]
            else:
                sig[i][k - n] = (q - int(a[i][j])) % q
    assert (p.galois_ntt(p.ntt_fwd(a.copy()), g) == p.ntt_fwd(sig.copy())).all()


def test_galois_elements(oracle):
    f = oracle.galois_elt_from_step
    n = 1 << 16
    assert f(0, n) == 2 * n - 1 and f(1, n) == 5 and f(2, n) == 25
    assert f(-1, n) == pow(5, n // 2 - 1, 2 * n) and f(-1, n) * 5 % (2 * n) == 1
    with pytest.raises(ValueError):
        f(n // 2, n)


def test_galois_table_formula(small, oracle):
    p = small
    g = 25
    t = p.galois_table(g)
    for i in range(p.n):
        r = oracle.bit_reverse(i, p.logn)
        assert int(t[i]) == oracle.bit_reverse(((g * (2 * r + 1)) >> 1) & (p.n - 1), p.logn)
