"""Pins the oracle's scalar arithmetic and host number theory.

Known answers are the ones the reference's own unit tests hold:
  cahel-main/unittest/util/uintarithsmallmod.cu:140-182 (BarrettReduce128), :184-210 (MultiplyUIntMod),
  :371-400 (MultiplyUIntModOperand), :442-480 (MultiplyUIntModLazy),
  cahel-main/unittest/util/numth.cu:92-110 (IsPrime), :197-216 (TryMinimalPrimitiveRootMod),
  cahel-main/unittest/util/common.cu:160-186 (ReverseBits),
  cahel-main/src/util/globals.cu:77-101,145-158 (default prime tables = largest NTT primes, descending).
Everything else is checked against Python big-integer arithmetic.
"""
import ctypes as C
import random

import numpy as np
import pytest


def ratio(O, q):
    lo, hi = O.barrett_ratio(q)
    return np.array([lo, hi], dtype=np.uint64)


def barrett128(O, lo, hi, q):
    r = ratio(O, q)
    return O.lib().orc_barrett128(lo, hi, q, r.ctypes.data_as(O.u64p))


def test_barrett128_known_answers(oracle):
    O = oracle
    M = 0xFFFFFFFFFFFFFFFF
    assert barrett128(O, 0, 0, 2) == 0
    assert barrett128(O, 1, 0, 2) == 1
    assert barrett128(O, M, M, 2) == 1
    assert barrett128(O, 123, 456, 3) == 0
    assert barrett128(O, M, M, 3) == 0
    q = 13131313131313
    assert barrett128(O, 1, 0, q) == 1
    assert barrett128(O, 123, 456, q) == 8722750765283
    assert barrett128(O, 24242424242424, 79797979797979, q) == 1010101010101


def test_mulmod_known_answers(oracle):
    O = oracle
    mm = lambda a, b, q: O.lib().orc_mulmod(a, b, q, ratio(O, q).ctypes.data_as(O.u64p))
    assert mm(7, 7, 10) == 9 and mm(6, 7, 10) == 2 and mm(1, 1, 2) == 1
    q = 2305843009211596801
    assert mm(1152921504605798400, 1152921504605798401, q) == 576460752302899200
    assert mm(1152921504605798401, 1152921504605798401, q) == 1729382256908697601
    assert mm(2305843009211596800, 2305843009211596800, q) == 1


def test_shoup_operand_known_answers(oracle):
    sq = oracle.lib().orc_shoup_quotient
    assert sq(1, 3) == 6148914691236517205 and sq(2, 3) == 12297829382473034410
    assert sq(1, 2147483647) == 8589934596 and sq(2147483646, 2147483647) == 18446744065119617019
    q = 2305843009211596801
    assert sq(1, q) == 8 and sq(q - 1, q) == 18446744073709551607


def test_mul_shoup_known_answers(oracle):
    L = oracle.lib()
    q = 2305843009211596801

    def ms(x, w, mod):
        return L.orc_mul_shoup(x, w, L.orc_shoup_quotient(w, mod), mod)

    assert ms(7, 6, 10) == 2 and ms(7, 7, 10) == 9 and ms(6, 7, 10) == 2
    assert ms(1152921504605798401, 1152921504605798400, q) == 576460752302899200
    assert ms(1152921504605798401, 1152921504605798401, q) == 1729382256908697601
    # the lazy form returns 2305843009211596802 = 1 + q for this pair (unittest :478); reduced it is 1
    assert ms(q - 1, q - 1, q) == 1


def test_scalar_random_against_bigint(oracle):
    O, L = oracle, oracle.lib()
    rng = random.Random(7)
    for bits in (30, 40, 50, 59, 60, 61):
        for _ in range(200):
            q = rng.randrange(1 << (bits - 1), 1 << bits) | 1
            a, b = rng.randrange(q), rng.randrange(q)
            r = ratio(O, q)
            assert L.orc_mulmod(a, b, q, r.ctypes.data_as(O.u64p)) == a * b % q
            x = rng.randrange(1 << 128)
            assert L.orc_barrett128(x & (2**64 - 1), x >> 64, q, r.ctypes.data_as(O.u64p)) == x % q
            y = rng.randrange(1 << 64)
            assert L.orc_barrett64(y, q, int(r[1])) == y % q
            w = rng.randrange(q)
            assert L.orc_shoup_quotient(w, q) == (w << 64) // q
            # Shoup multiply accepts any 64-bit left operand (lazy NTT values up to 4q)
            z = rng.randrange(4 * q)
            assert L.orc_mul_shoup(z, w, (w << 64) // q, q) == z * w % q


def test_is_prime_known_answers(oracle):
    ip = oracle.is_prime
    assert [ip(v) for v in (0, 2, 3, 4, 5, 221, 65537, 65536, 59399, 72307)] == \
        [False, True, True, False, True, False, True, False, True, True]
    assert not ip(72307 * 59399)
    assert ip(36893488147419103) and not ip(36893488147419107)


def test_primes_match_reference_default_tables(oracle):
    gp = oracle.get_primes
    assert gp(8192, 44, 3) == [0xfffffffc001, 0xffffff6c001, 0xfffffebc001]
    assert gp(8192, 43, 2) == [0x7fffffd8001, 0x7fffffc8001]
    assert gp(16384, 48, 3) == [0xfffffffd8001, 0xfffffffa0001, 0xfffffff00001]
    assert gp(16384, 49, 6) == [0x1fffffff68001, 0x1fffffff50001, 0x1ffffffee8001, 0x1ffffffea0001,
                                0x1ffffffe88001, 0x1ffffffe48001]
    assert gp(16384, 50, 6) == [0x3ffffffdf0001, 0x3ffffffd48001, 0x3ffffffd20001, 0x3ffffffd18001,
                                0x3ffffffcd0001, 0x3ffffffc70001]
    assert gp(32768, 55, 5) == [0x7fffffffe90001, 0x7fffffffbf0001, 0x7fffffffbd0001, 0x7fffffffba0001,
                                0x7fffffffaa0001]
    assert gp(32768, 56, 1) == [0xfffffffff70001]


def test_coeff_modulus_create_order(oracle):
    # first occurrence of a bit size takes the largest prime of that size (src/modulus.cu:121-131)
    n = 8192
    got = oracle.coeff_modulus_create(n, [60, 40, 40, 60])
    p60, p40 = oracle.get_primes(n, 60, 2), oracle.get_primes(n, 40, 2)
    assert got == [p60[0], p40[0], p40[1], p60[1]]
    assert all(q % (2 * n) == 1 and oracle.is_prime(q) for q in got)


def test_minimal_primitive_root_known_answers(oracle):
    mr = oracle.minimal_primitive_root
    assert mr(2, 11) == 10 and mr(2, 29) == 28 and mr(4, 29) == 12
    assert mr(2, 1234565441) == 1234565440 and mr(8, 1234565441) == 249725733


def test_minimal_primitive_root_is_minimal(oracle):
    q, deg = 0xffffff6c001, 64
    r = oracle.minimal_primitive_root(deg, q)
    roots = [x for x in (pow(g, (q - 1) // deg, q) for g in range(2, 400)) if pow(x, deg // 2, q) == q - 1]
    assert pow(r, deg // 2, q) == q - 1 and r == min(set(roots) | {r})
    # all primitive roots are odd powers of r: the minimum over them is r itself
    assert min(pow(r, k, q) for k in range(1, deg, 2)) == r


def test_reverse_bits_known_answers(oracle):
    rb = oracle.bit_reverse
    assert rb(1, 32) == 0x80000000 and rb(3, 32) == 0xC0000000 and rb(0x8000, 32) == 0x10000
    assert rb(0xFFFF, 32) == 0xFFFF0000 and rb(1, 16) == 0x8000 and rb(3, 16) == 0xC000 and rb(0x8000, 16) == 1
    assert list(oracle.bitrev_perm(3)) == [0, 4, 2, 6, 1, 5, 3, 7]


def test_barrett_ratio_is_floor_2_128_over_q(oracle):
    for q in (3, 13131313131313, 2305843009211596801):
        lo, hi = oracle.barrett_ratio(q)
        assert (hi << 64) | lo == (1 << 128) // q


def test_chacha20_block_rfc8439_vector(oracle):
    # RFC 8439 section 2.3.2: key 00..1f, block counter 1, nonce 00:00:00:09:00:00:00:4a:00:00:00:00
    key = np.frombuffer(bytes(range(32)), dtype="<u4").copy()
    out = np.zeros(16, dtype=np.uint32)
    counter = 1 | (0x09000000 << 32)   # state words 12, 13
    stream = 0x4a000000                # state words 14, 15
    oracle.lib().orc_chacha20_block(key.ctypes.data_as(oracle.u32p), C.c_uint64(counter), C.c_uint64(stream),
                                    out.ctypes.data_as(oracle.u32p))
    assert [int(v) for v in out] == [
        0xe4e7f110, 0x15593bd1, 0x1fdd0f50, 0xc47120a3, 0xc7f4d1c7, 0x0368c033, 0x9aaa2204, 0x4e6cd4c3,
        0x466482d2, 0x09aa9f07, 0x05d7c214, 0xa2028bd9, 0xd19c12b5, 0xb94e16de, 0xe883d0cb, 0x4e3c50a2]
