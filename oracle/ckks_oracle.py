"""CPU checker for the CKKS hot path of CAHEL (reference tree: cahel-main/).

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke check and by the benchmark's
cpu_baseline leg.  The product (lancelot_amd/) never imports it.

Host number theory is restated here with Python integers (primes, roots, CRT constants); the
per-coefficient loops run in oracle/ckks_oracle.c through ctypes.  Each function cites the reference
lines it follows.
"""
from __future__ import annotations

import ctypes as C
import math
import os
import subprocess
from dataclasses import dataclass, field

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libckks_oracle.so")
# a build of the same source to load instead (the sanitizer build of oracle/Makefile)
_LIB_OVERRIDE = os.environ.get("CKKS_ORACLE_LIB")

u64p = C.POINTER(C.c_uint64)
u32p = C.POINTER(C.c_uint32)


def build(force: bool = False) -> str:
    """Compile oracle/ckks_oracle.c (gcc) if the shared object is missing or stale."""
    src = os.path.join(_HERE, "ckks_oracle.c")
    if force or not os.path.exists(_LIB_PATH) or os.path.getmtime(_LIB_PATH) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libckks_oracle.so"], stdout=subprocess.DEVNULL)
    return _LIB_PATH


class _CParams(C.Structure):
    _fields_ = [("logn", C.c_uint32), ("size_q", C.c_uint32), ("size_p", C.c_uint32), ("reserved", C.c_uint32),
                ("mod", u64p), ("ratio", u64p), ("tw", u64p), ("twq", u64p), ("itw", u64p), ("itwq", u64p)]


_lib = None


def lib():
    global _lib
    if _lib is None:
        if _LIB_OVERRIDE:
            _lib = C.CDLL(_LIB_OVERRIDE)
        else:
            build()
            _lib = C.CDLL(_LIB_PATH)
        _lib.orc_shoup_quotient.restype = C.c_uint64
        _lib.orc_shoup_quotient.argtypes = [C.c_uint64, C.c_uint64]
        _lib.orc_mul_shoup.restype = C.c_uint64
        _lib.orc_mul_shoup.argtypes = [C.c_uint64] * 4
        _lib.orc_barrett128.restype = C.c_uint64
        _lib.orc_barrett128.argtypes = [C.c_uint64, C.c_uint64, C.c_uint64, u64p]
        _lib.orc_barrett64.restype = C.c_uint64
        _lib.orc_barrett64.argtypes = [C.c_uint64] * 3
        _lib.orc_mulmod.restype = C.c_uint64
        _lib.orc_mulmod.argtypes = [C.c_uint64, C.c_uint64, C.c_uint64, u64p]
        for name in ("orc_power_table", "orc_shoup_table", "orc_ntt_fwd", "orc_ntt_inv", "orc_ntt_fwd_limbs",
                     "orc_ntt_inv_limbs", "orc_elementwise", "orc_negate", "orc_mul_add", "orc_tensor_2x2",
                     "orc_tensor_square", "orc_tensor_mxn", "orc_galois_ntt", "orc_galois_table", "orc_rescale", "orc_modup",
                     "orc_inner_prod", "orc_moddown", "orc_evk_add_ps", "orc_chacha20_block", "orc_sample_ternary",
                     "orc_sample_error", "orc_sample_uniform", "orc_sample_gauss", "orc_decompose_coeffs"):
            getattr(_lib, name).restype = None
    return _lib


def _p64(a: np.ndarray):
    assert a.dtype == np.uint64 and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(u64p)


def _p32(a: np.ndarray):
    assert a.dtype == np.uint32 and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(u32p)


# ------------------------------------------------------------------------------------------------
# host number theory (cahel-main/src/util/numth.cu, src/modulus.cu)
# ------------------------------------------------------------------------------------------------

def is_prime(v: int) -> bool:
    """Deterministic Miller-Rabin for 64-bit inputs (src/util/numth.cu:131-207 uses trial division
    by 2..13 and randomised Miller-Rabin; both decide primality, so the results agree)."""
    if v < 2:
        return False
    for sp in (2, 3, 5, 7, 11, 13, 17, 19, 23, 29, 31, 37):
        if v % sp == 0:
            return v == sp
    d, r = v - 1, 0
    while d % 2 == 0:
        d //= 2
        r += 1
    for a in (2, 3, 5, 7, 11, 13, 17, 19, 23, 29, 31, 37):
        x = pow(a, d, v)
        if x in (1, v - 1):
            continue
        for _ in range(r - 1):
            x = x * x % v
            if x == v - 1:
                break
        else:
            return False
    return True


def get_primes(ntt_size: int, bit_size: int, count: int) -> list[int]:
    """src/util/numth.cu:209-235: primes 2^b - k*2N + 1, k = 1, 2, ..., above 2^(b-1), descending."""
    factor = 2 * ntt_size
    value = (1 << bit_size) - factor + 1
    lower = 1 << (bit_size - 1)
    out = []
    while count > 0 and value > lower:
        if is_prime(value):
            out.append(value)
            count -= 1
        value -= factor
    if count > 0:
        raise ValueError("failed to find enough qualifying primes")
    return out


def coeff_modulus_create(n: int, bit_sizes: list[int]) -> list[int]:
    """src/modulus.cu:93-133: per distinct bit size the largest primes, handed out in order of appearance."""
    counts: dict[int, int] = {}
    for b in bit_sizes:
        counts[b] = counts.get(b, 0) + 1
    table = {b: get_primes(n, b, c) for b, c in counts.items()}
    pos = {b: 0 for b in counts}
    out = []
    for b in bit_sizes:
        out.append(table[b][pos[b]])
        pos[b] += 1
    return out


def minimal_primitive_root(degree: int, q: int) -> int:
    """src/util/numth.cu:278-335: the smallest primitive degree-th root of unity mod q (degree a power
    of two).  Any primitive root r generates all of them as r^(odd); the minimum is unique."""
    if (q - 1) % degree:
        raise ValueError("no primitive root of that degree")
    quotient = (q - 1) // degree
    x = 2
    while True:
        r = pow(x, quotient, q)
        if pow(r, degree // 2, q) == q - 1:
            break
        x += 1
    sq = r * r % q
    best, cur = r, r
    for _ in range(degree // 2):
        if cur < best:
            best = cur
        cur = cur * sq % q
    return best


def bit_reverse(x: int, bits: int) -> int:
    r = 0
    for i in range(bits):
        r |= ((x >> i) & 1) << (bits - 1 - i)
    return r


def bitrev_perm(logn: int) -> np.ndarray:
    n = 1 << logn
    idx = np.arange(n, dtype=np.uint32)
    r = np.zeros(n, dtype=np.uint32)
    for i in range(logn):
        r |= ((idx >> i) & 1) << (logn - 1 - i)
    return r


def barrett_ratio(q: int) -> tuple[int, int]:
    """src/modulus.cu:36-48: floor(2^128 / q) as (low word, high word)."""
    r = (1 << 128) // q
    return r & ((1 << 64) - 1), r >> 64


# ------------------------------------------------------------------------------------------------
# parameter set + tables (src/context.cu:352-403, src/util/ntt.cu:32-80, src/util/rns.cu:433-556)
# ------------------------------------------------------------------------------------------------

@dataclass
class LevelTables:
    """Hybrid key-switch tables of the data level with L limbs (src/util/rns.cu:490-556)."""
    L: int
    beta: int
    digit_start: list[int]
    digit_size: list[int]
    hatinv: np.ndarray      # [L]   partQlHatInv_mod_Ql_concat
    mats: np.ndarray        # concatenated per-digit matrices, row-major [L+K-size][size]
    mat_off: np.ndarray     # [beta] offsets into mats (uint32)
    qlast_inv: np.ndarray   # [L-1] q_{L-1}^-1 mod q_j


class Params:
    """CKKS parameter set: moduli (Q then P), NTT tables, CRT constants for every data level.

    chain index 0 is the key level (Q u P), chain index c >= 1 has size_q - c + 1 limbs
    (src/context.cu:380-402)."""

    def __init__(self, logn: int, moduli: list[int], size_p: int):
        self.logn = logn
        self.n = 1 << logn
        self.moduli = [int(m) for m in moduli]
        self.size_p = size_p
        self.size_q = len(moduli) - size_p
        self.size_qp = len(moduli)
        n, qp = self.n, self.size_qp
        L = lib()
        self.mod = np.array(self.moduli, dtype=np.uint64)
        self.ratio = np.array([barrett_ratio(q) for q in self.moduli], dtype=np.uint64).reshape(qp, 2)
        self.psi = [minimal_primitive_root(2 * n, q) for q in self.moduli]
        rev = bitrev_perm(logn)
        self.tw = np.zeros((qp, n), dtype=np.uint64)
        self.itw = np.zeros((qp, n), dtype=np.uint64)
        powers = np.zeros(n, dtype=np.uint64)
        for i, q in enumerate(self.moduli):
            # src/util/ntt.cu:46-56: root_powers[bitrev(i)] = psi^i, entry 0 = 1
            L.orc_power_table(_p64(powers), C.c_uint64(1), C.c_uint64(self.psi[i]), C.c_uint64(q), C.c_size_t(n))
            self.tw[i][rev] = powers
            # src/util/ntt.cu:58-71: inv_root_powers_div2[bitrev(i)] = psi^-i / 2, entry 0 = psi^-1 / 2
            ipsi = pow(self.psi[i], -1, q)
            half = pow(2, -1, q)
            L.orc_power_table(_p64(powers), C.c_uint64(half), C.c_uint64(ipsi), C.c_uint64(q), C.c_size_t(n))
            self.itw[i][rev] = powers
            self.itw[i][0] = ipsi * half % q
        self.twq = np.zeros_like(self.tw)
        self.itwq = np.zeros_like(self.itw)
        for i, q in enumerate(self.moduli):
            L.orc_shoup_table(_p64(self.twq[i]), _p64(self.tw[i]), C.c_uint64(q), C.c_size_t(n))
            L.orc_shoup_table(_p64(self.itwq[i]), _p64(self.itw[i]), C.c_uint64(q), C.c_size_t(n))
        self.c = _CParams(logn, self.size_q, size_p, 0, _p64(self.mod), _p64(self.ratio.reshape(-1)),
                          _p64(self.tw.reshape(-1)), _p64(self.twq.reshape(-1)), _p64(self.itw.reshape(-1)),
                          _p64(self.itwq.reshape(-1)))
        self._build_hybrid()
        self._levels: dict[int, LevelTables] = {}

    # -- hybrid key switching constants that do not depend on the level (src/util/rns.cu:490-512, 553) --
    def _build_hybrid(self):
        q, p = self.moduli[: self.size_q], self.moduli[self.size_q:]
        self.P = math.prod(p) if p else 1
        self.p_mod_q = np.array([self.P % qi for qi in q], dtype=np.uint64)
        self.pinv_mod_q = np.array([pow(self.P % qi, -1, qi) for qi in q], dtype=np.uint64)
        self.phat_inv = np.array([pow((self.P // pk) % pk, -1, pk) for pk in p], dtype=np.uint64)
        # BaseConverter P -> Ql: QHatModp[j][k] = (P / p_k) mod q_j (src/util/rns.cu:374-392)
        self.mat_p2q = np.array([[(self.P // pk) % qj for pk in p] for qj in q], dtype=np.uint64).reshape(
            self.size_q, max(self.size_p, 1))

    def chain_limbs(self, chain_index: int) -> int:
        """Number of limbs of a ciphertext at chain_index (0 = key level)."""
        return self.size_qp if chain_index == 0 else self.size_q - chain_index + 1

    def level(self, L: int) -> LevelTables:
        """Tables of the data level with L limbs (src/util/rns.cu:514-551, :483-488)."""
        if L in self._levels:
            return self._levels[L]
        alpha = self.size_p
        q = self.moduli[:L]
        qlp = q + self.moduli[self.size_q:]
        beta = -(-L // alpha)
        starts, sizes, hatinv, mats, offs = [], [], [0] * L, [], []
        off = 0
        for d in range(beta):
            s = d * alpha
            sz = min(alpha, L - s)
            starts.append(s)
            sizes.append(sz)
            part = q[s:s + sz]
            prod = math.prod(part)
            for i, qi in enumerate(part):
                hatinv[s + i] = pow((prod // qi) % qi, -1, qi)
            compl = qlp[:s] + qlp[s + sz:]
            rows = [[(prod // qi) % m for qi in part] for m in compl]
            offs.append(off)
            mats.extend(v for row in rows for v in row)
            off += len(compl) * sz
        qlast = q[L - 1]
        lt = LevelTables(L, beta, starts, sizes, np.array(hatinv, dtype=np.uint64), np.array(mats, dtype=np.uint64),
                         np.array(offs, dtype=np.uint32),
                         np.array([pow(qlast % qj, -1, qj) for qj in q[:L - 1]], dtype=np.uint64))
        self._levels[L] = lt
        return lt

    def table_index(self, L: int, t: int) -> int:
        return t if t < L else self.size_q + (t - L)

    # ---------------------------------------------------------------------------------------------
    # integer stages
    # ---------------------------------------------------------------------------------------------
    def ntt_fwd(self, data: np.ndarray, tidx=None) -> np.ndarray:
        """In-place forward NTT of data [limbs][N]; limb i uses table tidx[i] (default i)."""
        d = data.reshape(-1, self.n)
        tidx = np.arange(d.shape[0], dtype=np.uint32) if tidx is None else np.asarray(tidx, dtype=np.uint32)
        lib().orc_ntt_fwd_limbs(C.byref(self.c), _p64(data.reshape(-1)), C.c_uint32(d.shape[0]), _p32(tidx))
        return data

    def ntt_inv(self, data: np.ndarray, tidx=None) -> np.ndarray:
        d = data.reshape(-1, self.n)
        tidx = np.arange(d.shape[0], dtype=np.uint32) if tidx is None else np.asarray(tidx, dtype=np.uint32)
        lib().orc_ntt_inv_limbs(C.byref(self.c), _p64(data.reshape(-1)), C.c_uint32(d.shape[0]), _p32(tidx))
        return data

    def _ew(self, op: int, a, b) -> np.ndarray:
        out = np.empty_like(a)
        lib().orc_elementwise(C.byref(self.c), C.c_int(op), _p64(a.reshape(-1)), _p64(b.reshape(-1)),
                              _p64(out.reshape(-1)), C.c_uint32(a.reshape(-1, self.n).shape[0]))
        return out

    def add(self, a, b):
        """[limbs][N] + [limbs][N]; limb i mod q_i (src/polymath.cu:40)."""
        return self._ew(0, a, b)

    def sub(self, a, b):
        return self._ew(1, a, b)

    def mul(self, a, b):
        return self._ew(2, a, b)

    def negate(self, a):
        out = np.empty_like(a)
        lib().orc_negate(C.byref(self.c), _p64(a.reshape(-1)), _p64(out.reshape(-1)),
                         C.c_uint32(a.reshape(-1, self.n).shape[0]))
        return out

    def mul_add(self, a, b, c, negate=False):
        out = np.empty_like(a)
        lib().orc_mul_add(C.byref(self.c), _p64(a.reshape(-1)), _p64(b.reshape(-1)), _p64(c.reshape(-1)),
                          _p64(out.reshape(-1)), C.c_uint32(a.reshape(-1, self.n).shape[0]), C.c_int(int(negate)))
        return out

    def tensor(self, ct1: np.ndarray, ct2: np.ndarray) -> np.ndarray:
        """(2,L,N) x (2,L,N) -> (3,L,N) (src/polymath.cu:531-566)."""
        L = ct1.shape[1]
        out = np.empty((3, L, self.n), dtype=np.uint64)
        lib().orc_tensor_2x2(C.byref(self.c), _p64(ct1.reshape(-1)), _p64(ct2.reshape(-1)), _p64(out.reshape(-1)),
                             C.c_uint32(L))
        return out

    def tensor_mxn(self, ct1: np.ndarray, ct2: np.ndarray) -> np.ndarray:
        """(s1,L,N) x (s2,L,N) -> (s1+s2-1,L,N), sizes up to 16 (src/polymath.cu:614-672)."""
        if not (1 <= ct1.shape[0] <= 16 and 1 <= ct2.shape[0] <= 16):
            raise ValueError("tensor_mxn takes 1 to 16 polynomials per operand")
        s1, L = ct1.shape[0], ct1.shape[1]
        s2 = ct2.shape[0]
        out = np.empty((s1 + s2 - 1, L, self.n), dtype=np.uint64)
        lib().orc_tensor_mxn(C.byref(self.c), _p64(np.ascontiguousarray(ct1).reshape(-1)), C.c_uint32(s1),
                             _p64(np.ascontiguousarray(ct2).reshape(-1)), C.c_uint32(s2), _p64(out.reshape(-1)),
                             C.c_uint32(L))
        return out

    def square(self, ct: np.ndarray) -> np.ndarray:
        L = ct.shape[1]
        out = np.empty((3, L, self.n), dtype=np.uint64)
        lib().orc_tensor_square(C.byref(self.c), _p64(ct.reshape(-1)), _p64(out.reshape(-1)), C.c_uint32(L))
        return out

    def galois_table(self, elt: int) -> np.ndarray:
        t = np.empty(self.n, dtype=np.uint32)
        lib().orc_galois_table(C.c_uint32(self.logn), C.c_uint32(elt), _p32(t))
        return t

    def galois_ntt(self, a: np.ndarray, elt: int) -> np.ndarray:
        """NTT-domain automorphism of every limb of a [..., N] (src/galois.cu:20-30)."""
        out = np.empty_like(a)
        lib().orc_galois_ntt(C.byref(self.c), _p64(a.reshape(-1)), _p64(out.reshape(-1)), _p32(self.galois_table(elt)),
                             C.c_uint32(a.reshape(-1, self.n).shape[0]))
        return out

    def rescale(self, ct: np.ndarray) -> np.ndarray:
        """(npoly,L,N) -> (npoly,L-1,N) (src/rns.cu:544-570)."""
        npoly, L, n = ct.shape
        lt = self.level(L)
        out = np.empty((npoly, L - 1, n), dtype=np.uint64)
        scratch = np.empty(n, dtype=np.uint64)
        lib().orc_rescale(C.byref(self.c), _p64(ct.reshape(-1)), _p64(out.reshape(-1)), C.c_uint32(npoly),
                          C.c_uint32(L), _p64(lt.qlast_inv), _p64(scratch))
        return out

    def modup(self, c: np.ndarray) -> np.ndarray:
        """(L,N) NTT -> (beta, L+K, N) NTT (src/rns_bconv.cu:668-792)."""
        L, n = c.shape
        lt = self.level(L)
        out = np.empty((lt.beta, L + self.size_p, n), dtype=np.uint64)
        scratch = np.empty(L * n, dtype=np.uint64)
        lib().orc_modup(C.byref(self.c), C.c_uint32(L), _p64(c.reshape(-1)), _p64(out.reshape(-1)), _p64(lt.hatinv),
                        _p64(lt.mats), _p32(lt.mat_off), _p64(scratch))
        return out

    def inner_prod(self, y: np.ndarray, evk: list[np.ndarray]) -> np.ndarray:
        """(beta,L+K,N) x beta keys (2,QP,N) -> (2,L+K,N) (src/eval_key_switch.cu:13-76)."""
        beta, LK, n = y.shape
        L = LK - self.size_p
        out = np.empty((2, LK, n), dtype=np.uint64)
        ptrs = (u64p * beta)(*[_p64(k.reshape(-1)) for k in evk[:beta]])
        lib().orc_inner_prod(C.byref(self.c), C.c_uint32(L), C.c_uint32(beta), _p64(y.reshape(-1)), ptrs,
                             _p64(out.reshape(-1)))
        return out

    def moddown(self, cx: np.ndarray) -> np.ndarray:
        """(L+K,N) NTT -> (L,N) NTT (src/rns_bconv.cu:965-1053)."""
        LK, n = cx.shape
        L = LK - self.size_p
        out = np.empty((L, n), dtype=np.uint64)
        scratch = np.empty(self.size_p * n, dtype=np.uint64)
        mat = np.ascontiguousarray(self.mat_p2q[:L])
        lib().orc_moddown(C.byref(self.c), C.c_uint32(L), _p64(cx.reshape(-1)), _p64(out.reshape(-1)),
                          _p64(self.phat_inv), _p64(mat.reshape(-1)), _p64(np.ascontiguousarray(self.pinv_mod_q[:L])),
                          _p64(scratch))
        return out

    # ---------------------------------------------------------------------------------------------
    # compositions (src/eval_key_switch.cu:80-216, src/evaluate.cu)
    # ---------------------------------------------------------------------------------------------
    def key_switch(self, c: np.ndarray, evk: list[np.ndarray]) -> np.ndarray:
        """Returns the (2,L,N) pair that switch_key_inplace adds onto (c0,c1)."""
        y = self.modup(c)
        cx = self.inner_prod(y, evk)
        return np.stack([self.moddown(cx[0]), self.moddown(cx[1])])

    def relinearize(self, ct3: np.ndarray, rlk: list[np.ndarray]) -> np.ndarray:
        """(3,L,N) -> (2,L,N) (src/evaluate.cu:2019-2056)."""
        ks = self.key_switch(ct3[2], rlk)
        return np.stack([self.add(ct3[0], ks[0]), self.add(ct3[1], ks[1])])

    def apply_galois(self, ct: np.ndarray, elt: int, glk: list[np.ndarray]) -> np.ndarray:
        """(sigma(c0), 0) + KeySwitch(sigma(c1)) (src/evaluate.cu:2631-2688)."""
        c0 = self.galois_ntt(ct[0], elt)
        c1 = self.galois_ntt(ct[1], elt)
        ks = self.key_switch(c1, glk)
        return np.stack([self.add(c0, ks[0]), ks[1]])

    def hoisting(self, ct: np.ndarray, elts: list[int], glks: list[list[np.ndarray]]) -> np.ndarray:
        """sum over elts of rot(ct) with one ModUp and one ModDown pair (src/evaluate.cu:2412-2629):
        the automorphism is applied to the lifted digits, not before the lift."""
        L = ct.shape[1]
        y = self.modup(ct[1])
        acc_c0 = None
        acc = None
        for elt, glk in zip(elts, glks):
            c0 = self.galois_ntt(ct[0], elt)
            acc_c0 = c0 if acc_c0 is None else self.add(acc_c0, c0)
            cx = self.inner_prod(self.galois_ntt(y, elt), glk)
            if acc is None:
                acc = cx
            else:
                tidx = [self.table_index(L, t) for t in range(L + self.size_p)]
                acc = np.stack([self._add_tidx(acc[b], cx[b], tidx) for b in range(2)])
        return np.stack([self.add(acc_c0, self.moddown(acc[0])), self.moddown(acc[1])])

    def _add_tidx(self, a, b, tidx):
        out = np.empty_like(a)
        for i, t in enumerate(tidx):
            q = np.uint64(self.moduli[t])
            s = a[i] + b[i]
            out[i] = np.where(s >= q, s - q, s)
        return out

    # ---------------------------------------------------------------------------------------------
    # samplers
    # ---------------------------------------------------------------------------------------------
    def _sample(self, fn, key: np.ndarray, stream: int, nlimbs: int, *extra) -> np.ndarray:
        out = np.empty((nlimbs, self.n), dtype=np.uint64)
        getattr(lib(), fn)(C.byref(self.c), _p32(key), C.c_uint64(stream), _p64(out.reshape(-1)), C.c_uint32(nlimbs),
                           *extra)
        return out

    def sample_ternary(self, key, stream, nlimbs):
        return self._sample("orc_sample_ternary", key, stream, nlimbs)

    def sample_error(self, key, stream, nlimbs):
        return self._sample("orc_sample_error", key, stream, nlimbs)

    def sample_uniform(self, key, stream, nlimbs):
        return self._sample("orc_sample_uniform", key, stream, nlimbs)

    def sample_gauss(self, key, stream, nlimbs, cdt: np.ndarray):
        return self._sample("orc_sample_gauss", key, stream, nlimbs, _p64(cdt), C.c_uint32(len(cdt)))


FLOODING_SIGMA = 5.574611952644673  # src/secretkey.cu:633


def gauss_cdt(sigma: float = FLOODING_SIGMA, tail: int = 12) -> np.ndarray:
    """cdt[i] = floor(2^63 * P(|X| <= i)) for the discrete Gaussian rho(x) ~ exp(-x^2 / (2 sigma^2)),
    truncated at tail*sigma.  Computed in double precision with a fixed operation order so that the
    product's C++ table (same formula) matches word for word."""
    bound = int(math.ceil(tail * sigma))
    w = [math.exp(-(x * x) / (2.0 * sigma * sigma)) for x in range(bound + 1)]
    total = w[0]
    for x in range(1, bound + 1):
        total += 2.0 * w[x]
    out, acc = [], 0.0
    for x in range(bound + 1):
        acc += w[x] if x == 0 else 2.0 * w[x]
        frac = acc / total
        out.append(int(frac * 9223372036854775808.0) if frac < 1.0 else (1 << 63) - 1)
    return np.array([min(v, (1 << 63) - 1) for v in out], dtype=np.uint64)


def chacha_key(seed: int) -> np.ndarray:
    """256-bit key from a 64-bit seed: word i = low/high halves of splitmix64 outputs."""
    mask = (1 << 64) - 1
    out, z = [], seed & mask
    for _ in range(4):
        z = (z + 0x9E3779B97F4A7C15) & mask
        x = z
        x = ((x ^ (x >> 30)) * 0xBF58476D1CE4E5B9) & mask
        x = ((x ^ (x >> 27)) * 0x94D049BB133111EB) & mask
        x ^= x >> 31
        out += [x & 0xFFFFFFFF, x >> 32]
    return np.array(out, dtype=np.uint32)


# ------------------------------------------------------------------------------------------------
# Galois elements (src/galois.cu:74-107, include/galois.cuh:158-195): generator 5
# ------------------------------------------------------------------------------------------------

def galois_elt_from_step(step: int, n: int) -> int:
    m = 2 * n
    if step == 0:
        return m - 1
    pos = abs(step)
    if pos >= n // 2:
        raise ValueError("step count too large")
    k = n // 2 - pos if step < 0 else pos
    return pow(5, k, m)


# ------------------------------------------------------------------------------------------------
# encoder (src/ckks.cu:104-209, src/fft.cu, src/rns_base.cu:121-156): canonical embedding over the
# orbit 5^j mod 2N, evaluated with numpy complex128
# ------------------------------------------------------------------------------------------------

class Encoder:
    def __init__(self, params: Params):
        self.p = params
        self.n = params.n
        self.slots = self.n // 2
        m = 2 * self.n
        self.rot_group = np.array([pow(5, j, m) for j in range(self.slots)], dtype=np.int64)
        self.ksi = np.exp(2j * np.pi * np.arange(m + 1) / m)

    def _fft_special_inv(self, vals: np.ndarray) -> np.ndarray:
        """HEAAN-style inverse special FFT (same transform as src/fft.cu:194-340 up to operation order)."""
        size = len(vals)
        m = 2 * self.n
        v = vals.astype(np.complex128).copy()
        ln = size
        while ln >= 2:
            lenh, lenq = ln >> 1, ln << 2
            gap = m // lenq
            j = np.arange(lenh)
            idx = (lenq - (self.rot_group[j] % lenq)) * gap
            w = self.ksi[idx]
            blk = v.reshape(-1, ln)
            u = blk[:, :lenh] + blk[:, lenh:]
            t = (blk[:, :lenh] - blk[:, lenh:]) * w
            blk[:, :lenh], blk[:, lenh:] = u, t
            ln >>= 1
        logs = int(math.log2(size))
        v = v[bitrev_perm(logs)] if size > 1 else v
        return v

    def _fft_special(self, vals: np.ndarray) -> np.ndarray:
        size = len(vals)
        m = 2 * self.n
        logs = int(math.log2(size))
        v = vals.astype(np.complex128)[bitrev_perm(logs)].copy()
        ln = 2
        while ln <= size:
            lenh, lenq = ln >> 1, ln << 2
            gap = m // lenq
            j = np.arange(lenh)
            idx = (self.rot_group[j] % lenq) * gap
            w = self.ksi[idx]
            blk = v.reshape(-1, ln)
            u = blk[:, :lenh].copy()
            t = blk[:, lenh:] * w
            blk[:, :lenh], blk[:, lenh:] = u + t, u - t
            ln <<= 1
        return v

    def encode_coeffs(self, values, scale: float, sparse_slots: int | None = None) -> np.ndarray:
        """Rounded real coefficients (float64, length N) of the plaintext polynomial."""
        values = np.asarray(values, dtype=np.complex128)
        ss = sparse_slots or max(2, 1 << int(math.ceil(math.log2(max(len(values), 1)))))
        z = np.zeros(ss, dtype=np.complex128)
        z[: len(values)] = values
        w = self._fft_special_inv(z) * (scale / ss)
        gap = self.slots // ss
        coeffs = np.zeros(self.n, dtype=np.float64)
        coeffs[0:ss * gap:gap] = np.round(w.real)
        coeffs[self.slots:self.slots + ss * gap:gap] = np.round(w.imag)
        return coeffs

    def encode(self, values, scale: float, nlimbs: int, sparse_slots: int | None = None) -> np.ndarray:
        """(nlimbs, N) NTT-form plaintext."""
        coeffs = self.encode_coeffs(values, scale, sparse_slots)
        out = np.empty((nlimbs, self.n), dtype=np.uint64)
        lib().orc_decompose_coeffs(C.byref(self.p.c), coeffs.ctypes.data_as(C.POINTER(C.c_double)),
                                   _p64(out.reshape(-1)), C.c_uint32(nlimbs))
        return self.p.ntt_fwd(out)

    def decode(self, plain: np.ndarray, scale: float, sparse_slots: int | None = None) -> np.ndarray:
        """(nlimbs, N) NTT-form plaintext -> complex slots (src/ckks.cu:292-465, src/rns_base.cu:325-459)."""
        nl = plain.shape[0]
        coeff = self.p.ntt_inv(plain.copy())
        q = self.p.moduli[:nl]
        Q = math.prod(q)
        hat = [Q // qi for qi in q]
        hinv = [pow(h % qi, -1, qi) for h, qi in zip(hat, q)]
        half = Q >> 1
        vals = np.empty(self.n, dtype=np.float64)
        cols = [coeff[i].tolist() for i in range(nl)]
        for j in range(self.n):
            v = 0
            for i in range(nl):
                v += (cols[i][j] * hinv[i] % q[i]) * hat[i]
            v %= Q
            if v > half:
                v -= Q
            vals[j] = float(v)
        vals /= scale
        ss = sparse_slots or self.slots
        gap = self.slots // ss
        z = vals[0:ss * gap:gap] + 1j * vals[self.slots:self.slots + ss * gap:gap]
        return self._fft_special(z)


# ------------------------------------------------------------------------------------------------
# keys, encryption, decryption (src/secretkey.cu) with the seeded samplers; stream ids are handed
# out in call order, one per sampled polynomial, mirroring the product's host code
# ------------------------------------------------------------------------------------------------

@dataclass
class KeySet:
    params: Params
    seed: int
    key: np.ndarray = field(init=False)
    stream: int = 0
    sk: np.ndarray = field(init=False, default=None)      # (QP, N) NTT

    def __post_init__(self):
        self.key = chacha_key(self.seed)

    def _next(self) -> int:
        s = self.stream
        self.stream += 1
        return s

    def gen_secret(self):
        """src/secretkey.cu:254-282"""
        p = self.params
        self.sk = p.ntt_fwd(p.sample_ternary(self.key, self._next(), p.size_qp))
        return self.sk

    def encrypt_zero_symmetric(self) -> np.ndarray:
        """Key-level (2,QP,N) pair (-(a s + e), a) (src/secretkey.cu:451-515, NTT branch)."""
        p = self.params
        e = p.ntt_fwd(p.sample_error(self.key, self._next(), p.size_qp))
        a = p.sample_uniform(self.key, self._next(), p.size_qp)
        c0 = p.mul_add(a, self.sk, e, negate=True)
        return np.stack([c0, a])

    def gen_public(self) -> np.ndarray:
        return self.encrypt_zero_symmetric()

    def gen_kswitch(self, sprime: np.ndarray) -> list[np.ndarray]:
        """dnum keys (src/secretkey.cu:328-372): evk_d = pk_d with [P]_{q_i} s' added on digit d's limbs."""
        p = self.params
        if p.size_q % p.size_p:
            raise ValueError("size_q must be a multiple of size_p (dnum = size_q / size_p, include/secretkey.h:141-144)")
        dnum = p.size_q // p.size_p
        keys = [self.encrypt_zero_symmetric() for _ in range(dnum)]
        for d, k in enumerate(keys):
            lib().orc_evk_add_ps(C.byref(p.c), C.c_uint32(d), _p64(k.reshape(-1)), _p64(sprime.reshape(-1)),
                                 _p64(p.p_mod_q))
        return keys

    def gen_relin(self) -> list[np.ndarray]:
        return self.gen_kswitch(self.params.mul(self.sk, self.sk))

    def gen_galois(self, elt: int) -> list[np.ndarray]:
        return self.gen_kswitch(self.params.galois_ntt(self.sk, elt))

    def encrypt_asymmetric(self, pk: np.ndarray, plain: np.ndarray) -> np.ndarray:
        """Encrypt at the key level, ModDown by P to the first data level, add the plaintext
        (src/secretkey.cu:47-246).  plain: (size_q, N) NTT form at chain index 1."""
        p = self.params
        qp = p.size_qp
        u = p.ntt_fwd(p.sample_ternary(self.key, self._next(), qp))
        parts = []
        for i in range(2):
            e = p.ntt_fwd(p.sample_error(self.key, self._next(), qp))
            parts.append(p.mul_add(u, pk[i], e))
        ct = np.stack([p.moddown(parts[0]), p.moddown(parts[1])])
        ct[0] = p.add(ct[0], plain)
        return ct

    def decrypt(self, ct: np.ndarray, flood_cdt: np.ndarray | None = None) -> np.ndarray:
        """c0 + c1 s (+ c2 s^2) over the ciphertext's limbs (src/secretkey.cu:594-654)."""
        p = self.params
        L = ct.shape[1]
        s = np.ascontiguousarray(self.sk[:L])
        acc = ct[0].copy()
        spow = s
        for i in range(1, ct.shape[0]):
            acc = p.mul_add(ct[i], spow, acc)
            spow = p.mul(spow, s)
        if flood_cdt is not None:
            noise = p.ntt_fwd(p.sample_gauss(self.key, self._next(), L, flood_cdt))
            acc = p.add(acc, noise)
        return acc
