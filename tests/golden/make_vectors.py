"""Writes tests/golden/ckks_n512.npz: inputs and expected outputs of every stage of the hot path on one small
parameter set (N = 512, four data primes of 40-50 bits, two special primes), computed with the CPU checker in
oracle/.  The checker itself is pinned by the reference's known-answer tests and by closed forms
(tests/test_oracle_*.py); these vectors freeze its answers so that neither the checker nor the HIP path can drift
unnoticed.  Run from the repository root:  python tests/golden/make_vectors.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle import ckks_oracle as O  # noqa: E402

LOGN, BITS, SIZE_P, SEED = 9, [50, 40, 45, 50, 50, 49], 2, 20251125


def rand_limbs(p, rng, tidx, n_polys=None):
    shape = (len(tidx), p.n) if n_polys is None else (n_polys, len(tidx), p.n)
    out = np.empty(shape, dtype=np.uint64)
    for i, t in enumerate(tidx):
        out[..., i, :] = rng.integers(0, p.moduli[t], size=shape[:-2] + (p.n,), dtype=np.uint64)
    return out


def build():
    O.build()
    n = 1 << LOGN
    moduli = O.coeff_modulus_create(n, BITS)
    p = O.Params(LOGN, moduli, SIZE_P)
    rng = np.random.default_rng(SEED)
    L = p.size_q
    c = rand_limbs(p, rng, range(L))
    ct = rand_limbs(p, rng, range(L), n_polys=2)
    ct2 = rand_limbs(p, rng, range(L), n_polys=2)
    evk = np.stack([rand_limbs(p, rng, range(p.size_qp), n_polys=2) for _ in range(L // SIZE_P)])
    elt = 5
    y = p.modup(c)
    cx = p.inner_prod(y, list(evk))
    ks = p.key_switch(c, list(evk))
    ks_rot = p.key_switch(p.galois_ntt(c, elt), list(evk))
    out = dict(
        moduli=np.array(moduli, dtype=np.uint64), logn=np.array(LOGN), size_p=np.array(SIZE_P), galois_elt=np.array(elt),
        c=c, ct=ct, ct2=ct2, evk=evk,
        ntt_fwd=p.ntt_fwd(c.copy()), ntt_inv=p.ntt_inv(c.copy()),
        tensor=p.tensor(ct, ct2), square=p.square(ct),
        galois=p.galois_ntt(c, elt),
        modup=y, inner=cx, moddown=np.stack([p.moddown(cx[b]) for b in range(2)]),
        keyswitch=np.stack([p.add(ct[b], ks[b]) for b in range(2)]),
        keyswitch_galois=np.stack([p.add(ct[b], ks_rot[b]) for b in range(2)]),
        rescale=p.rescale(ct),
        add=np.stack([p.add(ct[b], ct2[b]) for b in range(2)]),
        sub=np.stack([p.sub(ct[b], ct2[b]) for b in range(2)]),
    )
    return out


if __name__ == "__main__":
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "ckks_n512.npz")
    np.savez_compressed(path, **build())
    print("wrote", path, os.path.getsize(path), "bytes")
