"""Helpers for the GPU parity tests: device buffers through the C-ABI, paired product/oracle contexts."""
import ctypes as C

import numpy as np


class DeviceArray:
    """A uint64 device buffer owned by the test (he_malloc / he_free), mirrored from / to numpy."""

    def __init__(self, capi, shape=None, host=None, dtype=np.uint64):
        self.capi = capi
        if host is not None:
            host = np.ascontiguousarray(host)
            shape, dtype = host.shape, host.dtype
        self.shape, self.dtype = tuple(shape), np.dtype(dtype)
        self.nbytes = int(np.prod(self.shape)) * self.dtype.itemsize
        p = C.c_void_p()
        capi.check(capi.lib().he_malloc(C.byref(p), max(self.nbytes, 8)), "he_malloc")
        self.ptr = p.value
        if host is not None:
            capi.check(capi.lib().he_memcpy_h2d(self.ptr, host.ctypes.data, self.nbytes, None), "h2d")

    def numpy(self):
        out = np.empty(self.shape, dtype=self.dtype)
        self.capi.check(self.capi.lib().he_memcpy_d2h(out.ctypes.data, self.ptr, self.nbytes, None), "d2h")
        return out

    def at(self, word_offset):
        return self.ptr + 8 * int(word_offset)

    def free(self):
        if self.ptr:
            self.capi.lib().he_free(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def make_pair(oracle, logn, bit_sizes, size_p, seed=2025):
    """(pyCAHEL module, product context, oracle Params) over the same primes."""
    import lancelot_amd  # noqa: F401
    import pyCAHEL as cahel
    n = 1 << logn
    mods = cahel.coeff_modulus_create(n, bit_sizes)
    parms = cahel.params(cahel.scheme_type.ckks)
    parms.set_poly_modulus_degree(n)
    parms.set_coeff_modulus(mods)
    parms.set_special_modulus_size(size_p)
    ctx = cahel.context(parms, True, cahel.sec_level_type.none)
    ctx.set_seed(seed)
    values = [m.value() for m in mods]
    assert values == oracle.coeff_modulus_create(n, bit_sizes)
    return cahel, parms, ctx, oracle.Params(logn, values, size_p)


def rand_limbs(params, rng, tidx, n_polys=None):
    """Uniform residues, limb i below modulus tidx[i]; shape (len(tidx), N) or (n_polys, len(tidx), N)."""
    shape = (len(tidx), params.n) if n_polys is None else (n_polys, len(tidx), params.n)
    out = np.empty(shape, dtype=np.uint64)
    for i, t in enumerate(tidx):
        out[..., i, :] = rng.integers(0, params.moduli[t], size=shape[:-2] + (params.n,), dtype=np.uint64)
    return out
