"""Stream capture: the composite entry points enqueue only kernels and device-to-device copies on the caller's stream
(no allocation, no synchronisation, no memset), so a caller may record them into a HIP graph.  The graph is
replayed several times with eager work of the same library between the replays, and every replay must reproduce the
eager result."""
import ctypes as C

import numpy as np
import pytest

from gpu_util import DeviceArray, make_pair, rand_limbs

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("logn,bits,size_p,L", [(13, [50, 50, 49, 50, 50, 40, 50, 50], 2, 6), (12, [60, 40, 40, 60], 1, 3)])
def test_entry_points_under_stream_capture(oracle, logn, bits, size_p, L):
    from lancelot_amd import capi
    hip = C.CDLL("libamdhip64.so")
    cahel, parms, ctx, p = make_pair(oracle, logn, bits, size_p)
    lib, h = capi.lib(), ctx.he_handle()
    rng = np.random.default_rng(5)
    n = p.n
    beta = -(-L // size_p)
    host_evk = [rand_limbs(p, rng, range(p.size_qp), n_polys=2) for _ in range(p.size_q // size_p)]
    dev_evk = [DeviceArray(capi, host=k) for k in host_evk]
    ptrs = capi.evk_array([d.ptr for d in dev_evk])
    a, b = rand_limbs(p, rng, range(L), n_polys=2), rand_limbs(p, rng, range(L), n_polys=2)
    da, db = DeviceArray(capi, host=a), DeviceArray(capi, host=b)
    ws = DeviceArray(capi, shape=(lib.he_multiply_relin_rescale_workspace_words(h, L),))
    rws = DeviceArray(capi, shape=(lib.he_keyswitch_workspace_words(h, L),))
    prod, rot = DeviceArray(capi, shape=(2, L - 1, n)), DeviceArray(capi, shape=(2, L, n))
    elt = pow(5, 3, 2 * n)
    want_prod = p.rescale(p.relinearize(p.tensor(a, b), host_evk[:beta]))
    want_rot = p.apply_galois(a, elt, host_evk[:beta])

    # he_rescale_static: the entry point that takes no workspace (its scratch belongs to the library's device image)
    stat = DeviceArray(capi, shape=(2, L - 1, n))
    want_stat = p.rescale(a)

    st = C.c_void_p()
    capi.check(lib.he_stream_create(C.byref(st)))
    graph, gexec = C.c_void_p(), C.c_void_p()
    try:
        assert hip.hipStreamBeginCapture(st, 0) == 0            # hipStreamCaptureModeGlobal
        try:
            rcs = [lib.he_multiply_relin_rescale(h, L, da.ptr, db.ptr, ptrs, prod.ptr, ws.ptr, st),
                   lib.he_rotate(h, L, da.ptr, ptrs, rot.ptr, elt, rws.ptr, st),
                   lib.he_rescale_static(h, da.ptr, stat.ptr, 2, L, st)]
        finally:
            # always leave capture mode: a stream left capturing would fail every later call of the process
            end = hip.hipStreamEndCapture(st, C.byref(graph))
        assert rcs == [0, 0, 0] and end == 0
        assert hip.hipGraphInstantiate(C.byref(gexec), graph, None, None, C.c_size_t(0)) == 0
        scratch = DeviceArray(capi, shape=(2, L - 1, n))
        for replay in range(3):
            # clear the outputs, run other work of the library eagerly, then replay
            capi.check(lib.he_memset_zero(prod.ptr, 8 * 2 * (L - 1) * n, None))
            capi.check(lib.he_memset_zero(rot.ptr, 8 * 2 * L * n, None))
            capi.check(lib.he_memset_zero(stat.ptr, 8 * 2 * (L - 1) * n, None))
            capi.check(lib.he_multiply_relin_rescale(h, L, db.ptr, db.ptr, ptrs, scratch.ptr, ws.ptr, None))
            capi.check(lib.he_rescale_static(h, db.ptr, scratch.ptr, 2, L, None))
            capi.check(lib.he_stream_synchronize(None))
            assert hip.hipGraphLaunch(gexec, st) == 0
            capi.check(lib.he_stream_synchronize(st))
            assert (prod.numpy() == want_prod).all(), replay
            assert (rot.numpy() == want_rot).all(), replay
            assert (stat.numpy() == want_stat).all(), replay
    finally:
        if gexec:
            hip.hipGraphExecDestroy(gexec)
        if graph:
            hip.hipGraphDestroy(graph)
        capi.check(lib.he_stream_destroy(st))
