#!/usr/bin/env python3
"""Benchmark of the CKKS hot path on one MI355X.

    python bench.py --gpus 1 --steps K --warmup W

One "step" is one homomorphic multiplication with relinearisation and rescale (tensor product -> hybrid key
switch with dnum = 3 digits -> rescale) of two fresh ciphertexts at N = 2^16, L = 24 data limbs and 8 special
limbs of 50 bits, scale 2^40, on buffers that are resident in HBM before the timed region starts; the step goes
through the C-ABI of libcahel_hip.so exactly as the pyCAHEL evaluator drives it.  Prints ONE JSON line.

Extra objects on the line:
  roofline      the dominant kernel of the step (forward NTT, blocks pass, as launched by the key switch's
                ModUp) timed alone with HIP events: algorithmic bytes = limbs * N * 8 read + written
  ntt           config "batched forward + inverse NTT, 24 limbs x 2 polynomials": GB/s of limb data
  rotate        one rotation with key switch; hoisted and plain rotate-and-sum over 15 steps
  cpu_baseline  the CPU checker (oracle/, OpenMP) on the same HMult+relin+rescale workload, bounded sample
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

LOG_N, SIZE_Q, SIZE_P, BITS, SCALE = 16, 24, 8, 50, 2.0 ** 40
# HBM bytes of one 72-limb forward NTT call, from the FETCH_SIZE / WRITE_SIZE counters scaled by a copy of known
# size (profiles/ntt_forward_72limbs_n65536.md)
NTT72_TRAFFIC_BYTES = 164_057_088
HBM_PEAK_GBS = 8000.0


def sync(capi):
    capi.check(capi.lib().he_stream_synchronize(None), "sync")


class Timer:
    """HIP-event timer on the null stream (the stream every kernel here is launched on)."""

    def __init__(self, capi):
        self.capi, self.lib = capi, capi.lib()
        self.e0, self.e1 = C.c_void_p(), C.c_void_p()
        capi.check(self.lib.he_event_create(C.byref(self.e0)))
        capi.check(self.lib.he_event_create(C.byref(self.e1)))

    def time(self, fn, iters, warmup=3):
        for _ in range(warmup):
            fn()
        sync(self.capi)
        self.capi.check(self.lib.he_event_record(self.e0, None))
        for _ in range(iters):
            fn()
        self.capi.check(self.lib.he_event_record(self.e1, None))
        self.capi.check(self.lib.he_event_synchronize(self.e1))
        ms = C.c_float()
        self.capi.check(self.lib.he_event_elapsed_ms(self.e0, self.e1, C.byref(ms)))
        return ms.value / iters


class Buf:
    def __init__(self, capi, words):
        self.capi = capi
        p = C.c_void_p()
        capi.check(capi.lib().he_malloc(C.byref(p), 8 * words), "he_malloc")
        self.ptr, self.words = p.value, words

    def at(self, word):
        return self.ptr + 8 * word


def cpu_baseline(seconds_budget=12.0):
    """HMult + relinearise + rescale on the CPU checker at the benchmark's own shape (random residues)."""
    from oracle import ckks_oracle as O
    n = 1 << LOG_N
    mods = O.coeff_modulus_create(n, [BITS] * (SIZE_Q + SIZE_P))
    p = O.Params(LOG_N, mods, SIZE_P)
    rng = np.random.default_rng(1)

    def rnd(limbs, polys):
        out = np.empty((polys, limbs, n), dtype=np.uint64)
        for i in range(limbs):
            out[:, i] = rng.integers(0, mods[i], size=(polys, n), dtype=np.uint64)
        return out

    a, b = rnd(SIZE_Q, 2), rnd(SIZE_Q, 2)
    evk = [rnd(SIZE_Q + SIZE_P, 2) for _ in range(SIZE_Q // SIZE_P)]

    def op():
        return p.rescale(p.relinearize(p.tensor(a, b), evk))

    op()
    t0, iters = time.time(), 0
    while True:
        op()
        iters += 1
        if time.time() - t0 > seconds_budget or iters >= 2000:
            break
    dt = (time.time() - t0) / iters
    threads = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
    return {"value": 1.0 / dt, "unit": "HMult+relin+rescale ops/s", "cores": threads, "kind": "port",
            "sample": "%d iterations of the same workload (N=2^16, L=24, K=8, dnum=3, random residues) on "
                      "oracle/ckks_oracle.c with OpenMP" % iters,
            "ms_per_op": dt * 1e3}


def krum_round(seed: int = 2025, modulus_bits=(60, 40, 40, 60), sum_drop_levels=0):
    """One encrypted Krum round at its real shape (10 clients x 62,006 parameters, N = 2^16, moduli
    [60, 40, 40, 60], one special prime): seconds per phase and the error against the float64 closed form."""
    from lancelot_amd import krum
    rng = np.random.default_rng(seed)
    updates = [rng.normal(0.0, 0.01, 62006).astype(np.float32) for _ in range(10)]
    for k in (8, 9):
        updates[k] = updates[k] * 10
    t0 = time.perf_counter()
    state = krum.gpu_init(krum.KrumConfig(seed=seed, modulus_bits=tuple(modulus_bits), sum_drop_levels=sum_drop_levels))
    setup = time.perf_counter() - t0
    krum.gpu_krum_aggregate(updates, state=state)  # warm-up round (pool growth, first-touch of the keys)
    # the fastest of three rounds each (a round is about 12 ms of host-driven work: one scheduling hiccup of the host
    # threads would otherwise decide the figure)
    chosen_full, weights, full_timings = min((krum.gpu_krum_aggregate(updates, state=state) for _ in range(3)),
                                             key=lambda r: r[2]["total"])
    chosen, dist, timings = min((krum.gpu_krum(updates, state=state) for _ in range(3)), key=lambda r: r[2]["total"])
    plain = krum.plain_distance_matrix(updates)
    off = ~np.eye(10, dtype=bool)
    return {"workload": "Krum distance round, 10 clients x 62006 parameters, 2 ciphertexts per client, 45 pairs, N=2^16, "
                        "moduli of %s bits (the last one special); encode and encrypt are one batched pipeline, timed "
                        "under 'encode'" % (list(modulus_bits),),
            "setup_s": setup, "round_s": timings, "chosen": chosen, "chosen_plain": krum.krum_select(plain),
            "full_round_s": full_timings, "full_round_chosen": chosen_full,
            "aggregate_max_abs_err": float(np.max(np.abs(weights - updates[chosen_full].astype(np.float64)))),
            "max_rel_err_vs_float64": float(np.max(np.abs(dist[off] - plain[off]) / plain[off]))}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--lanes", type=int, default=3,
                    help="streams that the timed operations are dealt to (three and the null stream fill the four "
                         "hardware queues of a process; four measured slower than three or six)")
    ap.add_argument("--separate-rescale", action="store_true",
                    help="he_keyswitch then he_rescale instead of the merged he_keyswitch_rescale")
    ap.add_argument("--no-krum", action="store_true", help="skip the encrypted Krum round (BASELINE.json configs[4])")
    ap.add_argument("--only", choices=["all", "roofline", "krum"], default="all",
                    help="roofline: run just the kernel the roofline object describes (for rocprofv3)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)")

    import lancelot_amd  # noqa: F401  (raises if the native libraries are missing)
    import pyCAHEL as cahel
    from lancelot_amd import capi
    lib = capi.lib()

    n = 1 << LOG_N
    parms = cahel.params(cahel.scheme_type.ckks)
    parms.set_poly_modulus_degree(n)
    parms.set_coeff_modulus(cahel.coeff_modulus_create(n, [BITS] * (SIZE_Q + SIZE_P)))
    parms.set_special_modulus_size(SIZE_P)
    steps_pow2 = [1 << k for k in range(15)]
    parms.set_galois_elts(cahel.get_elts_from_steps(steps_pow2, n))
    ctx = cahel.context(parms, True, cahel.sec_level_type.tc128)
    ctx.set_seed(2025)
    if args.only == "krum":
        print(json.dumps(krum_round()))
        return
    if args.only == "roofline":
        # just the kernels the roofline object describes, plus one device-to-device copy of known size that
        # calibrates the FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run
        h = ctx.he_handle()
        words = 3 * (SIZE_Q + SIZE_P) * n
        big, ref = Buf(capi, words), Buf(capi, words)
        capi.check(lib.he_memset_zero(big.ptr, 8 * words, None))
        capi.check(lib.he_memcpy_d2d(ref.ptr, big.ptr, 8 * words, None))
        ms = Timer(capi).time(lambda: capi.check(lib.he_ntt_forward(h, big.ptr, 3, SIZE_Q + SIZE_P, SIZE_Q, 0, SIZE_Q, 0,
                                                                    None)), args.steps, args.warmup)
        print(json.dumps({"kernel": "forward NTT, 72 limbs (ntt_rows_kernel + ntt_blocks_kernel)", "ms_per_launch": ms,
                          "GBps": 72 * 8 * n * 2 / (ms * 1e-3) / 1e9, "calibration_copy_bytes": 8 * words}))
        return
    sk = cahel.secret_key(parms)
    sk.gen_secretkey(ctx)
    pk = cahel.public_key(ctx)
    sk.gen_publickey(ctx, pk)
    rlk = cahel.relin_key(ctx)
    sk.gen_relinkey(ctx, rlk)
    glk = cahel.galois_key(ctx)
    sk.create_galois_keys(ctx, glk)
    enc = cahel.ckks_encoder(ctx)
    rng = np.random.default_rng(2025)
    x, y = rng.uniform(-1, 1, n // 2), rng.uniform(-1, 1, n // 2)
    ct1 = pk.encrypt_asymmetric(ctx, enc.encode(ctx, x, SCALE))
    ct2 = pk.encrypt_asymmetric(ctx, enc.encode(ctx, y, SCALE))

    h = ctx.he_handle()
    L, K = SIZE_Q, SIZE_P
    LK = L + K
    limb_bytes = 8 * n
    evk = capi.evk_array([rlk.digit_ptr(d) for d in range(rlk.digit_count())])
    ws = Buf(capi, lib.he_keyswitch_workspace_words(h, L))
    t3 = Buf(capi, 3 * L * n)
    res = Buf(capi, 2 * (L - 1) * n)
    rs_ws = Buf(capi, 2 * n)
    a_ptr, b_ptr = ct1.data_ptr(), ct2.data_ptr()

    # relinearise + rescale: one C-ABI call (ModDown's and the rescale's forward transforms merged, same limbs), or,
    # with --separate-rescale, the two calls that the evaluator's relinearize_inplace / rescale_to_next_inplace make
    def relin_rescale(t3_, res_, ws_, rs_, st):
        if args.separate_rescale:
            capi.check(lib.he_keyswitch(h, L, t3_.at(2 * L * n), evk, t3_.ptr, 0, ws_.ptr, st))
            capi.check(lib.he_rescale(h, t3_.ptr, res_.ptr, 2, L, rs_.ptr, st))
        else:
            capi.check(lib.he_keyswitch_rescale(h, L, t3_.at(2 * L * n), evk, t3_.ptr, res_.ptr, 0, ws_.ptr, st))

    def step():
        capi.check(lib.he_tensor(h, a_ptr, b_ptr, t3.ptr, L, None))
        relin_rescale(t3, res, ws, rs_ws, None)

    # (1) one operation after the other on the null stream: the latency of a single HMult + relin + rescale
    for _ in range(args.warmup):
        step()
    sync(capi)
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    sync(capi)
    single_ms = (time.perf_counter() - t0) * 1e3 / args.steps

    # (2) the same K independent operations dealt round-robin to `lanes` streams, each with its own workspace and
    # output: kernels of different operations overlap (one loads while another computes), which a single
    # operation's kernels, all in the same phase at the same time, cannot do.  This is the throughput figure.
    lane_bufs, lane_streams = [], []
    for _ in range(args.lanes):
        st = C.c_void_p()
        capi.check(lib.he_stream_create(C.byref(st)))
        lane_streams.append(st)
        lane_bufs.append((Buf(capi, lib.he_keyswitch_workspace_words(h, L)), Buf(capi, 3 * L * n),
                          Buf(capi, 2 * (L - 1) * n), Buf(capi, 2 * n)))

    def lane_step(k):
        lws, lt3, lres, lrs = lane_bufs[k]
        st = lane_streams[k]
        capi.check(lib.he_tensor(h, a_ptr, b_ptr, lt3.ptr, L, st))
        relin_rescale(lt3, lres, lws, lrs, st)

    def lanes_sync():
        for st in lane_streams:
            capi.check(lib.he_stream_synchronize(st))

    for i in range(args.warmup):
        lane_step(i % args.lanes)
    lanes_sync()
    t0 = time.perf_counter()
    for i in range(args.steps):
        lane_step(i % args.lanes)
    lanes_sync()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps

    # the evaluator path must give the same limbs, and decrypt to x * y
    prod = cahel.ciphertext(ctx)
    cahel.multiply(ctx, ct1, ct2, prod)
    cahel.relinearize_inplace(ctx, prod, rlk)
    cahel.rescale_to_next_inplace(ctx, prod)
    got = np.empty((2, L - 1, n), dtype=np.uint64)
    capi.check(lib.he_memcpy_d2h(got.ctypes.data, res.ptr, got.nbytes, None))
    same = bool((got == prod.to_numpy()).all())
    for lws, lt3, lres, lrs in lane_bufs:
        capi.check(lib.he_memcpy_d2h(got.ctypes.data, lres.ptr, got.nbytes, None))
        same = same and bool((got == prod.to_numpy()).all())
    dec = np.array(enc.decode(ctx, sk.decrypt(ctx, prod)))
    max_err = float(np.max(np.abs(dec - x * y)))

    timer = Timer(capi)
    # dominant kernel: the forward NTT over the 72 converted limbs of ModUp (beta = 3 digits x 24 limbs); the same
    # two kernels also run in ModDown and rescale.  Timed alone on a 72-limb buffer.
    big = Buf(capi, 3 * LK * n)
    capi.check(lib.he_memset_zero(big.ptr, 8 * 3 * LK * n, None))
    fwd72 = timer.time(lambda: capi.check(lib.he_ntt_forward(h, big.ptr, 3, LK, L, 0, L, 0, None)), 50)
    ntt_bytes = 72 * limb_bytes * 2          # each limb read once and written once
    roof_gbs = ntt_bytes / (fwd72 * 1e-3) / 1e9

    # config "NTT alone": 24 limbs x 2 polynomials, forward + inverse
    two = Buf(capi, 2 * L * n)
    capi.check(lib.he_memcpy_d2d(two.ptr, a_ptr, 8 * 2 * L * n, None))
    f = timer.time(lambda: capi.check(lib.he_ntt_forward(h, two.ptr, 2, L, L, 0, L, 0, None)), 100)
    i = timer.time(lambda: capi.check(lib.he_ntt_inverse(h, two.ptr, 2, L, L, 0, L, 0, None)), 100)
    ntt = {"forward_ms": f, "inverse_ms": i, "bytes_fwd_plus_inv": 4 * 2 * L * limb_bytes,
           "GBps": 4 * 2 * L * limb_bytes / ((f + i) * 1e-3) / 1e9}
    ntt["frac_of_hbm_peak"] = ntt["GBps"] / HBM_PEAK_GBS
    # the same kernels over 6 ciphertexts in one call (288 limbs): a launch that spans several rounds of resident
    # workgroups overlaps the load, butterfly and store phases that a single round runs one after the other
    six = Buf(capi, 12 * L * n)
    capi.check(lib.he_memset_zero(six.ptr, 8 * 12 * L * n, None))
    f6 = timer.time(lambda: capi.check(lib.he_ntt_forward(h, six.ptr, 12, L, L, 0, L, 0, None)), 30)
    i6 = timer.time(lambda: capi.check(lib.he_ntt_inverse(h, six.ptr, 12, L, L, 0, L, 0, None)), 30)
    ntt["six_ciphertexts_per_call"] = {"forward_ms": f6, "inverse_ms": i6,
                                       "GBps": 4 * 12 * L * limb_bytes / ((f6 + i6) * 1e-3) / 1e9}
    ntt["six_ciphertexts_per_call"]["frac_of_hbm_peak"] = ntt["six_ciphertexts_per_call"]["GBps"] / HBM_PEAK_GBS

    # rotations (config "rotate-and-sum"): one keyed rotation; 15 dependent rotations + adds; hoisted form
    rot_in = ct1.copy()
    rot_out = cahel.ciphertext(ctx)

    def one_rot():
        cahel.rotate_vector(ctx, rot_in, 1, glk, rot_out)

    rot_ms = timer.time(one_rot, 20)

    def rotate_and_sum():
        acc = ct1.copy()
        tmp = cahel.ciphertext(ctx)
        for s in steps_pow2:
            cahel.rotate_vector(ctx, acc, s, glk, tmp)
            cahel.add_inplace(ctx, acc, tmp)
        return acc

    ras_ms = timer.time(rotate_and_sum, 5, warmup=1)
    total = np.array(enc.decode(ctx, sk.decrypt(ctx, rotate_and_sum())))
    rotate = {"one_rotation_ms": rot_ms, "rotate_and_sum_15_ms": ras_ms,
              "one_rotation_GBps": 288 * limb_bytes / (rot_ms * 1e-3) / 1e9,
              "rotate_and_sum_GBps": 15 * 432 * limb_bytes / (ras_ms * 1e-3) / 1e9,
              "slot_sum_rel_err": float(np.max(np.abs(total - x.sum())) / abs(x.sum()))}

    alg_bytes = 334 * limb_bytes
    line = {
        "metric": "HMult+relin+rescale ops/s at N=2^16, L=24 (dnum=3, 8 special primes)",
        "value": 1e3 / ms_per_step, "unit": "ops/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "u64", "data": "synthetic",
        "arithmetic": "64-bit residues; NTT and base conversion in exact FP64 (primes below 2^50), tensor and inner "
                      "product in 64-bit integers; every output bit-identical to the integer oracle",
        "config": {"workload": "HMult+relinearize+rescale, N=2^16, L=24 limbs of 50 bits, K=8, dnum=3, scale 2^40, "
                               "two fresh ciphertexts of 32768 uniform[-1,1] slots (BASELINE.json configs[2]); "
                               "independent operations issued round-robin on %d streams" % args.lanes,
                   "lanes": args.lanes},
        "single_stream": {"ms_per_step": single_ms, "ops_per_s": 1e3 / single_ms,
                          "frac_of_hbm_roofline": alg_bytes / (single_ms * 1e-3) / 1e9 / HBM_PEAK_GBS},
        "hmult_frac_of_hbm_roofline": alg_bytes / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS,
        "hmult_algorithmic_bytes": alg_bytes,
        "check": {"c_abi_equals_evaluator": same, "decrypt_max_abs_err_vs_xy": max_err},
        "roofline": {"bound": "hbm", "kernel": "ntt_rows_kernel + ntt_blocks_kernel (forward NTT, 72 limbs of ModUp)",
                     "achieved": roof_gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": roof_gbs / HBM_PEAK_GBS,
                     "traffic": NTT72_TRAFFIC_BYTES, "ms_per_launch": fwd72, "algorithmic_bytes_per_launch": ntt_bytes},
        "ntt": ntt, "rotate": rotate,
    }
    if not args.no_krum:
        line["krum"] = krum_round()
        # The same round with two settings that Lancelot's driver does not use (its own are the ones above): primes
        # below 2^50 (exact FP64 butterflies instead of 64-bit integer ones), and the slot sum one level further down
        # (mod_switch_to_next after the rescale: its key switches run over one limb instead of two).  The two do not
        # combine: one level down the whole modulus is the first prime, and the largest squared distances of this workload
        # (about 1,240 between two scaled-up clients) times the scale 2^40 are about 2^50.3: they fit below half of a
        # 60-bit prime but not below half of a 50-bit one.
        keep = ("round_s", "chosen", "max_rel_err_vs_float64")
        variants = {"primes_of_50_40_40_50_bits": dict(modulus_bits=(50, 40, 40, 50)),
                    "slot_sum_one_level_down": dict(sum_drop_levels=1)}
        line["krum_variants"] = {name: {k: v for k, v in krum_round(**kw).items() if k in keep}
                                 for name, kw in variants.items()}
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline()
    print(json.dumps(line))


if __name__ == "__main__":
    main()
