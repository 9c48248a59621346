#!/usr/bin/env python3
"""Benchmark of the CKKS hot path on one MI355X.

    python bench.py --gpus 1 --steps K --warmup W

One "step" is one homomorphic multiplication with relinearisation and rescale (tensor product -> hybrid key
switch with dnum = 3 digits -> rescale) of two fresh ciphertexts at N = 2^16, L = 24 data limbs and 8 special
limbs of 50 bits, scale 2^40 (BASELINE.json configs[2]), on buffers that are resident in HBM before the timed region
starts.  Every figure is the median of BLOCKS timed blocks of K steps each, after W warm-up steps.  Prints ONE JSON
line.

How the same step is driven (all give the same limbs, `check`):
  value / throughput   independent operations: dealt round-robin to `--lanes` streams (`streams`), or `--batch`
                       of them per call through he_multiply_relin_rescale_batch (`batch`); `value` is the better of
                       the two and `config.value_path` says which
  single_stream        one he_multiply_relin_rescale after the other on the null stream (HIP events)
  api_path             what lancelot-main-GPU's byzantine_fl.py gets: pyCAHEL multiply, relinearize_inplace,
                       rescale_to_next_inplace on the null stream

Extra objects on the line:
  roofline      the timed step on one stream against the HBM roofline: algorithmic bytes of the step / its duration
                (HIP events on the stream the kernels run on), with the VALU bound beside it (`valu`: wave
                instructions of the step's kernels from the committed counter profile, priced against the FP64
                issue rate that he_probe_fp64_issue_rate measures in this run); `frac` prices the 334 limbs of
                one operation (inputs, key, output), `frac_amortised_key` the bytes a launch of several operations
                has to move (the key once per launch)
  ntt           config "batched forward + inverse NTT, 24 limbs x 2 polynomials": GB/s of limb data
  rotate        one rotation with key switch; rotate-and-sum over 15 steps
  krum          the encrypted Krum round at its real shape, with the CPU checker's time for the same evaluate phase,
                and the distance phase driven call for call as lancelot-main-GPU's byzantine_fl.py does
                (`reference_call_sequence`: 55 pairs, operands encoded and encrypted again for every pair)
  cpu_baseline  the CPU checker (oracle/, OpenMP) on the same HMult+relin+rescale workload, bounded sample; and at
                BASELINE.json configs[0] (N = 2^14, 4 + 1 primes)
"""
import argparse
import ctypes as C
import json
import os
import statistics
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

LOG_N, SIZE_Q, SIZE_P, BITS, SCALE = 16, 24, 8, 50, 2.0 ** 40
HBM_PEAK_GBS = 8000.0
BLOCKS = 5
# From profiles/hmult_relin_rescale_n65536_l24_k8.md (rocprofv3 --pmc runs of `bench.py --only step` and
# `--only batch`), per operation: L2-miss traffic in limbs of 8 N bytes (FETCH_SIZE scaled by 2, WRITE_SIZE by 1: the
# factors a copy of known size gives) and SQ_INSTS_VALU summed over the kernels.  Constants of the profile, not
# measured in this run.
PROFILE = {"single": {"traffic_limbs": 1117.7, "valu_wave_instr": 30.88e6,
                      "kernels": "tensor_intt_blocks_fp, ntt_rows (inverse), bconv_rows_mx (ModUp, conversion on the int8 "
                                 "matrix cores), ntt_blocks_fp_inner, ntt_blocks_fp + ntt_rows (inverse), bconv_rows_fp, "
                                 "ntt_blocks_fp with the rescale epilogue"},
           "batch": {"traffic_limbs": 896.1, "valu_wave_instr": 27.3e6,
                     "kernels": "per call of 8 operations: tensor_fp, ntt_blocks_fp + ntt_rows (inverse), bconv_rows_mx, "
                                "ntt_blocks_fp_inner (items of a tile on one XCD, key tile shared through L2), "
                                "ntt_blocks_fp + ntt_rows (inverse), bconv_rows_mx, ntt_blocks_fp with the rescale "
                                "epilogue"}}


def issue_rates(capi):
    """he_probe_issue_rate for every kind at 2, 4 and 8 waves per SIMD of every CU: 10^12 lane-operations per second
    (multiply-adds for the matrix kinds)."""
    cus = 256   # MI355X
    kinds = ["v_fma_f64", "v_mad_u64_u32", "v_mul_lo_u32", "v_add_u32", "v_mfma_f64_16x16x4_f64",
             "v_mfma_f64_16x16x4_f64 + v_fma_f64 (equal work on each, sum of both)"]
    out = {"unit": "1e12 lane-operations per second", "compute_units": cus, "waves_per_simd": [2, 4, 8], "rates": {}}
    for kind, name in enumerate(kinds):
        row = []
        for waves in out["waves_per_simd"]:
            rate = C.c_double()
            capi.check(capi.probe_lib().he_probe_issue_rate(kind, cus * waves, 2000, C.byref(rate), None))
            row.append(round(rate.value / 1e12, 2))
        out["rates"][name] = row
    return out


def sync(capi):
    capi.check(capi.lib().he_stream_synchronize(None), "sync")


class Timer:
    """HIP-event timer on the null stream (the stream the timed kernels are launched on)."""

    def __init__(self, capi):
        self.capi, self.lib = capi, capi.lib()
        self.e0, self.e1 = C.c_void_p(), C.c_void_p()
        capi.check(self.lib.he_event_create(C.byref(self.e0)))
        capi.check(self.lib.he_event_create(C.byref(self.e1)))

    def once(self, fn, iters):
        self.capi.check(self.lib.he_event_record(self.e0, None))
        for _ in range(iters):
            fn()
        self.capi.check(self.lib.he_event_record(self.e1, None))
        self.capi.check(self.lib.he_event_synchronize(self.e1))
        ms = C.c_float()
        self.capi.check(self.lib.he_event_elapsed_ms(self.e0, self.e1, C.byref(ms)))
        return ms.value / iters

    def time(self, fn, iters, warmup=3, blocks=BLOCKS):
        for _ in range(warmup):
            fn()
        sync(self.capi)
        return statistics.median(self.once(fn, iters) for _ in range(blocks))


class Buf:
    def __init__(self, capi, words):
        self.capi = capi
        p = C.c_void_p()
        capi.check(capi.lib().he_malloc(C.byref(p), 8 * words), "he_malloc")
        self.ptr, self.words = p.value, words

    def at(self, word):
        return self.ptr + 8 * word


def cpu_hmult(log_n, size_q, size_p, seconds_budget):
    """HMult + relinearise + rescale on the CPU checker (random residues): (ops/s, iterations, threads)."""
    from oracle import ckks_oracle as O
    n = 1 << log_n
    mods = O.coeff_modulus_create(n, [BITS] * (size_q + size_p))
    p = O.Params(log_n, mods, size_p)
    rng = np.random.default_rng(1)

    def rnd(limbs, polys):
        out = np.empty((polys, limbs, n), dtype=np.uint64)
        for i in range(limbs):
            out[:, i] = rng.integers(0, mods[i], size=(polys, n), dtype=np.uint64)
        return out

    a, b = rnd(size_q, 2), rnd(size_q, 2)
    evk = [rnd(size_q + size_p, 2) for _ in range(size_q // size_p)]

    def op():
        return p.rescale(p.relinearize(p.tensor(a, b), evk))

    op()
    t0, iters = time.time(), 0
    while True:
        op()
        iters += 1
        if time.time() - t0 > seconds_budget or iters >= 5000:
            break
    dt = (time.time() - t0) / iters
    threads = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
    return 1.0 / dt, iters, threads


def cpu_baseline():
    # bounded samples (3 s + 2 s), so that most of a default run is GPU work
    v, iters, threads = cpu_hmult(LOG_N, SIZE_Q, SIZE_P, 3.0)
    v1, iters1, _ = cpu_hmult(14, 4, 1, 2.0)
    return {"value": v, "unit": "HMult+relin+rescale ops/s", "cores": threads, "kind": "port",
            "sample": "%d iterations of the same workload (N=2^16, L=24, K=8, dnum=3, random residues) on "
                      "oracle/ckks_oracle.c with OpenMP" % iters,
            "ms_per_op": 1e3 / v,
            "config_c1": {"value": v1, "unit": "HMult+relin+rescale ops/s", "cores": threads,
                          "workload": "BASELINE.json configs[0]: N=2^14, 4 limbs of 50 bits + 1 special prime",
                          "sample": "%d iterations" % iters1, "ms_per_op": 1e3 / v1}}


def gpu_c1(capi, cahel, timer, steps=400):
    """BASELINE.json configs[0] (the reference's own CPU-runnable case: N = 2^14, 4 limbs of 50 bits + 1 special
    prime) on the GPU: one operation after the other on the null stream, and batches of 32 per call."""
    lib = capi.lib()
    n, L, K = 1 << 14, 4, 1
    parms = cahel.params(cahel.scheme_type.ckks)
    parms.set_poly_modulus_degree(n)
    parms.set_coeff_modulus(cahel.coeff_modulus_create(n, [50] * (L + K)))
    parms.set_special_modulus_size(K)
    ctx = cahel.context(parms, True, cahel.sec_level_type.none)
    ctx.set_seed(2025)
    sk = cahel.secret_key(parms)
    sk.gen_secretkey(ctx)
    pk = cahel.public_key(ctx)
    sk.gen_publickey(ctx, pk)
    rlk = cahel.relin_key(ctx)
    sk.gen_relinkey(ctx, rlk)
    enc = cahel.ckks_encoder(ctx)
    rng = np.random.default_rng(14)
    x, y = rng.uniform(-1, 1, n // 2), rng.uniform(-1, 1, n // 2)
    ct1 = pk.encrypt_asymmetric(ctx, enc.encode(ctx, x, SCALE))
    ct2 = pk.encrypt_asymmetric(ctx, enc.encode(ctx, y, SCALE))
    h = ctx.he_handle()
    evk = capi.evk_array([rlk.digit_ptr(d) for d in range(rlk.digit_count())])
    ws, res = Buf(capi, lib.he_multiply_relin_rescale_workspace_words(h, L)), Buf(capi, 2 * (L - 1) * n)
    single = timer.time(lambda: capi.check(lib.he_multiply_relin_rescale(h, L, ct1.data_ptr(), ct2.data_ptr(), evk,
                                                                         res.ptr, ws.ptr, None)), steps, 20)
    B = 32
    ba, bb = Buf(capi, B * 2 * L * n), Buf(capi, B * 2 * L * n)
    for k in range(B):
        capi.check(lib.he_memcpy_d2d(ba.at(k * 2 * L * n), ct1.data_ptr(), 8 * 2 * L * n, None))
        capi.check(lib.he_memcpy_d2d(bb.at(k * 2 * L * n), ct2.data_ptr(), 8 * 2 * L * n, None))
    bres, bws = Buf(capi, B * 2 * (L - 1) * n), Buf(capi, lib.he_multiply_relin_rescale_batch_workspace_words(h, L, B))
    batch = timer.time(lambda: capi.check(lib.he_multiply_relin_rescale_batch(h, L, B, ba.ptr, bb.ptr, evk, bres.ptr,
                                                                              bws.ptr, None)), max(1, steps // B), 3) / B
    prod = cahel.ciphertext(ctx)
    cahel.multiply_relin_rescale(ctx, ct1, ct2, rlk, prod)
    got = np.empty((2, L - 1, n), dtype=np.uint64)
    capi.check(lib.he_memcpy_d2h(got.ctypes.data, bres.at((B - 1) * 2 * (L - 1) * n), got.nbytes, None))
    err = float(np.max(np.abs(np.array(enc.decode(ctx, sk.decrypt(ctx, prod))) - x * y)))
    return {"workload": "BASELINE.json configs[0]: HMult+relinearize+rescale, N=2^14, 4 limbs of 50 bits + 1 special prime",
            "single_stream": {"ms_per_step": single, "ops_per_s": 1e3 / single},
            "batch": {"ms_per_step": batch, "ops_per_s": 1e3 / batch, "ops_per_call": B},
            "batch_equals_single": bool((got == prod.to_numpy()).all()), "decrypt_max_abs_err_vs_xy": err}


def krum_cpu_evaluate(updates, pairs_sampled=2):
    """The evaluate phase of the Krum round on the CPU checker: per pair sub, square and add over the chunks,
    relinearise, rescale, and the slot sum as 15 rotations (each a key switch) + additions, with Lancelot's
    parameters; `pairs_sampled` pairs are timed and the figure is scaled to the 45 pairs of the round."""
    from oracle import ckks_oracle as O
    log_n, n = 16, 1 << 16
    mods = O.coeff_modulus_create(n, [60, 40, 40, 60])
    p = O.Params(log_n, mods, 1)
    ks = O.KeySet(p, seed=2025)
    ks.gen_secret()
    rlk = ks.gen_relin()
    elts = [O.galois_elt_from_step(1 << k, n) for k in range(15)]
    glk = [ks.gen_galois(e) for e in elts]
    rng = np.random.default_rng(3)
    L = p.size_q

    def rnd_ct():
        out = np.empty((2, L, n), dtype=np.uint64)
        for i in range(L):
            out[:, i] = rng.integers(0, mods[i], size=(2, n), dtype=np.uint64)
        return out

    chunks = 2
    cts = [[rnd_ct() for _ in range(chunks)] for _ in range(2)]
    t0 = time.time()
    for _ in range(pairs_sampled):
        acc = None
        for c in range(chunks):
            d = np.stack([p.sub(cts[1][c][k], cts[0][c][k]) for k in range(2)])
            sq = p.square(d)
            acc = sq if acc is None else np.stack([p.add(acc[k], sq[k]) for k in range(3)])
        r = p.rescale(p.relinearize(acc, rlk))
        for e, key in zip(elts, glk):
            rot = p.apply_galois(r, e, key)
            r = np.stack([p.add(r[k], rot[k]) for k in range(2)])
    per_pair = (time.time() - t0) / pairs_sampled
    return {"evaluate_s": per_pair * 45, "sample": "%d of the 45 pairs timed (%.3f s each) on oracle/ckks_oracle.c, "
            "%d threads; rotations one key switch each (the checker has no hoisting)"
            % (pairs_sampled, per_pair, int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1)))}


def krum_round(seed: int = 2025, modulus_bits=(60, 40, 40, 60), sum_drop_levels=0, with_cpu=False,
               with_reference_sequence=False):
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
    # the fastest of three rounds each (a round is a few ms of host-driven work: one scheduling hiccup of the host
    # threads would otherwise decide the figure)
    # (every round encrypts with fresh noise, so its errors are its own: the timings are the fastest round's, the
    # errors the largest over the three rounds, and the choice has to be the same in all of them)
    full_rounds = [krum.gpu_krum_aggregate(updates, state=state) for _ in range(3)]
    chosen_full, _, full_timings = min(full_rounds, key=lambda r: r[2]["total"])
    rounds = [krum.gpu_krum(updates, state=state) for _ in range(3)]
    chosen, _, timings = min(rounds, key=lambda r: r[2]["total"])
    plain = krum.plain_distance_matrix(updates)
    off = ~np.eye(10, dtype=bool)
    same_choice = all(r[0] == chosen for r in rounds) and all(r[0] == chosen_full for r in full_rounds)
    out = {"workload": "Krum distance round, 10 clients x 62006 parameters, 2 ciphertexts per client, 45 pairs, N=2^16, "
                       "moduli of %s bits (the last one special); encode and encrypt are one batched pipeline, timed "
                       "under 'encode'" % (list(modulus_bits),),
           "setup_s": setup, "round_s": timings, "chosen": chosen, "chosen_plain": krum.krum_select(plain),
           "full_round_s": full_timings, "full_round_chosen": chosen_full, "same_choice_in_every_round": same_choice,
           "aggregate_max_abs_err": max(float(np.max(np.abs(w - updates[c].astype(np.float64)))) for c, w, _ in full_rounds),
           "max_rel_err_vs_float64": max(float(np.max(np.abs(d[off] - plain[off]) / plain[off])) for _, d, _ in rounds)}
    if with_cpu:
        out["cpu_baseline"] = krum_cpu_evaluate(updates)
        out["cpu_baseline"]["gpu_evaluate_s"] = timings["evaluate"]
    if with_reference_sequence:
        # the same distances the way the unchanged caller computes them (lancelot-main-GPU/utils/byzantine_fl.py:173-321,
        # 466-514): 55 pairs, every pair encodes and encrypts its operands again, one pyCAHEL call per operation
        del state
        ref_state = krum.gpu_init(krum.KrumConfig(seed=seed, modulus_bits=tuple(modulus_bits), hoisting_radix=0,
                                                  batched=False, lanes=0))
        krum.reference_call_sequence(ref_state, updates[:2])        # warm-up: 3 pairs
        ref_dist, ref_t = krum.reference_call_sequence(ref_state, updates)
        out["reference_call_sequence"] = {
            "calls": "GPU_computing_distance_cipher as byzantine_fl.py issues it: 55 pairs (i <= j), per pair 2 encryptions "
                     "of zero + encode and encrypt of both operands per chunk, sub / square_inplace / add_inplace, "
                     "relinearize_inplace + rescale_to_next_inplace, hoisting(1..15) + add_inplace, 11 x (rotate_vector + "
                     "add_inplace); every call on the null stream, the phases timed with a synchronisation after each",
            "seconds": ref_t, "chosen": krum.krum_select(ref_dist),
            "max_rel_err_vs_float64": float(np.max(np.abs(ref_dist[off] - plain[off]) / plain[off])),
            "batched_driver_distance_phase_s": timings["encode"] + timings["evaluate"]}
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--lanes", type=int, default=3,
                    help="streams that the timed operations are dealt to (three and the null stream fill the four "
                         "hardware queues of a process)")
    ap.add_argument("--batch", type=int, default=8, help="operations per he_multiply_relin_rescale_batch call")
    ap.add_argument("--batch-streams", type=int, default=2, help="streams that the batch calls are dealt to")
    ap.add_argument("--no-krum", action="store_true", help="skip the encrypted Krum round (BASELINE.json configs[4])")
    ap.add_argument("--only", choices=["all", "step", "batch", "batch_streams", "rotate", "ntt", "krum", "krum_reference", "probe"], default="all",
                    help="step / batch / rotate / ntt: run just that workload on the null stream (for rocprofv3); "
                         "batch_streams: the batch calls dealt to --batch-streams streams, as `value` issues them; "
                         "krum_reference: the Krum round plus the distance phase by the reference's own call sequence; "
                         "probe: the issue rates of the instruction kinds that the kernels' bounds are argued with")
    ap.add_argument("--prime-bits", type=int, default=BITS,
                    help="with --only ntt: size of the 32 primes (50: the benchmark's, FP64 back end; 51 to 60: the "
                         "integer back end; the context is then built without the security check)")
    args = ap.parse_args()
    if args.prime_bits != BITS and args.only != "ntt":
        sys.exit("--prime-bits applies to --only ntt")
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)")

    import lancelot_amd  # noqa: F401  (raises if the native libraries are missing)
    import pyCAHEL as cahel
    from lancelot_amd import capi
    lib = capi.lib()

    if args.only == "krum":
        print(json.dumps(krum_round()))
        return
    if args.only == "krum_reference":
        print(json.dumps(krum_round(with_reference_sequence=True)))
        return
    if args.only == "probe":
        print(json.dumps(issue_rates(capi)))
        return
    n = 1 << LOG_N
    parms = cahel.params(cahel.scheme_type.ckks)
    parms.set_poly_modulus_degree(n)
    parms.set_coeff_modulus(cahel.coeff_modulus_create(n, [args.prime_bits] * (SIZE_Q + SIZE_P)))
    parms.set_special_modulus_size(SIZE_P)
    steps_pow2 = [1 << k for k in range(15)]
    # the same slot sum as five hoisted rounds of radix 8 (`hoisting` of the reference's API): steps 8^r times 1..7.
    # A round costs about 0.19 ms besides its steps' 0.022 ms each at this shape (a key is 192 limbs): five rounds of 7
    # steps measure 1.71 ms, four of 7 + 3 x 15 steps 1.89, six of radix 4, 4, 4, 8, 8, 8 1.76, three of radix 32 2.67
    hoist_rounds = [[8 ** r * k for k in range(1, 8)] for r in range(5)]
    all_steps = sorted(set(steps_pow2) | {s for rnd in hoist_rounds for s in rnd})
    parms.set_galois_elts(cahel.get_elts_from_steps(all_steps if args.only == "all" else
                                                    (steps_pow2 if args.only == "rotate" else [1]), n))
    ctx = cahel.context(parms, True, cahel.sec_level_type.tc128 if args.prime_bits == BITS else cahel.sec_level_type.none)
    ctx.set_seed(2025)
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
    limb_bytes = 8 * n
    evk = capi.evk_array([rlk.digit_ptr(d) for d in range(rlk.digit_count())])
    ws_words = lib.he_multiply_relin_rescale_workspace_words(h, L)
    ws, res = Buf(capi, ws_words), Buf(capi, 2 * (L - 1) * n)
    a_ptr, b_ptr = ct1.data_ptr(), ct2.data_ptr()
    timer = Timer(capi)
    K_steps, W = args.steps, args.warmup

    def step():
        capi.check(lib.he_multiply_relin_rescale(h, L, a_ptr, b_ptr, evk, res.ptr, ws.ptr, None))

    rot_in, rot_out = ct1.copy(), cahel.ciphertext(ctx)

    def one_rot():
        cahel.rotate_vector(ctx, rot_in, 1, glk, rot_out)

    two = Buf(capi, 2 * L * n)
    capi.check(lib.he_memcpy_d2d(two.ptr, a_ptr, 8 * 2 * L * n, None))

    # operands of the batch entry point: `batch` independent products per call
    B = args.batch
    ba, bb = Buf(capi, B * 2 * L * n), Buf(capi, B * 2 * L * n)
    for k in range(B):
        capi.check(lib.he_memcpy_d2d(ba.at(k * 2 * L * n), a_ptr, 8 * 2 * L * n, None))
        capi.check(lib.he_memcpy_d2d(bb.at(k * 2 * L * n), b_ptr, 8 * 2 * L * n, None))
    bres = Buf(capi, B * 2 * (L - 1) * n)
    bws = Buf(capi, lib.he_multiply_relin_rescale_batch_workspace_words(h, L, B))

    def batch_call():
        capi.check(lib.he_multiply_relin_rescale_batch(h, L, B, ba.ptr, bb.ptr, evk, bres.ptr, bws.ptr, None))

    def make_batch_lanes(streams):
        """Per stream: its own operands, output and workspace for he_multiply_relin_rescale_batch."""
        lanes = []
        for st in streams:
            la, lb = Buf(capi, B * 2 * L * n), Buf(capi, B * 2 * L * n)
            capi.check(lib.he_memcpy_d2d(la.ptr, ba.ptr, 8 * B * 2 * L * n, None))
            capi.check(lib.he_memcpy_d2d(lb.ptr, bb.ptr, 8 * B * 2 * L * n, None))
            lanes.append((st, la, lb, Buf(capi, B * 2 * (L - 1) * n),
                          Buf(capi, lib.he_multiply_relin_rescale_batch_workspace_words(h, L, B))))
        return lanes

    if args.only == "batch_streams":
        # what `value` times, alone (for rocprofv3): batch calls dealt round-robin to the streams
        streams = []
        for _ in range(args.batch_streams):
            st = C.c_void_p()
            capi.check(lib.he_stream_create(C.byref(st)))
            streams.append(st)
        lanes = make_batch_lanes(streams)
        capi.check(lib.he_memcpy_d2d(ws.ptr, ws.at(48 * n), 8 * 48 * n, None))
        sync(capi)

        def issue(i):
            st, la, lb, lres, lws = lanes[i % len(lanes)]
            capi.check(lib.he_multiply_relin_rescale_batch(h, L, B, la.ptr, lb.ptr, evk, lres.ptr, lws.ptr, st))

        calls = max(2 * len(lanes), -(-K_steps // B))
        for i in range(2 * len(lanes)):
            issue(i)
        for st in streams:
            capi.check(lib.he_stream_synchronize(st))
        t0 = time.perf_counter()
        for i in range(calls):
            issue(i)
        for st in streams:
            capi.check(lib.he_stream_synchronize(st))
        ms = (time.perf_counter() - t0) * 1e3 / calls
        print(json.dumps({"only": args.only, "ms_per_call": ms, "ms_per_operation": ms / B, "calls": calls,
                          "operations_per_call": B, "streams": len(lanes), "calibration_copy_bytes": 8 * 48 * n}))
        return
    if args.only in ("step", "batch", "rotate", "ntt"):
        fn = {"step": step, "batch": batch_call, "rotate": one_rot,
              "ntt": lambda: (capi.check(lib.he_ntt_forward(h, two.ptr, 2, L, L, 0, L, 0, None)),
                              capi.check(lib.he_ntt_inverse(h, two.ptr, 2, L, L, 0, L, 0, None)))}[args.only]
        # one device-to-device copy of known size calibrates FETCH_SIZE / WRITE_SIZE of a rocprofv3 --pmc run
        capi.check(lib.he_memcpy_d2d(ws.ptr, ws.at(48 * n), 8 * 48 * n, None))
        ms = timer.time(fn, K_steps, W, blocks=1)
        print(json.dumps({"only": args.only, "ms_per_step": ms, "steps": K_steps, "calibration_copy_bytes": 8 * 48 * n}))
        return

    # (1) one operation after the other on the null stream
    single_ms = timer.time(step, K_steps, W)

    # (2) the same independent operations dealt round-robin to `lanes` streams, each with its own workspace and output
    lane_bufs, lane_streams = [], []
    for _ in range(args.lanes):
        st = C.c_void_p()
        capi.check(lib.he_stream_create(C.byref(st)))
        lane_streams.append(st)
        lane_bufs.append((Buf(capi, ws_words), Buf(capi, 2 * (L - 1) * n)))

    def lane_step(k):
        lws, lres = lane_bufs[k]
        capi.check(lib.he_multiply_relin_rescale(h, L, a_ptr, b_ptr, evk, lres.ptr, lws.ptr, lane_streams[k]))

    def lanes_sync():
        for st in lane_streams:
            capi.check(lib.he_stream_synchronize(st))

    def timed_wall(issue, count):
        blocks = []
        for _ in range(BLOCKS):
            sync(capi)
            lanes_sync()
            t0 = time.perf_counter()
            for i in range(count):
                issue(i)
            lanes_sync()
            sync(capi)
            blocks.append((time.perf_counter() - t0) * 1e3 / count)
        return statistics.median(blocks), blocks

    for i in range(W):
        lane_step(i % args.lanes)
    streams_ms, streams_blocks = timed_wall(lambda i: lane_step(i % args.lanes), K_steps)

    # (3) `batch` operations per call, one launch per stage for all of them.  A timed block holds at least 20 calls
    # whatever --steps says: a block of a few calls would be a few milliseconds of GPU time
    calls = max(20, -(-K_steps // B))
    batch_ms = timer.time(batch_call, calls, max(1, W // B)) / B

    # (3b) the same batch calls dealt to two streams (each with its own operands, workspace and output): the tail of
    # one call's kernels overlaps the head of the other's
    batch_lanes = make_batch_lanes(lane_streams[:min(args.batch_streams, len(lane_streams))])

    def batch_lane_call(i):
        st, la, lb, lres, lws = batch_lanes[i % len(batch_lanes)]
        capi.check(lib.he_multiply_relin_rescale_batch(h, L, B, la.ptr, lb.ptr, evk, lres.ptr, lws.ptr, st))

    for i in range(2 * len(batch_lanes)):
        batch_lane_call(i)
    bs_calls = max(20, 2 * len(batch_lanes), calls)
    bs_ms, bs_blocks = timed_wall(batch_lane_call, bs_calls)
    bs_ms /= B

    # (4) the reference's own call sequence through pyCAHEL on the null stream
    prod = cahel.ciphertext(ctx)

    def api_step():
        cahel.multiply(ctx, ct1, ct2, prod)
        cahel.relinearize_inplace(ctx, prod, rlk)
        cahel.rescale_to_next_inplace(ctx, prod)

    api_ms = timer.time(api_step, K_steps, W)

    # every path gives the evaluator's limbs, and they decrypt to x * y
    api_step()
    want = prod.to_numpy()
    got = np.empty((2, L - 1, n), dtype=np.uint64)
    same = True
    views = [type("B", (), {"ptr": bres.at(k * 2 * (L - 1) * n)}) for k in (0, B - 1)]
    views += [type("B", (), {"ptr": lane[3].at((B - 1) * 2 * (L - 1) * n)}) for lane in batch_lanes]
    for buf in [res] + [lres for _, lres in lane_bufs] + views:
        capi.check(lib.he_memcpy_d2h(got.ctypes.data, buf.ptr, got.nbytes, None))
        same = same and bool((got == want).all())
    fused = cahel.ciphertext(ctx)
    cahel.multiply_relin_rescale(ctx, ct1, ct2, rlk, fused)
    same = same and bool((fused.to_numpy() == want).all())
    dec = np.array(enc.decode(ctx, sk.decrypt(ctx, prod)))
    max_err = float(np.max(np.abs(dec - x * y)))

    # measured FP64 issue rate of this GPU (8 waves per SIMD of independent multiply-add chains)
    rate = C.c_double()
    capi.check(capi.probe_lib().he_probe_fp64_issue_rate(2048, 2000, C.byref(rate), None))

    # config "NTT alone": 24 limbs x 2 polynomials, forward + inverse
    f = timer.time(lambda: capi.check(lib.he_ntt_forward(h, two.ptr, 2, L, L, 0, L, 0, None)), 100)
    i = timer.time(lambda: capi.check(lib.he_ntt_inverse(h, two.ptr, 2, L, L, 0, L, 0, None)), 100)
    ntt = {"forward_ms": f, "inverse_ms": i, "bytes_fwd_plus_inv": 4 * 2 * L * limb_bytes,
           "GBps": 4 * 2 * L * limb_bytes / ((f + i) * 1e-3) / 1e9}
    ntt["frac_of_hbm_peak"] = ntt["GBps"] / HBM_PEAK_GBS
    six = Buf(capi, 12 * L * n)
    capi.check(lib.he_memset_zero(six.ptr, 8 * 12 * L * n, None))
    f6 = timer.time(lambda: capi.check(lib.he_ntt_forward(h, six.ptr, 12, L, L, 0, L, 0, None)), 30)
    i6 = timer.time(lambda: capi.check(lib.he_ntt_inverse(h, six.ptr, 12, L, L, 0, L, 0, None)), 30)
    ntt["six_ciphertexts_per_call"] = {"forward_ms": f6, "inverse_ms": i6,
                                       "GBps": 4 * 12 * L * limb_bytes / ((f6 + i6) * 1e-3) / 1e9}
    ntt["six_ciphertexts_per_call"]["frac_of_hbm_peak"] = ntt["six_ciphertexts_per_call"]["GBps"] / HBM_PEAK_GBS

    # rotations (config "rotate-and-sum"): one keyed rotation; 15 dependent rotations + adds
    rot_ms = timer.time(one_rot, 50)

    def rotate_and_sum():
        acc = ct1.copy()
        tmp = cahel.ciphertext(ctx)
        for s in steps_pow2:
            cahel.rotate_vector(ctx, acc, s, glk, tmp)
            cahel.add_inplace(ctx, acc, tmp)
        return acc

    ras_ms = timer.time(rotate_and_sum, 5, warmup=1)
    total = np.array(enc.decode(ctx, sk.decrypt(ctx, rotate_and_sum())))

    def hoisted_sum():
        acc = ct1.copy()
        for steps in hoist_rounds:
            cahel.add_inplace(ctx, acc, cahel.hoisting(ctx, acc, glk, steps))
        return acc

    hs_ms = timer.time(hoisted_sum, 5, warmup=1)
    total_h = np.array(enc.decode(ctx, sk.decrypt(ctx, hoisted_sum())))
    rotate = {"one_rotation_ms": rot_ms, "rotate_and_sum_15_ms": ras_ms,
              "one_rotation_GBps": 288 * limb_bytes / (rot_ms * 1e-3) / 1e9,
              "one_rotation_frac_of_hbm_roofline": 288 * limb_bytes / (rot_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
              "rotate_and_sum_GBps": 15 * 432 * limb_bytes / (ras_ms * 1e-3) / 1e9,
              "slot_sum_rel_err": float(np.max(np.abs(total - x.sum())) / abs(x.sum())),
              "slot_sum_hoisted_rounds_ms": hs_ms, "hoisted_rounds": "5 rounds of steps 8^r x (1..7)",
              "slot_sum_hoisted_rel_err": float(np.max(np.abs(total_h - x.sum())) / abs(x.sum()))}

    alg_bytes = 334 * limb_bytes

    def frac(ms):
        return alg_bytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS

    def roofline(ms_per_op, kind, what, ops_per_launch):
        """The step as the roofline unit: its kernels run back to back, so algorithmic bytes over the step's
        duration is the traffic-weighted rate of its kernels."""
        prof = PROFILE[kind]
        issue_ms = prof["valu_wave_instr"] * 64 / rate.value * 1e3
        floor_ms = 920 * limb_bytes / 6.0e12 * 1e3
        return {"bound": "hbm", "kernel": what + prof["kernels"],
                "achieved": alg_bytes / (ms_per_op * 1e-3) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": frac(ms_per_op),
                # the same with the bytes that a launch has to move: the key is read once per launch, not per operation
                "frac_amortised_key": (96 + 46 + 192.0 / ops_per_launch) * limb_bytes / (ms_per_op * 1e-3) / 1e9 / HBM_PEAK_GBS,
                "compulsory_bytes_per_launch": int((96 + 46) * limb_bytes * ops_per_launch + 192 * limb_bytes),
                "ms_per_launch": ms_per_op * ops_per_launch,
                "operations_per_launch": ops_per_launch,
                "algorithmic_bytes_per_launch": alg_bytes * ops_per_launch,
                "traffic": int(prof["traffic_limbs"] * limb_bytes * ops_per_launch),
                "traffic_source": "profiles/hmult_relin_rescale_n65536_l24_k8.md (counter profile, not this run)",
                "frac_of_dataflow_floor": floor_ms / ms_per_op,
                "dataflow_floor": "920 limbs of traffic per operation (two-pass transforms, every fusion of "
                                  "neighbouring pointwise stages) at the 6 TB/s a streaming kernel reaches on this GPU",
                "valu": {"wave_instructions_per_operation": prof["valu_wave_instr"],
                         "source": "SQ_INSTS_VALU summed over the kernels, same profile",
                         "fp64_issue_peak_lane_ops_per_s": rate.value, "issue_bound_ms": issue_ms,
                         "frac_of_issue_bound": issue_ms / ms_per_op}}

    best_ms, path = min((streams_ms, "streams"), (batch_ms, "batch"), (bs_ms, "batch_streams"))
    line = {
        "metric": "HMult+relin+rescale ops/s at N=2^16, L=24 (dnum=3, 8 special primes)",
        "value": 1e3 / best_ms, "unit": "ops/s", "n_gpus": 1, "steps": K_steps, "warmup": W,
        "ms_per_step": best_ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "u64", "data": "synthetic",
        "arithmetic": "64-bit residues; every stage in exact FP64 (primes below 2^50) with canonical 64-bit results; "
                      "every output bit-identical to the integer oracle",
        "timing": "median of %d timed blocks after %d warm-up steps; a block is %d steps for the single-call paths, %d "
                  "calls of %d operations for `batch` and %d such calls for `batch_streams` (`value`), whatever --steps says"
                  % (BLOCKS, W, K_steps, calls, B, bs_calls),
        "config": {"workload": "HMult+relinearize+rescale, N=2^16, L=24 limbs of 50 bits, K=8, dnum=3, scale 2^40, "
                               "two fresh ciphertexts of 32768 uniform[-1,1] slots (BASELINE.json configs[2]); "
                               "independent operations, the best of %d streams of single calls, batches of %d per "
                               "call on one stream, and such batches dealt to %d streams"
                               % (args.lanes, B, len(batch_lanes)),
                   "value_path": path, "lanes": args.lanes, "batch": B},
        "hmult_frac_of_hbm_roofline": frac(best_ms),
        "hmult_algorithmic_bytes": alg_bytes,
        "streams": {"ms_per_step": streams_ms, "ops_per_s": 1e3 / streams_ms, "frac_of_hbm_roofline": frac(streams_ms),
                    "blocks_ms": streams_blocks},
        "batch": {"ms_per_step": batch_ms, "ops_per_s": 1e3 / batch_ms, "frac_of_hbm_roofline": frac(batch_ms),
                  "ops_per_call": B},
        "batch_streams": {"ms_per_step": bs_ms, "ops_per_s": 1e3 / bs_ms, "frac_of_hbm_roofline": frac(bs_ms),
                          "ops_per_call": B, "streams": len(batch_lanes), "blocks_ms": [b / B for b in bs_blocks]},
        "single_stream": {"ms_per_step": single_ms, "ops_per_s": 1e3 / single_ms, "frac_of_hbm_roofline": frac(single_ms)},
        "api_path": {"calls": "pyCAHEL multiply, relinearize_inplace, rescale_to_next_inplace on the null stream",
                     "ms_per_step": api_ms, "ops_per_s": 1e3 / api_ms, "frac_of_hbm_roofline": frac(api_ms)},
        "check": {"all_paths_equal_the_evaluator": same, "decrypt_max_abs_err_vs_xy": max_err},
        "roofline": roofline(best_ms, "single" if path == "streams" else "batch",
                             "value path (%s): " % path, 1 if path == "streams" else B),
        "single_stream_roofline": roofline(single_ms, "single", "one operation after the other on one stream: ", 1),
        "ntt": ntt, "rotate": rotate,
        "config_c1": gpu_c1(capi, cahel, timer),
    }
    if not args.no_krum:
        line["krum"] = krum_round(with_cpu=not args.no_cpu_baseline, with_reference_sequence=True)
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
