"""Encrypted Krum distance computation over pyCAHEL: the caller side of the hot path.

Restates the protocol of lancelot-main-GPU/utils/byzantine_fl.py (GPU_init :432-462,
GPU_compute_pair_distance :173-321, GPU_computing_distance_cipher :466-514, GPU_decrypt_sort_mask :327-369,
GPU_mul_mask_weight :371-429, GPU_krum :517-525) on top of the same pyCAHEL calls, with two differences that do not change the result:
every client chunk is encoded and encrypted once (the reference re-encrypts both operands for every pair) and
the i == j pairs, whose distance is zero, are not evaluated.

Per pair (i, j): for every chunk  d = ct_j - ct_i ; d = d^2 (size 3) ; acc += d   ("lazy relinearisation"),
then one relinearise + rescale, then rotate-and-sum so that every slot holds sum_k (u_i[k] - u_j[k])^2.
The score of a client is the plain row sum of its distances (no nearest-neighbour truncation), as in
byzantine_fl.py:344-353 and :531-533; the chosen client is the argmin.

Two ways through the same arithmetic (KrumConfig.batched): all chunks / pairs / results through every stage together,
one launch per stage (encode_encrypt_many, pair_square_distances, decrypt_decode_many: three- and four-limb
ciphertexts are too small to fill the GPU one at a time), or call by call as the reference does, spread over the
lanes of the host layer.
"""
from __future__ import annotations

import math
import time
from dataclasses import dataclass, field

import numpy as np


@dataclass
class KrumConfig:
    log_n: int = 16
    modulus_bits: tuple = (60, 40, 40, 60)   # GPU_init: modulus_chain = [60, 40, 40, 60]
    special_modulus_size: int = 1            # GPU_init: size_P = 1
    scale: float = 2.0 ** 40
    hoisting: bool = True                    # byzantine_fl.py: Hoisting_flag = 1
    hoisting_radix: int = 16                 # every round of the slot sum is a hoisted sum of radix - 1 rotations;
                                             # 0: the reference's split, hoisting(1..15) then one rotation per doubling
    sum_drop_levels: int = 0                 # limbs dropped without scaling (mod_switch_to_next) after the rescale:
                                             # the slot sum's key switches then run over fewer limbs; 0 = as the
                                             # reference, which rotates at the level the rescale leaves.  The
                                             # moduli that remain must still hold distance * scale (with one limb
                                             # left that is the first prime alone: 60 bits are enough for the
                                             # benchmark's distances at scale 2^40, 50 bits are not)
    batched: bool = True                     # all pairs go through every stage together, one launch per stage
                                             # (pair_square_distances); False: pair by pair over the lanes
    lanes: int = 3                           # host threads / streams that the pairs are dealt to (0: null stream);
                                             # three streams and the null stream fill the four hardware queues
    sec_level: str = "tc128"
    seed: int | None = None
    reproducible: bool = False               # with a seed: encrypt on the calling thread, so that every ciphertext
                                             # draws the same randomness in every run


@dataclass
class KrumState:
    cahel: object
    config: KrumConfig
    context: object
    pk: object
    sk: object
    glk: object
    rlk: object
    encoder: object
    slots: int
    timings: dict = field(default_factory=lambda: {"encode": 0.0, "encrypt": 0.0, "evaluate": 0.0, "decrypt": 0.0})


def _sync(cahel):
    cahel._synchronize()


def gpu_init(config: KrumConfig | None = None) -> KrumState:
    """Context, keys and encoder (byzantine_fl.py:432-462)."""
    import lancelot_amd  # noqa: F401
    import pyCAHEL as cahel
    config = config or KrumConfig()
    n = 1 << config.log_n
    log_slots = config.log_n - 1
    steps = sorted({s for rnd in rotate_sum_plan(log_slots, config) for s in rnd if s < n // 2})
    params = cahel.params(cahel.scheme_type.ckks)
    params.set_poly_modulus_degree(n)
    params.set_coeff_modulus(cahel.coeff_modulus_create(n, list(config.modulus_bits)))
    params.set_special_modulus_size(config.special_modulus_size)
    params.set_galois_elts(cahel.get_elts_from_steps(steps, n))
    context = cahel.context(params, True, getattr(cahel.sec_level_type, config.sec_level))
    if config.seed is not None:
        context.set_seed(config.seed)
    sk = cahel.secret_key(params)
    sk.gen_secretkey(context)
    pk = cahel.public_key(context)
    sk.gen_publickey(context, pk)
    rlk = cahel.relin_key(context)
    sk.gen_relinkey(context, rlk)
    glk = cahel.galois_key(context)
    sk.create_galois_keys(context, glk)
    encoder = cahel.ckks_encoder(context)
    return KrumState(cahel, config, context, pk, sk, glk, rlk, encoder, encoder.slot_count())


def rotate_sum_plan(log_slots: int, config: KrumConfig):
    """Rounds of the slot sum: after round r every slot holds the sum of a block of prod(len(round) + 1) slots.
    A round [s1, s2, ...] is acc += sum_k rot(acc, s_k): hoisted when it has several steps, one rotation otherwise.
    The reference (byzantine_fl.py:252-300) hoists the first four doublings, steps 1..15, and rotates for the rest."""
    if not config.hoisting:
        return [[2 ** k] for k in range(log_slots)]
    if config.hoisting_radix < 2 or log_slots <= 4:
        head = [list(range(1, 16))] if log_slots > 4 else []
        return head + [[2 ** k] for k in range(4 if head else 0, log_slots)]
    # The short round comes first: rounds whose steps are multiples of N / 512 permute the NTT order inside blocks of
    # 256 words, which the hoisting kernel serves from LDS; the rounds before them gather from memory once per step,
    # so those get the fewer steps.
    log_radix = max(1, int(math.log2(config.hoisting_radix)))
    n_rounds = -(-log_slots // log_radix)
    rounds, block = [], 1
    for r in range(n_rounds):
        radix = 1 << (log_slots - (n_rounds - 1) * log_radix if r == 0 else log_radix)
        rounds.append([block * s for s in range(1, radix)])
        block *= radix
    return rounds


def split_updates(vectors, slots: int):
    """Zero-pad every flattened update to a multiple of `slots` and split it (byzantine_fl.py:474-490): one float64
    matrix [client][padded length], the chunks are views of its rows."""
    length = int(np.asarray(vectors[0]).size)
    if any(int(np.asarray(v).size) != length for v in vectors):
        raise ValueError("all client updates must have the same length")
    whole = length if length % slots == 0 else (length // slots + 1) * slots
    padded = np.zeros((len(vectors), whole), dtype=np.float64)
    for row, v in zip(padded, vectors):
        row[:length] = np.asarray(v).reshape(-1)
    return [[row[k:k + slots] for k in range(0, whole, slots)] for row in padded]


def encrypt_updates(state: KrumState, chunks):
    """One ciphertext per (client, chunk).  Batched: all chunks through encode and encrypt together.  Otherwise the
    chunks go over the lanes (unless the run is to be reproducible); the first one is then encoded on the calling
    thread because the first message fixes the encoder's slot count."""
    import threading
    ctx = state.context
    spent = {"encode": 0.0, "encrypt": 0.0}
    spent_lock = threading.Lock()

    def one(item):
        t0 = time.perf_counter()
        pt = state.encoder.encode(ctx, np.ascontiguousarray(item, dtype=np.float64), state.config.scale)
        t1 = time.perf_counter()
        ct = state.pk.encrypt_asymmetric(ctx, pt)
        t2 = time.perf_counter()
        with spent_lock:                    # summed over the threads; scaled to the wall time below
            spent["encode"] += t1 - t0
            spent["encrypt"] += t2 - t1
        return ct

    t0 = time.perf_counter()
    flat = [chunk for client in chunks for chunk in client]
    if state.config.batched:
        # all chunks through encode and encrypt together, one launch per stage; the chunks of split_updates are the
        # rows of one matrix already
        base = flat[0].base
        if base is not None and base.ndim == 2 and base.size == len(flat) * state.slots and base.flags.c_contiguous \
                and all(c.base is base for c in flat):
            matrix = base.reshape(len(flat), state.slots)
        else:
            matrix = np.ascontiguousarray(np.stack([np.asarray(c, dtype=np.float64) for c in flat]))
        cts = state.encoder.encode_encrypt_many(ctx, state.pk, matrix, state.config.scale)
        _sync(state.cahel)
        wall = time.perf_counter() - t0
        state.timings["encode"] += wall        # encode and encrypt are one pipeline here
        it = iter(cts)
        return [[next(it) for _ in client] for client in chunks]
    if state.config.reproducible:
        cts = [one(item) for item in flat]      # the encryption randomness is drawn in a fixed order
    else:
        cts = [one(flat[0])] + _map_lanes(state, flat[1:], one)
    wall = time.perf_counter() - t0
    busy = max(spent["encode"] + spent["encrypt"], 1e-12)
    for k in spent:
        state.timings[k] += wall * spent[k] / busy
    it = iter(cts)
    return [[next(it) for _ in client] for client in chunks]


def pair_distance(state: KrumState, cts_i, cts_j):
    """Ciphertext whose every slot holds ||u_i - u_j||^2 (byzantine_fl.py:173-321)."""
    c, ctx, cfg = state.cahel, state.context, state.config
    acc = None
    tmp = c.ciphertext(ctx)
    for ct1, ct2 in zip(cts_i, cts_j):
        c.sub(ctx, ct2, ct1, tmp)
        c.square_inplace(ctx, tmp)
        if acc is None:
            acc = tmp
            tmp = c.ciphertext(ctx)
        else:
            c.add_inplace(ctx, acc, tmp)
    c.relinearize_rescale_inplace(ctx, acc, state.rlk)     # = relinearize_inplace + rescale_to_next_inplace
    acc.set_scale(cfg.scale)
    for _ in range(cfg.sum_drop_levels):
        c.mod_switch_to_next_inplace(ctx, acc)
    rot = c.ciphertext(ctx)
    for steps in rotate_sum_plan(int(math.log2(state.slots)), cfg):
        if len(steps) > 1:
            c.add_inplace(ctx, acc, c.hoisting(ctx, acc, state.glk, steps))
        else:
            c.rotate_vector(ctx, acc, steps[0], state.glk, rot)
            c.add_inplace(ctx, acc, rot)
    return acc


def reference_call_sequence(state: KrumState, updates):
    """The distance phase exactly as lancelot-main-GPU/utils/byzantine_fl.py drives the library, call for call, on the
    null stream: GPU_computing_distance_cipher (:466-514) runs GPU_compute_pair_distance (:173-321) for the 55 pairs
    i <= j, and every pair encodes and encrypts both operands again, chunk by chunk, besides two encryptions of zero
    (one of them unused on the lazy-relinearisation branch that the file takes); then sub, square_inplace, add_inplace
    onto the squared zero, relinearize_inplace, rescale_to_next_inplace, set_scale, hoisting of steps 1..15 +
    add_inplace, and one rotate_vector + add_inplace per doubling from 2^4 on.  `state` must come from a KrumConfig
    with hoisting_radix = 0 (that key set).  Returns (decrypted distance matrix, seconds per phase)."""
    c, ctx, cfg = state.cahel, state.context, state.config
    enc, pk, scale = state.encoder, state.pk, cfg.scale
    log_slots = int(math.log2(state.slots))
    chunks = split_updates(updates, state.slots)
    n_clients = len(chunks)
    spent = {"encode": 0.0, "encrypt": 0.0, "square_accumulate": 0.0, "relinearize_rescale": 0.0, "rotate_and_sum": 0.0}
    zero = np.zeros(state.slots)

    def lap(key, t0):
        _sync(c)                      # the reference's timers bracket asynchronous calls; these wait for the work
        now = time.perf_counter()
        spent[key] += now - t0
        return now

    def pair(msg1, msg2):
        t = time.perf_counter()
        tmp = c.ciphertext(ctx)
        pt_tmp1 = enc.encode(ctx, zero, scale)
        t = lap("encode", t)
        tmp1 = pk.encrypt_asymmetric(ctx, pt_tmp1)
        c.mod_switch_to_inplace(ctx, tmp1, 2)
        t = lap("encrypt", t)
        pt_zero = enc.encode(ctx, zero, scale)
        t = lap("encode", t)
        acc = pk.encrypt_asymmetric(ctx, pt_zero)
        t = lap("encrypt", t)
        c.square_inplace(ctx, acc)
        t = lap("square_accumulate", t)
        for x1, x2 in zip(msg1, msg2):
            pt1 = enc.encode(ctx, x1, scale)
            pt2 = enc.encode(ctx, x2, scale)
            t = lap("encode", t)
            ct1 = pk.encrypt_asymmetric(ctx, pt1)
            ct2 = pk.encrypt_asymmetric(ctx, pt2)
            t = lap("encrypt", t)
            c.sub(ctx, ct2, ct1, tmp)
            c.square_inplace(ctx, tmp)
            c.add_inplace(ctx, acc, tmp)
            t = lap("square_accumulate", t)
        c.relinearize_inplace(ctx, acc, state.rlk)
        c.rescale_to_next_inplace(ctx, acc)
        acc.set_scale(scale)
        t = lap("relinearize_rescale", t)
        rot = c.ciphertext(ctx)
        hoisted = c.hoisting(ctx, acc, state.glk, list(range(1, 16)))
        c.add_inplace(ctx, acc, hoisted)
        for k in range(4, log_slots):
            c.rotate_vector(ctx, acc, 2 ** k, state.glk, rot)
            c.add_inplace(ctx, acc, rot)
        lap("rotate_and_sum", t)
        return acc

    _sync(c)
    t0 = time.perf_counter()
    enc_dist = [[None] * n_clients for _ in range(n_clients)]
    for i in range(n_clients):
        for j in range(i, n_clients):
            enc_dist[i][j] = enc_dist[j][i] = pair(chunks[i], chunks[j])
    _sync(c)
    timings = dict(spent, distance_phase=time.perf_counter() - t0, pairs=n_clients * (n_clients + 1) // 2)
    dist = np.zeros((n_clients, n_clients))
    for i in range(n_clients):
        for j in range(i + 1, n_clients):
            dist[i, j] = dist[j, i] = state.encoder.decode_array(ctx, state.sk.decrypt(ctx, enc_dist[i][j]), 1)[0]
    return dist, timings


def _map_lanes(state: KrumState, items, fn):
    """[fn(item) for item in items], the items dealt round-robin to `lanes` host threads, each issuing on its own
    lane (stream) of the host layer (the evaluator, decrypt and decode calls release the interpreter lock);
    everything is synchronised before and after."""
    c = state.cahel
    lanes = min(state.config.lanes, c._lane_count(), max(len(items), 1))
    _sync(c)
    if lanes <= 0:
        out = [fn(item) for item in items]
        _sync(c)
        return out

    def worker(w):
        c._set_lane(1 + w)          # the current lane is per host thread
        return [fn(item) for item in items[w::lanes]]

    from concurrent.futures import ThreadPoolExecutor
    out = [None] * len(items)
    with ThreadPoolExecutor(max_workers=lanes) as pool:
        for w, part in enumerate(pool.map(worker, range(lanes))):
            out[w::lanes] = part
    _sync(c)
    return out


def all_pair_distances(state: KrumState, cts, enc):
    """enc[i][j] = enc[j][i] = pair_distance(i, j) for every i < j.  The pairs are independent, and at Lancelot's
    sizes (three or four limbs) one of them neither fills the GPU nor keeps one host thread's launch rate busy, so
    they go through every stage together (one launch per stage for all pairs) or, pair by pair, over the lanes."""
    n_clients = len(cts)
    pairs = [(i, j) for i in range(n_clients) for j in range(i + 1, n_clients)]
    if state.config.batched:
        c = state.cahel
        rounds = rotate_sum_plan(int(math.log2(state.slots)), state.config)
        out = c.pair_square_distances(state.context, cts, pairs, state.rlk, state.glk, rounds, state.config.scale,
                                      state.config.sum_drop_levels)
        _sync(c)
    else:
        out = _map_lanes(state, pairs, lambda ij: pair_distance(state, cts[ij[0]], cts[ij[1]]))
    for (i, j), ct in zip(pairs, out):
        enc[i][j] = enc[j][i] = ct


def distance_matrix(state: KrumState, updates):
    """Encrypted pairwise squared distances and their decryptions (slot 0 of every pair)."""
    c = state.cahel
    chunks = split_updates(updates, state.slots)
    cts = encrypt_updates(state, chunks)
    n_clients = len(updates)
    enc = [[None] * n_clients for _ in range(n_clients)]
    t0 = time.perf_counter()
    all_pair_distances(state, cts, enc)
    state.timings["evaluate"] += time.perf_counter() - t0
    t0 = time.perf_counter()
    dist = np.zeros((n_clients, n_clients))
    pairs = [(i, j) for i in range(n_clients) for j in range(i + 1, n_clients)]
    # every slot holds the distance: slot 0 is downloaded
    if state.config.batched:
        values = state.sk.decrypt_decode_many(state.context, [enc[i][j] for i, j in pairs], state.slots, 1)[:, 0]
    else:
        values = _map_lanes(state, pairs, lambda ij: state.encoder.decode_array(
            state.context, state.sk.decrypt(state.context, enc[ij[0]][ij[1]]), 1)[0])
    for (i, j), value in zip(pairs, values):
        dist[i, j] = dist[j, i] = value
    state.timings["decrypt"] += time.perf_counter() - t0
    return dist, enc


def _encrypt_constant(state: KrumState, value: float):
    c = state.cahel
    pt = state.encoder.encode(state.context, np.full(state.slots, value, dtype=np.float64), state.config.scale)
    return state.pk.encrypt_asymmetric(state.context, pt)


def decrypt_sort_mask(state: KrumState, enc):
    """Row sums of the encrypted distances, decrypted scores, and the one-hot mask ciphertexts
    (byzantine_fl.py:327-369): mask[r][k] encrypts 1 when client k has the r-th smallest score, else 0.
    Returns (mask, order, scores)."""
    c, ctx = state.cahel, state.context
    n_clients = len(enc)
    t0 = time.perf_counter()

    def row_sum(i):
        # the i == j distance is zero and was never evaluated; the reference starts from an encryption of zero
        row = [ct for ct in enc[i] if ct is not None]
        total = row[0]
        if len(row) > 1:
            total = c.ciphertext(ctx)
            c.add(ctx, row[0], row[1], total)
            for ct in row[2:]:
                c.add_inplace(ctx, total, ct)
        return total

    if state.config.batched:
        totals = [row_sum(i) for i in range(n_clients)]
        scores = list(state.sk.decrypt_decode_many(ctx, totals, state.slots, 1)[:, 0])
    else:
        scores = _map_lanes(state, list(range(n_clients)), lambda i: state.encoder.decode_array(
            ctx, state.sk.decrypt(ctx, row_sum(i)), 1)[0])
    order = np.argsort(np.asarray(scores), kind="stable")
    zero, one = _encrypt_constant(state, 0.0), _encrypt_constant(state, 1.0)
    mask = [[one if order[r] == k else zero for k in range(n_clients)] for r in range(n_clients)]
    _sync(c)
    state.timings["mask"] = state.timings.get("mask", 0.0) + time.perf_counter() - t0
    return mask, order, np.asarray(scores)


def mul_mask_weight(state: KrumState, cts, mask_row):
    """sum_k mask_row[k] * update_k chunk by chunk with lazy relinearisation: the products stay size-3
    ciphertexts, are added, and are decrypted as such (byzantine_fl.py:371-429, lazy_relin_flag branch).
    `cts[k][chunk]` are the cached client ciphertexts.  Returns the decoded weights (all chunks, padded)."""
    c, ctx = state.cahel, state.context
    t0 = time.perf_counter()
    n_chunks = len(cts[0])
    out = []
    prod = c.ciphertext(ctx)
    for chunk in range(n_chunks):
        acc = None
        for k, ct_mask in enumerate(mask_row):
            c.multiply(ctx, cts[k][chunk], ct_mask, prod)
            if acc is None:
                acc = prod
                prod = c.ciphertext(ctx)
            else:
                c.add_inplace(ctx, acc, prod)
        out.append(state.encoder.decode_array(ctx, state.sk.decrypt(ctx, acc)))
    _sync(c)
    state.timings["mask_multiply"] = state.timings.get("mask_multiply", 0.0) + time.perf_counter() - t0
    return np.concatenate(out)


def plain_distance_matrix(updates):
    """float64 closed form ||u_i - u_j||^2 (byzantine_fl.py:129-131, 162-171)."""
    v = [np.asarray(u, dtype=np.float64).reshape(-1) for u in updates]
    n = len(v)
    d = np.zeros((n, n))
    for i in range(n):
        for j in range(i + 1, n):
            d[i, j] = d[j, i] = float(np.sum((v[i] - v[j]) ** 2))
    return d


def krum_select(dist: np.ndarray) -> int:
    """Row sums, argsort, first entry (byzantine_fl.py:531-533)."""
    return int(np.argsort(dist.sum(axis=0), kind="stable")[0])


def gpu_krum(updates, config: KrumConfig | None = None, state: KrumState | None = None):
    """One encrypted Krum round: returns (chosen client index, distance matrix, timings in seconds)."""
    state = state or gpu_init(config)
    for k in state.timings:
        state.timings[k] = 0.0
    t0 = time.perf_counter()
    dist, _ = distance_matrix(state, updates)
    total = time.perf_counter() - t0
    timings = dict(state.timings, total=total)
    return krum_select(dist), dist, timings


def gpu_krum_aggregate(updates, config: KrumConfig | None = None, state: KrumState | None = None):
    """The full round of the reference's driver: encrypted distances, decrypt-sort-mask, and the masked sum of
    the encrypted updates, which is the update of the chosen client (byzantine_fl.py:517-525 followed by
    :327-429).  Returns (chosen client index, aggregated weights of len(updates[0]), timings in seconds)."""
    state = state or gpu_init(config)
    for k in list(state.timings):
        state.timings[k] = 0.0
    t0 = time.perf_counter()
    chunks = split_updates(updates, state.slots)
    cts = encrypt_updates(state, chunks)
    n_clients = len(updates)
    enc = [[None] * n_clients for _ in range(n_clients)]
    t1 = time.perf_counter()
    all_pair_distances(state, cts, enc)
    state.timings["evaluate"] += time.perf_counter() - t1
    mask, order, _ = decrypt_sort_mask(state, enc)
    weights = mul_mask_weight(state, cts, mask[0])
    total = time.perf_counter() - t0
    length = len(np.asarray(updates[0]).reshape(-1))
    return int(order[0]), weights[:length], dict(state.timings, total=total)
