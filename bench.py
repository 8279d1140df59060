#!/usr/bin/env python3
"""Benchmark of the sparse pull + push hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--resident KEYS] [--config cfg3]

A step is one SparseTablePull followed by one SparseTablePush over one seeded
synthetic batch whose inputs (signs, labels, gradients) and outputs (mapped
ids, variables) are already resident in HBM.  The default workload is the one
the headline metric is quoted on: dim-16 AdaGrad, batch 16384 x 100 slots with
Poisson(3) id lists (~5 M lookups), Zipf(1.1) signs over a 1e9 vocabulary and
5e8 resident keys.  Prints ONE JSON line.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK = 8.0e12  # bytes/s, MI355X


def log(msg):
    print("[bench] " + msg, file=sys.stderr, flush=True)


# HBM bytes per launch (read + written) of the cfg3 kernels at 5e8 resident keys come from the rocprofv3 --pmc
# FETCH_SIZE / WRITE_SIZE runs that `python3 -m tensornet_amd.profile_summary` condenses into this file beside
# profiles/cfg3_adagrad_dim16_pull_push.md (counters cannot be read from inside this script).
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "cfg3_traffic.json")
# launched by a step, a few microseconds each, no traffic worth counting
SMALL_STEP_KERNELS = ("k_stage_in", "k_publish", "k_init_new_recs", "k_group_offsets", "k_scan_tiles")


def measured_traffic(step_kernels):
    """{kernel: HBM bytes per launch} of the committed profile, its provenance, and a loud failure if a kernel the
    step launches is not in it (the profile is older than the kernels: refresh it)."""
    if not os.path.exists(TRAFFIC_FILE):
        raise SystemExit("bench.py: %s is missing (python3 -m tensornet_amd.profile_summary writes it)" % TRAFFIC_FILE)
    with open(TRAFFIC_FILE) as f:
        t = json.load(f)
    per_launch = t["bytes_per_launch"]
    missing = sorted(k.split("<")[0] for k in step_kernels
                     if k.split("<")[0] not in per_launch and not k.startswith(SMALL_STEP_KERNELS))
    if missing:
        raise SystemExit("bench.py: the step launches %s, which %s does not cover: refresh the profile "
                         "(python3 -m tensornet_amd.profile_summary)" % (", ".join(missing), TRAFFIC_FILE))
    return per_launch, {"file": os.path.relpath(TRAFFIC_FILE, ROOT), "profiled_at_commit": t.get("commit"),
                        "fetch_factor": t.get("fetch_factor"), "write_factor": t.get("write_factor")}


def state_bytes(opt, dim):
    """Optimizer state bytes read+written per applied row (beyond w and the gradient)."""
    return 28 if opt == "AdaGrad" else 16 * dim + 8


def step_algorithmic_bytes(opt, dim, L, U):
    """Bytes one pull + one push must move, counting each datum once:
    pull = 8L (signs) + 8L (mapped ids) + U*(8 key + 4D row + 4D var);
    push = 8L (signs) + 8L (labels) + U*(4D grad + 8 key + 8D w r/w + state)."""
    return 32 * L + U * (8 + 8 * dim + 4 * dim + 8 + 8 * dim + state_bytes(opt, dim))


# Launched on the table's side streams, concurrently with kernels of the caller's stream (the other
# update kernels; the ranking kernels of the remap).
SIDE_STREAM_KERNELS = ("k_apply_single", "k_group_count", "k_group_offsets", "k_probe_recs")
BIG_GROUP = 16  # records from which a sign is applied by k_apply_big (sparse_table.hip)


def kernel_algorithmic_bytes(name, opt, dim, shape):
    """Algorithmic bytes of one launch of each kernel of the step: what the kernel has to
    read and write once, from the sizes of the batch.  shape: L lookups, U per-slot distinct
    signs (records), G distinct signs of the whole batch (groups); G1 groups with one record,
    Rm / Gm records / groups with 2..15 records, Rb / Gb records / groups with 16 or more."""
    L, U, G = shape["L"], shape["U"], shape["G"]
    row = 4 * dim
    st = state_bytes(opt, dim)

    def apply_bytes(records, groups):  # gradient + member entry per record; row and state read and written per group
        return records * (row + 16) + groups * (2 * row + st)

    table = {
        # remap through LDS (T: distinct signs per 2048-lookup tile, summed over the tiles)
        "k_tile_dedup": 12 * L + L // 32 + 16 * shape["T"],  # reads every sign, leaves its first position in the tile,
                                                             # 16 bytes of fingerprint per 64 signs and a record per
                                                             # distinct sign of a tile
        "k_lds_dedup": 16 * shape["T"] + 4 * (shape["T"] - U) + 16 * U,  # the tiles' records in; first positions for the
                                                                         # tiles' repeats and the distinct records out
        "k_lds_flags": 4 * L,
        "k_lds_assign": 4 * U,
        "k_lds_mapped": 12 * L,                # first position in, mapped id out
        "k_group_count": 24 * U,               # distinct records in, per-record placement out
        "k_group_emit": 52 * U + 20 * G,       # records, placement and rows in; member lists, per-record index and
                                               # row, groups out
        # global-table fallback
        "k_remap_insert": 8 * L, "k_assign_rank": 8 * U, "k_write_mapped": 8 * L, "k_count_show": 8 * L,
        "k_mask_insert": 16 * U, "k_mask_compact": 16 * G, "k_mask_fill": 32 * U,
        "k_group_insert": 16 * U,
        # table
        "k_probe": 8 * G + 4 * G,              # one stored-key compare per distinct sign, row number out
        "k_probe_recs": 8 * U + 8 * U + 4 * U, # the record's sign in, one stored-key compare, row number out
        "k_gather_vars": U * (2 * row + 4),    # row read + variable row write
        # push
        # the op's signs and labels, against the pull's copy of the signs (COPY) or its fingerprints of them
        "k_verify_values": (24 * L if name.endswith(", true>") else 16 * L + L // 32),
        "k_reset_counts": 8 * U,
        "k_apply_single": apply_bytes(shape["G1"], shape["G1"]),
        "k_apply_vec": apply_bytes(shape["Rm"], shape["Gm"]),
        "k_apply_big": apply_bytes(shape["Rb"], shape["Gb"]),
        "k_apply_big_adagrad": apply_bytes(shape["Rb"], shape["Gb"]),
        "k_apply_scalar": apply_bytes(U, G),
    }
    return table.get(name.split("<")[0], 0)


def batch_shape(values):
    """Sizes of one batch (torch on the GPU, harness only): see kernel_algorithmic_bytes."""
    import torch

    per_slot = [torch.unique(v) for v in values]
    _, k = torch.unique(torch.cat(per_slot), return_counts=True)
    # distinct (tile, slot, sign) triples: what the tiles of 2048 consecutive lookups hand on
    tile_recs, pos = 0, 0
    for v in values:
        tiles = (torch.arange(v.numel(), device=v.device) + pos) // 2048
        tile_recs += int(torch.unique(torch.stack([tiles, v], 1), dim=0).shape[0])
        pos += v.numel()
    mid = (k > 1) & (k < BIG_GROUP)
    big = k >= BIG_GROUP
    return {
        "L": sum(v.numel() for v in values), "U": sum(u.numel() for u in per_slot), "G": int(k.numel()),
        "T": tile_recs,
        "G1": int((k == 1).sum()), "Gm": int(mid.sum()), "Rm": int(k[mid].sum()),
        "Gb": int(big.sum()), "Rb": int(k[big].sum()),
    }


def populate(tn, handle, resident, dim):
    """Loads splitmix64(1..resident) with the synthetic snapshot rows."""
    from tensornet_amd import synth

    t0 = time.time()
    synth.populate_table(tn, handle, resident, dim)
    log("populated %d keys in %.1f s" % (resident, time.time() - t0))


def host_cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_baseline(cfg, values, grads_sigma):
    """Times the CPU oracle (the reference's data structures, one thread) on one
    full batch: pull op then push op.  The CPU table only holds the keys the batch
    touches (the host cannot hold the full resident set)."""
    import numpy as np

    from oracle import cpu as oracle
    from tensornet_amd import synth

    oracle.load(timed=True)  # the build with the reference's Release flags
    kinds = {"AdaGrad": oracle.ADAGRAD, "Adam": oracle.ADAM, "Ftrl": oracle.FTRL}
    dim = cfg["dim"]
    t = oracle.Table(kinds[cfg["opt"]], dim, buckets=15485863, **cfg["hyper"])
    signs = np.unique(np.concatenate(values).view(np.uint64))
    t.set_rows(signs, synth.snapshot_rows(signs, dim))
    L = sum(len(v) for v in values)
    vars_ = [np.zeros((len(v) + 1, dim), np.float32) for v in values]
    t0 = time.perf_counter()
    rc, mapped, counts = t.pull_op(values, vars_)
    t1 = time.perf_counter()
    assert rc == 0
    grads = synth.make_grads(counts, dim, grads_sigma)
    labels = synth.make_labels(values, 0)
    t2 = time.perf_counter()
    rc, _ = t.push_op(values, grads, labels)
    t3 = time.perf_counter()
    assert rc == 0
    secs = (t1 - t0) + (t3 - t2)
    log("cpu baseline: pull %.2f s, push %.2f s, %d lookups, %d rows" % (t1 - t0, t3 - t2, L, int(counts.sum())))
    from oracle import cpu as oracle_front

    return {
        "value": L / secs,
        "unit": "keys/s",
        "cores": 1,
        "threads": 1,
        "cpu_model": host_cpu_model(),
        "host_cores": os.cpu_count(),
        "flags": oracle_front.TIMED_FLAGS,
        "kind": "port",
        "sample": "1 full batch (%d lookups, %d per-slot distinct rows), pull op + push op, CPU table "
                  "pre-populated with only the %d keys the batch touches" % (L, int(counts.sum()), len(signs)),
        "pull_s": t1 - t0,
        "push_s": t3 - t2,
    }


# The other configurations the path is stated on: optimizers, dims and resident keys of the tables one step pulls
# from and pushes to (cfg4: the wide Ftrl weights and the deep AdaGrad embeddings of the same signs).
OTHER_TABLES = {
    "cfg1": [("AdaGrad", 8, dict(learning_rate=0.01, initial_g2sum=0.1, epsilon=1e-8))],
    "cfg2": [("Adam", 16, dict(learning_rate=1e-3, beta1=0.9, beta2=0.999, epsilon=1e-8))],
    "cfg4": [("Ftrl", 1, dict(learning_rate=0.05, beta=1.0, lambda1=1.0, lambda2=1.0)),
             ("AdaGrad", 64, dict(learning_rate=0.01, initial_g2sum=0.1, epsilon=1e-8))],
    "cfg5": [("AdaGrad", 16, dict(learning_rate=0.01, initial_g2sum=0.1, epsilon=1e-8))],
}


def other_config(tn, name, steps=10, warmup=2, small_path=True):
    """Pull + push steps of one of the other configurations at its stated shape and resident keys, each step on a
    seeded batch of its own (the new keys of a step are inserted inside it); the tables are given back afterwards."""
    import torch

    from tensornet_amd import synth

    cfg = synth.CONFIGS[name]
    rng = torch.Generator(device="cuda")
    rng.manual_seed(1)
    tables = []
    for opt_name, dim, hyper in OTHER_TABLES[name]:
        h = tn.core.create_sparse_table(getattr(tn.core, opt_name)(**hyper), "", dim, False, "")
        tn.core.reserve_sparse_table(h, int(cfg["resident"] * 1.02) + (1 << 22))
        tn.core.set_sparse_table_small_batch_path(h, small_path)
        synth.populate_table(tn, h, cfg["resident"], dim)
        tables.append((h, opt_name, dim))
    bound, Ls, Us = [], [], []
    for b in range(warmup + steps):
        hb = synth.make_batch(cfg, b)
        values = [torch.from_numpy(v).cuda() for v in hb]
        labels = [torch.from_numpy(l).cuda() for l in synth.make_labels(hb, b)]
        ops = []
        for h, opt_name, dim in tables:
            grads = [torch.randn((len(v), dim), device="cuda", generator=rng) * cfg["grad_sigma"] for v in values]
            vars_ = [torch.zeros((len(v) + 1, dim), device="cuda") for v in values]
            ops.append((tn.ops.BoundSparseTablePull(vars_, values, h), tn.ops.BoundSparseTablePush(values, grads, labels, h)))
        bound.append(ops)
        Ls.append(sum(v.numel() for v in values))
        Us.append(sum(int(torch.unique(v).numel()) for v in values))

    def step(i):
        for pull, push in bound[i]:
            pull()
            push()

    for i in range(warmup):
        step(i)
    for h, _, _ in tables:
        tn.ops.sparse_table_sync(h)
    torch.cuda.synchronize()
    keys_before = [tn.core.sparse_table_key_count(h) for h, _, _ in tables]
    t0 = time.perf_counter()
    for i in range(warmup, warmup + steps):
        step(i)
    for h, _, _ in tables:
        tn.ops.sparse_table_sync(h)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    new_keys = [tn.core.sparse_table_key_count(h) - k for (h, _, _), k in zip(tables, keys_before)]
    total_L = sum(Ls[warmup:])
    total_U = sum(Us[warmup:])
    alg = sum(step_algorithmic_bytes(opt_name, dim, total_L, total_U) for _, opt_name, dim in tables)
    for h, _, _ in tables:
        tn.core.clear_sparse_table(h)
    del bound
    torch.cuda.empty_cache()
    return {
        "tables": ["%s dim %d" % (o, d) for _, o, d in tables],
        "resident_keys": cfg["resident"],
        "lookups_per_step": total_L / steps,
        "ms_per_step": wall * 1e3 / steps,
        "keys_per_s": total_L / wall,
        "new_keys_per_step": new_keys[0] / steps,
        "step_frac_of_hbm_peak": alg / wall / HBM_PEAK,
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--config", default="cfg3")
    ap.add_argument("--resident", type=int, default=None, help="resident keys (default: the config's)")
    ap.add_argument("--profile-steps", type=int, default=8,
                    help="further steps, on batches of their own, run with HIP events around every launch")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-dense", action="store_true", help="skip the dense Adam side measurement")
    ap.add_argument("--no-combiner", action="store_true", help="skip the combiner side measurement")
    ap.add_argument("--no-traffic", action="store_true",
                    help="leave roofline.traffic out (development runs on kernels newer than the committed profile)")
    ap.add_argument("--no-fallback", action="store_true", help="skip the side measurement of a pull whose buckets overflow")
    ap.add_argument("--no-decay", action="store_true", help="skip the ShowDecay side measurement")
    ap.add_argument("--no-others", action="store_true",
                    help="skip the side measurement of the other configurations (cfg1, cfg2, cfg4, cfg5)")
    ap.add_argument("--detached-updates", action="store_true",
                    help="the timed steps with the push's update kernels detached (tn_sparse_table_set_detached_updates)")
    ap.add_argument("--detached", action="store_true", help="add the side measurement of detached updates")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU's share of the path; --gpus %d is not supported "
              "(every box has one GPU, nothing here uses collectives)" % args.gpus, file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch

    import tensornet_amd as tn
    from tensornet_amd import _lib, synth

    tn.load()
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(2)
    import tensornet_amd.ops  # noqa: F401

    torch.cuda.set_device(0)
    cfg = synth.CONFIGS[args.config]
    dim, opt_name = cfg["dim"], cfg["opt"]
    resident = args.resident if args.resident is not None else cfg["resident"]

    opt = getattr(tn.core, opt_name)(**cfg["hyper"])
    h = tn.core.create_sparse_table(opt, "bench", dim, False, "")
    tn.core.reserve_sparse_table(h, int(resident * 1.02) + 16 * 1024 * 1024)
    if args.detached_updates:
        tn.core.set_sparse_table_detached_updates(h, True)
    populate(tn, h, resident, dim)

    # ---- inputs, resident in HBM -------------------------------------------------
    # One seeded batch per step, none used twice: every step, timed or not, meets its own share of signs the
    # table does not hold yet (cfg3: the Zipf tail beyond the 5e8 resident ids, about 1 % of the lookups) and
    # inserts them inside the step (SparseKernelBlock::GetWeight, core/ps/optimizer/optimizer_kernel.h:299-308).
    psteps = max(1, min(args.profile_steps, args.steps))
    nb = args.warmup + args.steps + psteps
    rng = torch.Generator(device="cuda")
    rng.manual_seed(0)
    t_gen = time.time()
    host_batch0 = None
    batches = []
    for b in range(nb):
        hb = synth.make_batch(cfg, b)
        if b == 0:
            host_batch0 = hb
        values = [torch.from_numpy(v).cuda() for v in hb]
        labels = [torch.from_numpy(l).cuda() for l in synth.make_labels(hb, b)]
        # gradient matrices have one row per possible distinct sign; the op reads the first U_s
        grads = [torch.randn((len(v), dim), device="cuda", generator=rng) * cfg["grad_sigma"] for v in values]
        vars_ = [torch.zeros((len(v) + 1, dim), device="cuda") for v in values]
        batches.append((values, labels, grads, vars_))
    log("generated %d batches in %.1f s" % (nb, time.time() - t_gen))
    n_slots = len(batches[0][0])

    # The ops are bound to their tensors once, as an op kernel of a built graph is: the timed
    # region holds the calls through the C ABI, not Python's per-tensor argument marshalling.
    bound = [(tn.ops.BoundSparseTablePull(vars_, values, h), tn.ops.BoundSparseTablePush(values, grads, labels, h))
             for values, labels, grads, vars_ in batches]

    def step(i):
        pull, push = bound[i]
        pull()
        push()

    for i in range(args.warmup):
        step(i)
    tn.ops.sparse_table_sync(h)
    torch.cuda.synchronize()
    timed = range(args.warmup, args.warmup + args.steps)
    Ls = [sum(v.numel() for v in batches[i][0]) for i in timed]
    keys_before = tn.core.sparse_table_key_count(h)

    # ---- timed region ------------------------------------------------------------
    ev0 = torch.cuda.Event(enable_timing=True)
    ev1 = torch.cuda.Event(enable_timing=True)
    Us = []
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    ev0.record()
    for i in timed:
        step(i)
    ev1.record()
    tn.ops.sparse_table_sync(h)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / args.steps
    new_keys = tn.core.sparse_table_key_count(h) - keys_before
    # per-slot distinct signs of the timed batches: counted by torch on the device, after the clock has stopped
    Us = [sum(int(torch.unique(v).numel()) for v in batches[i][0]) for i in timed]
    total_L, total_U = sum(Ls), sum(Us)
    value = total_L / wall
    alg = step_algorithmic_bytes(opt_name, dim, total_L, total_U)
    log("timed %d steps: %.3f ms/step (events %.3f ms/step), %.3e keys/s, %.0f new keys per step" %
        (args.steps, ms_per_step, ev0.elapsed_time(ev1) / args.steps, value, new_keys / args.steps))

    # ---- per-kernel durations, HIP events around every launch --------------------
    lib = tn.load()
    lib.tn_profile_reset()
    lib.tn_profile_enable(1)
    prof_range = range(args.warmup + args.steps, nb)
    for i in prof_range:
        step(i)
    tn.ops.sparse_table_sync(h)
    torch.cuda.synchronize()
    lib.tn_profile_enable(0)
    prof = _lib.profile_summary()
    lib.tn_profile_reset()
    per_step = {k: (c / psteps, ms / psteps) for k, (c, ms) in prof.items()}
    kernel_ms = sum(ms for _, ms in per_step.values())
    # the dominant kernel: the one with the largest duration in the step
    shapes = [batch_shape(batches[i][0]) for i in list(prof_range)[:2]]
    G0 = shapes[0]["G"]
    mean_shape = {k: sum(sh[k] for sh in shapes) / len(shapes) for k in shapes[0]}
    dominant = max((kv for kv in per_step.items() if kernel_algorithmic_bytes(kv[0], opt_name, dim, mean_shape) > 0),
                   key=lambda kv: kv[1][1])
    dname, (dcount, dms) = dominant
    avg_launch_s = dms / dcount * 1e-3
    mean_L, mean_U = total_L / args.steps, total_U / args.steps
    dbytes = kernel_algorithmic_bytes(dname, opt_name, dim, mean_shape)
    achieved = dbytes / avg_launch_s
    for k, (c, ms) in sorted(per_step.items(), key=lambda kv: -kv[1][1]):
        log("  %-28s %5.1f launches/step %9.3f ms/step" % (k, c, ms))
    log("  sum of kernel time %.3f ms/step" % kernel_ms)

    # measured HBM traffic of the dominant kernel: from the committed profile of this workload (none of the others)
    traffic, traffic_source = (measured_traffic(per_step.keys())
                               if args.config == "cfg3" and resident == cfg["resident"] and not args.no_traffic
                               else (None, None))

    out = {
        "metric": "sparse pull+push keys/sec (dim16 AdaGrad); achieved HBM GB/s vs ~8 TB/s peak",
        "value": value,
        "unit": "keys/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": "%s: batch %d x %d slots, %s id lists, Zipf(%.2f) over %.0e vocab, dim %d %s, %d resident keys, "
                        "feature labels 1 on %.0f %% of the lookups"
                        % (args.config, cfg["batch"], cfg["slots"], cfg["lens"], cfg["zipf_s"], cfg["vocab"], dim,
                           opt_name, resident, 100 * synth.CLICK_RATE),
            "optimizer": opt_name,
            "dim": dim,
            "lookups_per_step": mean_L,
            "distinct_rows_per_step": mean_U,
            "globally_distinct_keys_of_a_batch": G0,
            "distinct_batches": nb,
            "new_keys_per_step": new_keys / args.steps,
            "push_updates": "detached" if args.detached_updates else "in the order of the caller's stream",
        },
        "rows_per_s": total_U / wall,
        "step_algorithmic_GBps": alg / wall / 1e9,
        "step_frac_of_hbm_peak": alg / wall / HBM_PEAK,
        "roofline": {
            "bound": "hbm",
            "kernel": dname,
            "achieved": achieved / 1e9,
            "peak": HBM_PEAK / 1e9,
            "unit": "GB/s",
            "frac": achieved / HBM_PEAK,
            "traffic": traffic.get(dname.split("<")[0]) if traffic else None,
            "traffic_source": traffic_source,
            "avg_launch_us": avg_launch_s * 1e6,
            "algorithmic_bytes_per_launch": dbytes,
        },
        "kernels_ms_per_step": {k: round(ms, 4) for k, (c, ms) in per_step.items()},
        "kernels_frac_of_hbm_peak": {
            k: round(kernel_algorithmic_bytes(k, opt_name, dim, mean_shape) / (ms / c * 1e-3) / HBM_PEAK, 4)
            for k, (c, ms) in per_step.items() if kernel_algorithmic_bytes(k, opt_name, dim, mean_shape) > 0},
        "side_stream_kernels": [k for k in per_step if k.startswith(SIDE_STREAM_KERNELS)],
        "batch_shape": mean_shape,
    }

    # ---- side measurement: a batch that overflows the buckets sized from the recent pulls ----------
    # A batch small enough for the path of few launches: the same steps once more on the path every other batch
    # takes (the library has a switch for that), to be quoted beside it.
    if any(k.startswith("k_small") for k in per_step):
        tn.core.set_sparse_table_small_batch_path(h, False)
        reps = [i for i in timed]
        for i in reps[:max(1, args.warmup)]:
            step(i)
        tn.ops.sparse_table_sync(h)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in reps:
            step(i)
        tn.ops.sparse_table_sync(h)
        torch.cuda.synchronize()
        other = (time.perf_counter() - t0) * 1e3 / len(reps)
        tn.core.set_sparse_table_small_batch_path(h, True)
        out["small_batch_path"] = {
            "what": "the timed steps ran on the path of few launches that small batches take; the same batches again "
                    "on the path every other batch takes",
            "ms_per_step": ms_per_step,
            "other_path_ms_per_step": other,
        }
        log("small-batch path %.4f ms/step, the other path %.4f ms/step" % (ms_per_step, other))

    # ---- side measurement: the same step with the push's update kernels detached from the caller's stream ------
    # (tn_sparse_table_set_detached_updates: they then run beside the analysis of the next pull's batch; the
    # gradient tensors must outlive the call, which is why the timed steps above do not use it.)  Batches of
    # their own again, so that the steps insert their share of new signs.
    if mean_L >= (3 << 20) and args.detached and not args.detached_updates:
        dsteps, dwarm = 10, 2
        more = []
        for b in range(nb + 2, nb + 2 + dwarm + dsteps):
            hb = synth.make_batch(cfg, b)
            values = [torch.from_numpy(v).cuda() for v in hb]
            labels = [torch.from_numpy(l).cuda() for l in synth.make_labels(hb, b)]
            grads = [torch.randn((len(v), dim), device="cuda", generator=rng) * cfg["grad_sigma"] for v in values]
            vars_ = [torch.zeros((len(v) + 1, dim), device="cuda") for v in values]
            more.append((tn.ops.BoundSparseTablePull(vars_, values, h),
                         tn.ops.BoundSparseTablePush(values, grads, labels, h), sum(v.numel() for v in values)))
        tn.core.set_sparse_table_detached_updates(h, True)
        for pull, push, _ in more[:dwarm]:
            pull()
            push()
        tn.ops.sparse_table_sync(h)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for pull, push, _ in more[dwarm:]:
            pull()
            push()
        tn.ops.sparse_table_sync(h)
        torch.cuda.synchronize()
        dwall = time.perf_counter() - t0
        tn.core.set_sparse_table_detached_updates(h, False)
        out["detached_updates"] = {
            "what": "the same step with tn_sparse_table_set_detached_updates: the push's update kernels run on the "
                    "table's own streams beside the analysis of the next pull's batch (the gradients must then stay "
                    "untouched until the table's next waiting call returns)",
            "steps": dsteps,
            "ms_per_step": dwall * 1e3 / dsteps,
            "keys_per_s": sum(n for _, _, n in more[dwarm:]) / dwall,
        }
        log("detached updates: %.4f ms/step" % (dwall * 1e3 / dsteps))
        del more

    # The second-level buckets follow the share of distinct records of the recent pulls.  A dozen pulls of a
    # batch that repeats a thousand signs shrink them; the next ordinary batch then overflows, and its pull is
    # repeated with buckets sized for a batch of distinct signs only.
    if not args.no_fallback:
        few = synth.splitmix64(np.arange(1, 1001, dtype=np.uint64)).view(np.int64)
        frng = np.random.default_rng(5)
        rep_values = [torch.from_numpy(few[frng.integers(0, len(few), v.numel())]).cuda() for v in batches[0][0]]
        rep_vars = [torch.zeros((v.numel() + 1, dim), device="cuda") for v in rep_values]
        rep_pull = tn.ops.BoundSparseTablePull(rep_vars, rep_values, h)
        fresh = []
        for b in (nb, nb + 1):
            hb = synth.make_batch(cfg, b)
            values = [torch.from_numpy(v).cuda() for v in hb]
            labels = [torch.from_numpy(l).cuda() for l in synth.make_labels(hb, b)]
            grads = [torch.randn((len(v), dim), device="cuda", generator=rng) * cfg["grad_sigma"] for v in values]
            vars_ = [torch.zeros((len(v) + 1, dim), device="cuda") for v in values]
            fresh.append((tn.ops.BoundSparseTablePull(vars_, values, h),
                          tn.ops.BoundSparseTablePush(values, grads, labels, h)))
        for _ in range(12):
            rep_pull()
        tn.ops.sparse_table_sync(h)
        torch.cuda.synchronize()
        times = []
        for pull, push in fresh:  # the first overflows and is redone, the second runs on worst-case buckets
            t0 = time.perf_counter()
            pull()
            t1 = time.perf_counter()
            push()
            tn.ops.sparse_table_sync(h)
            torch.cuda.synchronize()
            times.append((time.perf_counter() - t0) * 1e3)
            log("  pull %.3f ms, push %.3f ms" % ((t1 - t0) * 1e3, (time.perf_counter() - t1) * 1e3))
        out["fallback_step"] = {
            "what": "pull + push of an ordinary batch right after 12 pulls of a batch that repeats 1000 signs (buckets "
                    "sized for those overflow; the pull is redone with buckets sized for distinct signs only), and of "
                    "the batch after it; single steps, host waits included",
            "overflowing_step_ms": times[0],
            "step_after_ms": times[1],
            "ordinary_step_ms": ms_per_step,
        }
        log("fallback: overflowing step %.3f ms, the step after %.3f ms (ordinary %.3f ms)" % (times[0], times[1], ms_per_step))

    # ---- side measurement: the combiner around the ops on the device ---------------
    # pull -> embedding_lookup_sparse (mean) -> push of the pooled gradients, same batches
    if not args.no_combiner:
        crng = np.random.default_rng(0)
        cb = []
        for values, labels, grads, vars_ in batches[:4]:  # batches the table has seen: a side measurement
            ex = [torch.from_numpy(np.sort(crng.integers(0, cfg["batch"], v.numel()))).cuda() for v in values]
            pooled = [torch.randn((cfg["batch"], dim), device="cuda", generator=rng) * cfg["grad_sigma"] for _ in values]
            pull = tn.ops.BoundSparseTablePull(vars_, values, h)
            combine = tn.ops.BoundEmbeddingLookupSparse(vars_, pull.mapped, ex, cfg["batch"], h, "mean")
            push = tn.ops.BoundSparseTablePushPooled(values, ex, pooled, labels, h, "mean")
            cb.append((pull, combine, push))

        def cstep(i):
            pull, combine, push = cb[i % len(cb)]
            pull()
            combine()
            push()

        for i in range(2):
            cstep(i)
        tn.ops.sparse_table_sync(h)
        torch.cuda.synchronize()
        csteps = min(args.steps, 10)
        t0 = time.perf_counter()
        for i in range(csteps):
            cstep(i)
        tn.ops.sparse_table_sync(h)
        torch.cuda.synchronize()
        cms = (time.perf_counter() - t0) * 1e3 / csteps
        lib.tn_profile_reset()
        lib.tn_profile_enable(1)
        for i in range(csteps):
            cstep(i)
        tn.ops.sparse_table_sync(h)
        torch.cuda.synchronize()
        lib.tn_profile_enable(0)
        cprof = {k: ms / csteps for k, (c, ms) in _lib.profile_summary().items()}
        lib.tn_profile_reset()
        comb_bytes = {
            # signs' ids + example ids in, one output row per (slot, example) out, variable rows read once
            "k_combine_fwd": 16 * mean_L + 4 * dim * (cfg["batch"] * n_slots + mean_U),
            # example ids in, value out
            "k_lookup_keys": 16 * mean_L,
            # distinct index (twice: count, place) + value in, index + value out at their place in the sign's segment
            "k_place_lookups": 28 * mean_L,
            # index + value in, value out at its rank in the segment
            "k_rank_short": 20 * mean_L,
            # sorted values in, pooled rows read once, one reduced row per distinct sign out
            "k_reduce_pooled": 8 * mean_L + 4 * dim * (cfg["batch"] * n_slots + mean_U),
        }
        out["combiner_step"] = {
            "what": "pull + embedding_lookup_sparse(mean) + push of pooled gradients, same workload",
            "ms_per_step": cms,
            "keys_per_s": mean_L / (cms * 1e-3),
            "kernels_ms_per_step": {k: round(v, 4) for k, v in cprof.items()
                                    if k.startswith(("k_combine", "k_example", "k_lookup_keys", "k_place", "k_rank", "k_order", "k_reduce"))},
            "kernels_frac_of_hbm_peak": {k: round(comb_bytes[k.split("<")[0]] / (v * 1e-3) / HBM_PEAK, 4)
                                         for k, v in cprof.items() if k.split("<")[0] in comb_bytes},
        }
        log("combiner step: %.3f ms/step; %s" % (cms, out["combiner_step"]["kernels_ms_per_step"]))

    # ---- side measurement: ShowDecay, one streaming pass over the whole table -------
    if not args.no_decay:
        cap = tn.core.sparse_table_capacity(h)
        keys_now = tn.core.sparse_table_key_count(h)
        tn.core.show_decay(h, 1)
        torch.cuda.synchronize()
        d0 = torch.cuda.Event(enable_timing=True)
        d1 = torch.cuda.Event(enable_timing=True)
        d0.record()
        for _ in range(3):
            tn.core.show_decay(h, 1)
        d1.record()
        torch.cuda.synchronize()
        dms = d0.elapsed_time(d1) / 3
        # every slot's key is read; a resident row's state (16 B for AdaGrad) is read and written
        dbytes_decay = 8 * cap + 32 * keys_now
        out["show_decay"] = {
            "slots": cap, "resident_keys": keys_now, "ms": dms,
            "algorithmic_GBps": dbytes_decay / (dms * 1e-3) / 1e9,
            "frac_of_hbm_peak": dbytes_decay / (dms * 1e-3) / HBM_PEAK,
        }
        log("show_decay over %d slots: %.2f ms" % (cap, dms))

    # ---- dense Adam side measurement (cfg5's flat array) --------------------------
    if not args.no_dense:
        total = synth.CONFIGS["cfg5"]["dense_total"]
        dh = tn.core.create_dense_table(tn.core.Adam(learning_rate=1e-3, beta1=0.9, beta2=0.999))
        w = (torch.rand(total, device="cuda") - 0.5) * 0.1
        g = torch.randn(total, device="cuda") * 1e-4
        tn.ops.dense_table_init([w], dh)
        for _ in range(3):
            tn.ops.dense_table_push_pull([w], [g], 1e-3, dh)
        torch.cuda.synchronize()
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(20):
            tn.ops.dense_table_push_pull([w], [g], 1e-3, dh)
        e1.record()
        torch.cuda.synchronize()
        dsec = e0.elapsed_time(e1) / 20 * 1e-3
        out["dense_adam"] = {
            "params": total,
            "ms_per_step": dsec * 1e3,
            "algorithmic_GBps": 28 * total / dsec / 1e9,  # read g,w,m,v ; write w,m,v
            "frac_of_hbm_peak": 28 * total / dsec / HBM_PEAK,
            # with the new weights also written back into the op's variable (the pull half of the op),
            # which is what FETCH_SIZE / WRITE_SIZE show for the kernel: 16 B read, 16 B written per parameter
            "hbm_traffic_GBps": 32 * total / dsec / 1e9,
            "traffic_frac_of_hbm_peak": 32 * total / dsec / HBM_PEAK,
        }
        # the same array under dense AdaGrad: g, w, d2sum, g2sum, m read; w, d2sum, g2sum, m written (+ the variable)
        gh = tn.core.create_dense_table(tn.core.AdaGrad(learning_rate=1e-3, initial_g2sum=0.1))
        tn.ops.dense_table_init([w], gh)
        for _ in range(3):
            tn.ops.dense_table_push_pull([w], [g], 1e-3, gh)
        torch.cuda.synchronize()
        e0.record()
        for _ in range(20):
            tn.ops.dense_table_push_pull([w], [g], 1e-3, gh)
        e1.record()
        torch.cuda.synchronize()
        gsec = e0.elapsed_time(e1) / 20 * 1e-3
        out["dense_adagrad"] = {
            "params": total,
            "ms_per_step": gsec * 1e3,
            "algorithmic_GBps": 36 * total / gsec / 1e9,
            "frac_of_hbm_peak": 36 * total / gsec / HBM_PEAK,
            "hbm_traffic_GBps": 40 * total / gsec / 1e9,
            "traffic_frac_of_hbm_peak": 40 * total / gsec / HBM_PEAK,
        }
        del w, g

    # ---- side measurement: the other configurations, on tables of their own ---------------------------
    if args.config == "cfg3" and not args.no_others:
        del bound, batches
        tn.core.clear_sparse_table(h)  # (cfg5's table takes 176 GB)
        torch.cuda.empty_cache()
        others = {}
        for name in ("cfg1", "cfg2", "cfg4", "cfg5"):
            t_cfg = time.time()
            others[name] = other_config(tn, name)
            if name in ("cfg1", "cfg2"):  # small enough for the path of few launches: the other path beside it
                others[name]["other_path_ms_per_step"] = other_config(tn, name, small_path=False)["ms_per_step"]
            log("%s: %.4f ms/step, %.3e keys/s, %.0f new keys per step, %.3f of the HBM roofline (%.1f s)" %
                (name, others[name]["ms_per_step"], others[name]["keys_per_s"], others[name]["new_keys_per_step"],
                 others[name]["step_frac_of_hbm_peak"], time.time() - t_cfg))
        if "dense_adam" in out:  # cfg5's step also applies the dense Adam update measured above
            others["cfg5"]["with_dense_adam_ms_per_step"] = others["cfg5"]["ms_per_step"] + out["dense_adam"]["ms_per_step"]
        out["other_configs"] = others

    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(cfg, host_batch0, cfg["grad_sigma"])
    else:
        out["cpu_baseline"] = None
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
