#!/usr/bin/env python3
"""Benchmark of the MASCOT SGD hot path on one MI355X.

A step is one epoch of the product's own training driver (mf_session_epoch: the update launches of
`quantized_mf -synth 4 -v 1 -k 128 -ug 100 -ig 100 -s 0.05 -it 2 -e 20 -l 50`, error estimate and precision
switching included as the epochs reach them) over the seeded synthetic stand-in of BASELINE.json's fourth
configuration: 480,000 x 17,800, 100M training ratings (user Zipf(0.8), item Zipf(1.1), integers 1-5 from a rank-32
truth plus N(0,0.9) noise), generated on the device by mf_generate_ratings -- the ratings the command line, the
full-size tests and the committed CPU reference curve (tests/golden/) use.  The ratings and the model are resident in
HBM before the timed region.  `value` counts the time of the update launches (hipEvent, as the driver reports it
and as the reference times its kernels, mf_methods.cu:187-241); every row update is carried out.  Everything goes
through the C ABI of libmascot_hip.so.  One JSON line on stdout.
"""
import argparse
import ctypes as C
import glob
import hashlib
import importlib
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
PEAK_HBM_GBS = 8000.0
TRAIN = dict(epochs=50, lr=0.01, decay=0.1, lam=0.015, sample_ratio=0.05, interval=2, ug=100, ig=100, threshold=20.0)
# rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of a plain epoch's update kernels, recorded with the workload and the digest of
# the kernel sources they were taken with; reported only for that workload and those sources
PROFILED_TRAFFIC = os.path.join(ROOT, "profiles", "hogwild_mascot_k128_config4_hbm_traffic.json")
KERNEL_SOURCES = os.path.join(ROOT, "icdm-2021_mascot_amd", "csrc")


def kernel_sources_digest():
    """sha256 over the sources of the library (file names and contents, in name order): the kernels, and the host code
    whose defaults decide how rows are treated."""
    h = hashlib.sha256()
    for name in sorted(os.listdir(KERNEL_SOURCES)):
        if name.endswith((".h", ".hip", ".cpp")):
            h.update(name.encode())
            with open(os.path.join(KERNEL_SOURCES, name), "rb") as f:
                h.update(f.read())
    return h.hexdigest()


def profiled_traffic(config, n_train, k, seed, workers):
    """The committed HBM-side bytes per plain epoch of this workload, or None when the record is of another workload or
    of other kernel sources than the ones this library was built from."""
    try:
        rec = json.load(open(PROFILED_TRAFFIC))
    except (OSError, ValueError):
        return None
    same = (rec.get("config"), rec.get("n_train"), rec.get("k"), rec.get("seed"), rec.get("workers")) == (config, n_train, k, seed, workers)
    if not same or rec.get("kernel_sources_sha256") != kernel_sources_digest():
        return None
    return rec


def generate(h, config, seed, n_train, n_test):
    """The first n_train + n_test ratings of the configuration's stream, split as the command line does; the test set
    goes through the reference's test-set rules (unseen users / items dropped, (user, item) order, io_utils.h:183-198)."""
    cfg = h.synth_config(config)
    node = importlib.import_module("icdm-2021_mascot_amd.capi").NODE
    allr = np.empty(n_train + n_test, node)
    h.mf_generate_ratings_host(C.addressof(cfg), seed, 0, allr.size, allr.ctypes.data)
    train, test = allr[:n_train], allr[n_train:]
    seen_u = np.zeros(cfg.n_users, bool); seen_u[train["u"]] = True
    seen_i = np.zeros(cfg.n_items, bool); seen_i[train["i"]] = True
    test = test[seen_u[test["u"]] & seen_i[test["i"]]]
    key = test["u"].astype(np.int64) * (1 << 32) + test["i"].astype(np.int64)
    order = np.argsort(key, kind="stable")
    test, key = test[order], key[order]
    last = np.ones(test.size, bool)
    last[:-1] = key[1:] != key[:-1]
    return cfg, np.ascontiguousarray(train), np.ascontiguousarray(test[last])


def params(h, a, version, **kw):
    args = dict(k=a.k, num_workers=a.workers, epoch=TRAIN["epochs"], learning_rate=TRAIN["lr"], lam=TRAIN["lam"], decay=TRAIN["decay"],
                version=version, seed=a.seed, user_group_num=TRAIN["ug"], item_group_num=TRAIN["ig"], sample_ratio=TRAIN["sample_ratio"],
                interval=TRAIN["interval"], error_threshold=TRAIN["threshold"])
    args.update(kw)
    return h.default_params(**args)


def run_session(torch, capi, h, prm, cfg, train, test, seed, warmup, steps, run_to=0, half_init=False):
    """W untimed epochs, K timed ones (wall clock bracketed by synchronisations; per epoch the driver's hipEvent time of
    its update launches), then untimed on to `run_to` epochs.  Returns the figures and the still open session."""
    p, q = h.init_model(cfg.n_users, cfg.n_items, prm.k, seed, half_init)
    s = capi.Session(h, prm, train, cfg.n_users, cfg.n_items, test, p, q)
    rmse, ms, prec = [], [], []

    def epoch():
        # the precision of every group while this epoch's updates run (switching comes after them)
        prec.append((s.groups(0)[0], s.groups(1)[0]))
        r, m = s.epoch(); rmse.append(r); ms.append(m)
    for _ in range(warmup):
        epoch()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        epoch()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    while s.epochs_done < run_to:
        epoch()
    return dict(session=s, rmse=rmse, ms=ms, wall_s=wall, timed=ms[warmup:warmup + steps], prec=prec)


def epoch_bytes(k, updates, prec, ratings):
    """Algorithmic bytes of one MASCOT epoch: every update reads 12 bytes of rating and reads and writes one row per side,
    2 k bytes for a binary16 row and 4 k for a binary32 one (mascot_sgd_kernel.h:188-443, the four cases).  The case of
    an update follows from the groups of its two rows, so the sum over the epoch's updates is, per side, the share of
    the ratings that falls on binary32 groups.  Returns (bytes, user share, item share)."""
    share = []
    for side in (0, 1):
        r = ratings[side].astype(np.float64)
        share.append(float((r * (prec[side] != 0)).sum() / r.sum()) if r.size else 0.0)
    per_update = 12 + 2 * k * (2 + 2 * share[0]) + 2 * k * (2 + 2 * share[1])
    return updates * per_update, share[0], share[1]


def is_check_epoch(e):
    return e >= 5 and e % TRAIN["interval"] == 5 % TRAIN["interval"] and e != TRAIN["epochs"] - 1


def reference_curve(config, n_train, k, seed, version=1):
    """Per-epoch test RMSE of the reference rule on the CPU (tests/golden/make_reference_curve.py): mean and spread of the
    committed runs of this workload, or None."""
    runs = []
    for path in sorted(glob.glob(os.path.join(ROOT, "tests", "golden", "reference_curve_config%d*_run*.json" % config))):
        d = json.load(open(path))
        if d["n_train"] == n_train and d["train"]["k"] == k and d["seed"] == seed and d["scale"] == 1.0 and d.get("version", 1) == version:
            runs.append(d)
    if not runs:
        return None
    epochs = min(len(d["test_rmse"]) for d in runs)
    curves = np.array([d["test_rmse"][:epochs] for d in runs])
    return dict(mean=curves.mean(0), spread=curves.max(0) - curves.min(0), runs=len(runs), threads=runs[0]["threads"], workers=runs[0]["workers"],
                user_groups_binary32=[d.get("user_groups_binary32") for d in runs] if "user_groups_binary32" in runs[0] else None,
                item_groups_binary32=[d.get("item_groups_binary32") for d in runs] if "item_groups_binary32" in runs[0] else None)


def probe_ms(torch, h, sess, n, n_users, n_items, row_bytes, workers, seed, epoch, reps=3, item_row_bytes=0):
    """mf_row_traffic_probe on the session's ratings and launch options: the epoch's memory traffic without the arithmetic."""
    dev = torch.device("cuda:0")
    item_row_bytes = item_row_bytes or row_bytes
    P = torch.zeros(n_users * row_bytes, dtype=torch.uint8, device=dev)
    Q = torch.zeros(n_items * item_row_bytes, dtype=torch.uint8, device=dev)
    r_ptr, o_ptr = sess.device_state(epoch)
    st = torch.cuda.current_stream().cuda_stream
    run = lambda: h.mf_row_traffic_probe_sides(r_ptr, n, P.data_ptr(), Q.data_ptr(), row_bytes, item_row_bytes, workers, seed, st, o_ptr)
    run(); torch.cuda.synchronize()
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(reps)]
    for x, y in ev:
        x.record(); run(); y.record()
    torch.cuda.synchronize()
    return float(np.mean([x.elapsed_time(y) for x, y in ev]))


def cpu_baseline(cfg, train, k, seed, threads, sample):
    """The checker's MASCOT epoch (reference update rule, binary16 through F16C) as an OpenMP Hogwild loop over the first
    `sample` training ratings: its own shuffle, histogram, sort, grouping and re-index, then one timed epoch."""
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import mfutil
    from oracle import oracle as om
    orc = om.get()
    R = np.ascontiguousarray(train[:sample])
    Rs = orc.shuffle(seed, R)
    ucnt, icnt = orc.histogram(Rs, cfg.n_users, cfg.n_items)
    suc, sui = orc.sort_by_count(ucnt)
    sic, sii = orc.sort_by_count(icnt)
    uend, iend = orc.grouping(suc, TRAIN["ug"]), orc.grouping(sic, TRAIN["ig"])
    u2s, _, _ = orc.reindex_tables(sui, uend)
    i2s, _, _ = orc.reindex_tables(sii, iend)
    orc.lib.orc_reindex(Rs.ctypes.data, Rs.size, u2s.ctypes.data, i2s.ctypes.data)
    P = orc.init_normal(seed, 0, cfg.n_users * k).reshape(cfg.n_users, k)
    Q = orc.init_normal(seed, 1, cfg.n_items * k).reshape(cfg.n_items, k)
    Ps = np.empty_like(P); Ps[u2s] = P
    Qs = np.empty_like(Q); Qs[i2s] = Q
    gu = mfutil.host_grouped(orc, k, Ps, uend, np.zeros(uend.size, np.uint8))
    gi = mfutil.host_grouped(orc, k, Qs, iend, np.zeros(iend.size, np.uint8))
    W = threads * 8
    uc = orc.lib.orc_update_count(Rs.size, W, 128)
    z = [np.zeros(m, np.float32) for m in (gu.groups * k, gi.groups * k, gu.groups, gi.groups)]
    t0 = time.perf_counter()
    orc.lib.orc_mascot_epoch(k, Rs.ctypes.data, Rs.size, gu.ptrs, gi.ptrs, gu.end_idx.ctypes.data, gi.end_idx.ctypes.data,
                             gu.prec.ctypes.data, gi.prec.ctypes.data, gu.groups, gi.groups, W, uc, 128, TRAIN["lr"], TRAIN["lam"], uc * 128,
                             z[0].ctypes.data, z[1].ctypes.data, z[2].ctypes.data, z[3].ctypes.data, seed, 0, None, threads)
    dt = time.perf_counter() - t0
    done = W * uc * 128
    return done / dt, done, dt


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--config", type=int, default=4, choices=(2, 3, 4, 5), help="BASELINE.json configuration (4 = the one the metric is quoted on)")
    ap.add_argument("--ratings", type=int, default=0, help="training ratings (default: the configuration's; the test set is scaled alike)")
    ap.add_argument("--k", type=int, default=128, choices=(64, 128))
    ap.add_argument("--workers", type=int, default=0, help="-wg (default 0: mf_auto_workers(ratings); 48832 at config 4)")
    ap.add_argument("--seed", type=int, default=2021)
    ap.add_argument("--replicate", type=float, default=-1.0, help="mf_params.replicate_inflight (default: derived from learning rate and mean rating)")
    ap.add_argument("--merges", type=int, default=0, help="mf_params.replica_merges (default: the library's)")
    ap.add_argument("--step-epochs", type=int, default=-1, help="mf_params.replica_step_epochs (default: the library's 1; 0 = every epoch)")
    ap.add_argument("--replicate-late", type=float, default=-1.0, help="mf_params.replicate_inflight_late (default: a quarter of --replicate's value; 0 = the same bar throughout)")
    ap.add_argument("--late-from", type=int, default=-1, help="mf_params.replicate_late_from (default: the library's 1, the second epoch)")
    ap.add_argument("--early", type=float, default=-1.0, help="mf_params.early_inflight: fraction of the updates in flight during the first epoch (default: the library's 0.5; 1 = off)")
    ap.add_argument("--step-scale", type=float, default=-1.0, help="mf_params.replica_step_scale (default: the library's; 0 = unscaled steps on replicated rows)")
    ap.add_argument("--thin", type=float, default=0.0, help="mf_params.hot_row_inflight: opt-in thinning of hot rows (0 = every update carried out)")
    ap.add_argument("--cpu-updates", type=int, default=32_000_000, help="size of the CPU baseline sample (about 10 s on 16 threads)")
    ap.add_argument("--skip-cpu", action="store_true")
    ap.add_argument("--skip-fp32", action="store_true", help="skip the fp32-SGD leg")
    ap.add_argument("--skip-ceiling", action="store_true", help="skip the access-pattern probe")
    ap.add_argument("--skip-full-run", action="store_true", help="stop after the timed epochs instead of running on to epoch 50")
    ap.add_argument("--skip-reference-semantics", action="store_true", help="skip the two epochs without hot rows (-hot 0: every row stored, last writer wins; 0.25 s per epoch)")
    ap.add_argument("--every-rule", action="store_true", help="also run MPT, MuPPET, AFP and binary16 storage (-v 4, 3, 2, 7) for eight epochs each")
    ap.add_argument("--rules", default="mpt,muppet,afp,mem_quant", help="the rules --every-rule runs")
    ap.add_argument("--pmc-copy", action="store_true", help="profiling aid: also run three 1 GiB device copies, the known-size kernel that FETCH_SIZE / WRITE_SIZE are scaled by")
    ap.add_argument("--only-timed", action="store_true", help="profiling aid: the MASCOT warm-up and timed epochs only")
    a = ap.parse_args()
    if a.gpus != 1:
        print("bench.py: this build runs on one GPU only (one process, one device; sharding over several GPUs is a design "
              "note, not code); run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    if a.warmup + a.steps > TRAIN["epochs"]:
        print("bench.py: warmup + steps is at most %d, the epochs of the configured run" % TRAIN["epochs"], file=sys.stderr)
        sys.exit(2)
    if a.only_timed:
        a.skip_cpu = a.skip_fp32 = a.skip_ceiling = a.skip_full_run = a.skip_reference_semantics = True
    import torch
    capi = importlib.import_module("icdm-2021_mascot_amd.capi")
    h = importlib.import_module("icdm-2021_mascot_amd").load()
    torch.cuda.init()
    t0 = time.perf_counter()
    preset = h.synth_config(a.config)
    n_train = a.ratings or preset.n_train
    n_test = int(preset.n_test * n_train / preset.n_train)
    cfg, train, test = generate(h, a.config, a.seed, n_train, n_test)
    k = a.k
    yahoo = 1 if a.config == 5 else 0       # 0..100 ratings already mapped to r/25+1 by the generator; MuPPET starts at 12 bit
    extra = dict(replicate_inflight=a.replicate, hot_row_inflight=a.thin, is_yahoo=yahoo)
    if a.merges:
        extra["replica_merges"] = a.merges
    if a.step_scale >= 0:
        extra["replica_step_scale"] = a.step_scale
    if a.step_epochs >= 0:
        extra["replica_step_epochs"] = a.step_epochs
    if a.replicate_late >= 0:
        extra["replicate_inflight_late"] = a.replicate_late
    if a.late_from >= 0:
        extra["replicate_late_from"] = a.late_from
    if a.early >= 0:
        extra["early_inflight"] = a.early
    if a.pmc_copy:
        src = torch.empty(1 << 28, dtype=torch.float32, device="cuda").normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    prm = params(h, a, 1, **extra)
    run_to = 0 if a.skip_full_run else TRAIN["epochs"]
    main_run = run_session(torch, capi, h, prm, cfg, train, test, a.seed, a.warmup, a.steps, run_to)
    sess = main_run["session"]
    setup_s = time.perf_counter() - t0
    W = sess.workers
    rep_u, rep_v, inflight = sess.hot_rows()
    replicate_bar = float(h.mf_replicate_threshold(TRAIN["lr"], float(np.abs(train["r"][:4_000_000]).mean()))) if a.replicate < 0 else a.replicate
    uc = h.mf_update_count(n_train, W, 128)
    updates = W * uc * 128
    timed = np.array(main_run["timed"], np.float64)
    ms = float(timed.mean())
    # a rating reads 12 B and one row per side and writes both rows back: 12 + 2 k (s_user + s_item) bytes, s = 2 for a
    # binary16 row and 4 for a binary32 one; per epoch the sum over its updates follows from the precision of the groups
    # during that epoch and the ratings that fall on each group (epoch_bytes)
    group_ratings = (sess.groups(0)[1], sess.groups(1)[1])
    per_epoch = [epoch_bytes(k, updates, pr, group_ratings) for pr in main_run["prec"]]
    timed_bytes = float(np.mean([b for b, _, _ in per_epoch[a.warmup:a.warmup + a.steps]]))
    bytes_per_update = timed_bytes / updates
    gbs = timed_bytes / (ms / 1e3) / 1e9
    epochs_done_timed = a.warmup + a.steps
    launches = capi.HogwildOptions.from_address(sess.device_state(a.warmup)[1]).launches or 1
    plain = [m for i, m in enumerate(main_run["timed"]) if not is_check_epoch(a.warmup + i)] or list(main_run["timed"])
    out = {
        "metric": "SGD ratings/sec/epoch & % HBM roofline at k=128 on 1 MI355X; test RMSE delta",
        "value": n_train / (ms / 1e3), "unit": "ratings/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16", "data": "synthetic",
        "config": {"workload": "config %d: %d users x %d items, user Zipf(%.1f), item Zipf(%.1f), %d train / %d test ratings from mf_generate_ratings; "
                               "mf_train -v 1 -k %d -ug 100 -ig 100 -s 0.05 -it 2 -e 20 -l 50 -a 0.01 -d 0.1, one epoch per step"
                               % (a.config, cfg.n_users, cfg.n_items, cfg.user_alpha, cfg.item_alpha, train.size, test.size, k),
                   "workers": W, "row_access": "device-coherent stores; rows with several updates in flight: added in memory, or one copy per XCD",
                   "update_vector_size": 128, "epochs_timed": "%d..%d of 50" % (a.warmup, a.warmup + a.steps - 1), "seed": a.seed,
                   "row_updates_carried_out": 1.0 if a.thin == 0 else None,
                   "updates_in_flight": inflight, "replicated_rows": {"user": rep_u, "item": rep_v},
                   "replicate_above_in_flight": {"epochs_before": prm.replicate_late_from, "bar": replicate_bar,
                                                 "later_bar": (replicate_bar / 4.0 if prm.replicate_inflight_late < 0 else (prm.replicate_inflight_late or replicate_bar))},
                   "first_epochs": {"epochs": prm.early_inflight_epochs, "updates_in_flight_fraction": prm.early_inflight, "replica_step_scale": "library default" if a.step_scale < 0 else a.step_scale},
                   "setup_s": round(setup_s, 1)},
        "roofline": {"bound": "hbm", "achieved": gbs, "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": gbs / PEAK_HBM_GBS,
                     "note": "algorithmic bytes: every update reads and writes both rows (12 + 2k(s_user + s_item) bytes, s = 2 for a binary16 "
                             "and 4 for a binary32 row, summed over the epoch's updates by the precision of their groups; 1036 B while "
                             "every group is binary16).  Rows that are re-used while they sit in an L2 never reach HBM, so `frac` is the "
                             "rate the update stream is served at over the HBM peak, not HBM utilisation: the profiled HBM-side share is "
                             "`hbm_side.frac`",
                     "traffic": None,
                     "kernel": "hogwild_kernel<MascotRuleT<%d,true,false,false>,true>" % k,
                     "bytes_per_update": bytes_per_update, "updates_per_step": updates,
                     "kernel_launches_per_step": launches,
                     "per": "step: achieved, traffic and updates are those of one epoch = the driver's update call, which cuts the epoch into "
                            "kernel_launches_per_step launches of this kernel with the replica averaging between them; the time is the driver's "
                            "hipEvent time around that call on its stream (check epochs add the sampled launch)"},
        "ms_steps": [round(float(x), 3) for x in timed],
        "epoch_wall_ms": main_run["wall_s"] * 1e3 / a.steps,
        "plain_epoch_ms": float(np.mean(plain)),
        "test_rmse_after_timed_epochs": {"value": main_run["rmse"][epochs_done_timed - 1], "epochs": epochs_done_timed, "test_ratings": int(test.size)},
        "test_rmse_per_epoch": [round(float(x), 5) for x in main_run["rmse"]],
    }
    traffic = profiled_traffic(a.config, n_train, k, a.seed, W)
    if traffic is not None and a.replicate < 0 and a.thin == 0 and a.step_scale < 0 and a.step_epochs < 0 and not a.merges \
            and a.replicate_late < 0 and a.late_from < 0 and a.early < 0:
        out["roofline"]["traffic"] = traffic["bytes_per_epoch"]
        out["roofline"]["traffic_source"] = traffic["source"]
        out["roofline"]["hbm_side"] = {"frac": traffic["bytes_per_epoch"] / (float(np.mean(plain)) / 1e3) / 1e9 / PEAK_HBM_GBS,
                                       "note": "profiled HBM bytes of a plain all-binary16 epoch (FETCH_SIZE + WRITE_SIZE, not re-measured by this run) "
                                               "over this run's mean plain epoch, against the 8 TB/s peak: algorithmic %.2f / HBM-side %.2f"
                                               % (gbs / PEAK_HBM_GBS, traffic["bytes_per_epoch"] / (float(np.mean(plain)) / 1e3) / 1e9 / PEAK_HBM_GBS)}
    ref = reference_curve(a.config, n_train, k, a.seed)
    if ref is not None:
        def delta(epochs):
            i = epochs - 1
            return {"value": main_run["rmse"][i] - float(ref["mean"][i]), "epochs": epochs, "test_rmse": main_run["rmse"][i],
                    "reference_rule_test_rmse": float(ref["mean"][i]), "reference_runs": ref["runs"], "reference_spread": float(ref["spread"][i])}
        if epochs_done_timed <= len(ref["mean"]):
            out["test_rmse_delta"] = delta(epochs_done_timed)
            out["test_rmse_delta"]["source"] = ("reference update rule on the CPU (checker under oracle/, %d host threads racing over the windows of %d workers), "
                                                "curves committed under tests/golden/" % (ref["threads"], ref["workers"]))
        if len(main_run["rmse"]) >= TRAIN["epochs"] and len(ref["mean"]) >= TRAIN["epochs"]:
            out["test_rmse_delta_epoch50"] = delta(TRAIN["epochs"])
            worst = int(np.argmax(np.abs(np.array(main_run["rmse"][:len(ref["mean"])]) - ref["mean"][:len(main_run["rmse"])])))
            out["test_rmse_delta_largest"] = delta(worst + 1)
    if len(main_run["rmse"]) >= TRAIN["epochs"]:
        rep = sess.report
        out["whole_job"] = {"note": "the 50-epoch run this session ended up being: update launches of all epochs, switching included",
                            "epochs": TRAIN["epochs"], "sgd_ms_total": float(np.sum(main_run["ms"])), "sgd_ms_per_epoch": float(np.mean(main_run["ms"])),
                            "sgd_ms_epochs": [round(float(x), 2) for x in main_run["ms"]],
                            "ratings_per_s": n_train * TRAIN["epochs"] / (float(np.sum(main_run["ms"])) / 1e3),
                            "preprocess_ms": rep.preprocess_ms, "error_ms": rep.error_ms, "switching_ms": rep.switching_ms,
                            "final_test_rmse": main_run["rmse"][-1],
                            # the four precision cases per epoch: groups in binary32 while the epoch ran, the share of the
                            # ratings on them, and the algorithmic bytes that follow (epoch_bytes)
                            "user_groups_binary32": [int(pu.sum()) for pu, _ in main_run["prec"]],
                            "item_groups_binary32": [int(pi.sum()) for _, pi in main_run["prec"]],
                            "groups": {"user": int(group_ratings[0].size), "item": int(group_ratings[1].size)},
                            "ratings_on_binary32_user_rows": [round(su, 4) for _, su, _ in per_epoch],
                            "ratings_on_binary32_item_rows": [round(si, 4) for _, _, si in per_epoch],
                            "algorithmic_gb_epochs": [round(b / 1e9, 2) for b, _, _ in per_epoch],
                            "roofline_frac_epochs": [round(b / (m / 1e3) / 1e9 / PEAK_HBM_GBS, 3) for (b, _, _), m in zip(per_epoch, main_run["ms"])],
                            "roofline_frac": float(sum(b for b, _, _ in per_epoch) / (float(np.sum(main_run["ms"])) / 1e3) / 1e9 / PEAK_HBM_GBS)}
        if ref is not None and ref.get("user_groups_binary32") is not None:
            out["whole_job"]["reference_rule_groups_binary32_after_50_epochs"] = {"user": ref["user_groups_binary32"], "item": ref["item_groups_binary32"]}
    if not a.skip_ceiling:
        ceil_ms = probe_ms(torch, h, sess, n_train, cfg.n_users, cfg.n_items, k * 2, W, a.seed, a.warmup)
        out["roofline"]["access_pattern_ceiling"] = {
            "note": "mf_row_traffic_probe: the same ratings, workers, hot-row tables, replicas and store policy, rows read and written "
                    "back without the arithmetic, one launch; kernel_vs_ceiling = this time / mean plain epoch",
            "ms": ceil_ms, "plain_epoch_ms": float(np.mean(plain)), "kernel_vs_ceiling": ceil_ms / float(np.mean(plain))}
    sess.close()
    del main_run["session"]

    def side_leg(version, epochs_w, epochs_k, note, half_init=False, **kw):
        e = dict(extra); e.update(kw)
        r = run_session(torch, capi, h, params(h, a, version, **e), cfg, train, test, a.seed, epochs_w, epochs_k, 0, half_init)
        s2 = r.pop("session")
        row = k * (2 if version in (1, 7) else 4)
        leg_ms = float(np.mean(r["timed"]))
        probe = None if a.skip_ceiling else probe_ms(torch, h, s2, n_train, cfg.n_users, cfg.n_items, row, s2.workers, a.seed, epochs_w)
        s2.close()
        res = {"note": note, "value": n_train / (leg_ms / 1e3), "unit": "ratings/s", "ms_per_step": leg_ms, "workers": W,
               "roofline_frac": updates * (12 + 4 * row) / (leg_ms / 1e3) / 1e9 / PEAK_HBM_GBS,
               "test_rmse_after_timed_epochs": r["rmse"][-1], "epochs": epochs_w + epochs_k, "test_rmse_per_epoch": [round(float(x), 5) for x in r["rmse"]]}
        if probe is not None:
            res["access_pattern_ceiling_ms"] = probe
        return res

    def switched_leg():
        """MASCOT epochs with every group of both sides promoted to binary32 after two binary16 epochs: the update kernel
        on the bytes of the fp32 rule (2060 B per update at k = 128)."""
        r = run_session(torch, capi, h, params(h, a, 1, **dict(extra, interval=0)), cfg, train, test, a.seed, 2, 0, 0)
        s2 = r.pop("session")
        for side in (0, 1):
            s2.promote_groups(side, np.ones(s2.groups(side)[0].size, np.uint8))
        t = [s2.epoch() for _ in range(4)]
        probe = None if a.skip_ceiling else probe_ms(torch, h, s2, n_train, cfg.n_users, cfg.n_items, k * 4, s2.workers, a.seed, 2)
        s2.close()
        leg_ms = float(np.mean([m for _, m in t[1:]]))
        res = {"note": "mf_train -v 1 with every group promoted to binary32 (mf_session_promote_groups) after epoch 2; epochs 4..6",
               "ms_per_step": leg_ms, "value": n_train / (leg_ms / 1e3), "unit": "ratings/s",
               "roofline_frac": updates * (12 + 4 * k * 4) / (leg_ms / 1e3) / 1e9 / PEAK_HBM_GBS}
        if probe is not None:
            res["access_pattern_ceiling_ms"] = probe
        return res

    if not a.skip_fp32:
        out["mascot_all_binary32"] = switched_leg()
        out["fp32_sgd"] = side_leg(5, a.warmup, a.steps, "fp32 SGD (mf_train -v 5) on the same ratings, workers and hot-row treatment, every row update carried out")
        out["fp32_sgd"]["mascot_speedup"] = out["fp32_sgd"]["ms_per_step"] / ms
        out["mascot_all_binary32"]["vs_fp32_sgd_epoch"] = out["mascot_all_binary32"]["ms_per_step"] / out["fp32_sgd"]["ms_per_step"]
        if "whole_job" in out:
            out["whole_job"]["speedup_vs_50_fp32_sgd_epochs"] = TRAIN["epochs"] * out["fp32_sgd"]["ms_per_step"] / out["whole_job"]["sgd_ms_total"]
    if not a.skip_reference_semantics:
        out["reference_semantics"] = side_leg(1, 0, 2, "mf_train -v 1 without hot rows (-hot 0): every row stored with a device-coherent store, last writer "
                                              "wins -- bound by the serialisation of the stores to the hottest row at the memory side",
                                              hot_rows=0, replicate_inflight=0.0, hot_row_inflight=0.0)
    if a.every_rule:
        out["every_rule"] = {}
        for name, version, half in (("mpt", 4, True), ("muppet", 3, False), ("afp", 2, False), ("mem_quant", 7, True)):
            if name not in a.rules.split(","):
                continue
            out["every_rule"][name] = side_leg(version, 2, 6, "mf_train -v %d, epochs 2..7" % version, half)
    if not a.skip_cpu:
        threads = min(os.cpu_count() or 1, 16)
        sample = min(n_train, a.cpu_updates)
        rate, done, dt = cpu_baseline(cfg, train, k, a.seed, threads, sample)
        out["cpu_baseline"] = {"value": rate, "unit": "ratings/s", "cores": threads, "kind": "port",
                               "sample": "one epoch over the first %d training ratings (%d updates: %d workers x %d windows of 128; binary16 model, "
                                         "100+100 groups), %.1f s, OpenMP Hogwild loop of the checker" % (sample, done, threads * 8, done // (threads * 8 * 128), dt)}
    print(json.dumps(out))


if __name__ == "__main__":
    main()
