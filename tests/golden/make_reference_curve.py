"""Writes reference_curve_config<N>*.json: the per-epoch test RMSE of the reference's training drivers
(mascot_training_mf, mf_methods.cu:36-434; training_single_mf :820-924; mixed_precision_training_mf :713-818) run by
the CPU checker under oracle/ as a multithreaded Hogwild loop -- the curves bench.py and the GPU tests hold the HIP
training run against.

    python tests/golden/make_reference_curve.py [--config 4] [--version 1] [--k 128] [--run 1] [--threads 8] [--epochs 50]

Configurations 2, 3 and 4 of BASELINE.json (8M, 20M and 100M training ratings); versions 1 (MASCOT), 5 (fp32 SGD) and
4 (MPT), the variants configuration 3 names.  Files: reference_curve_config<N>[_v<V>][_k64]_run<R>.json.

The run mirrors `quantized_mf -synth 4 -v 1 -k 128 -ug 100 -ig 100 -s 0.05 -it 2 -e 20 -l 50 -a 0.01 -d 0.1
-seed 2021` step by step on the host: the seeded synthetic ratings of BASELINE configuration 4 (checker twin of
mf_generate_ratings), the reference's test-set rules (io_utils.h:183-198, preprocess_utils.h:38-52), the seeded
N(0, 0.01^2) initial model, the seeded shuffle, histogram / sort / grouping / re-index, 50 epochs of the
reference update rule over the windows of 6104 workers with the sampled error estimate and precision switching.
Only the number of updates in flight differs: `threads` host threads race instead of thousands of wavefronts, so
the curve is the reference rule close to its sequential limit.  The CPU loop races as well: two runs differ in the
fourth decimal, which is why several runs are kept (`--run N` names the output file).

No GPU and no HIP library are involved; about an hour per run on 8 cores."""
import argparse
import json
import os
import sys
import time

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

# BASELINE configuration 4 (the table of mf_synth_baseline_config): 480,000 users x 17,800 items, 100M training and
# 1.4M test ratings, user Zipf(0.8), item Zipf(1.1), integers 1..5 from a rank-32 truth + N(0, 0.9), mean 3.6
CONFIGS = {
    # configurations 2 and 3: 70,000 x 10,700 with 8M / 2M ratings, Zipf(0.9); 162,000 x 59,000 with 20M / 5M, Zipf(1.0);
    # ratings 0.5..5.0 in half steps from a rank-16 truth + N(0, 0.8), mean 3.5
    2: dict(n_users=70_000, n_items=10_700, n_train=8_000_000, n_test=2_000_000, user_alpha=0.9, item_alpha=0.9,
            rank=16, noise=0.8, mean=3.5, step=0.5, lo=0.5, hi=5.0, bimodal=0),
    3: dict(n_users=162_000, n_items=59_000, n_train=20_000_000, n_test=5_000_000, user_alpha=1.0, item_alpha=1.0,
            rank=16, noise=0.8, mean=3.5, step=0.5, lo=0.5, hi=5.0, bimodal=0),
    4: dict(n_users=480_000, n_items=17_800, n_train=100_000_000, n_test=1_400_000, user_alpha=0.8, item_alpha=1.1,
            rank=32, noise=0.9, mean=3.6, step=1.0, lo=1.0, hi=5.0, bimodal=0),
}
CONFIG4 = CONFIGS[4]
# workers: the windows the CPU threads race over.  Configuration 4's curves were taken with 6104 (one resident set of
# the GPU); configurations 2 and 3 use mf_auto_workers(n) = n / 16384 rounded up to a multiple of four (488, 1220),
# which is what the GPU run of the same command line uses.
TRAIN = dict(k=128, workers=6104, lr=0.01, lam=0.015, decay=0.1, ug=100, ig=100, sample_ratio=0.05, interval=2, threshold=20.0)


def auto_workers(n):
    return max(16, (n // 16384 + 3) // 4 * 4)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--config", type=int, default=4, choices=(2, 3, 4))
    ap.add_argument("--version", type=int, default=1, choices=(1, 4, 5), help="1 MASCOT, 4 MPT, 5 fp32 SGD")
    ap.add_argument("--k", type=int, default=128, choices=(64, 128))
    ap.add_argument("--run", type=int, default=1)
    ap.add_argument("--threads", type=int, default=8)
    ap.add_argument("--epochs", type=int, default=50)
    ap.add_argument("--seed", type=int, default=2021)
    ap.add_argument("--scale", type=float, default=1.0, help="fraction of the ratings (and of the workers): smoke runs of this script")
    a = ap.parse_args()
    import mfutil
    from oracle import oracle as om
    orc = om.get()
    shape = CONFIGS[a.config]
    cfg = om.SynthConfig(**shape)
    n_train, n_test = int(shape["n_train"] * a.scale), int(shape["n_test"] * a.scale)
    W = TRAIN["workers"] if a.config == 4 else auto_workers(n_train)
    if a.scale != 1.0:
        cfg.n_train, cfg.n_test = n_train, n_test
        W = auto_workers(n_train)
    t0 = time.time()
    allr = orc.generate_ratings(cfg, a.seed, 0, n_train + n_test)
    train, test = allr[:n_train], allr[n_train:]
    # read_test_dataset: ratings of unseen users / items are dropped; duplicates: last wins; order (user, item)
    seen_u = np.zeros(cfg.n_users, bool); seen_u[train["u"]] = True
    seen_i = np.zeros(cfg.n_items, bool); seen_i[train["i"]] = True
    test = mfutil.test_set_order(test[seen_u[test["u"]] & seen_i[test["i"]]])
    k = a.k
    P = orc.init_normal(a.seed, 0, cfg.n_users * k).reshape(cfg.n_users, k)
    Q = orc.init_normal(a.seed, 1, cfg.n_items * k).reshape(cfg.n_items, k)
    print("data ready: %d train, %d test ratings, %.0f s" % (train.size, test.size, time.time() - t0), flush=True)
    tag = ("" if a.version == 1 else "_v%d" % a.version) + ("" if k == 128 else "_k%d" % k) + ("" if a.scale == 1.0 else "_scale%g" % a.scale)
    out_name = os.path.join(HERE, "reference_curve_config%d%s_run%d.json" % (a.config, tag, a.run))
    rmse = []
    t1 = time.time()
    progress = lambda e, r: print("epoch %d rmse %.6f (%.0f s)" % (e + 1, r, time.time() - t1), flush=True)
    train_args = dict(TRAIN, k=k, workers=W)
    if a.version != 1:
        # -v 4 starts from an initial model rounded to binary16 (init_model_half, main.cu:152-153)
        if a.version == 4:
            P, Q = orc.h2f(orc.f2h(P)).reshape(P.shape), orc.h2f(orc.f2h(Q)).reshape(Q.shape)
        curve, _ = mfutil.oracle_train_dense(orc, a.version, train, test, P, Q, k, W, a.epochs, TRAIN["lr"], TRAIN["lam"], TRAIN["decay"], a.seed,
                                             threads=a.threads, progress=progress)
        out = dict(config=a.config, version=a.version, scale=a.scale, seed=a.seed, threads=a.threads, epochs=a.epochs, workers=W,
                   n_train=int(train.size), n_test=int(test.size), train=train_args, test_rmse=[float(x) for x in curve], seconds=round(time.time() - t0),
                   source="tests/golden/make_reference_curve.py: reference update rule (CPU checker), %d host threads" % a.threads)
        with open(out_name, "w") as f:
            json.dump(out, f, indent=1)
        print("wrote", out_name)
        return

    # oracle_train_mascot one epoch at a time would redo the preprocessing; run it whole and log from its result
    curve, info = mfutil.oracle_train_mascot(orc, train, test, P, Q, k, W, a.epochs, TRAIN["lr"], TRAIN["lam"], TRAIN["decay"], a.seed,
                                             TRAIN["ug"], TRAIN["ig"], TRAIN["sample_ratio"], TRAIN["interval"], TRAIN["threshold"],
                                             threads=a.threads, progress=progress)
    rmse = [float(x) for x in curve]
    out = dict(config=a.config, version=1, scale=a.scale, seed=a.seed, threads=a.threads, epochs=a.epochs, workers=W, n_train=int(train.size), n_test=int(test.size),
               train=train_args, user_groups=int(info["uend"].size), item_groups=int(info["iend"].size),
               user_groups_binary32=int(info["gu"].prec.sum()), item_groups_binary32=int(info["gi"].prec.sum()),
               user_groups_binary32_per_epoch=[int(x[0]) for x in info["switched_per_epoch"]],
               item_groups_binary32_per_epoch=[int(x[1]) for x in info["switched_per_epoch"]],
               test_rmse=rmse, seconds=round(time.time() - t0),
               source="tests/golden/make_reference_curve.py: reference update rule (CPU checker), %d host threads" % a.threads)
    with open(out_name, "w") as f:
        json.dump(out, f, indent=1)
    print("wrote", out_name)


if __name__ == "__main__":
    main()
