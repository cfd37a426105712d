#!/usr/bin/env python3
"""Benchmark of the MASCOT SGD hot path on one MI355X.

A step is one epoch's update launch of MASCOT (k=128, ug=ig=100, sample ratio 0.05, period 2) over the
synthetic 480,000 x 17,800 matrix with 100M training ratings (item popularity Zipf(1.1), integers 1-5 from a
rank-32 truth plus N(0,0.9) noise) -- the fourth configuration of BASELINE.json.  Inputs are resident in HBM
before the timed region.  Everything goes through the C ABI of libmascot_hip.so; torch only owns the device
memory and the stream.  One JSON line on stdout.
"""
import argparse
import ctypes as C
import importlib
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
PEAK_HBM_GBS = 8000.0


def zipf_ranks(torch, count, size, alpha, gen, dev):
    w = 1.0 / torch.arange(1, count + 1, device=dev, dtype=torch.float64) ** alpha
    cdf = torch.cumsum(w, 0)
    cdf = cdf / cdf[-1]
    out = torch.empty(size, dtype=torch.int64, device=dev)
    step = 20_000_000
    for s in range(0, size, step):
        r = torch.rand(min(step, size - s), device=dev, generator=gen, dtype=torch.float64)
        out[s:s + r.numel()] = torch.searchsorted(cdf, r).clamp_(max=count - 1)
    return out


# The synthetic configurations of BASELINE.json that fit one GPU (config 1 is the CPU-runnable plumbing case of the
# tests).  Config 5's ratings are integers 0..100; like the reference does for its 0..100 data set (io_utils.h:75)
# they are mapped to r / 25 + 1 so that the N(0, 0.01^2) start and lr 0.01 stay in binary16 range.
CONFIGS = {
    2: dict(n_users=70_000, n_items=10_700, n_train=8_000_000, n_test=2_000_000, user_alpha=0.9, item_alpha=0.9, rank=16, noise=0.8,
            mean=3.5, step=0.5, lo=0.5, hi=5.0, text="70000 users x 10700 items, Zipf(0.9), 0.5-5.0 in half steps from rank-16 truth + N(0,0.8)"),
    3: dict(n_users=162_000, n_items=59_000, n_train=20_000_000, n_test=5_000_000, user_alpha=1.0, item_alpha=1.0, rank=16, noise=0.8,
            mean=3.5, step=0.5, lo=0.5, hi=5.0, text="162000 users x 59000 items, Zipf(1.0), 0.5-5.0 in half steps from rank-16 truth + N(0,0.8)"),
    4: dict(n_users=480_000, n_items=17_800, n_train=100_000_000, n_test=1_400_000, user_alpha=0.8, item_alpha=1.1, rank=32, noise=0.9,
            mean=3.6, step=1.0, lo=1.0, hi=5.0, text="480000 users x 17800 items, item Zipf(1.1), user Zipf(0.8), ints 1-5 from rank-32 truth + N(0,0.9)"),
    5: dict(n_users=1_000_000, n_items=625_000, n_train=250_000_000, n_test=4_000_000, user_alpha=1.2, item_alpha=1.2, rank=0, noise=15.0,
            mean=0.0, step=1.0, lo=0.0, hi=100.0, text="1000000 users x 625000 items, Zipf(1.2), ints 0-100 from 0.5 N(20,15) + 0.5 N(80,15), mapped to r/25+1"),
}


def make_workload(torch, n_users, n_items, n, seed, dev, user_alpha, item_alpha, rank, noise, mean, step=1.0, lo=1.0, hi=5.0):
    """COO ratings [n][3] int32 (float bits, user, item) on the device, ids in random (unsorted) order.  rank = 0: the
    bimodal 0..100 ratings of config 5 (no low-rank truth), mapped to r / 25 + 1."""
    gen = torch.Generator(device=dev)
    gen.manual_seed(seed)
    uperm = torch.randperm(n_users, device=dev, generator=gen)
    iperm = torch.randperm(n_items, device=dev, generator=gen)
    u = uperm[zipf_ranks(torch, n_users, n, user_alpha, gen, dev)]
    i = iperm[zipf_ranks(torch, n_items, n, item_alpha, gen, dev)]
    if rank:
        U = torch.randn(n_users, rank, device=dev, generator=gen) * 0.5
        V = torch.randn(n_items, rank, device=dev, generator=gen) * 0.5
    R = torch.empty((n, 3), dtype=torch.int32, device=dev)
    chunk = 10_000_000
    for s in range(0, n, chunk):
        e = min(n, s + chunk)
        if rank:
            val = (U[u[s:e]] * V[i[s:e]]).sum(1) + mean + torch.randn(e - s, device=dev, generator=gen) * noise
            val = (val / step).round_().mul_(step).clamp_(lo, hi)
        else:
            mode = torch.where(torch.rand(e - s, device=dev, generator=gen) < 0.5, 20.0, 80.0)
            val = (mode + torch.randn(e - s, device=dev, generator=gen) * noise).round_().clamp_(lo, hi) / 25.0 + 1.0
        R[s:e, 0] = val.to(torch.float32).view(torch.int32)
    R[:, 1] = u.to(torch.int32)
    R[:, 2] = i.to(torch.int32)
    return R


class MascotProblem:
    """Device-resident MASCOT training state built with the library's own pre-processing kernels."""

    def __init__(self, torch, h, R, n_users, n_items, k, ug, ig, seed, test=None):
        self.torch, self.h, self.k = torch, h, k
        dev = R.device
        st = torch.cuda.current_stream().cuda_stream
        n = R.shape[0]
        self.n, self.n_users, self.n_items = n, n_users, n_items
        # seeded shuffle (mf_methods.cu:38-39)
        self.R = torch.empty_like(R)
        h.mf_shuffle_ratings(R.data_ptr(), self.R.data_ptr(), n, seed, st)
        # histogram -> sort -> grouping -> re-index (preprocess_utils.h:54-255)
        ucnt = torch.zeros(n_users, dtype=torch.int32, device=dev)
        icnt = torch.zeros(n_items, dtype=torch.int32, device=dev)
        h.mf_user_item_histogram(self.R.data_ptr(), n, ucnt.data_ptr(), icnt.data_ptr(), st)
        self.sides = []
        for cnt, num, req in ((ucnt, n_users, ug), (icnt, n_items, ig)):
            idx = torch.empty(num, dtype=torch.int32, device=dev)
            h.mf_init_idx_arr(idx.data_ptr(), num, st)
            h.mf_sort_by_count(cnt.data_ptr(), idx.data_ptr(), num, st)
            sorted_cnt = cnt.cpu().numpy().view(np.uint32)
            sorted_id = idx.cpu().numpy().view(np.uint32)
            end = np.zeros(num, np.uint32)
            g = h.mf_group_end_indices(sorted_cnt.ctypes.data, num, req, end.ctypes.data)
            end = end[:g].copy()
            id2sorted = np.empty(num, np.uint32)
            id2sorted[sorted_id] = np.arange(num, dtype=np.uint32)
            id2group = np.searchsorted(end, id2sorted).astype(np.uint32)
            self.sides.append(dict(end=end, id2sorted=id2sorted, id2group=id2group, groups=g, num=num, sorted_cnt=sorted_cnt.copy()))
        du2s = torch.from_numpy(self.sides[0]["id2sorted"].view(np.int32)).to(dev)
        di2s = torch.from_numpy(self.sides[1]["id2sorted"].view(np.int32)).to(dev)
        h.mf_matrix_reconst_triplet(self.R.data_ptr(), du2s.data_ptr(), di2s.data_ptr(), n, st)
        self.test = None
        if test is not None:
            self.test = test.clone()
            h.mf_matrix_reconst_triplet(self.test.data_ptr(), du2s.data_ptr(), di2s.data_ptr(), self.test.shape[0], st)
        # model init (model_init.cu:114-173) and scatter into binary16 groups (model_init.cu:175-222)
        for side, (s, d_id2sorted) in enumerate(zip(self.sides, (du2s, di2s))):
            num, g, end = s["num"], s["groups"], s["end"]
            dense = torch.empty(num * k, dtype=torch.float32, device=dev)
            h.mf_init_rand_feature(dense.data_ptr(), num * k, seed, side, st)
            sizes = np.diff(np.concatenate([[-1], end.astype(np.int64)]))
            offs = np.concatenate([[0], np.cumsum((sizes * k * 2 + 255) // 256 * 256)[:-1]])
            arena = torch.zeros(int((sizes * k * 2 + 255).sum() // 1 + 256 * g), dtype=torch.uint8, device=dev)
            ptrs = torch.tensor([arena.data_ptr() + int(o) for o in offs], dtype=torch.int64, device=dev)
            d_end = torch.from_numpy(end.view(np.int32)).to(dev)
            d_prec = torch.zeros(g, dtype=torch.uint8, device=dev)
            d_id2group = torch.from_numpy(s["id2group"].view(np.int32)).to(dev)
            h.mf_cpyparams2grouped_params(dense.data_ptr(), ptrs.data_ptr(), d_end.data_ptr(), d_id2group.data_ptr(),
                                          d_id2sorted.data_ptr(), k, num, g, st)
            s.update(arena=arena, ptrs=ptrs, d_end=d_end, d_prec=d_prec, sizes=sizes, offs=offs)
            torch.cuda.synchronize()
            s["initial"] = arena.clone()
        self.stats = None
        self.hot = None

    def reset(self):
        for s in self.sides:
            s["arena"].copy_(s["initial"])

    def hot_tables(self, W, inflight_cap):
        """Hot-row tables from the rating counts (rows are in popularity-sorted order), as mf_train builds them:
        255 = ordinary row; rows with more than one update in flight are hot rows (updates added in memory), thinned to
        at most `inflight_cap` updates in flight.  Returns (user table, item table, fraction of row updates carried out)."""
        tabs, kept = [], 0.0
        for s in self.sides:
            cnt = np.ascontiguousarray(s["sorted_cnt"], np.uint32)
            t = np.empty(cnt.size, np.uint8)
            self.h.mf_hot_row_table(cnt.ctypes.data, cnt.size, self.n, W, inflight_cap, t.ctypes.data)
            kept += float((cnt.astype(np.float64) * np.where(t == 255, 1.0, (t.astype(np.float64) + 1) / 255.0)).sum()) / self.n
            tabs.append(self.torch.from_numpy(t).to(self.R.device))
        return tabs[0], tabs[1], kept / 2

    def set_hot_rows(self, W, cap, early_cap=0.0, early_epochs=0):
        """The hot-row schedule of a leg: `early_cap` during the first `early_epochs` epochs, `cap` afterwards (0 = off)."""
        self.hot = None
        self.h.mf_set_hot_row_thinning(None, None)
        if cap:
            steady = self.hot_tables(W, cap)
            early = self.hot_tables(W, early_cap) if early_epochs and early_cap > cap else steady
            self.hot = dict(steady=steady, early=early, early_epochs=early_epochs if early is not steady else 0)

    def select_hot_rows(self, e):
        """Installs the tables of epoch e; returns the fraction of row updates that epoch carries out."""
        if self.hot is None:
            return 1.0
        u, v, kept = self.hot["early"] if e < self.hot["early_epochs"] else self.hot["steady"]
        self.h.mf_set_hot_row_thinning(u.data_ptr(), v.data_ptr())
        return kept

    def alloc_stats(self, W):
        torch, h, k = self.torch, self.h, self.k
        nb = h.mf_mascot_norm_blocks(W)
        U, I = self.sides
        dev = self.R.device
        self.stats = dict(W=W, nb=nb,
                          gsp=torch.zeros(U["groups"] * k, device=dev), gsq=torch.zeros(I["groups"] * k, device=dev),
                          nsp=torch.zeros(U["groups"] * nb, device=dev), nsq=torch.zeros(I["groups"] * nb, device=dev))

    def epoch(self, e, W, epochs, lr0, decay, lam, sample_ratio, interval, seed):
        h, U, I, s = self.h, self.sides[0], self.sides[1], self.stats
        st = self.torch.cuda.current_stream().cuda_stream
        uc = h.mf_update_count(self.n, W, 128)
        first = h.mf_first_sample_rating_idx(e, interval, epochs, uc, 128, sample_ratio)
        if first < uc * 128:
            s["gsp"].zero_()
            s["gsq"].zero_()
        h.mf_mascot_sgd_hogwild(self.R.data_ptr(), self.n, U["ptrs"].data_ptr(), I["ptrs"].data_ptr(), self.k, W, uc, 128,
                                h.mf_lr_schedule(lr0, decay, e), lam, U["d_end"].data_ptr(), I["d_end"].data_ptr(),
                                U["d_prec"].data_ptr(), I["d_prec"].data_ptr(), s["gsp"].data_ptr(), s["gsq"].data_ptr(),
                                s["nsp"].data_ptr(), s["nsq"].data_ptr(), first, U["groups"], I["groups"], seed, e, None, st)
        return uc

    def rmse(self):
        torch, h, U, I = self.torch, self.h, self.sides[0], self.sides[1]
        acc = torch.zeros(1, dtype=torch.float64, device=self.R.device)
        h.mf_test_rmse_grouped(self.test.data_ptr(), self.test.shape[0], U["ptrs"].data_ptr(), I["ptrs"].data_ptr(), self.k,
                               U["d_end"].data_ptr(), I["d_end"].data_ptr(), U["d_prec"].data_ptr(), I["d_prec"].data_ptr(),
                               U["groups"], I["groups"], acc.data_ptr(), torch.cuda.current_stream().cuda_stream)
        return float(np.sqrt(acc.item() / self.test.shape[0]))

    def host_grouped(self):
        """Host mirror of the grouped model for the CPU checker."""
        from oracle import oracle as om
        out = []
        for s in self.sides:
            host = s["arena"].cpu().numpy()
            arrays = [host[int(o):int(o) + int(sz) * self.k * 2].view(np.uint16).copy() for o, sz in zip(s["offs"], s["sizes"])]
            out.append(om.GroupedModel(self.k, s["end"], np.zeros(s["groups"], np.uint8), arrays))
        return out


def time_steps(torch, prob, W, warmup, steps, cfg, seed):
    """W untimed epochs, then K epochs each bracketed by events on the launch stream."""
    prob.reset()
    prob.alloc_stats(W)
    for e in range(warmup):
        prob.select_hot_rows(e)
        prob.epoch(e, W, cfg["epochs"], cfg["lr"], cfg["decay"], cfg["lam"], cfg["sample_ratio"], cfg["interval"], seed)
    torch.cuda.synchronize()
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    t0 = time.perf_counter()
    uc = 0
    kept = []
    for i in range(steps):
        kept.append(prob.select_hot_rows(warmup + i))
        ev[i][0].record()
        uc = prob.epoch(warmup + i, W, cfg["epochs"], cfg["lr"], cfg["decay"], cfg["lam"], cfg["sample_ratio"], cfg["interval"], seed)
        ev[i][1].record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    per = np.array([a.elapsed_time(b) for a, b in ev])
    return per, wall, uc, float(np.mean(kept))


def access_pattern_ceiling(torch, h, prob, W, tables, coherent, seed, reps=3):
    """Time of mf_row_traffic_probe on the same ratings, hot-row tables and store policy: the epoch's memory traffic
    without the arithmetic (all rows binary16, as in the timed epochs)."""
    dev = prob.R.device
    n = prob.R.shape[0]
    P = torch.zeros(prob.n_users * prob.k, dtype=torch.float16, device=dev)
    Q = torch.zeros(prob.n_items * prob.k, dtype=torch.float16, device=dev)
    ku, kv = (tables[0].data_ptr(), tables[1].data_ptr()) if tables is not None else (None, None)
    st = torch.cuda.current_stream().cuda_stream
    run = lambda: h.mf_row_traffic_probe(prob.R.data_ptr(), n, P.data_ptr(), Q.data_ptr(), prob.k * 2, W, ku, kv, seed, 1 if coherent else 0, st)
    run()
    torch.cuda.synchronize()
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(reps)]
    for a, b in ev:
        a.record(); run(); b.record()
    torch.cuda.synchronize()
    return float(np.mean([a.elapsed_time(b) for a, b in ev]))


def cpu_baseline(prob, cfg, seed, threads, target_updates):
    """The checker's MASCOT epoch (reference update rule, binary16 through F16C) as a Hogwild CPU loop."""
    from oracle import oracle as om
    orc = om.get()
    R = prob.R.cpu().numpy().view(np.uint8).reshape(-1).view(om.NODE)
    gu, gi = prob.host_grouped()
    W = threads * 8
    uc = max(1, target_updates // (W * 128))
    z = [np.zeros(n, np.float32) for n in (gu.groups * prob.k, gi.groups * prob.k, gu.groups, gi.groups)]
    t0 = time.perf_counter()
    orc.lib.orc_mascot_epoch(prob.k, R.ctypes.data, R.size, gu.ptrs, gi.ptrs, gu.end_idx.ctypes.data, gi.end_idx.ctypes.data,
                             gu.prec.ctypes.data, gi.prec.ctypes.data, gu.groups, gi.groups, W, uc, 128,
                             cfg["lr"], cfg["lam"], uc * 128, z[0].ctypes.data, z[1].ctypes.data, z[2].ctypes.data, z[3].ctypes.data,
                             seed, 0, None, threads)
    dt = time.perf_counter() - t0
    done = W * uc * 128
    return done / dt, done, dt


def cpu_baseline_fp32(prob, h, cfg, seed, threads, target_updates):
    """The checker's fp32 SGD epoch (reference rule of -v 5) as the same Hogwild CPU loop, dense fp32 P and Q."""
    from oracle import oracle as om
    orc = om.get()
    R = prob.R.cpu().numpy().view(np.uint8).reshape(-1).view(om.NODE)
    P = orc.init_normal(seed, 0, prob.n_users * prob.k)
    Q = orc.init_normal(seed, 1, prob.n_items * prob.k)
    W = threads * 8
    uc = max(1, target_updates // (W * 128))
    t0 = time.perf_counter()
    orc.lib.orc_sgd_epoch(prob.k, R.ctypes.data, R.size, P.ctypes.data, Q.ctypes.data, W, uc, 128, cfg["lr"], cfg["lam"], seed, 0, None, threads)
    dt = time.perf_counter() - t0
    return W * uc * 128 / dt, W * uc * 128, dt


def time_fp32_sgd(torch, h, prob, W, warmup, steps, cfg, seed):
    """The fp32-SGD update (-v 5) on the same ratings, schedule and hot-row tables: dense fp32 P and Q."""
    dev, k, st = prob.R.device, prob.k, torch.cuda.current_stream().cuda_stream
    P = torch.empty(prob.n_users * k, dtype=torch.float32, device=dev)
    Q = torch.empty(prob.n_items * k, dtype=torch.float32, device=dev)
    h.mf_init_rand_feature(P.data_ptr(), P.numel(), seed, 0, st)
    h.mf_init_rand_feature(Q.data_ptr(), Q.numel(), seed, 1, st)
    uc = h.mf_update_count(prob.n, W, 128)
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    kept = []
    for e in range(warmup + steps):
        kept_e = prob.select_hot_rows(e)
        if e >= warmup:
            kept.append(kept_e)
            ev[e - warmup][0].record()
        h.mf_single_sgd_hogwild(prob.R.data_ptr(), prob.n, P.data_ptr(), Q.data_ptr(), k, W, uc, 128,
                                h.mf_lr_schedule(cfg["lr"], cfg["decay"], e), cfg["lam"], seed, e, None, st)
        if e >= warmup:
            ev[e - warmup][1].record()
    torch.cuda.synchronize()
    acc = torch.zeros(1, dtype=torch.float64, device=dev)
    h.mf_test_rmse(prob.test.data_ptr(), prob.test.shape[0], P.data_ptr(), Q.data_ptr(), k, acc.data_ptr(), st)
    rmse = float(np.sqrt(acc.item() / prob.test.shape[0]))
    return np.array([a.elapsed_time(b) for a, b in ev]), uc, rmse, float(np.mean(kept))


def time_every_rule(torch, h, prob, W, cfg, seed, epochs=6):
    """Every update kernel on the same ratings, workers and hot-row schedule (dense P and Q in the rule's storage format):
    mean time of the steady plain epochs 2..epochs-1 and the test RMSE after `epochs` epochs, with the access-pattern
    probe of the rule's row size beside it."""
    dev, k, st = prob.R.device, prob.k, torch.cuda.current_stream().cuda_stream
    uc = h.mf_update_count(prob.n, W, 128)
    lr = lambda e: h.mf_lr_schedule(cfg["lr"], cfg["decay"], e)
    lam_h = int(np.array([np.float32(cfg["lam"]) * np.float32(1000.0)], np.float32).astype(np.float16).view(np.uint16)[0])
    R, n = prob.R.data_ptr(), prob.n
    sums = torch.zeros(k, dtype=torch.float32, device=dev)
    norms = torch.zeros(W, dtype=torch.float32, device=dev)
    rules = {
        "fp32_sgd": (4, lambda P, Q, e: h.mf_single_sgd_hogwild(R, n, P, Q, k, W, uc, 128, lr(e), cfg["lam"], seed, e, None, st)),
        "mpt": (4, lambda P, Q, e: h.mf_mpt_sgd_hogwild(R, n, P, Q, k, W, uc, 128, lr(e), lam_h, 1000.0, seed, e, None, st)),
        "muppet_8bit": (4, lambda P, Q, e: h.mf_muppet_sgd_hogwild(R, n, P, Q, k, W, uc, 128, lr(e), cfg["lam"], uc * 128, sums.data_ptr(),
                                                                  norms.data_ptr(), 8, 8, seed, e, None, st)),
        "muppet_16bit": (4, lambda P, Q, e: h.mf_muppet_sgd_hogwild(R, n, P, Q, k, W, uc, 128, lr(e), cfg["lam"], uc * 128, sums.data_ptr(),
                                                                   norms.data_ptr(), 16, 16, seed, e, None, st)),
        "afp": (4, lambda P, Q, e: h.mf_afp_sgd_hogwild(R, n, P, Q, k, W, uc, 128, lr(e), cfg["lam"], e, seed, e, None, st)),
        "mem_quant": (2, lambda P, Q, e: h.mf_mem_quant_sgd_hogwild(R, n, P, Q, k, W, uc, 128, lr(e), cfg["lam"], seed, e, None, st)),
    }
    out, ceilings = {}, {}
    steady = prob.hot["steady"] if prob.hot else None
    for name, (elem, call) in rules.items():
        P32 = torch.empty(prob.n_users * k, dtype=torch.float32, device=dev)
        Q32 = torch.empty(prob.n_items * k, dtype=torch.float32, device=dev)
        h.mf_init_rand_feature(P32.data_ptr(), P32.numel(), seed, 0, st)
        h.mf_init_rand_feature(Q32.data_ptr(), Q32.numel(), seed, 1, st)
        P, Q = P32, Q32
        if elem == 2:
            P, Q = torch.empty(P32.numel(), dtype=torch.float16, device=dev), torch.empty(Q32.numel(), dtype=torch.float16, device=dev)
            h.mf_transform_float2half(P32.data_ptr(), P.data_ptr(), P32.numel(), st)
            h.mf_transform_float2half(Q32.data_ptr(), Q.data_ptr(), Q32.numel(), st)
        ms = []
        for e in range(epochs):
            prob.select_hot_rows(e)
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record(); call(P.data_ptr(), Q.data_ptr(), e); b.record()
            torch.cuda.synchronize()
            ms.append(a.elapsed_time(b))
        if elem == 2:
            h.mf_transform_half2float(P.data_ptr(), P32.data_ptr(), P32.numel(), st)
            h.mf_transform_half2float(Q.data_ptr(), Q32.data_ptr(), Q32.numel(), st)
        acc = torch.zeros(1, dtype=torch.float64, device=dev)
        h.mf_test_rmse(prob.test.data_ptr(), prob.test.shape[0], P32.data_ptr(), Q32.data_ptr(), k, acc.data_ptr(), st)
        row_bytes = k * elem
        if row_bytes not in ceilings:
            ku, kv = (steady[0].data_ptr(), steady[1].data_ptr()) if steady else (None, None)
            probe = lambda: h.mf_row_traffic_probe(R, n, P.data_ptr(), Q.data_ptr(), row_bytes, W, ku, kv, seed, h.mf_get_row_coherence(), st)
            probe(); torch.cuda.synchronize()
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record(); probe(); probe(); b.record(); torch.cuda.synchronize()
            ceilings[row_bytes] = a.elapsed_time(b) / 2
        steady_ms = float(np.mean(ms[2:]))
        out[name] = {"ms_per_epoch": steady_ms, "row_bytes": row_bytes, "access_pattern_ceiling_ms": ceilings[row_bytes],
                     "kernel_vs_ceiling": ceilings[row_bytes] / steady_ms, "test_rmse": float(np.sqrt(acc.item() / prob.test.shape[0])), "epochs": epochs}
        del P, Q, P32, Q32
    return out


def reference_rule_rmse(prob, h, cfg, seed, threads, epochs, workers):
    """Test RMSE of the reference update rule (the checker's MASCOT epoch as an OpenMP Hogwild loop, `threads` updates
    in flight) after `epochs` epochs on the same shuffled ratings, initial model, schedule and learning rates."""
    from oracle import oracle as om
    orc = om.get()
    prob.reset()
    R = prob.R.cpu().numpy().view(np.uint8).reshape(-1).view(om.NODE)
    gu, gi = prob.host_grouped()
    uc = h.mf_update_count(prob.n, workers, 128)
    z = [np.zeros(n, np.float32) for n in (gu.groups * prob.k, gi.groups * prob.k, gu.groups, gi.groups)]
    for e in range(epochs):
        t0 = time.perf_counter()
        orc.lib.orc_mascot_epoch(prob.k, R.ctypes.data, R.size, gu.ptrs, gi.ptrs, gu.end_idx.ctypes.data, gi.end_idx.ctypes.data,
                                 gu.prec.ctypes.data, gi.prec.ctypes.data, gu.groups, gi.groups, workers, uc, 128,
                                 h.mf_lr_schedule(cfg["lr"], cfg["decay"], e), cfg["lam"], uc * 128,
                                 z[0].ctypes.data, z[1].ctypes.data, z[2].ctypes.data, z[3].ctypes.data, seed, e, None, threads)
        print("bench.py: reference rule on the CPU, epoch %d of %d, %.1f s" % (e + 1, epochs, time.perf_counter() - t0), file=sys.stderr, flush=True)
    for s, g in zip(prob.sides, (gu, gi)):                      # score it with the same device RMSE kernel
        host = s["arena"].cpu().numpy()
        for o, sz, arr in zip(s["offs"], s["sizes"], g.arrays):
            host[int(o):int(o) + int(sz) * prob.k * 2] = arr.view(np.uint8)
        s["arena"].copy_(prob.torch.from_numpy(host))
    rmse = prob.rmse()
    prob.reset()
    return rmse


def measured_traffic(a, leg):
    """HBM bytes per launch of a plain epoch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (KiB per dispatch, scaled by
    2.0 / 1.0, the factors a 1 GiB device copy gives; summaries under profiles/).  Counters cannot be read from inside
    this process, so the figures are the profiled ones and only reported for the exact workload they were taken on."""
    if a.config != 4 or a.k != 128 or a.ratings != 100_000_000 or a.seed != 2021:
        return None
    if a.skip_coherent:
        return (13_996_993 * 2.0 + 24_209_347) * 1024 if leg["workers"] == 16384 else None
    if leg["workers"] == 6104 and a.hot_row_inflight == 2.0 and a.warmup >= a.hot_row_early_epochs:
        return (15_952_590 * 2.0 + 27_557_537) * 1024
    return None


# Test RMSE of the reference update rule on the CPU (`--reference-rmse`: the checker's MASCOT epoch as a 16-thread
# Hogwild loop over the same ratings, shuffle, initial model and windows), recorded so that the default run can report
# the delta without six minutes of CPU work (two recorded runs gave 0.88717 and 0.88760: the CPU loop races too).  Key: (config, train ratings, k, seed, epochs, workers).  A run with
# other settings reports no delta unless --reference-rmse computes it.
RECORDED_REFERENCE_RMSE = {
    (4, 100_000_000, 128, 2021, 12, 6104): 0.88760,
    (4, 100_000_000, 128, 2021, 30, 6104): 0.88079,
}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--config", type=int, default=4, choices=sorted(CONFIGS), help="BASELINE.json configuration (4 = the one the metric is quoted on)")
    ap.add_argument("--ratings", type=int, default=0, help="training ratings (default: the configuration's)")
    ap.add_argument("--k", type=int, default=128, choices=(64, 128))
    ap.add_argument("--workers", type=int, default=0, help="-wg of the measured run (default: mf_auto_workers(ratings); 6104 at config 4)")
    ap.add_argument("--cached-workers", type=int, default=16384)
    ap.add_argument("--cpu-updates", type=int, default=32_000_000, help="size of the CPU baseline sample (about 10 s on 16 threads)")
    ap.add_argument("--skip-cpu", action="store_true")
    ap.add_argument("--skip-cached", action="store_true")
    ap.add_argument("--skip-coherent", action="store_true", help="profiling aid: time only the cached-rows leg")
    ap.add_argument("--skip-exact", action="store_true", help="skip the leg with every row update carried out (no thinning)")
    ap.add_argument("--hot-row-inflight", type=float, default=2.0, help="hot rows of the measured run are thinned to this many updates in flight (0 = no hot rows)")
    ap.add_argument("--hot-row-inflight-early", type=float, default=8.0, help="the same cap during the first epochs")
    ap.add_argument("--hot-row-early-epochs", type=int, default=2, help="number of epochs that run with the early cap")
    ap.add_argument("--pmc-copy", action="store_true",
                    help="profiling aid: also run three 1 GiB device copies, the known-size kernel that FETCH_SIZE / WRITE_SIZE are scaled by")
    ap.add_argument("--skip-fp32", action="store_true", help="skip the fp32-SGD leg")
    ap.add_argument("--skip-ceiling", action="store_true", help="skip the access-pattern probe")
    ap.add_argument("--every-rule", action="store_true",
                    help="also time every update kernel (fp32 SGD, MPT, MuPPET, AFP, mem_quant) for six epochs on the same workload")
    ap.add_argument("--reference-rmse", action="store_true",
                    help="also train with the reference rule on the CPU for warmup+steps epochs (minutes) and report the test RMSE delta")
    ap.add_argument("--seed", type=int, default=2021)
    a = ap.parse_args()
    if a.gpus != 1:
        print("bench.py: this build runs on one GPU only (one process, one device; sharding over several GPUs is a design "
              "note, not code); run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    import torch
    h = importlib.import_module("icdm-2021_mascot_amd").load()
    dev = torch.device("cuda:0")
    wc = CONFIGS[a.config]
    n_users, n_items, k = wc["n_users"], wc["n_items"], a.k
    a.ratings = a.ratings or wc["n_train"]
    a.workers = a.workers or h.mf_auto_workers(a.ratings)
    cfg = dict(epochs=50, lr=0.01, decay=0.1, lam=0.015, sample_ratio=0.05, interval=2, ug=100, ig=100)
    t0 = time.perf_counter()
    n_test = wc["n_test"]
    R = make_workload(torch, n_users, n_items, a.ratings + n_test, a.seed, dev, **{key: wc[key] for key in
                      ("user_alpha", "item_alpha", "rank", "noise", "mean", "step", "lo", "hi")})
    prob = MascotProblem(torch, h, R[:a.ratings].contiguous(), n_users, n_items, k, cfg["ug"], cfg["ig"], a.seed, test=R[a.ratings:].contiguous())
    del R
    torch.cuda.synchronize()
    setup_s = time.perf_counter() - t0
    # All groups are still binary16 in the measured epochs: a rating reads 12 B and two 256 B rows, and writes the
    # two rows back (1036 B) unless hot-row thinning skips a write (then that row is read only).
    read_bytes, row_bytes = 12 + 2 * k * 2, 2 * k * 2

    def leg(coherent, W, inflight_cap=0.0):
        h.mf_set_row_coherence(1 if coherent else 0)
        prob.set_hot_rows(W, inflight_cap, a.hot_row_inflight_early, a.hot_row_early_epochs)
        per, wall, uc, kept = time_steps(torch, prob, W, a.warmup, a.steps, cfg, a.seed)
        rmse = prob.rmse()
        prob.set_hot_rows(W, 0.0)
        updates = W * uc * 128
        ms = float(per.mean())
        bytes_per_update = read_bytes + row_bytes * kept
        return dict(ms_per_step=ms, ms_steps=[round(float(x), 3) for x in per], wall_s=wall, updates_per_step=updates,
                    ratings_per_s=a.ratings / (ms / 1e3), gbs=updates * bytes_per_update / (ms / 1e3) / 1e9, workers=W,
                    rmse=rmse, row_updates_kept=kept, bytes_per_update=bytes_per_update)

    if a.pmc_copy:
        src = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    main_leg = leg(False, a.cached_workers) if a.skip_coherent else leg(True, a.workers, a.hot_row_inflight)
    if a.skip_coherent:
        a.skip_cached = True
    out = {
        "metric": "SGD ratings/sec/epoch & % HBM roofline at k=128 on 1 MI355X; test RMSE delta",
        "value": main_leg["ratings_per_s"], "unit": "ratings/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": main_leg["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16", "data": "synthetic",
        "config": {"workload": "config %d: %s, %d train ratings; MASCOT -v 1 -k %d -ug 100 -ig 100 -s 0.05 -it 2 -e 20"
                               % (a.config, wc["text"], a.ratings, k),
                   "workers": main_leg["workers"], "row_access": "cached" if a.skip_coherent else "device-coherent", "update_vector_size": 128,
                   "epochs_timed": "%d..%d of 50" % (a.warmup, a.warmup + a.steps - 1), "seed": a.seed,
                   "hot_row_inflight": 0.0 if a.skip_coherent else a.hot_row_inflight,
                   "hot_row_inflight_early": 0.0 if a.skip_coherent else a.hot_row_inflight_early, "hot_row_early_epochs": a.hot_row_early_epochs,
                   "row_updates_carried_out": round(main_leg["row_updates_kept"], 4),
                   "user_groups": int(prob.sides[0]["groups"]), "item_groups": int(prob.sides[1]["groups"]), "setup_s": round(setup_s, 1)},
        "roofline": {"bound": "hbm", "achieved": main_leg["gbs"], "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": main_leg["gbs"] / PEAK_HBM_GBS,
                     "traffic": measured_traffic(a, main_leg),
                     "kernel": "hogwild_kernel<MascotRuleT<%d,%s,false>>" % (k, "false" if a.skip_coherent else "true"),
                     "bytes_per_update": round(main_leg["bytes_per_update"], 1),
                     "updates_per_launch": main_leg["updates_per_step"]},
        "ms_steps": main_leg["ms_steps"],
        "test_rmse_after_timed_epochs": {"value": main_leg["rmse"], "epochs": a.warmup + a.steps, "test_ratings": n_test},
    }
    recorded = RECORDED_REFERENCE_RMSE.get((a.config, a.ratings, k, a.seed, a.warmup + a.steps, main_leg["workers"]))
    if recorded is not None and not a.skip_coherent:
        out["test_rmse_delta"] = {"value": main_leg["rmse"] - recorded, "reference_rule_test_rmse": recorded,
                                  "source": "reference rule on the CPU, recorded from `bench.py --reference-rmse` with the same "
                                            "configuration, seed, epochs and workers (16 host threads)"}
    if not a.skip_ceiling:
        # what the memory system sustains for this epoch's addresses and store policy, beside the plain (non-check) epochs
        is_check = lambda e: e >= 5 and e % cfg["interval"] == 5 % cfg["interval"] and e != cfg["epochs"] - 1
        plain = [ms for i, ms in enumerate(main_leg["ms_steps"]) if not is_check(a.warmup + i)] or main_leg["ms_steps"]
        tables = None if a.skip_coherent or not a.hot_row_inflight else prob.hot_tables(main_leg["workers"], a.hot_row_inflight)
        ceil_ms = access_pattern_ceiling(torch, h, prob, main_leg["workers"], tables, not a.skip_coherent, a.seed)
        out["roofline"]["access_pattern_ceiling"] = {
            "note": "mf_row_traffic_probe: the same ratings, workers, hot-row tables and store policy, rows read and written "
                    "back without the arithmetic; kernel_vs_ceiling = this time / mean plain epoch",
            "ms": ceil_ms, "plain_epoch_ms": float(np.mean(plain)), "kernel_vs_ceiling": ceil_ms / float(np.mean(plain))}
    if not a.skip_coherent and not a.skip_exact and a.hot_row_inflight:
        e = leg(True, a.workers, 0.0)
        out["exact_coherent"] = {"note": "same workload, device-coherent rows, every row update carried out (no hot-row thinning): bound by "
                                         "the serialisation of accesses to the hottest row at the memory side",
                                 "value": e["ratings_per_s"], "unit": "ratings/s", "ms_per_step": e["ms_per_step"], "workers": e["workers"],
                                 "roofline_frac": e["gbs"] / PEAK_HBM_GBS, "test_rmse_after_timed_epochs": e["rmse"]}
    if not a.skip_cached:
        c = leg(False, a.cached_workers)
        out["cached_rows"] = {"note": "same workload with ordinary cached row accesses (each XCD trains its own L2-resident copy of hot "
                                      "rows; faster, converges worse); its algorithmic bytes can exceed the HBM peak because "
                                      "hot rows are served and overwritten in L2 without reaching memory",
                              "value": c["ratings_per_s"], "unit": "ratings/s", "ms_per_step": c["ms_per_step"], "workers": c["workers"],
                              "roofline": {"bound": "hbm", "achieved": c["gbs"], "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": c["gbs"] / PEAK_HBM_GBS,
                                           "kernel": "hogwild_kernel<MascotRuleT<%d,false,false>>" % k},
                              "ms_steps": c["ms_steps"], "test_rmse_after_timed_epochs": c["rmse"]}
        h.mf_set_row_coherence(1)
    if not a.skip_fp32 and not a.skip_coherent:
        h.mf_set_row_coherence(1)
        prob.set_hot_rows(a.workers, a.hot_row_inflight, a.hot_row_inflight_early, a.hot_row_early_epochs)
        per, uc, rmse, kept = time_fp32_sgd(torch, h, prob, a.workers, a.warmup, a.steps, cfg, a.seed)
        prob.set_hot_rows(a.workers, 0.0)
        ms = float(per.mean())
        bpu = 12 + 2 * k * 4 + 2 * k * 4 * kept
        out["fp32_sgd"] = {"note": "fp32 SGD (-v 5) on the same ratings, workers, row access and hot-row tables",
                           "value": a.ratings / (ms / 1e3), "unit": "ratings/s", "ms_per_step": ms, "workers": a.workers,
                           "roofline_frac": a.workers * uc * 128 * bpu / (ms / 1e3) / 1e9 / PEAK_HBM_GBS,
                           "test_rmse_after_timed_epochs": rmse, "mascot_speedup": ms / main_leg["ms_per_step"]}
    if a.every_rule and not a.skip_coherent:
        h.mf_set_row_coherence(1)
        prob.set_hot_rows(a.workers, a.hot_row_inflight, a.hot_row_inflight_early, a.hot_row_early_epochs)
        out["every_rule"] = time_every_rule(torch, h, prob, a.workers, cfg, a.seed)
        prob.set_hot_rows(a.workers, 0.0)
    if a.reference_rmse:
        threads = min(os.cpu_count() or 1, 16)
        ref = reference_rule_rmse(prob, h, cfg, a.seed, threads, a.warmup + a.steps, a.workers)
        out["reference_rule"] = {"test_rmse": ref, "epochs": a.warmup + a.steps, "threads": threads,
                                 "rmse_delta": main_leg["rmse"] - ref}
        out["test_rmse_delta"] = {"value": main_leg["rmse"] - ref, "reference_rule_test_rmse": ref,
                                  "source": "reference rule on the CPU, computed in this run (%d host threads)" % threads}
    if not a.skip_cpu:
        threads = min(os.cpu_count() or 1, 16)
        prob.reset()
        rate, done, dt = cpu_baseline(prob, cfg, a.seed, threads, a.cpu_updates)
        out["cpu_baseline"] = {"value": rate, "unit": "ratings/s", "cores": threads, "kind": "port",
                               "sample": "%d updates of the same shuffled ratings and binary16 model (%d workers x %d windows of 128), "
                                         "%.1f s, OpenMP Hogwild loop of the checker" % (done, threads * 8, done // (threads * 8 * 128), dt)}
        if not a.skip_fp32:
            rate, done, dt = cpu_baseline_fp32(prob, h, cfg, a.seed, threads, a.cpu_updates // 2)
            out["cpu_baseline"]["fp32_sgd"] = {"value": rate, "unit": "ratings/s", "cores": threads, "kind": "port",
                                               "sample": "%d updates of the same shuffled ratings, dense fp32 model, %.1f s" % (done, dt)}
    print(json.dumps(out))


if __name__ == "__main__":
    main()
