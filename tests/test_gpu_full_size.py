"""The hot path at BASELINE.json's full size (configuration 4: 480,000 x 17,800, 100M training ratings), checked through
properties that do not need a CPU run of that size: range independence of the generator, exact integer invariants of
the pre-processing kernels, and an epoch with learning rate 0, which must leave every value of the model as it was
(every row address of 100M updates stays inside its row) before a real epoch lowers the test RMSE."""
import ctypes as C
import os
import sys

import numpy as np
import pytest

import mfutil

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def full():
    import torch
    sys.path.insert(0, ROOT)
    import bench
    h = mfutil.hip()
    c = h.synth_config(4)
    n, nt = int(c.n_train), int(c.n_test)
    R = torch.empty((n + nt, 3), dtype=torch.int32, device="cuda")
    h.mf_generate_ratings(C.addressof(c), 2021, 0, n + nt, R.data_ptr(), mfutil.stream_ptr())
    return dict(torch=torch, bench=bench, h=h, c=c, n=n, nt=nt, R=R)


def test_generator_ranges_and_marginals(full):
    torch, h, c, n, R = full["torch"], full["h"], full["c"], full["n"], full["R"]
    # two halves generated on their own are the two halves of the stream
    half = torch.empty((n // 2, 3), dtype=torch.int32, device="cuda")
    for first in (0, n // 2):
        h.mf_generate_ratings(C.addressof(c), 2021, first, n // 2, half.data_ptr(), mfutil.stream_ptr())
        assert torch.equal(half, R[first:first + n // 2])
    u, i, r = R[:n, 1], R[:n, 2], R[:n, 0].view(torch.float32)
    assert int(u.max()) < c.n_users and int(i.max()) < c.n_items and int(u.min()) >= 0 and int(i.min()) >= 0
    assert torch.equal(torch.unique(r), torch.arange(1, 6, device="cuda", dtype=torch.float32))
    # the most popular item's share is the Zipf(1.1) head: 1 / sum_j j^-1.1 over 17,800 items
    share = 1.0 / float((torch.arange(1, c.n_items + 1, dtype=torch.float64) ** -1.1).sum())
    top = int(torch.bincount(i).max())
    assert abs(top - n * share) < 6 * np.sqrt(n * share)


def test_preprocessing_invariants(full):
    torch, h, c, n = full["torch"], full["h"], full["c"], full["n"]
    st = mfutil.stream_ptr()
    R = full["R"][:n].contiguous()
    # shuffle: a permutation of the ratings (checksums of keyed sums agree, order differs)
    S = torch.empty_like(R)
    h.mf_shuffle_ratings(R.data_ptr(), S.data_ptr(), n, 77, st)
    key = lambda X: (X[:, 0].to(torch.int64) * 1000003 + X[:, 1].to(torch.int64) * 7919 + X[:, 2].to(torch.int64))
    ka, kb = key(R), key(S)
    assert int(ka.sum()) == int(kb.sum()) and int((ka * ka % 1000000007).sum()) == int((kb * kb % 1000000007).sum())
    assert not torch.equal(R[:1000], S[:1000])
    # histogram: exact counts
    ucnt = torch.zeros(c.n_users, dtype=torch.int32, device="cuda")
    icnt = torch.zeros(c.n_items, dtype=torch.int32, device="cuda")
    h.mf_user_item_histogram(S.data_ptr(), n, ucnt.data_ptr(), icnt.data_ptr(), st)
    assert torch.equal(ucnt.to(torch.int64), torch.bincount(S[:, 1], minlength=c.n_users))
    assert torch.equal(icnt.to(torch.int64), torch.bincount(S[:, 2], minlength=c.n_items))
    # sort by count: ascending, stable, a permutation of the ids
    for cnt, num in ((ucnt, c.n_users), (icnt, c.n_items)):
        idx = torch.empty(num, dtype=torch.int32, device="cuda")
        h.mf_init_idx_arr(idx.data_ptr(), num, st)
        before = cnt.clone()
        h.mf_sort_by_count(cnt.data_ptr(), idx.data_ptr(), num, st)
        assert bool((cnt[1:] >= cnt[:-1]).all())
        assert torch.equal(torch.sort(idx.to(torch.int64)).values, torch.arange(num, device="cuda"))
        assert torch.equal(before[idx.to(torch.int64)], cnt)
        ties = cnt[1:] == cnt[:-1]
        assert bool((idx[1:][ties] > idx[:-1][ties]).all())
        # re-index with the inverse permutation and back
    del S, ka, kb


def test_epoch_with_zero_learning_rate_changes_nothing_then_training_learns(full):
    torch, bench, h, n = full["torch"], full["bench"], full["h"], full["n"]
    R = full["R"]
    prob = bench.MascotProblem(torch, h, R[:n].contiguous(), 480_000, 17_800, 128, 100, 100, 2021, test=R[n:].contiguous())
    W = h.mf_auto_workers(n)
    prob.alloc_stats(W)
    before = [s["arena"].clone() for s in prob.sides]
    rmse0 = prob.rmse()
    prob.set_hot_rows(W, 2.0, 8.0, 2)
    for e in (0, 5):                      # an early plain epoch (cap 8) and a check epoch (sampled launch, cap 2)
        prob.select_hot_rows(e)
        prob.epoch(e, W, 50, 0.0, 0.1, 0.015, 0.05, 2, 2021)
    torch.cuda.synchronize()
    for s, b in zip(prob.sides, before):
        # value for value; the only bytes that may differ are signs of zeros (-0 + lr * g = +0 when lr = 0)
        even = s["arena"].numel() // 2 * 2
        now, was = s["arena"][:even].view(torch.float16), b[:even].view(torch.float16)
        assert bool((now == was).all())
        assert bool((was[now.view(torch.int16) != was.view(torch.int16)] == 0).all())
    assert abs(prob.rmse() - rmse0) < 1e-9                     # partial sums meet in a different order
    # the sampled sums of the check epoch are finite and non-zero for binary16 groups
    assert bool(torch.isfinite(prob.stats["gsp"]).all()) and float(prob.stats["nsp"].sum()) > 0
    # two real epochs: the test RMSE falls
    for e in (0, 1):
        prob.select_hot_rows(e)
        prob.epoch(e, W, 50, 0.01, 0.1, 0.015, 0.05, 2, 2021)
    r2 = prob.rmse()
    prob.set_hot_rows(W, 0.0)
    assert np.isfinite(r2) and r2 < rmse0 - 0.5
