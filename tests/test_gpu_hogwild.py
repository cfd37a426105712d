"""GPU parity of the five Hogwild update kernels against the CPU checker, through the C ABI.

Schedules are conflict-free (each worker owns its users and items), so any interleaving of the
wavefronts must equal the checker's sequential run.  Bar: bit-exact for every variant (the kernels
reproduce the reference's order of roundings); sampled float sums that go through atomics are compared
to 1e-5 relative."""
import ctypes as C

import numpy as np
import pytest

import mfutil
from mfutil import to_dev, from_dev

pytestmark = pytest.mark.gpu

LR, LAM = 0.01, 0.05


def _run_dense(variant, k, R, starts, P, Q, uc, window, extra=()):
    h = mfutil.hip()
    W = starts.shape[1]
    dR, dS, dP, dQ = to_dev(R), to_dev(starts), to_dev(P), to_dev(Q)
    fn = getattr(h, "mf_%s_sgd_hogwild" % variant)
    fn(dR.data_ptr(), R.size, dP.data_ptr(), dQ.data_ptr(), k, W, uc, window, *extra, 1234, 0, dS.data_ptr(), mfutil.stream_ptr())
    import torch
    torch.cuda.synchronize()
    return from_dev(dP, np.float32, P.shape), from_dev(dQ, np.float32, Q.shape)


@pytest.mark.parametrize("k", [64, 128])
@pytest.mark.parametrize("W,uc,window", [(1, 1, 1), (6, 3, 128), (9, 2, 70), (64, 2, 128)])
def test_sgd_fp32_bit_exact(orc, k, W, uc, window):
    R, starts, P, Q = mfutil.conflict_free_problem(10 + k + W, k, W, uc, window)
    gp, gq = _run_dense("single", k, R, starts, P, Q, uc, window, (LR, LAM))
    orc.lib.orc_sgd_epoch(k, R.ctypes.data, R.size, P.ctypes.data, Q.ctypes.data, W, uc, window, LR, LAM, 0, 0, starts.ctypes.data, 1)
    assert np.array_equal(gp.view(np.uint32), P.view(np.uint32))
    assert np.array_equal(gq.view(np.uint32), Q.view(np.uint32))


@pytest.mark.parametrize("k", [64, 128])
@pytest.mark.parametrize("W,uc,window", [(1, 1, 1), (6, 3, 128), (9, 2, 70), (64, 2, 128)])
def test_mem_quant_bit_exact(orc, k, W, uc, window):
    """-v 7: dense binary16 rows, binary32 arithmetic, per-lane products summed left to right."""
    import torch
    h = mfutil.hip()
    R, starts, P, Q = mfutil.conflict_free_problem(15 + k + W, k, W, uc, window)
    Ph, Qh = orc.f2h(P).reshape(P.shape), orc.f2h(Q).reshape(Q.shape)
    dR, dS, dP, dQ = to_dev(R), to_dev(starts), to_dev(Ph), to_dev(Qh)
    h.mf_mem_quant_sgd_hogwild(dR.data_ptr(), R.size, dP.data_ptr(), dQ.data_ptr(), k, W, uc, window, LR, LAM, 1234, 0, dS.data_ptr(), mfutil.stream_ptr())
    torch.cuda.synchronize()
    orc.lib.orc_mem_quant_epoch(k, R.ctypes.data, R.size, Ph.ctypes.data, Qh.ctypes.data, W, uc, window, LR, LAM, 0, 0, starts.ctypes.data, 1)
    assert np.array_equal(from_dev(dP, np.uint16, P.shape), Ph)
    assert np.array_equal(from_dev(dQ, np.uint16, Q.shape), Qh)


@pytest.mark.parametrize("k", [64, 128])
@pytest.mark.parametrize("W,uc,window", [(1, 1, 1), (7, 3, 128), (64, 2, 128)])
def test_mpt_bit_exact(orc, k, W, uc, window):
    R, starts, P, Q = mfutil.conflict_free_problem(20 + k + W, k, W, uc, window)
    # MPT's master copy starts from binary16-representable values (main.cu:152-153, mf_methods.cu:730-733)
    P = orc.h2f(orc.f2h(P)); Q = orc.h2f(orc.f2h(Q))
    lam_h = orc.lib.orc_float2half(np.float32(LAM) * np.float32(1000.0))
    gp, gq = _run_dense("mpt", k, R, starts, P, Q, uc, window, (LR, lam_h, 1000.0))
    orc.lib.orc_mpt_epoch(k, R.ctypes.data, R.size, P.ctypes.data, Q.ctypes.data, W, uc, window, LR, LAM, 1000.0, 0, 0, starts.ctypes.data, 1)
    assert np.array_equal(gp.view(np.uint32), P.view(np.uint32))
    assert np.array_equal(gq.view(np.uint32), Q.view(np.uint32))


@pytest.mark.parametrize("k", [64, 128])
@pytest.mark.parametrize("bits", [8, 12, 14, 16, 32])
def test_muppet_bit_exact(orc, k, bits):
    W, uc, window = 10, 2, 128
    R, starts, P, Q = mfutil.conflict_free_problem(30 + k + bits, k, W, uc, window)
    first_sample = window  # second window of every worker is sampled
    import torch
    h = mfutil.hip()
    dR, dS, dP, dQ = to_dev(R), to_dev(starts), to_dev(P), to_dev(Q)
    d_sum = torch.zeros(k, dtype=torch.float32, device="cuda")
    d_norm = torch.full((W,), -7.0, dtype=torch.float32, device="cuda")
    h.mf_muppet_sgd_hogwild(dR.data_ptr(), R.size, dP.data_ptr(), dQ.data_ptr(), k, W, uc, window, LR, LAM, first_sample,
                            d_sum.data_ptr(), d_norm.data_ptr(), bits, bits, 0, 0, dS.data_ptr(), mfutil.stream_ptr())
    torch.cuda.synchronize()
    sum_ref = np.zeros(k, np.float32)
    norm_ref = np.zeros(W, np.float32)
    orc.lib.orc_muppet_epoch(k, R.ctypes.data, R.size, P.ctypes.data, Q.ctypes.data, W, uc, window, LR, LAM, first_sample,
                             sum_ref.ctypes.data, norm_ref.ctypes.data, bits, bits, 0, 0, starts.ctypes.data, 1)
    assert np.array_equal(from_dev(dP, np.float32, P.shape).view(np.uint32), P.view(np.uint32))
    assert np.array_equal(from_dev(dQ, np.float32, Q.shape).view(np.uint32), Q.view(np.uint32))
    assert np.array_equal(d_norm.cpu().numpy().view(np.uint32), norm_ref.view(np.uint32))
    got = d_sum.cpu().numpy()
    if bits == 32:
        assert np.all(got == 0) and np.all(sum_ref == 0)
    else:
        scale = np.abs(sum_ref).max()
        assert np.allclose(got, sum_ref, rtol=1e-5, atol=1e-5 * scale)


@pytest.mark.parametrize("k", [64, 128])
@pytest.mark.parametrize("afp_epoch", [0, 3])
def test_afp_bit_exact(orc, k, afp_epoch):
    W, uc, window = 10, 3, 128
    R, starts, P, Q = mfutil.conflict_free_problem(40 + k + afp_epoch, k, W, uc, window)
    gp, gq = _run_dense("afp", k, R, starts, P, Q, uc, window, (LR, LAM, afp_epoch))
    orc.lib.orc_afp_epoch(k, R.ctypes.data, R.size, P.ctypes.data, Q.ctypes.data, W, uc, window, LR, LAM, afp_epoch, 0, 0, starts.ctypes.data, 1)
    assert np.array_equal(gp.view(np.uint32), P.view(np.uint32))
    assert np.array_equal(gq.view(np.uint32), Q.view(np.uint32))


def _special_rows(seed, k, nan_elements=False):
    """A conflict-free problem whose workers own rows with special contents: all zeros (scale index 0 by definition),
    huge values (the int8 conversion saturates), infinities (a ratio of 0, whose logarithm is -inf), exact .5 ties
    after scaling (roundf's halves away from zero) and tiny values (scale indices near 100).  nan_elements: a seventh
    worker whose otherwise ordinary rows hold a NaN element each (the extrema drop it, as fmaxf does; its int8 value
    is 0)."""
    W, uc, window = 7 if nan_elements else 6, 1, 128
    R, starts, P, Q = mfutil.conflict_free_problem(seed, k, W, uc, window)
    if nan_elements:
        up, ip = P.shape[0] // W, Q.shape[0] // W
        P[6 * up:7 * up:2, 5] = np.nan; Q[6 * ip:7 * ip:3, k - 3] = np.nan
    up, ip = P.shape[0] // W, Q.shape[0] // W
    P[1 * up] = 0.0; Q[1 * ip] = 0.0; P[1 * up + 1] = 0.0
    P[2 * up, ::3] = 1e30; Q[2 * ip, 1::5] = -3e29
    Q[3 * ip, 7] = np.inf; P[3 * up, 11] = -np.inf
    P[4 * up] = (np.arange(k) % 9 - 4).astype(np.float32) * 0.0625 + 0.03125; Q[4 * ip] = 0.5 - (np.arange(k) % 5) * 0.25
    P[5 * up:6 * up] *= 1e-29; Q[5 * ip:6 * ip] *= 1e-29
    return R, starts, P, Q, uc, window


def _same_values(got, want):
    """Bit-exact where the checker's value is a number; the same positions hold NaN (payloads are not compared)."""
    nan = np.isnan(want)
    return np.array_equal(np.isnan(got), nan) and np.array_equal(got.view(np.uint32)[~nan], want.view(np.uint32)[~nan])


def _half_edge_rows(seed, k):
    """A conflict-free problem whose workers own rows at the edges of binary16: zeros, values whose products and
    scaled gradients overflow binary16, values in its subnormal range, and an infinity."""
    W, uc, window = 5, 1, 128
    R, starts, P, Q = mfutil.conflict_free_problem(seed, k, W, uc, window)
    up, ip = P.shape[0] // W, Q.shape[0] // W
    P[1 * up] = 0.0; Q[1 * ip] = -0.0
    P[2 * up:3 * up] *= 3000.0; Q[2 * ip:3 * ip] *= 2000.0
    P[3 * up:4 * up] *= 3e-5; Q[3 * ip:4 * ip] *= 1e-4
    Q[4 * ip, 3] = np.inf
    return R, starts, P, Q, uc, window


@pytest.mark.parametrize("k", [64, 128])
@pytest.mark.parametrize("variant", ["single", "mpt", "mem_quant"])
def test_dense_rules_special_values(orc, k, variant):
    """fp32 SGD, MPT (binary16 arithmetic on values scaled by 1000) and -v 7 (binary16 storage) on such rows."""
    import torch
    h = mfutil.hip()
    R, starts, P, Q, uc, window = _half_edge_rows(900 + k, k)
    W = starts.shape[1]
    with np.errstate(all="ignore"):
        if variant == "mem_quant":
            Ph, Qh = orc.f2h(P).reshape(P.shape), orc.f2h(Q).reshape(Q.shape)
            dR, dS, dP, dQ = to_dev(R), to_dev(starts), to_dev(Ph), to_dev(Qh)
            h.mf_mem_quant_sgd_hogwild(dR.data_ptr(), R.size, dP.data_ptr(), dQ.data_ptr(), k, W, uc, window, LR, LAM, 1234, 0, dS.data_ptr(), mfutil.stream_ptr())
            torch.cuda.synchronize()
            orc.lib.orc_mem_quant_epoch(k, R.ctypes.data, R.size, Ph.ctypes.data, Qh.ctypes.data, W, uc, window, LR, LAM, 0, 0, starts.ctypes.data, 1)
            assert _same_storage(from_dev(dP, np.uint16, P.shape), Ph)
            assert _same_storage(from_dev(dQ, np.uint16, Q.shape), Qh)
            return
        if variant == "mpt":
            P = orc.h2f(orc.f2h(P)).reshape(P.shape); Q = orc.h2f(orc.f2h(Q)).reshape(Q.shape)
            lam_h = orc.lib.orc_float2half(np.float32(LAM) * np.float32(1000.0))
            gp, gq = _run_dense("mpt", k, R, starts, P, Q, uc, window, (LR, lam_h, 1000.0))
            orc.lib.orc_mpt_epoch(k, R.ctypes.data, R.size, P.ctypes.data, Q.ctypes.data, W, uc, window, LR, LAM, 1000.0, 0, 0, starts.ctypes.data, 1)
        else:
            gp, gq = _run_dense("single", k, R, starts, P, Q, uc, window, (LR, LAM))
            orc.lib.orc_sgd_epoch(k, R.ctypes.data, R.size, P.ctypes.data, Q.ctypes.data, W, uc, window, LR, LAM, 0, 0, starts.ctypes.data, 1)
    assert _same_values(gp, P)
    assert _same_values(gq, Q)


@pytest.mark.parametrize("k", [64, 128])
@pytest.mark.parametrize("bits", [8, 16])
def test_muppet_special_values(orc, k, bits):
    """The saturating conversions and the scale index on inputs that reach their edges (zeros, saturation, infinities,
    ties, very small values): the kernel uses the hardware's conversions, the checker spells CUDA's cast rules out."""
    import torch
    h = mfutil.hip()
    R, starts, P, Q, uc, window = _special_rows(700 + k + bits, k, nan_elements=True)
    W = starts.shape[1]
    dR, dS, dP, dQ = to_dev(R), to_dev(starts), to_dev(P), to_dev(Q)
    d_sum = torch.zeros(k, dtype=torch.float32, device="cuda")
    d_norm = torch.zeros(W, dtype=torch.float32, device="cuda")
    h.mf_muppet_sgd_hogwild(dR.data_ptr(), R.size, dP.data_ptr(), dQ.data_ptr(), k, W, uc, window, LR, LAM, uc * window,
                            d_sum.data_ptr(), d_norm.data_ptr(), bits, bits, 0, 0, dS.data_ptr(), mfutil.stream_ptr())
    torch.cuda.synchronize()
    sum_ref, norm_ref = np.zeros(k, np.float32), np.zeros(W, np.float32)
    with np.errstate(all="ignore"):
        orc.lib.orc_muppet_epoch(k, R.ctypes.data, R.size, P.ctypes.data, Q.ctypes.data, W, uc, window, LR, LAM, uc * window,
                                 sum_ref.ctypes.data, norm_ref.ctypes.data, bits, bits, 0, 0, starts.ctypes.data, 1)
    assert _same_values(from_dev(dP, np.float32, P.shape), P)
    assert _same_values(from_dev(dQ, np.float32, Q.shape), Q)


@pytest.mark.parametrize("k", [64, 128])
def test_afp_special_values(orc, k):
    R, starts, P, Q, uc, window = _special_rows(800 + k, k)
    W = starts.shape[1]
    gp, gq = _run_dense("afp", k, R, starts, P, Q, uc, window, (LR, LAM, 0))
    orc.lib.orc_afp_epoch(k, R.ctypes.data, R.size, P.ctypes.data, Q.ctypes.data, W, uc, window, LR, LAM, 0, 0, 0, starts.ctypes.data, 1)
    assert _same_values(gp, P)
    assert _same_values(gq, Q)


def _mascot_case(orc, k, W, uc, window, user_groups, item_groups, prec_mode, first_sample, seed, lr=LR, row_classes=None, all_binary16=0, step_scale=0.0, resident_workers=0):
    """row_classes: keep-table values drawn at random per row (mf_hogwild_options); with them the call goes through the
    _opt entry point, with the all_binary16 hint, the step factor of replicated rows' copies and the cap on resident
    workers as given."""
    import torch
    h = mfutil.hip()
    R, starts, P, Q = mfutil.conflict_free_problem(seed, k, W, uc, window)
    n_users, n_items = P.shape[0], Q.shape[0]
    uend, iend = mfutil.equal_end_idx(n_users, user_groups), mfutil.equal_end_idx(n_items, item_groups)
    rng = np.random.default_rng(seed)
    if prec_mode == "half":
        uprec, iprec = np.zeros(user_groups, np.uint8), np.zeros(item_groups, np.uint8)
    elif prec_mode == "float":
        uprec, iprec = np.ones(user_groups, np.uint8), np.ones(item_groups, np.uint8)
    else:
        uprec, iprec = rng.integers(0, 2, user_groups).astype(np.uint8), rng.integers(0, 2, item_groups).astype(np.uint8)
    gmp, gmq = mfutil.host_grouped(orc, k, P, uend, uprec), mfutil.host_grouped(orc, k, Q, iend, iprec)
    dp, dq = mfutil.DeviceGrouped(gmp), mfutil.DeviceGrouped(gmq)
    nb = h.mf_mascot_norm_blocks(W)
    dR, dS = to_dev(R), to_dev(starts)
    d_gsp = torch.zeros(user_groups * k, dtype=torch.float32, device="cuda")
    d_gsq = torch.zeros(item_groups * k, dtype=torch.float32, device="cuda")
    d_nsp = torch.full((user_groups * nb,), -3.0, dtype=torch.float32, device="cuda")
    d_nsq = torch.full((item_groups * nb,), -3.0, dtype=torch.float32, device="cuda")
    args = (dR.data_ptr(), R.size, dp.ptrs.data_ptr(), dq.ptrs.data_ptr(), k, W, uc, window, lr, LAM,
            dp.end.data_ptr(), dq.end.data_ptr(), dp.prec.data_ptr(), dq.prec.data_ptr(),
            d_gsp.data_ptr(), d_gsq.data_ptr(), d_nsp.data_ptr(), d_nsq.data_ptr(),
            first_sample, user_groups, item_groups, 0, 0, dS.data_ptr(), mfutil.stream_ptr())
    if row_classes is None and not all_binary16 and not resident_workers:
        h.mf_mascot_sgd_hogwild(*args)
    else:
        values = np.array(row_classes if row_classes is not None else [255], np.uint8)
        keep = [values[rng.integers(0, values.size, n)] for n in (n_users, n_items)] if row_classes is not None else [None, None]
        opt = mfutil.HogwildOptions(k, keep[0], keep[1], launches=2, step_scale=step_scale)
        opt.o.all_binary16 = all_binary16
        opt.o.resident_workers = resident_workers
        h.mf_mascot_sgd_hogwild_opt(*args, opt.ptr)
    torch.cuda.synchronize()
    gsp, gsq = np.zeros(user_groups * k, np.float32), np.zeros(item_groups * k, np.float32)
    nsp, nsq = np.zeros(user_groups, np.float32), np.zeros(item_groups, np.float32)
    orc.lib.orc_mascot_epoch(k, R.ctypes.data, R.size, gmp.ptrs, gmq.ptrs, gmp.end_idx.ctypes.data, gmq.end_idx.ctypes.data,
                             gmp.prec.ctypes.data, gmq.prec.ctypes.data, user_groups, item_groups, W, uc, window, lr, LAM,
                             first_sample, gsp.ctypes.data, gsq.ctypes.data, nsp.ctypes.data, nsq.ctypes.data,
                             0, 0, starts.ctypes.data, 1)
    for got, want in zip(dp.download() + dq.download(), gmp.arrays + gmq.arrays):
        assert got.dtype == want.dtype
        assert np.array_equal(got.view(np.uint8), want.view(np.uint8))
    got_nsp = d_nsp.cpu().numpy().reshape(user_groups, nb).astype(np.float64).sum(1)
    got_nsq = d_nsq.cpu().numpy().reshape(item_groups, nb).astype(np.float64).sum(1)
    assert np.allclose(got_nsp, nsp, rtol=1e-5, atol=1e-7)
    assert np.allclose(got_nsq, nsq, rtol=1e-5, atol=1e-7)
    for got, want in ((d_gsp.cpu().numpy(), gsp), (d_gsq.cpu().numpy(), gsq)):
        scale = max(np.abs(want).max(), 1e-6)
        assert np.allclose(got, want, rtol=1e-5, atol=2e-5 * scale)
    return nsp, nsq


@pytest.mark.parametrize("k", [64, 128])
@pytest.mark.parametrize("prec_mode", ["half", "float", "mixed"])
def test_mascot_bit_exact(orc, k, prec_mode):
    W, uc, window = 12, 3, 128
    nsp, nsq = _mascot_case(orc, k, W, uc, window, 7, 5, prec_mode, first_sample=2 * window - 40, seed=50 + k)
    if prec_mode == "half":
        assert nsp.sum() > 0 and nsq.sum() > 0
    if prec_mode == "float":
        assert nsp.sum() == 0 and nsq.sum() == 0


@pytest.mark.parametrize("k", [64, 128])
@pytest.mark.parametrize("prec_mode", ["half", "mixed", "float"])
def test_mascot_row_classes_and_hints_keep_the_checkers_result(orc, k, prec_mode):
    """The straight-line path for chunks of mixed precisions and the kernel build for all-binary16 runs with the hot-row
    code in them.  Every worker owns its rows, so a replicated row (253) changes in one XCD's copy only and the merge
    returns that copy: with ordinary and replicated rows mixed at random the result is the checker's, bit for bit --
    whatever the all_binary16 hint says (a wrong hint sends mixed chunks down the general path: slower, not different),
    and with a step factor for the copies as long as the launch is one workgroup (one copy in play: factor 1)."""
    W, uc, window = 12, 3, 128
    for hint in (0, 1):
        _mascot_case(orc, k, W, uc, window, 7, 5, prec_mode, first_sample=2 * window - 40, seed=150 + k, row_classes=(255, 253), all_binary16=hint)
        _mascot_case(orc, k, W, uc, window, 7, 5, prec_mode, first_sample=uc * window, seed=151 + k, all_binary16=hint)
    _mascot_case(orc, k, 4, uc, window, 7, 5, prec_mode, first_sample=2 * window - 40, seed=152 + k, row_classes=(255, 253), step_scale=4.0)


@pytest.mark.parametrize("k", [64, 128])
def test_resident_worker_cap_changes_when_not_what(orc, k):
    """mf_hogwild_options.resident_workers holds a launch to fewer resident workers by asking for LDS it does not use.
    1100 workers that own their rows, held to one workgroup per compute unit: the results are the checker's bit for bit
    (fp32 SGD without tables; MASCOT with row classes, its own LDS tables inside the padded allocation).  And the number
    of updates in flight the library reports for such a launch: whole workgroups per compute unit, never more than the
    uncapped launch, unchanged for a launch that is below the cap anyway."""
    import torch
    h = mfutil.hip()
    W, uc, window = 1100, 1, 64
    R, starts, P, Q = mfutil.conflict_free_problem(170 + k, k, W, uc, window)
    dR, dS, dP, dQ = to_dev(R), to_dev(starts), to_dev(P), to_dev(Q)
    opt = mfutil.HogwildOptions(k)
    opt.o.resident_workers = 1
    h.mf_single_sgd_hogwild_opt(dR.data_ptr(), R.size, dP.data_ptr(), dQ.data_ptr(), k, W, uc, window, LR, LAM, 1234, 0, dS.data_ptr(), mfutil.stream_ptr(), opt.ptr)
    torch.cuda.synchronize()
    orc.lib.orc_sgd_epoch(k, R.ctypes.data, R.size, P.ctypes.data, Q.ctypes.data, W, uc, window, LR, LAM, 0, 0, starts.ctypes.data, 1)
    assert np.array_equal(from_dev(dP, np.float32, P.shape).view(np.uint32), P.view(np.uint32))
    assert np.array_equal(from_dev(dQ, np.float32, Q.shape).view(np.uint32), Q.view(np.uint32))
    _mascot_case(orc, k, W, uc, window, 7, 5, "mixed", first_sample=uc * window, seed=171 + k, row_classes=(255, 253), resident_workers=1)
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    for version, per_worker in ((5, 4), (1, 4), (3, 2)):
        full = h.lib.mf_hogwild_inflight(version, k, 1000000, 7, 5)
        assert full > 0 and full % (4 * cus * per_worker) == 0
        resident = int(full) // per_worker
        assert h.lib.mf_hogwild_inflight_capped(version, k, 1000000, 7, 5, 0) == full
        assert h.lib.mf_hogwild_inflight_capped(version, k, 1000000, 7, 5, resident) == full
        assert h.lib.mf_hogwild_inflight_capped(version, k, 1000000, 7, 5, 1) == 4 * cus * per_worker          # one workgroup per compute unit
        half = h.lib.mf_hogwild_inflight_capped(version, k, 1000000, 7, 5, resident // 2)
        assert half == (resident // 2) // (4 * cus) * (4 * cus) * per_worker
        assert h.lib.mf_hogwild_inflight_capped(version, k, 500, 7, 5, 100) == 500 * per_worker                 # 125 workgroups: below any cap


@pytest.mark.parametrize("k", [64, 128])
def test_mascot_sampled_ranges_in_pieces(orc, k):
    """More workers than the sampled launch has wavefronts (4096): every worker's sampled range is cut into pieces
    that different wavefronts play.  With a learning rate of 0 the model does not move, so the pieces may run in
    any order and the sums must still hold every sampled rating exactly once."""
    W, uc, window = 4100, 2, 192
    nsp, nsq = _mascot_case(orc, k, W, uc, window, 9, 6, "half", first_sample=100, seed=90 + k, lr=0.0)
    assert nsp.sum() > 0 and nsq.sum() > 0


@pytest.mark.parametrize("k", [64, 128])
def test_mascot_group_table_sizes(orc, k):
    # one group per side, and more groups than a 64-lane compare could hold
    _mascot_case(orc, k, 4, 1, 128, 1, 1, "half", first_sample=128, seed=61)
    _mascot_case(orc, k, 40, 1, 64, 150, 101, "mixed", first_sample=0, seed=62)
    # more groups than the sampled sums have room for in LDS: the whole epoch runs with the sums in global memory
    _mascot_case(orc, k, 100, 1, 64, 400, 350, "mixed", first_sample=10, seed=63)


@pytest.mark.parametrize("k", [64, 128])
def test_single_update_mascot_four_cases(orc, k):
    for up in (0, 1):
        for ip in (0, 1):
            import torch
            h = mfutil.hip()
            rng = np.random.default_rng(70 + 2 * up + ip)
            P = (rng.standard_normal((1, k)) * 0.1).astype(np.float32)
            Q = (rng.standard_normal((1, k)) * 0.1).astype(np.float32)
            R = np.zeros(1, mfutil.NODE); R["r"] = 4.0
            gmp = mfutil.host_grouped(orc, k, P, np.array([0], np.uint32), np.array([up], np.uint8))
            gmq = mfutil.host_grouped(orc, k, Q, np.array([0], np.uint32), np.array([ip], np.uint8))
            dp, dq = mfutil.DeviceGrouped(gmp), mfutil.DeviceGrouped(gmq)
            dR = to_dev(R); dS = to_dev(np.zeros((1, 1), np.uint32))
            z = torch.zeros(4 * k, dtype=torch.float32, device="cuda")
            h.mf_mascot_sgd_hogwild(dR.data_ptr(), 1, dp.ptrs.data_ptr(), dq.ptrs.data_ptr(), k, 1, 1, 1, LR, LAM,
                                    dp.end.data_ptr(), dq.end.data_ptr(), dp.prec.data_ptr(), dq.prec.data_ptr(),
                                    z.data_ptr(), z[k:].data_ptr(), z[2 * k:].data_ptr(), z[3 * k:].data_ptr(),
                                    1, 1, 1, 0, 0, dS.data_ptr(), mfutil.stream_ptr())
            torch.cuda.synchronize()
            orc.lib.orc_mascot_update(k, gmp.arrays[0].ctypes.data, up, gmq.arrays[0].ctypes.data, ip, 4.0, LR, LAM, None, None, None, None)
            assert np.array_equal(dp.download()[0].view(np.uint8), gmp.arrays[0].view(np.uint8)), (up, ip)
            assert np.array_equal(dq.download()[0].view(np.uint8), gmq.arrays[0].view(np.uint8)), (up, ip)


def _same_storage(got, want):
    """Bit-exact where the checker's value is a number; NaN in the same positions (payloads are not compared)."""
    if want.dtype == np.uint16:
        nan = (want & 0x7fff) > 0x7c00
        return np.array_equal((got & 0x7fff) > 0x7c00, nan) and np.array_equal(got[~nan], want[~nan])
    return _same_values(got.view(np.float32), want.view(np.float32))


@pytest.mark.parametrize("k", [64, 128])
@pytest.mark.parametrize("case", ["subnormal", "overflow", "largest", "zeros"])
def test_single_update_mascot_special_values(orc, k, case):
    """One update in each of the four precision cases on rows at the edges of binary16: products and sums in the
    subnormal range (nothing may be flushed to zero), values whose products overflow to infinity (and the NaN that
    follows), the largest finite binary16 value, and signed zeros."""
    import torch
    h = mfutil.hip()
    rng = np.random.default_rng(170 + k)
    g = rng.standard_normal((2, 1, k)).astype(np.float32)
    if case == "subnormal":
        P, Q, r = g[0] * 3e-6, g[1] * 0.5, 1e-5
    elif case == "overflow":
        P, Q, r = g[0] * 200.0, g[1] * 300.0, 4.0
    elif case == "largest":
        P, Q, r = np.full((1, k), 65504.0, np.float32), g[1] * 1e-3, 4.0
        P[0, ::2] = -65504.0
    else:
        P, Q, r = np.zeros((1, k), np.float32), g[1] * 0.1, 0.0
        P[0, ::3] = -0.0
    for up in (0, 1):
        for ip in (0, 1):
            R = np.zeros(1, mfutil.NODE); R["r"] = r
            gmp = mfutil.host_grouped(orc, k, P.astype(np.float32), np.array([0], np.uint32), np.array([up], np.uint8))
            gmq = mfutil.host_grouped(orc, k, Q.astype(np.float32), np.array([0], np.uint32), np.array([ip], np.uint8))
            dp, dq = mfutil.DeviceGrouped(gmp), mfutil.DeviceGrouped(gmq)
            dR = to_dev(R); dS = to_dev(np.zeros((1, 1), np.uint32))
            z = torch.zeros(4 * k, dtype=torch.float32, device="cuda")
            h.mf_mascot_sgd_hogwild(dR.data_ptr(), 1, dp.ptrs.data_ptr(), dq.ptrs.data_ptr(), k, 1, 1, 1, LR, LAM,
                                    dp.end.data_ptr(), dq.end.data_ptr(), dp.prec.data_ptr(), dq.prec.data_ptr(),
                                    z.data_ptr(), z[k:].data_ptr(), z[2 * k:].data_ptr(), z[3 * k:].data_ptr(),
                                    1, 1, 1, 0, 0, dS.data_ptr(), mfutil.stream_ptr())
            torch.cuda.synchronize()
            with np.errstate(all="ignore"):
                orc.lib.orc_mascot_update(k, gmp.arrays[0].ctypes.data, up, gmq.arrays[0].ctypes.data, ip, r, LR, LAM, None, None, None, None)
            assert _same_storage(dp.download()[0], gmp.arrays[0]), (case, up, ip)
            assert _same_storage(dq.download()[0], gmq.arrays[0]), (case, up, ip)


@pytest.mark.parametrize("k", [64, 128])
def test_counter_rng_schedule_matches_checker(orc, k):
    """window_start == NULL: the kernel's own generator must pick the windows the checker's twin picks."""
    h = mfutil.hip()
    rng = np.random.default_rng(80)
    R = mfutil.make_ratings(81, 50, 40, 3000)
    P = (rng.standard_normal((50, k)) * 0.1).astype(np.float32)
    Q = (rng.standard_normal((40, k)) * 0.1).astype(np.float32)
    for e in range(3):
        for w in range(5):
            assert h.mf_window_start(99, e, w, 7, R.size) == orc.lib.orc_window_start(99, e, w, 7, R.size)
    import torch
    dR, dP, dQ = to_dev(R), to_dev(P), to_dev(Q)
    h.mf_single_sgd_hogwild(dR.data_ptr(), R.size, dP.data_ptr(), dQ.data_ptr(), k, 1, 6, 128, LR, LAM, 99, 2, None, mfutil.stream_ptr())
    torch.cuda.synchronize()
    orc.lib.orc_sgd_epoch(k, R.ctypes.data, R.size, P.ctypes.data, Q.ctypes.data, 1, 6, 128, LR, LAM, 99, 2, None, 1)
    assert np.array_equal(from_dev(dP, np.float32, P.shape).view(np.uint32), P.view(np.uint32))
    assert np.array_equal(from_dev(dQ, np.float32, Q.shape).view(np.uint32), Q.view(np.uint32))


def test_window_wraps_past_end_of_ratings(orc):
    """nnz smaller than the window: offset = (start + i) % nnz wraps several times (sgd_kernel.h:33)."""
    k = 64
    rng = np.random.default_rng(90)
    R = mfutil.make_ratings(91, 6, 5, 50)
    P = (rng.standard_normal((6, k)) * 0.1).astype(np.float32)
    Q = (rng.standard_normal((5, k)) * 0.1).astype(np.float32)
    starts = np.array([[47], [3]], np.uint32)
    gp, gq = _run_dense("single", k, R, starts, P, Q, 2, 128, (LR, LAM))
    orc.lib.orc_sgd_epoch(k, R.ctypes.data, R.size, P.ctypes.data, Q.ctypes.data, 1, 2, 128, LR, LAM, 0, 0, starts.ctypes.data, 1)
    assert np.array_equal(gp.view(np.uint32), P.view(np.uint32))
    assert np.array_equal(gq.view(np.uint32), Q.view(np.uint32))


def test_argument_errors_launch_nothing():
    h = mfutil.hip()
    from importlib import import_module
    MfError = import_module("icdm-2021_mascot_amd.capi").MfError
    with pytest.raises(MfError, match="k must be 64 or 128"):
        h.mf_single_sgd_hogwild(1, 1, 1, 1, 32, 1, 1, 1, LR, LAM, 0, 0, None, None)
    with pytest.raises(MfError, match="empty rating array"):
        h.mf_single_sgd_hogwild(None, 0, 1, 1, 64, 1, 1, 1, LR, LAM, 0, 0, None, None)


@pytest.mark.parametrize("k", [64, 128])
@pytest.mark.parametrize("variant", ["single", "mascot", "mascot_ff", "mascot_hf"])
def test_hot_row_thinning_drops_whole_row_updates(orc, k, variant):
    """mf_hogwild_options keep tables: 255 = ordinary row, nothing changes; 254 = hot row, every update carried out (added
    in memory: with one update per row the sum equals the stored row, up to the extra rounding of the binary16
    change); 63 carries out a quarter of a row's updates, a skipped row is left untouched while the other side of
    the rating is updated exactly as without thinning."""
    import torch
    h = mfutil.hip()
    n = 4096
    rng = np.random.default_rng(123 + k)
    R = np.zeros(n, mfutil.NODE)
    R["u"], R["i"], R["r"] = np.arange(n), rng.permutation(n), rng.integers(1, 6, n)      # every row is touched exactly once
    P0 = (rng.standard_normal((n, k)) * 0.1).astype(np.float32)
    Q0 = (rng.standard_normal((n, k)) * 0.1).astype(np.float32)
    starts = np.arange(0, n, 128, dtype=np.uint32).reshape(-1, 1)          # one worker, consecutive windows
    uc = starts.shape[0]
    uprec = np.array([1 if variant == "mascot_ff" else 0], np.uint8)       # binary32 user rows / item rows
    iprec = np.array([0 if variant == "mascot" else 1], np.uint8)
    if variant != "single":
        if not uprec[0]:
            P0 = orc.h2f(orc.f2h(P0)).reshape(P0.shape)
        if not iprec[0]:
            Q0 = orc.h2f(orc.f2h(Q0)).reshape(Q0.shape)
        end = np.array([n - 1], np.uint32)

    def rows(a):
        return (a if a.dtype == np.float32 else orc.h2f(a)).reshape(n, k).astype(np.float32)

    def run(keep_u, keep_v):
        dR, dS = to_dev(R), to_dev(starts)
        opt = mfutil.HogwildOptions(k, np.full(n, keep_u, np.uint8), np.full(n, keep_v, np.uint8))
        if variant == "single":
            dP, dQ = to_dev(P0), to_dev(Q0)
            h.mf_single_sgd_hogwild_opt(dR.data_ptr(), n, dP.data_ptr(), dQ.data_ptr(), k, 1, uc, 128, LR, LAM, 5, 0, dS.data_ptr(), mfutil.stream_ptr(), opt.ptr)
            torch.cuda.synchronize()
            return from_dev(dP, np.float32, P0.shape), from_dev(dQ, np.float32, Q0.shape)
        gp = mfutil.host_grouped(orc, k, P0, end, uprec)
        gq = mfutil.host_grouped(orc, k, Q0, end, iprec)
        dp, dq = mfutil.DeviceGrouped(gp), mfutil.DeviceGrouped(gq)
        z = torch.zeros(4 * k + 16, dtype=torch.float32, device="cuda")
        h.mf_mascot_sgd_hogwild_opt(dR.data_ptr(), n, dp.ptrs.data_ptr(), dq.ptrs.data_ptr(), k, 1, uc, 128, LR, LAM,
                                    dp.end.data_ptr(), dq.end.data_ptr(), dp.prec.data_ptr(), dq.prec.data_ptr(),
                                    z.data_ptr(), z[k:].data_ptr(), z[2 * k:].data_ptr(), z[3 * k:].data_ptr(),
                                    uc * 128, 1, 1, 5, 0, dS.data_ptr(), mfutil.stream_ptr(), opt.ptr)
        torch.cuda.synchronize()
        return rows(dp.download()[0]), rows(dq.download()[0])

    # the checker's result with every update carried out
    if variant == "single":
        Pw, Qw = P0.copy(), Q0.copy()
        orc.lib.orc_sgd_epoch(k, R.ctypes.data, n, Pw.ctypes.data, Qw.ctypes.data, 1, uc, 128, LR, LAM, 5, 0, starts.ctypes.data, 1)
    else:
        gp = mfutil.host_grouped(orc, k, P0, end, uprec)
        gq = mfutil.host_grouped(orc, k, Q0, end, iprec)
        z = [np.zeros(k, np.float32) for _ in range(4)]
        orc.lib.orc_mascot_epoch(k, R.ctypes.data, n, gp.ptrs, gq.ptrs, gp.end_idx.ctypes.data, gq.end_idx.ctypes.data,
                                 gp.prec.ctypes.data, gq.prec.ctypes.data, 1, 1, 1, uc, 128, LR, LAM, uc * 128,
                                 z[0].ctypes.data, z[1].ctypes.data, z[2].ctypes.data, z[3].ctypes.data, 5, 0, starts.ctypes.data, 1)
        Pw, Qw = rows(gp.arrays[0]), rows(gq.arrays[0])

    def same(got, want, old, binary32=False):
        if variant == "single":                                     # fp32 SGD: old + change is the stored value
            return np.array_equal(got, want)
        # MASCOT: memory adds round(lr*g) to the row, the rule stores fma(lr, g, row); the extra rounding is the one of
        # the change, so the two are within one ulp (of the row's format) of the larger of the change and the result
        fmt = np.float32 if binary32 else np.float16
        scale = np.maximum(np.abs(want), np.abs(want - old)).astype(fmt)
        return np.all(np.abs(got.astype(np.float64) - want) <= np.spacing(scale).astype(np.float64))

    P1, Q1 = run(255, 255)
    assert np.array_equal(P1, Pw) and np.array_equal(Q1, Qw)
    P4, Q4 = run(254, 254)
    assert same(P4, Pw, P0, uprec[0]) and same(Q4, Qw, Q0, iprec[0])
    assert np.all(np.any(P4 != P0, axis=1)) and np.all(np.any(Q4 != Q0, axis=1))
    P2, Q2 = run(63, 255)
    assert np.array_equal(Q2, Qw)                                   # item side: every update, computed from the old user row
    changed = np.any(P2 != P0, axis=1)
    assert same(P2[changed], Pw[changed], P0[changed], uprec[0])                           # a user row is either untouched or fully updated
    assert np.array_equal(P2[~changed], P0[~changed])
    assert 0.20 < changed.mean() < 0.30                             # (63+1)/255 of the updates
    P3, Q3 = run(255, 0)
    assert np.array_equal(P3, Pw)
    assert np.any(Q3 != Q0, axis=1).mean() < 0.02                   # (0+1)/255
    # 253 = replicated rows: the one worker runs on one XCD, whose copies are the only ones that change, so the rows come
    # back as that XCD left them -- the reference rule's result, bit for bit (every update carried out, stored, not added)
    for sides in ((253, 255), (255, 253), (253, 253)):
        P5, Q5 = run(*sides)
        assert np.array_equal(P5, Pw) and np.array_equal(Q5, Qw), sides
    # 252 = replicated rows whose updates are added to the copy: as 254, through the copy and the merge
    P6, Q6 = run(252, 252)
    assert same(P6, Pw, P0, uprec[0]) and same(Q6, Qw, Q0, iprec[0])
    assert np.all(np.any(P6 != P0, axis=1)) and np.all(np.any(Q6 != Q0, axis=1))


@pytest.mark.parametrize("k", [64, 128])
@pytest.mark.parametrize("variant", ["single", "mpt", "muppet", "afp", "mem_quant"])
def test_chunks_with_skipped_updates_take_the_general_loop_to_the_same_rows(k, variant):
    """The dense rules run a chunk of 64 ratings in which no update is skipped in a loop without the selects for skipped
    updates, and any other chunk in the general loop.  One worker, every row touched exactly once, so no update depends
    on another: with a quarter of the user updates carried out (keep 63) every item row and every updated user row must
    come out as in the run without thinning (bit for bit for binary32 rows), and a skipped user row as it went in."""
    import torch
    h = mfutil.hip()
    n = 4096
    rng = np.random.default_rng(321 + k)
    R = np.zeros(n, mfutil.NODE)
    R["u"], R["i"], R["r"] = np.arange(n), rng.permutation(n), rng.integers(1, 6, n)
    P0 = (rng.standard_normal((n, k)) * 0.1).astype(np.float32)
    Q0 = (rng.standard_normal((n, k)) * 0.1).astype(np.float32)
    dt = np.float32
    if variant == "mem_quant":
        P0, Q0, dt = P0.astype(np.float16), Q0.astype(np.float16), np.float16
    starts = np.arange(0, n, 128, dtype=np.uint32).reshape(-1, 1)
    uc = starts.shape[0]

    def run(keep_u):
        dR, dS, dP, dQ = to_dev(R), to_dev(starts), to_dev(P0), to_dev(Q0)
        opt = mfutil.HogwildOptions(k, np.full(n, keep_u, np.uint8), np.full(n, 255, np.uint8))
        head = (dR.data_ptr(), n, dP.data_ptr(), dQ.data_ptr(), k, 1, uc, 128)
        tail = (5, 0, dS.data_ptr(), mfutil.stream_ptr(), opt.ptr)
        if variant == "single":
            h.mf_single_sgd_hogwild_opt(*head, LR, LAM, *tail)
        elif variant == "mpt":
            h.mf_mpt_sgd_hogwild_opt(*head, LR, 0x5240, 1000.0, *tail)          # binary16 50 = lambda x 1000
        elif variant == "muppet":
            sm, sn = torch.zeros(k, dtype=torch.float32, device="cuda"), torch.zeros(1, dtype=torch.float32, device="cuda")
            h.mf_muppet_sgd_hogwild_opt(*head, LR, LAM, uc * 128, sm.data_ptr(), sn.data_ptr(), 8, 8, *tail)
        elif variant == "afp":
            h.mf_afp_sgd_hogwild_opt(*head, LR, LAM, 1, *tail)
        else:
            h.mf_mem_quant_sgd_hogwild_opt(*head, LR, LAM, *tail)
        torch.cuda.synchronize()
        return from_dev(dP, dt, P0.shape), from_dev(dQ, dt, Q0.shape)

    P1, Q1 = run(255)
    assert np.all(np.any(P1 != P0, axis=1)) and np.all(np.any(Q1 != Q0, axis=1))
    P2, Q2 = run(63)
    assert np.array_equal(Q2.view(np.uint8), Q1.view(np.uint8))
    changed = np.any(P2 != P0, axis=1)
    assert 0.20 < changed.mean() < 0.30
    if variant == "mem_quant":
        # an update of a thinned row that is carried out is added to the row in memory, rounded to binary16 first, where
        # the run without thinning stores the rounded sum: within one binary16 ulp of the larger of change and result
        got, want, old = P2[changed].astype(np.float64), P1[changed].astype(np.float64), P0[changed].astype(np.float64)
        scale = np.maximum(np.abs(want), np.abs(want - old)).astype(np.float16)
        assert np.all(np.abs(got - want) <= np.spacing(scale).astype(np.float64))
    else:
        assert np.array_equal(P2[changed].view(np.uint8), P1[changed].view(np.uint8))      # binary32: old + change is the stored value
    assert np.array_equal(P2[~changed].view(np.uint8), P0[~changed].view(np.uint8))


@pytest.mark.parametrize("k", [64, 128])
@pytest.mark.parametrize("variant", ["single", "mpt", "mascot", "muppet", "afp"])
def test_hot_row_updates_add_up(orc, k, variant):
    """k wavefronts in k/4 workgroups update one hot item row at the same time.  User u's row is 0.5 * e_u, the item
    row starts at zero and lambda is zero, so every update sees a zero dot product whatever the others have done
    and adds lr * r_u * 0.5 to element u only: all k updates must land, exactly, in any order."""
    import torch
    h = mfutil.hip()
    n, lr = k, 2.0 ** -6
    rng = np.random.default_rng(7 + k)
    R = np.zeros(n, mfutil.NODE)
    R["u"], R["i"], R["r"] = rng.permutation(n), 0, rng.integers(1, 6, n)
    P0 = (0.5 * np.eye(n, k)).astype(np.float32)
    Q0 = np.zeros((1, k), np.float32)
    if variant == "afp":        # AFP measures a relative quantisation error, 0/0 on an all-zero row: start from 2^-10
        Q0 += 2.0 ** -10
    starts = np.arange(n, dtype=np.uint32).reshape(1, n)            # n workers, one rating each
    want = np.zeros(k, np.float32)
    want[R["u"]] = lr * R["r"] * 0.5
    dR, dS = to_dev(R), to_dev(starts)
    opt = mfutil.HogwildOptions(k, np.full(n, 255, np.uint8), np.full(1, 254, np.uint8))
    if True:
        if variant == "mascot":
            end_u, end_i = np.array([n - 1], np.uint32), np.array([0], np.uint32)
            gp = mfutil.host_grouped(orc, k, P0, end_u, np.zeros(1, np.uint8))
            gq = mfutil.host_grouped(orc, k, Q0, end_i, np.zeros(1, np.uint8))
            dp, dq = mfutil.DeviceGrouped(gp), mfutil.DeviceGrouped(gq)
            z = torch.zeros(4 * k + 4 * n, dtype=torch.float32, device="cuda")
            h.mf_mascot_sgd_hogwild_opt(dR.data_ptr(), n, dp.ptrs.data_ptr(), dq.ptrs.data_ptr(), k, n, 1, 1, lr, 0.0,
                                        dp.end.data_ptr(), dq.end.data_ptr(), dp.prec.data_ptr(), dq.prec.data_ptr(),
                                        z.data_ptr(), z[k:].data_ptr(), z[2 * k:].data_ptr(), z[2 * k + n:].data_ptr(),
                                        1, 1, 1, 5, 0, dS.data_ptr(), mfutil.stream_ptr(), opt.ptr)
            torch.cuda.synchronize()
            got = orc.h2f(dq.download()[0]).reshape(k)
        else:
            dP, dQ = to_dev(P0), to_dev(Q0)
            if variant == "single":
                h.mf_single_sgd_hogwild_opt(dR.data_ptr(), n, dP.data_ptr(), dQ.data_ptr(), k, n, 1, 1, lr, 0.0, 5, 0, dS.data_ptr(), mfutil.stream_ptr(), opt.ptr)
            elif variant == "muppet":       # 32 bit forward and backward: the plain binary32 gradient
                sm, sn = torch.zeros(k, dtype=torch.float32, device="cuda"), torch.zeros(n, dtype=torch.float32, device="cuda")
                h.mf_muppet_sgd_hogwild_opt(dR.data_ptr(), n, dP.data_ptr(), dQ.data_ptr(), k, n, 1, 1, lr, 0.0, 1, sm.data_ptr(), sn.data_ptr(),
                                            32, 32, 5, 0, dS.data_ptr(), mfutil.stream_ptr(), opt.ptr)
            elif variant == "afp":          # quantised on a power-of-two grid that holds 0.5 and the ratings 1..5
                h.mf_afp_sgd_hogwild_opt(dR.data_ptr(), n, dP.data_ptr(), dQ.data_ptr(), k, n, 1, 1, lr, 0.0, 0, 5, 0, dS.data_ptr(), mfutil.stream_ptr(), opt.ptr)
            else:
                h.mf_mpt_sgd_hogwild_opt(dR.data_ptr(), n, dP.data_ptr(), dQ.data_ptr(), k, n, 1, 1, lr, 0, 1024.0, 5, 0, dS.data_ptr(), mfutil.stream_ptr(), opt.ptr)
            torch.cuda.synchronize()
            got = from_dev(dQ, np.float32, Q0.shape).reshape(k)
    if variant == "afp":        # quantised arithmetic and a small non-zero dot product: every update landed, to 2 %
        assert np.all(np.isfinite(got)) and np.all(np.abs(got - Q0.reshape(k) - want) < 0.02 * want)
    else:
        assert np.array_equal(got, want)


@pytest.mark.parametrize("k", [64, 128])
@pytest.mark.parametrize("elem", [2, 4])
def test_replica_sync_copies_out_and_averages_changed_copies(orc, k, elem):
    """mf_replica_sync_dense, the step the update calls run around every kernel launch for replicated rows: merge = 0
    fills all eight copies of every slot with its row; merge = 1 sets the row and its copies to the mean of the copies
    that differ from the row (binary32 sum in XCD order, one division, one rounding), and leaves a row alone when none does."""
    import torch
    h = mfutil.hip()
    rng = np.random.default_rng(k + elem)
    rows, slots = 40, 6
    dt = np.float32 if elem == 4 else np.float16
    M = (rng.standard_normal((rows, k)) * 0.3).astype(dt)
    slot_row = np.array([3, 39, 0, 17, 18, 5], np.uint32)
    dM, dS = to_dev(M), to_dev(slot_row)
    rep = torch.full((8 * slots * k * 4,), 0xAB, dtype=torch.uint8, device="cuda")
    h.mf_replica_sync_dense(dM.data_ptr(), elem, k, rep.data_ptr(), dS.data_ptr(), slots, 0, mfutil.stream_ptr())
    torch.cuda.synchronize()
    R = rep.cpu().numpy().reshape(8, slots, k * 4)
    for x in range(8):
        for sl in range(slots):
            assert np.array_equal(R[x, sl, :k * elem].view(dt), M[slot_row[sl]])
    assert np.array_equal(from_dev(dM, dt, M.shape), M)
    # change some copies: slot 0 in XCDs 1, 4, 6; slot 1 in all eight; slot 2 in XCD 7 only; slot 3 in none; slots 4, 5 in two
    touched = {0: [1, 4, 6], 1: list(range(8)), 2: [7], 3: [], 4: [0, 1], 5: [2, 3]}
    for sl, xs in touched.items():
        for x in xs:
            R[x, sl, :k * elem] = (rng.standard_normal(k) * 0.3).astype(dt).view(np.uint8)
    rep.copy_(torch.from_numpy(R.reshape(-1)))
    h.mf_replica_sync_dense(dM.data_ptr(), elem, k, rep.data_ptr(), dS.data_ptr(), slots, 1, mfutil.stream_ptr())
    torch.cuda.synchronize()
    got, R2 = from_dev(dM, dt, M.shape), rep.cpu().numpy().reshape(8, slots, k * 4)
    want = M.copy()
    for sl, xs in touched.items():
        if xs:
            acc = np.zeros(k, np.float32)
            for x in xs:
                acc = acc + R[x, sl, :k * elem].view(dt).astype(np.float32)
            want[slot_row[sl]] = (acc / np.float32(len(xs))).astype(dt)
    assert np.array_equal(got.view(np.uint8), want.view(np.uint8))
    for x in range(8):
        for sl in range(slots):
            assert np.array_equal(R2[x, sl, :k * elem].view(dt).view(np.uint8), want[slot_row[sl]].view(np.uint8))


@pytest.mark.parametrize("variant", ["single", "mem_quant", "mascot"])
def test_replicated_rows_under_many_workers(orc, variant):
    """2048 workers on every XCD race on a few replicated rows (each XCD on its own copies) while the other rows are
    ordinary: the ordinary side of a conflict-free schedule must come out as the checker computes it when the
    replicated side is not updated at all (learning rate 0 on it is not available, so the check is structural): every
    value finite, every replicated row moved, the copies of a row equal the row after the call, and a second call
    with the same inputs starts from the rows, not from stale copies."""
    import torch
    h = mfutil.hip()
    k, n_users, n_items, n = 128, 4096, 8, 2048 * 128
    rng = np.random.default_rng(99)
    R = np.zeros(n, mfutil.NODE)
    R["u"], R["i"], R["r"] = rng.integers(0, n_users, n), rng.integers(0, n_items, n), rng.integers(1, 6, n)
    P0 = (rng.standard_normal((n_users, k)) * 0.1).astype(np.float32)
    Q0 = (rng.standard_normal((n_items, k)) * 0.1).astype(np.float32)
    keep_u, keep_v = np.full(n_users, 255, np.uint8), np.full(n_items, 253, np.uint8)
    keep_u[:5] = 253
    opt = mfutil.HogwildOptions(k, keep_u, keep_v, launches=2)
    dR = to_dev(R)
    W, uc = 2048, 1

    def call(dP, dQ, epoch):
        if variant == "single":
            h.mf_single_sgd_hogwild_opt(dR.data_ptr(), n, dP.data_ptr(), dQ.data_ptr(), k, W, uc, 128, 0.01, 0.02, 5, epoch, None, mfutil.stream_ptr(), opt.ptr)
        elif variant == "mem_quant":
            h.mf_mem_quant_sgd_hogwild_opt(dR.data_ptr(), n, dP.data_ptr(), dQ.data_ptr(), k, W, uc, 128, 0.01, 0.02, 5, epoch, None, mfutil.stream_ptr(), opt.ptr)
        torch.cuda.synchronize()

    if variant == "mascot":
        end_u, end_i = mfutil.equal_end_idx(n_users, 3), np.array([n_items - 1], np.uint32)
        uprec = np.array([0, 1, 0], np.uint8)
        gp = mfutil.host_grouped(orc, k, P0, end_u, uprec)
        gq = mfutil.host_grouped(orc, k, Q0, end_i, np.zeros(1, np.uint8))
        dp, dq = mfutil.DeviceGrouped(gp), mfutil.DeviceGrouped(gq)
        nb = h.mf_mascot_norm_blocks(W)
        z = torch.zeros(4 * k + 4 * nb, dtype=torch.float32, device="cuda")
        for epoch in range(2):
            h.mf_mascot_sgd_hogwild_opt(dR.data_ptr(), n, dp.ptrs.data_ptr(), dq.ptrs.data_ptr(), k, W, uc, 128, 0.01, 0.02,
                                        dp.end.data_ptr(), dq.end.data_ptr(), dp.prec.data_ptr(), dq.prec.data_ptr(),
                                        z.data_ptr(), z[3 * k:].data_ptr(), z[4 * k:].data_ptr(), z[4 * k + 3 * nb:].data_ptr(),
                                        uc * 128, 3, 1, 5, epoch, None, mfutil.stream_ptr(), opt.ptr)
            torch.cuda.synchronize()
        Qg = orc.h2f(dq.download()[0]).reshape(n_items, k)
        Pg = np.concatenate([(a if a.dtype == np.float32 else orc.h2f(a)).reshape(-1, k) for a in dp.download()])
        P0 = np.concatenate([(a if a.dtype == np.float32 else orc.h2f(a)).reshape(-1, k) for a in gp.arrays])
        Q0 = orc.h2f(gq.arrays[0]).reshape(n_items, k)
        elem_q = 2
    else:
        if variant == "mem_quant":
            dP, dQ = to_dev(orc.f2h(P0)), to_dev(orc.f2h(Q0))
            P0, Q0 = orc.h2f(orc.f2h(P0)).reshape(P0.shape), orc.h2f(orc.f2h(Q0)).reshape(Q0.shape)
        else:
            dP, dQ = to_dev(P0), to_dev(Q0)
        call(dP, dQ, 0)
        call(dP, dQ, 1)
        if variant == "mem_quant":
            Pg, Qg = orc.h2f(from_dev(dP, np.uint16)).reshape(P0.shape), orc.h2f(from_dev(dQ, np.uint16)).reshape(Q0.shape)
            elem_q = 2
        else:
            Pg, Qg = from_dev(dP, np.float32, P0.shape), from_dev(dQ, np.float32, Q0.shape)
            elem_q = 4
    assert np.all(np.isfinite(Pg)) and np.all(np.isfinite(Qg))
    assert np.all(np.any(Qg != Q0, axis=1)) and np.all(np.any(Pg[:5] != P0[:5], axis=1))
    # two epochs of lr 0.01 on ratings 1..5 from rows of size 0.1: the rows grow, nothing explodes
    assert np.abs(Qg).max() < 5 and np.abs(Pg).max() < 5
    touched = np.bincount(R["u"], minlength=n_users) > 0
    assert np.all(np.any(Pg[touched] != P0[touched], axis=1))
    # the copies of every item row equal the row after the call (the last merge wrote them)
    rep = opt.replicas[1].cpu().numpy().reshape(8, n_items, k * 4)
    dtq = np.float32 if elem_q == 4 else np.float16
    for x in range(8):
        for sl in range(n_items):
            assert np.array_equal(rep[x, sl, :k * elem_q].view(dtq).astype(np.float32), Qg[sl])
