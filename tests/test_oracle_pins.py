"""Pins of the CPU checker's MPT, MuPPET and AFP updates and of the MuPPET ladder that do not share code or a
transcription with oracle/mascot_oracle.c.  Each rule is restated here from the reference with independent engines --
numpy.float16 for every binary16 rounding, Python integers for the int8 dot products, math.frexp for floor/ceil of
log2 (exact for a binary32 argument, no logarithm evaluated) -- lane by lane in the reference's warp order, and the
quantities a slip would change (scale indices, quantised values, bit widths, intervals) are also stated by hand on
crafted rows, chosen so that floor <-> ceil, an index off by one or a dropped rounding changes the result.

Reference: mpt/mpt_sgd_kernel.h:38-91, muppet/muppet_sgd_kernel.h:7-32,110-285 (+ _k64.h), afp/afp_sgd_kernel.h:8-125,
196-374 (+ _k64.h), reduce_kernel.h, mf_methods.cu:586-601,659-697."""
import ctypes as C
import math

import numpy as np
import pytest

f32, f16 = np.float32, np.float16


# ---- independent engines ------------------------------------------------------------------------------------------
def roundf(x):
    """C roundf on binary32: to the nearest integer, halves away from zero."""
    x = np.asarray(x, f32)
    return (np.sign(x) * np.floor(np.abs(x).astype(np.float64) + 0.5)).astype(f32)


def floor_log2(x):
    """floor(log2(x)) of a positive binary32 value, exactly (frexp: x = m * 2^e, 0.5 <= m < 1)."""
    m, e = math.frexp(float(f32(x)))
    return e - 1


def ceil_log2(x):
    m, e = math.frexp(float(f32(x)))
    return e - 1 if m == 0.5 else e


def away_from_power_of_two(x, rel=2e-6):
    """True when floor/ceil(log2f(x)) cannot depend on the last bits of a log2f implementation (16 binary32 ulps away)."""
    m, _ = math.frexp(float(x))
    return abs(m - 0.5) > rel and abs(m - 1.0) > rel


def tree(x, add):
    """The reference's shfl_down 16, 8, 4, 2, 1 reduction; lane 0's value."""
    x = list(x)
    for off in (16, 8, 4, 2, 1):
        for lane in range(off):
            x[lane] = add(x[lane], x[lane + off])
    return x[0]


def h(x):
    return f16(f32(x))


def hmul(a, b):
    return f16(f32(a) * f32(b))          # the product of two binary16 values is exact in binary32: one rounding


def hadd(a, b):
    return f16(f32(a) + f32(b))


def hsub(a, b):
    return f16(f32(a) - f32(b))


def lanes(v, k):
    """v[l + 32 j] as [j][l]: what warp lane l holds."""
    return np.asarray(v).reshape(k // 32, 32)


# ---- MPT ----------------------------------------------------------------------------------------------------------
def mpt_numpy(k, p, q, r, lr, lam_scaled_h, scale):
    """mpt/mpt_sgd_kernel.h:38-91 with numpy.float16."""
    ph, qh = p.astype(f16), q.astype(f16)
    P, Q = lanes(ph, k), lanes(qh, k)
    m = [[hmul(P[j][l], Q[j][l]) for l in range(32)] for j in range(k // 32)]
    if k == 128:
        per_lane = [hadd(hadd(m[0][l], m[1][l]), hadd(m[2][l], m[3][l])) for l in range(32)]
    else:
        per_lane = [hadd(m[0][l], m[1][l]) for l in range(32)]
    dot = tree(per_lane, hadd)
    ruv = hmul(h(scale), hsub(h(r), dot))
    rev = f32(1) / f32(scale)
    newp, newq = np.empty(k, f32), np.empty(k, f32)
    for e in range(k):
        gp = hsub(hmul(ruv, qh[e]), hmul(lam_scaled_h, ph[e]))
        gq = hsub(hmul(ruv, ph[e]), hmul(lam_scaled_h, qh[e]))
        newp[e] = p[e] + f32(lr) * (rev * f32(gp))
        newq[e] = q[e] + f32(lr) * (rev * f32(gq))
    return newp, newq


@pytest.mark.parametrize("k", [64, 128])
def test_mpt_update_against_numpy_float16(orc, k):
    rng = np.random.default_rng(31 + k)
    lam_h = h(f32(0.05) * f32(1000))                       # mf_methods.cu:764-765
    lam_bits = int(lam_h.view(np.uint16))
    assert orc.lib.orc_float2half(f32(0.05) * f32(1000)) == lam_bits
    for trial in range(30):
        # fp32 master values that are NOT binary16-representable, so the conversion's rounding matters
        p = (rng.standard_normal(k) * 0.3).astype(f32)
        q = (rng.standard_normal(k) * 0.3).astype(f32)
        r = float(rng.integers(1, 6)) if trial % 3 else float(rng.integers(1, 11)) / 2
        want_p, want_q = mpt_numpy(k, p, q, r, 0.01, lam_h, 1000.0)
        p1, q1 = p.copy(), q.copy()
        orc.lib.orc_mpt_update(k, p1.ctypes.data, q1.ctypes.data, r, 0.01, lam_bits, 1000.0)
        assert np.array_equal(p1.view(np.uint32), want_p.view(np.uint32))
        assert np.array_equal(q1.view(np.uint32), want_q.view(np.uint32))


def test_mpt_hand_worked_row(orc):
    """One row whose every intermediate is written out: p = 0.5 e_0, q = 0.25 e_0 + 0.5 e_33, r = 3, loss scale 1000.
    dot = 0.125; ruv = rn16(1000 * 2.875) = rn16(2875) = 2876 (binary16 spacing 2 above 2048, tie to even 2876);
    lambda_s = rn16(50) = 50.  p0: g = rn16(rn16(2876 * 0.25) - rn16(50 * 0.5)) = 719 - 25 = 694,
    p0' = 0.5 + 0.01 * (0.001 * 694); q0: g = rn16(1438 - 12.5) = rn16(1425.5) = 1426 (spacing 1, tie to even);
    q33: g = rn16(0 - 25) = -25; p33 (zero before): g = rn16(2876 * 0.5) - 0 = 1438."""
    k = 64
    p, q = np.zeros(k, f32), np.zeros(k, f32)
    p[0], q[0], q[33] = 0.5, 0.25, 0.5
    orc.lib.orc_mpt_update(k, p.ctypes.data, q.ctypes.data, 3.0, 0.01, int(h(50.0).view(np.uint16)), 1000.0)
    rev = f32(1) / f32(1000)
    assert p[0] == f32(0.5) + f32(0.01) * (rev * f32(694))
    assert q[0] == f32(0.25) + f32(0.01) * (rev * f32(1426))
    assert q[33] == f32(0.5) + f32(0.01) * (rev * f32(-25))
    assert p[33] == f32(0.01) * (rev * f32(1438))
    assert np.all(np.delete(p, [0, 33]) == 0) and np.all(np.delete(q, [0, 33]) == 0)


# ---- MuPPET -------------------------------------------------------------------------------------------------------
def muppet_index(bits, vmax, vmin):
    """get_only_scaling_factor, muppet_sgd_kernel.h:7-18, stored in an unsigned: negative results become 0."""
    if vmax == 0 and vmin == 0:
        return 0
    val = f32(1 << (bits - 1))
    max_val, min_val = (val - f32(1)) + f32(0.5), (-val) - f32(0.5)
    with np.errstate(divide="ignore"):
        best = min(abs(max_val / f32(vmax)), abs(min_val / f32(vmin)))
    assert away_from_power_of_two(best), "test input within an ulp of a power of two: parity unpinned there"
    return max(0, floor_log2(best))


def grid_h(v, s):
    return h(roundf(f32(v) * f32(s)) * (f32(1) / f32(s)))


def i8(x):
    x = float(x)
    assert -128 <= x <= 127, "int8 overflow: conversion behaviour is unpinned there, keep test inputs inside"
    return int(x)


def muppet_numpy(k, p, q, r, lr, lam, fb, bb):
    """muppet_sgd_kernel.h:110-285 / _k64.h for bit widths below 32; returns new rows, gradients and scale indices."""
    J = k // 32
    P, Q = lanes(p, k), lanes(q, k)
    p_min, p_max, q_min, q_max = f32(p.min()), f32(p.max()), f32(q.min()), f32(q.max())
    ip, iq = muppet_index(fb, p_max, p_min), muppet_index(fb, q_max, q_min)
    sp, sq = f32(2.0 ** ip), f32(2.0 ** iq)
    if fb == 8:
        per_lane = [sum(i8(roundf(P[j][l] * sp)) * i8(roundf(Q[j][l] * sq)) for j in range(J)) for l in range(32)]
        pred = f32(tree(per_lane, lambda a, b: a + b)) / (sp * sq)
    else:
        m = [[hmul(grid_h(P[j][l], sp), grid_h(Q[j][l], sq)) for l in range(32)] for j in range(J)]
        # half2 lanes: .x = element l (+ element l+64), .y = element l+32 (+ l+96); the tree runs on both halves
        if k == 128:
            x = [hadd(m[0][l], m[2][l]) for l in range(32)]
            y = [hadd(m[1][l], m[3][l]) for l in range(32)]
        else:
            x, y = m[0], m[1]
        pred = f32(hadd(tree(x, hadd), tree(y, hadd)))
    ruv = f32(r) - pred
    neg_lam = f32(-1) * f32(lam)
    bmin = min(min(p_min, q_min), min(neg_lam, ruv))
    bmax = max(max(p_max, q_max), max(neg_lam, ruv))
    ib = muppet_index(bb, bmax, bmin)
    sb = f32(2.0 ** ib)
    gp, gq = np.empty(k, f32), np.empty(k, f32)
    if bb == 8:
        rev = f32(1) / (sb * sb)
        ruv_i, lam_i = i8(roundf(ruv * sb)), i8(roundf(f32(-1.0) * f32(lam) * sb))
        for e in range(k):
            pi, qi = i8(roundf(p[e] * sb)), i8(roundf(q[e] * sb))
            gp[e] = f32(qi * ruv_i + pi * lam_i) * rev
            gq[e] = f32(pi * ruv_i + qi * lam_i) * rev
    else:
        t_ruv, t_lam = grid_h(ruv, sb), grid_h(neg_lam, sb)
        for e in range(k):
            ph, qh = grid_h(p[e], sb), grid_h(q[e], sb)
            gp[e] = f32(hadd(hmul(qh, t_ruv), hmul(ph, t_lam)))
            gq[e] = f32(hadd(hmul(ph, t_ruv), hmul(qh, t_lam)))
    newp = (p + f32(lr) * gp).astype(f32)
    newq = (q + f32(lr) * gq).astype(f32)
    GP, GQ = lanes(gp, k), lanes(gq, k)
    fadd = lambda a, b: f32(a + b)
    if k == 128:
        n = [fadd(fadd(fadd(GP[0][l] * GP[0][l], GP[1][l] * GP[1][l]), fadd(GP[2][l] * GP[2][l], GP[3][l] * GP[3][l])),
                  fadd(fadd(GQ[0][l] * GQ[0][l], GQ[1][l] * GQ[1][l]), fadd(GQ[2][l] * GQ[2][l], GQ[3][l] * GQ[3][l]))) for l in range(32)]
    else:
        n = [fadd(fadd(GP[0][l] * GP[0][l], GP[1][l] * GP[1][l]), fadd(GQ[0][l] * GQ[0][l], GQ[1][l] * GQ[1][l])) for l in range(32)]
    return newp, newq, gp, gq, tree(n, fadd), (ip, iq, ib)


def run_muppet(orc, k, p, q, r, lr, lam, fb, bb):
    p1, q1 = p.copy(), q.copy()
    s, nrm = np.zeros(k, f32), C.c_float(0)
    orc.lib.orc_muppet_update(k, p1.ctypes.data, q1.ctypes.data, r, lr, lam, fb, bb, s.ctypes.data, C.byref(nrm))
    return p1, q1, s, nrm.value


@pytest.mark.parametrize("k", [64, 128])
@pytest.mark.parametrize("bits", [8, 12, 14, 16])
def test_muppet_update_against_numpy(orc, k, bits):
    rng = np.random.default_rng(100 * bits + k)
    done = 0
    for trial in range(200):
        p = (rng.standard_normal(k) * 0.2).astype(f32)
        q = (rng.standard_normal(k) * 0.2).astype(f32)
        r = float(rng.integers(1, 6))
        try:
            want_p, want_q, gp, gq, norm, idx = muppet_numpy(k, p, q, r, 0.01, 0.05, bits, bits)
        except AssertionError:
            continue                                   # a scale decision within an ulp of a power of two, or an int8 overflow
        got_p, got_q, s, nrm = run_muppet(orc, k, p, q, r, 0.01, 0.05, bits, bits)
        assert np.array_equal(got_p.view(np.uint32), want_p.view(np.uint32)), (trial, idx)
        assert np.array_equal(got_q.view(np.uint32), want_q.view(np.uint32)), (trial, idx)
        assert np.array_equal(s, (gp + gq).astype(f32)) and f32(nrm) == f32(norm)
        done += 1
        if done == 25:
            break
    assert done == 25


@pytest.mark.parametrize("k", [64, 128])
@pytest.mark.parametrize("bits", [8, 12, 14, 16])
def test_muppet_hand_worked_scale_and_grid(orc, k, bits):
    """Rows whose scale indices and quantised values are written out by hand.

    Forward: max p = max q = 1, min = -1, so range_best = (2^(b-1) - 0.5) / 1 and the index is floor(log2) = b - 2
    (a ceil would give b - 1): scale 2^(b-2).  p[1] = 1.5 / scale lies half a step off the grid and rounds away from
    zero to 2 / scale (with index b - 1 it would be representable, with b - 3 it would round to 4 / that scale = 1 / ...:
    both change p[1] * q[1]); q[1] = 1.  p[0] = 1, q[0] = -1, p[2] = -1, q[2] = 0.5 / scale ... rounds to 1 / scale.
    pred = -1 + 2/scale - 1/scale = -1 + 1/scale; at 8 bit the int8 products are 64*-64 + 2*64 - 64*1 = -4032 over 64*64.
    Backward: r = 2 gives ruv = 3 - 1/scale, the largest magnitude among {p, q, -lambda, ruv}; range_best =
    (2^(b-1) - 0.5) / ruv, a little above 2^(b-1) / 4 ... index b - 3, scale 2^(b-3)."""
    scale = 2.0 ** (bits - 2)
    p, q = np.zeros(k, f32), np.zeros(k, f32)
    p[0], q[0] = 1.0, -1.0
    p[1], q[1] = 1.5 / scale, 1.0
    p[2], q[2] = -1.0, 0.5 / scale
    r, lr, lam = 2.0, 0.01, 0.0625
    want_p, want_q, gp, gq, norm, (ip, iq, ib) = muppet_numpy(k, p, q, r, lr, lam, bits, bits)
    assert (ip, iq, ib) == (bits - 2, bits - 2, bits - 3)            # the restatement agrees with the hand-worked indices
    # hand-worked forward: quantised p[1] = 2/scale, q[2] = 1/scale
    assert grid_h(p[1], scale) == h(2.0 / scale) and grid_h(q[2], scale) == h(1.0 / scale)
    pred = -1.0 + 1.0 / scale
    ruv = f32(r) - f32(pred)
    got_p, got_q, s, nrm = run_muppet(orc, k, p, q, r, lr, lam, bits, bits)
    assert np.array_equal(got_p.view(np.uint32), want_p.view(np.uint32)) and np.array_equal(got_q.view(np.uint32), want_q.view(np.uint32))
    # the gradient of an element the oracle must reproduce, from the hand-worked values only (backward scale 2^(b-3)):
    sb = 2.0 ** (bits - 3)
    if bits == 8:
        ruv_i, lam_i = int(roundf(ruv * f32(sb))), int(roundf(f32(-lam * sb)))      # 3 - 1/64 -> round(95.5) = 96; -0.0625 * 32 = -2
        assert (ruv_i, lam_i) == (96, -2)
        g0 = f32(-32 * ruv_i + 32 * lam_i) * (f32(1) / f32(sb * sb))                 # gp[0] = (q0_i * ruv_i + p0_i * lam_i) / sb^2, q0_i = -32, p0_i = 32
        assert got_p[0] == f32(1.0) + f32(lr) * g0
        assert (g0, float(gp[0])) == (f32(-3136 / 1024), float(g0))
    else:
        t_ruv, t_lam = grid_h(ruv, sb), grid_h(-lam, sb)
        g0 = f32(hadd(hmul(h(-1.0), t_ruv), hmul(h(1.0), t_lam)))
        assert got_p[0] == f32(1.0) + f32(lr) * g0
    assert np.array_equal(s, (gp + gq).astype(f32)) and f32(nrm) == f32(norm)
    # the same rows with the forward index forced wrong would differ: the crafted elements do discriminate
    for wrong in (bits - 1, bits - 3):
        assert grid_h(p[1], 2.0 ** wrong) != grid_h(p[1], scale) or grid_h(q[2], 2.0 ** wrong) != grid_h(q[2], scale)


@pytest.mark.parametrize("k", [64, 128])
def test_muppet_scale_bounds_hand_worked(orc, k):
    """The two bounds of get_only_scaling_factor are (2^(b-1) - 1) + 0.5 and -2^(b-1) - 0.5 (127.5 and -128.5 at 8 bit).
    max p = 127/64 with a small minimum: 127.5 / 1.984375 = 64.25 -> index 6, scale 64, p_i = 127 (126.5 as the bound
    would give 63.7 -> index 5).  min q = -2 with a small maximum: 128.5 / 2 = 64.25 -> index 6, q_i = -128 (127.5 as
    the bound would give index 5).  The int8 product of elements 0: 127 * -128."""
    p, q = np.zeros(k, f32), np.zeros(k, f32)
    p[0], p[1], q[0], q[1] = 127 / 64, -0.5, -2.0, 0.5
    r = 0.98125                                               # chosen so that the two candidate predictions round ruv differently
    want_p, want_q, gp, gq, norm, idx = muppet_numpy(k, p, q, r, 0.01, 0.0625, 8, 8)
    assert idx[:2] == (6, 6)
    # pred = (127 * -128 + (-32) * 32) / 4096 = -4.21875; ruv = 5.2 dominates the backward range: 127.5 / 5.2 = 24.5 -> index 4
    # (with forward index 5 on the p side: (64 * -128 - 16 * 32) / 2048 = -4.25, ruv = 5.23125, ruv_i = round(83.7) = 84)
    assert idx[2] == 4
    got_p, got_q, s, nrm = run_muppet(orc, k, p, q, r, 0.01, 0.0625, 8, 8)
    assert np.array_equal(got_p.view(np.uint32), want_p.view(np.uint32)) and np.array_equal(got_q.view(np.uint32), want_q.view(np.uint32))
    ruv_i, lam_i = 83, -1                                     # round(5.2 * 16) = round(83.2) = 83; round(-0.0625 * 16) = -1
    assert got_p[0] == f32(127 / 64) + f32(0.01) * (f32(-32 * ruv_i + 32 * lam_i) * (f32(1) / f32(256)))      # q0_i = -32, p0_i = round(31.75) = 32
    # the q side's bound: the same rows with the roles of p and q exchanged (min p = -2 decides p's index)
    want = muppet_numpy(k, q, p, r, 0.01, 0.0625, 8, 8)
    got = run_muppet(orc, k, q, p, r, 0.01, 0.0625, 8, 8)
    assert want[5][:2] == (6, 6) and np.array_equal(got[0], want[0]) and np.array_equal(got[1], want[1])


def test_muppet_scale_index_edge_cases(orc):
    """All-zero rows give index 0 (scale 1), and an index that would be negative is stored in an unsigned: 0.
    p = q = 0: pred = 0, ruv = r = 200; backward range_best = 127.5 / 200 < 1, floor(log2) = -1 -> 0: scale 1,
    ruv_i = round(200) saturates -- kept out of the pinned set; use r = 100: 127.5 / 100 = 1.275 -> index 0, ruv_i = 100."""
    k = 64
    p, q = np.zeros(k, f32), np.zeros(k, f32)
    got_p, got_q, _, _ = run_muppet(orc, k, p, q, 100.0, 0.01, 0.05, 8, 8)
    # gp = (q_i * ruv_i + p_i * lam_i) / 1 = 0: lam_i = round(-0.05) = 0
    assert np.all(got_p == 0) and np.all(got_q == 0)
    p[3], q[3] = 1.0, 2.0                                    # forward: index 6 for p (127.5/1), 5 for q (127.5/2 = 63.75)
    want = muppet_numpy(k, p, q, 100.0, 0.01, 0.05, 8, 8)
    assert want[5][:2] == (6, 5) and want[5][2] == 0         # backward: ruv = 98 dominates, 127.5/98 = 1.3 -> 0
    got_p, got_q, _, _ = run_muppet(orc, k, p, q, 100.0, 0.01, 0.05, 8, 8)
    assert np.array_equal(got_p, want[0]) and np.array_equal(got_q, want[1])
    assert got_p[3] == f32(1.0) + f32(0.01) * f32(2 * 98 + 1 * 0)      # p_i = 1, q_i = 2, ruv_i = 98, lam_i = 0, scale 1


# ---- AFP ----------------------------------------------------------------------------------------------------------
def afp_index(bits, vmax):
    """get_only_scaling_factor_cvpr, afp_sgd_kernel.h:8-16: |ceil(log2(max / (2^(b-1) - 1)))|."""
    if vmax == 0:
        return 0
    ratio = f32(vmax) / (f32(2.0 ** (bits - 1)) - f32(1))
    assert away_from_power_of_two(ratio)
    return abs(ceil_log2(ratio))


def afp_qem(vals_per_lane, vmax):
    """QEM / QEM_BP, afp_sgd_kernel.h:32-102: vals_per_lane[l] = the values lane l holds, summed left to right."""
    s = f32(2.0 ** afp_index(8, vmax))
    rev = f32(1) / s
    fadd = lambda a, b: f32(a + b)

    def lane_sum(vs, quantise):
        acc = None
        for v in vs:
            t = abs(roundf(f32(v) * s) * rev) if quantise else abs(f32(v))
            acc = f32(t) if acc is None else fadd(acc, t)
        return acc
    sum_q = tree([lane_sum(vs, True) for vs in vals_per_lane], fadd)
    sum_v = tree([lane_sum(vs, False) for vs in vals_per_lane], fadd)
    return f32(math.log2(float(f32(abs(f32(sum_v - sum_q) / sum_v) + f32(1))))), sum_v, sum_q


def afp_qpa(diff, rng_, prev):
    """QPA, afp_sgd_kernel.h:104-125; returns (r, n, itv, mov_avg_range)."""
    n = 8 if diff <= f32(0.0005) else 16
    r = abs(ceil_log2(f32(rng_) / (f32(2.0 ** (n - 1)) - f32(1))))
    mov = f32(f32(0.04) * f32(rng_) + f32(f32(1.0) - f32(0.04)) * f32(prev))
    i1 = f32(f32(f32(100) * f32(diff)) * f32(diff))
    i2 = abs(f32(mov - f32(prev)))
    with np.errstate(divide="ignore"):
        itv_f = f32(f32(0.1) / max(i1, i2)) - f32(2)
    itv = 2147483647 if itv_f >= 2147483648.0 else int(itv_f)          # float -> int conversion saturates (cvt.rzi.s32.f32)
    return r, n, itv, mov


def test_afp_first_update_hand_worked(orc):
    """The first update of a launch (cur_iter = 0, epoch 0, first tenth) on a row where everything is a dyadic value.

    k = 64; p = 0.5 on elements 0 and 32, q = 0.25 on element 0 and 0.75 on element 33; r = 3; lambda = 0.0625.
    user side: max |p| = 0.5; QEM scale index |ceil(log2(0.5 / 127))| = |ceil(-7.99)| = 7, scale 128: every value is on
    the grid, diff = log2(0 + 1) = 0 <= 0.0005 -> n = 8, r = 7 (same formula), mov_avg = 0.04*0.5 + 0.96*0.5 = 0.5,
    itv = 0.1 / max(0, 0) - 2 = inf -> saturates, but epoch 0 and cur_iter < threshold force itv = 1.
    item side: max |q| = 0.75: index |ceil(log2(0.75/127))| = |ceil(-7.4)| = 7: same.
    forward (both 8 bit): p_i = 64, q_i = 32, 96: dot = 64*32 = 2048 -> pred = 2048 / 128^2 = 0.125; ruv = 2.875.
    backward: max(|p|, |q|, lambda, |ruv|) = 2.875: index |ceil(log2(2.875/127))| = |ceil(-5.47)| = 5, scale 32;
    QEM_BP on {p, q, lambda, ruv} per lane: all on the 1/32 grid (0.0625 = 2/32, 2.875 = 92/32) -> diff 0 -> n = 8.
    gp[0] = (q_i*ruv_i + p_i*lam_i)/32^2 = (8*92 + 16*(-2))/1024 = 0.6875; gq[33] = (0*92 + 24*(-2))/1024 = -0.046875."""
    from oracle.oracle import AfpState
    k = 64
    p, q = np.zeros(k, f32), np.zeros(k, f32)
    p[0], p[32], q[0], q[33] = 0.5, 0.5, 0.25, 0.75
    st = AfpState()
    orc.lib.orc_afp_state_init(C.byref(st))
    orc.lib.orc_afp_update(k, C.byref(st), p.ctypes.data, q.ctypes.data, 3.0, 0.01, 0.0625, 0, 10)
    ema = lambda x: float(f32(f32(0.04) * f32(x) + f32(f32(1.0) - f32(0.04)) * f32(x)))      # alpha*range + (1-alpha)*range in binary32: not always x
    assert (st.user.r, st.user.n, st.user.itv, st.user.mov_avg_range) == (7, 8, 1, ema(0.5))
    assert (st.item.r, st.item.n, st.item.itv, st.item.mov_avg_range) == (7, 8, 1, ema(0.75))
    assert (st.backward.r, st.backward.n, st.backward.itv, st.backward.mov_avg_range) == (5, 8, 1, ema(2.875))
    assert ema(0.5) == 0.5 and abs(ema(0.75) - 0.75) < 1e-7
    assert (st.cur_iter, st.update_user_params_iter, st.update_item_params_iter, st.update_backward_iter) == (1, 1, 1, 1)
    assert (st.scaling_factor_p, st.scaling_factor_q, st.scaling_factor_back_prop) == (128.0, 128.0, 32.0)
    assert p[0] == f32(0.5) + f32(0.01) * f32(0.6875)
    assert p[32] == f32(0.5) + f32(0.01) * f32((0 * 92 + 16 * -2) / 1024)
    assert q[0] == f32(0.25) + f32(0.01) * f32((16 * 92 + 8 * -2) / 1024)
    assert q[33] == f32(0.75) + f32(0.01) * f32(-0.046875)
    assert q[1] == 0 and p[1] == 0
    # the same update in a later epoch keeps the measured interval: inf saturates to INT_MAX
    p2, q2 = np.zeros(k, f32), np.zeros(k, f32)
    p2[0], p2[32], q2[0], q2[33] = 0.5, 0.5, 0.25, 0.75
    st2 = AfpState()
    orc.lib.orc_afp_state_init(C.byref(st2))
    orc.lib.orc_afp_update(k, C.byref(st2), p2.ctypes.data, q2.ctypes.data, 3.0, 0.01, 0.0625, 1, 10)
    assert st2.user.itv == 2147483647 and st2.update_user_params_iter == 2147483647
    assert np.array_equal(p2, p) and np.array_equal(q2, q)


def test_afp_qem_qpa_16bit_branch_and_interval(orc):
    """A row off the 8-bit grid: the measured error exceeds 0.0005, so the quantiser moves to 16 bit with its own
    scale index, and the interval comes out of the formula.  k = 64, p = 0.3 everywhere (one value per element):
    max = 0.3, QEM index |ceil(log2(0.3/127))| = |ceil(-8.73)| = 8, scale 256: 0.3*256 = 76.8 -> 77 -> 0.30078125;
    relative error (0.30078125 - 0.3)/0.3 = 0.0026 -> diff = log2(1.0026) = 0.00375 > 0.0005 -> n = 16,
    r = |ceil(log2(0.3/32767))| = |ceil(-16.74)| = 16; first update: mov_avg = 0.3, i2 = 0, i1 = 100 * diff^2 = 0.0014,
    itv = 0.1/0.0014 - 2 = 69 (later epoch, so not forced to 1)."""
    from oracle.oracle import AfpState
    k = 64
    p = np.full(k, 0.3, f32)
    q = np.full(k, 0.3, f32)
    per_lane = [[p[l], p[l + 32]] for l in range(32)]
    diff, sum_v, sum_q = afp_qem(per_lane, f32(0.3))
    assert afp_index(8, f32(0.3)) == 8 and 0.0035 < diff < 0.0040
    r, n, itv, mov = afp_qpa(diff, f32(0.3), f32(0.3))
    assert (r, n) == (16, 16) and mov == f32(f32(0.04) * f32(0.3) + f32(0.96) * f32(0.3)) and 60 < itv < 80
    st = AfpState()
    orc.lib.orc_afp_state_init(C.byref(st))
    orc.lib.orc_afp_update(k, C.byref(st), p.ctypes.data, q.ctypes.data, 3.0, 0.01, 0.05, 1, 10)
    assert (st.user.r, st.user.n, st.user.mov_avg_range) == (r, n, mov)
    assert abs(st.user.itv - itv) <= 1            # the value of log2f (not its floor) sets the interval: last-bit differences move it by one
    assert (st.item.r, st.item.n) == (16, 16)
    assert st.update_user_params_iter == st.user.itv and st.scaling_factor_p == 65536.0


@pytest.mark.parametrize("k", [64, 128])
def test_afp_forward_backward_against_numpy(orc, k):
    """Random rows through the first update of a later epoch (all three quantisers measured), restated with the engines
    above: both the all-8-bit path with saturating int8 products and the binary16-grid path occur."""
    from oracle.oracle import AfpState
    rng = np.random.default_rng(77 + k)
    J = k // 32
    seen = set()
    done = 0
    for trial in range(300):
        coarse = trial % 2 == 0
        if coarse:      # values on a 1/128 grid below 1: the 8-bit measurement is exact -> int8 path
            p = (rng.integers(-100, 101, k) / 128.0).astype(f32)
            q = (rng.integers(-100, 101, k) / 128.0).astype(f32)
        else:
            p = (rng.standard_normal(k) * 0.2).astype(f32)
            q = (rng.standard_normal(k) * 0.2).astype(f32)
        r, lr, lam = float(rng.integers(1, 6)), 0.01, 0.0625
        try:
            P, Q = lanes(p, k), lanes(q, k)
            pmax, qmax = f32(np.abs(p).max()), f32(np.abs(q).max())
            du, _, _ = afp_qem([[P[j][l] for j in range(J)] for l in range(32)], pmax)
            di, _, _ = afp_qem([[Q[j][l] for j in range(J)] for l in range(32)], qmax)
            ur, un, uitv, umov = afp_qpa(du, pmax, pmax)
            ir, in_, iitv, imov = afp_qpa(di, qmax, qmax)
            sp, sq = f32(2.0 ** ur), f32(2.0 ** ir)
            sat = lambda x: int(min(127.0, max(-128.0, float(x))))
            if un == 8 and in_ == 8:
                per_lane = [sum(sat(roundf(P[j][l] * sp)) * sat(roundf(Q[j][l] * sq)) for j in range(J)) for l in range(32)]
                pred = f32(tree(per_lane, lambda a, b: a + b)) / (sp * sq)
            else:
                m = [[hmul(grid_h(P[j][l], sp), grid_h(Q[j][l], sq)) for l in range(32)] for j in range(J)]
                x = [hadd(m[0][l], m[2][l]) for l in range(32)] if k == 128 else m[0]
                y = [hadd(m[1][l], m[3][l]) for l in range(32)] if k == 128 else m[1]
                pred = f32(hadd(tree(x, hadd), tree(y, hadd)))
            ruv = f32(r) - pred
            bmax = max(max(pmax, qmax), max(abs(f32(lam)), abs(ruv)))
            db, _, _ = afp_qem([[P[j][l] for j in range(J)] + [Q[j][l] for j in range(J)] + [f32(lam), ruv] for l in range(32)], bmax)
            br, bn, bitv, bmov = afp_qpa(db, bmax, bmax)
        except AssertionError:
            continue
        sb = f32(2.0 ** br)
        gp, gq = np.empty(k, f32), np.empty(k, f32)
        if bn == 8:
            rev = f32(1) / (sb * sb)
            ruv_i, lam_i = sat(roundf(ruv * sb)), sat(roundf(f32(-1.0) * f32(lam) * sb))
            for e in range(k):
                pi, qi = sat(roundf(p[e] * sb)), sat(roundf(q[e] * sb))
                gp[e] = f32(qi * ruv_i + pi * lam_i) * rev
                gq[e] = f32(pi * ruv_i + qi * lam_i) * rev
        else:
            t_ruv, t_lam = grid_h(ruv, sb), grid_h(f32(-1.0) * f32(lam), sb)
            for e in range(k):
                ph, qh = grid_h(p[e], sb), grid_h(q[e], sb)
                gp[e] = f32(hadd(hmul(qh, t_ruv), hmul(ph, t_lam)))
                gq[e] = f32(hadd(hmul(ph, t_ruv), hmul(qh, t_lam)))
        want_p, want_q = (p + f32(lr) * gp).astype(f32), (q + f32(lr) * gq).astype(f32)
        st = AfpState()
        orc.lib.orc_afp_state_init(C.byref(st))
        p1, q1 = p.copy(), q.copy()
        orc.lib.orc_afp_update(k, C.byref(st), p1.ctypes.data, q1.ctypes.data, r, lr, lam, 1, 10)
        assert (st.user.r, st.user.n, st.item.r, st.item.n, st.backward.r, st.backward.n) == (ur, un, ir, in_, br, bn), trial
        assert abs(st.user.itv - uitv) <= 1 and abs(st.item.itv - iitv) <= 1 and abs(st.backward.itv - bitv) <= 1
        assert np.array_equal(p1.view(np.uint32), want_p.view(np.uint32)) and np.array_equal(q1.view(np.uint32), want_q.view(np.uint32)), trial
        seen.add((un, in_, bn))
        done += 1
        if done >= 40 and len(seen) >= 2:
            break
    # the int8 forward path (both sides 8 bit), the int8 backward path and the binary16-grid paths all occurred
    # (all three at 8 bit together is the hand-worked row of test_afp_first_update_hand_worked)
    assert done >= 40 and any(s[0] == 8 and s[1] == 8 for s in seen) and any(s[2] == 8 for s in seen) and any(s[0] == 16 or s[1] == 16 for s in seen) and any(s[2] == 16 for s in seen), seen


def test_afp_interval_schedule(orc):
    """The quantisers are re-measured when cur_iter reaches their update iteration, and not in between: run five updates
    of a later epoch on the hand-worked 16-bit row (interval about 69) -- only the first measures; and five updates in the
    first tenth of epoch 0 (threshold 10) -- every one measures (itv forced to 1), the sixth onwards would not be."""
    from oracle.oracle import AfpState
    k = 64
    for epoch, expect in ((1, None), (0, 1)):
        p, q = np.full(k, 0.3, f32), np.full(k, 0.3, f32)
        st = AfpState()
        orc.lib.orc_afp_state_init(C.byref(st))
        first_itv = None
        for it in range(5):
            orc.lib.orc_afp_update(k, C.byref(st), p.ctypes.data, q.ctypes.data, 3.0, 0.01, 0.05, epoch, 10)
            if it == 0:
                first_itv = st.user.itv
            assert st.cur_iter == it + 1
            if epoch == 1:
                assert st.update_user_params_iter == first_itv and first_itv > 5      # not re-measured: still the first interval
            else:
                assert st.user.itv == 1 and st.update_user_params_iter == it + 1      # measured on every update
    # past the first tenth of epoch 0 the measured interval applies again
    p, q = np.full(k, 0.3, f32), np.full(k, 0.3, f32)
    st = AfpState()
    orc.lib.orc_afp_state_init(C.byref(st))
    for it in range(3):
        orc.lib.orc_afp_update(k, C.byref(st), p.ctypes.data, q.ctypes.data, 3.0, 0.01, 0.05, 0, 2)      # threshold 2: updates 0 and 1 are forced
    assert st.user.itv > 1 and st.update_user_params_iter == 2 + st.user.itv


# ---- MuPPET ladder ------------------------------------------------------------------------------------------------
def test_muppet_ladder_hand_worked_history(orc):
    """mf_methods.cu:659-697 on a five-epoch history with k = 2 whose every figure can be followed by hand.

    Diversity of epochs e-2..e: (sum of the three epochs' norm sums) / |sum of the three epochs' gradient sums|^2.
    epoch  norms  gradient sum   window                      diversity            max     ratio   threshold 1 + 1.5 e^(-0.3 e)
      0     12     (2, 0)         -- (fewer than 3 epochs since the start: switched_epoch = -1, e - (-1) = 1)
      1     12     (2, 0)         -- (2)
      2     12     (2, 0)         36 / |(6, 0)|^2 = 1        1       1       1.823  no switch
      3     24     (1, 1)         48 / |(5, 1)|^2 = 48/26    1.846   1       1.610  no switch
      4      6     (3, 4)         42 / |(6, 5)|^2 = 42/61    0.689   1.846 / 0.689 = 2.68 > 1.452: switch, state reset
      5      6     (3, 4)         -- (5 - 4 = 1 epoch since the switch)
      7      ...   first window after the switch is epochs 5..7"""
    k = 2
    norms = np.array([12, 12, 12, 24, 6, 6, 6, 6], f32)
    sums = np.array([[2, 0], [2, 0], [2, 0], [1, 1], [3, 4], [3, 4], [3, 4], [3, 4]], f32)
    switched, pidx, viol, maxdiv = C.c_int(-1), C.c_int(0), C.c_int(0), C.c_float(-1.0)
    trace = []
    for e in range(8):
        moved = orc.lib.orc_muppet_ladder_step(k, e, C.byref(switched), C.byref(pidx), C.byref(maxdiv), C.byref(viol),
                                               norms.ctypes.data, sums.ctypes.data)
        trace.append((moved, pidx.value, switched.value, round(float(maxdiv.value), 4)))
    assert trace[0] == (0, 0, -1, -1.0) and trace[1] == (0, 0, -1, -1.0)
    assert trace[2] == (0, 0, -1, 1.0)
    assert trace[3] == (0, 0, -1, round(48 / 26, 4))
    assert trace[4] == (1, 1, 4, -1.0)                       # ratio 2.68 against 1 + 1.5 exp(-1.2) = 1.452
    assert trace[5] == (0, 1, 4, -1.0) and trace[6] == (0, 1, 4, -1.0)
    assert trace[7] == (0, 1, 4, round(18 / (81 + 144), 4))  # epochs 5..7: 18 / |(9, 12)|^2 = 0.08; ratio 1, no switch
    # one notch below the threshold does not switch: same history with epoch 4's gradient sum scaled so that the ratio is 1.4
    # (diversity_4 = 1.846 / 1.4 = 1.3187 = 42 / |v|^2 -> |v|^2 = 31.85 with v = (2, 0) + (1, 1) + g: g = (2.55, 0) gives 31.80,
    # ratio 1.398 against 1.452)
    sums2 = sums.copy(); sums2[4] = (2.55, 0.0)
    switched, pidx, viol, maxdiv = C.c_int(-1), C.c_int(0), C.c_int(0), C.c_float(-1.0)
    for e in range(5):
        moved = orc.lib.orc_muppet_ladder_step(k, e, C.byref(switched), C.byref(pidx), C.byref(maxdiv), C.byref(viol),
                                               norms.ctypes.data, sums2.ctypes.data)
    assert moved == 0 and pidx.value == 0 and switched.value == -1
    assert abs(maxdiv.value / (42 / 31.8025) - 1.398) < 1e-3
    # and one notch above does: g = (2.3, 0) -> |v|^2 = 29.09, diversity 1.4438, ratio 1.2787 ... against epoch 4's threshold that
    # is still below; the threshold decays, so the same ratio 1.398 switches from epoch 6 on (1 + 1.5 exp(-1.8) = 1.248)
    norms3 = np.array([12, 12, 12, 24, 24, 24, 6], f32)
    sums3 = np.array([[2, 0], [2, 0], [2, 0], [1, 1], [1, 1], [1, 1], [3.55, 1]], f32)
    # windows: e=2: 36/36 = 1; e=3: 48/26 = 1.846; e=4: 60/|(4,2)|^2 = 3 (new max); e=5: 72/|(3,3)|^2 = 4 (new max);
    # e=6: 54/|(5.55,3)|^2 = 54/39.80 = 1.3567 -> ratio 4/1.3567 = 2.948 > 1.248: switch in epoch 6
    switched, pidx, viol, maxdiv = C.c_int(-1), C.c_int(1), C.c_int(0), C.c_float(-1.0)      # precision_idx starts at 1 (Yahoo, mf_methods.cu:600)
    moves = [orc.lib.orc_muppet_ladder_step(k, e, C.byref(switched), C.byref(pidx), C.byref(maxdiv), C.byref(viol),
                                            norms3.ctypes.data, sums3.ctypes.data) for e in range(7)]
    assert moves == [0, 0, 0, 0, 0, 0, 1] and pidx.value == 2 and switched.value == 6
