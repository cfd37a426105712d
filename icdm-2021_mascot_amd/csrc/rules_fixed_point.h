// MuPPET (block fixed point, muppet/muppet_sgd_kernel.h) and AFP (adaptive fixed point,
// afp/afp_sgd_kernel.h) update rules over dense fp32 P/Q.
//
// Both rules derive per-rating scale factors from warp-wide statistics whose value depends on how
// the reference groups elements per lane (lane l owns elements l, l+32, l+64, l+96 and sums them left
// to right before the tree).  To keep those sums bit-identical, the wavefront mirrors the 32-lane
// warp: lane L loads elements L and L+64, swaps with lane L^32, and then both half-waves hold, per
// lane, the same 2 (k=64) or 4 (k=128) values the reference lane (L mod 32) holds.  All statistics are
// computed redundantly in both halves with the reference's 16,8,4,2,1 tree; each lane finally
// updates and stores only the elements it loaded.
#pragma once
#include "rules_fp32.h"

namespace mf {

__device__ __forceinline__ uint32_t f2u_sat(float f)
{
    if (!(f > 0.0f)) return 0u;
    if (f >= 4294967296.0f) return 0xffffffffu;
    return (uint32_t)f;
}
__device__ __forceinline__ int f2i_sat(float f)
{
    if (f != f) return 0;
    if (f >= 2147483648.0f) return 2147483647;
    if (f <= -2147483648.0f) return (int)0x80000000;
    return (int)f;
}
__device__ __forceinline__ int f2i8_sat(float f)
{
    if (f != f) return 0;
    if (f > 127.0f) return 127;
    if (f < -128.0f) return -128;
    return (int)f;
}
// 2^n for an integer-valued exponent, exact (exp2f of an integer in the reference).
__device__ __forceinline__ float pow2u(uint32_t n) { return __builtin_ldexpf(1.0f, n > 1000u ? 1000 : (int)n); }
__device__ __forceinline__ float pow2i(int n) { return __builtin_ldexpf(1.0f, n > 1000 ? 1000 : (n < -1000 ? -1000 : n)); }

// Mirror: v[j] = element (L mod 32) + 32 j of the row, own[] = which of them this lane stores.
template <int K> struct Mirror {
    static constexpr int E = K / 64;
    static constexpr int J = K / 32;
    float v[J];
    __device__ __forceinline__ void build(const float* own, bool upper)
    {
#pragma unroll
        for (int e = 0; e < E; ++e) {
            const float other = lane_xor32(own[e]);
            v[2 * e] = upper ? other : own[e];
            v[2 * e + 1] = upper ? own[e] : other;
        }
    }
    __device__ __forceinline__ float own(int e, bool upper) const { return upper ? v[2 * e + 1] : v[2 * e]; }
};

template <class T, class Op> __device__ __forceinline__ T tree32(T x, Op op) { return reduce_half_wave(x, op); }

// get_only_scaling_factor, muppet_sgd_kernel.h:7-18, stored in an unsigned (:71-73)
__device__ __forceinline__ uint32_t muppet_scale_index(unsigned bitwidth, float max_v, float min_v)
{
    if (max_v == 0 && min_v == 0) return 0u;
    float val = (float)(1 << (bitwidth - 1));
    float max_val = (val - 1) + 0.5f;
    float min_val = (-val) - 0.5f;
    float range_best = fminf(fabsf(max_val / max_v), fabsf(min_val / min_v));
    return f2u_sat(floorf(__builtin_log2f(range_best)));
}
__device__ __forceinline__ half_t grid_h(float v, float s, float s_rev) { return (half_t)(roundf(v * s) * s_rev); }

template <int K, bool COH> struct MuppetRule : DenseBase<K, COH> {
    using Base = DenseBase<K, COH>;
    using typename Base::Row;
    using typename Base::Info;
    static constexpr int E = Base::E;
    static constexpr int J = K / 32;
    static constexpr int kAhead = 1, kRing = 4;
    struct Params {
        float* p; float* q; float lrate; float lambda; uint32_t first_sample;
        float* sum_updated_val; float* sum_norms; uint32_t num_workers; int fwd; int bwd; bool accumulate;
    };
    static constexpr bool kSplittable = false;     // per-worker statistics span the whole launch
    float lrate, lambda; uint32_t first_sample; float* sum_updated_val; int fwd, bwd;
    float sum_norms_reg;
    float grad_acc[K / 64];
    bool upper;

    __device__ __forceinline__ void init(const Params& a, uint8_t*, int lane_, uint32_t)
    {
        this->P = a.p; this->Q = a.q; this->lane = lane_; lrate = a.lrate; lambda = a.lambda;
        first_sample = a.first_sample; sum_updated_val = a.sum_updated_val; fwd = a.fwd; bwd = a.bwd;
        sum_norms_reg = 0.f; upper = lane_ >= 32;
#pragma unroll
        for (int e = 0; e < E; ++e) grad_acc[e] = 0.f;
    }
    template <int CLS> __device__ __forceinline__ void update(Row& row, const Info& i, uint32_t processed)
    {
        Mirror<K> p, q;
        p.build(row.p, upper); q.build(row.q, upper);
        float p_min = 0, p_max = 0, q_min = 0, q_max = 0, sp = 0, sq = 0, pred;
        if (fwd != 32) {
            p_min = p_max = p.v[0]; q_min = q_max = q.v[0];
#pragma unroll
            for (int j = 1; j < J; ++j) {
                p_min = fminf(p_min, p.v[j]); p_max = fmaxf(p_max, p.v[j]);
                q_min = fminf(q_min, q.v[j]); q_max = fmaxf(q_max, q.v[j]);
            }
            p_min = tree32(p_min, OpMin()); q_min = tree32(q_min, OpMin());
            p_max = tree32(p_max, OpMax()); q_max = tree32(q_max, OpMax());
            sp = pow2u(muppet_scale_index((unsigned)fwd, p_max, p_min));
            sq = pow2u(muppet_scale_index((unsigned)fwd, q_max, q_min));
        }
        if (fwd == 8) {
            int acc = 0;
#pragma unroll
            for (int j = 0; j < J; ++j) acc += f2i8_sat(roundf(p.v[j] * sp)) * f2i8_sat(roundf(q.v[j] * sq));
            acc = tree32(acc, OpAdd());
            pred = acc / (sp * sq);
        } else if (fwd == 32) {
            float a = p.v[0] * q.v[0] + p.v[1] * q.v[1];
            if constexpr (J == 4) { float b = p.v[2] * q.v[2] + p.v[3] * q.v[3]; a = a + b; }
            pred = tree32(a, OpAdd());
        } else {
            const float sp_rev = 1 / sp, sq_rev = 1 / sq;
            // half2 lanes of the reference: .x = elements l (and l+64), .y = elements l+32 (and l+96)
            half2_t t;
            t.x = grid_h(p.v[0], sp, sp_rev) * grid_h(q.v[0], sq, sq_rev);
            t.y = grid_h(p.v[1], sp, sp_rev) * grid_h(q.v[1], sq, sq_rev);
            if constexpr (J == 4) {
                half2_t t2;
                t2.x = grid_h(p.v[2], sp, sp_rev) * grid_h(q.v[2], sq, sq_rev);
                t2.y = grid_h(p.v[3], sp, sp_rev) * grid_h(q.v[3], sq, sq_rev);
                t = t + t2;
            }
            t = tree32(t, OpAdd());
            pred = (float)(half_t)(t.x + t.y);
        }
        const float ruv = i.r - pred;
        float sb = 0;
        if (bwd != 32) {
            const float neg_lambda = -1 * lambda;
            const float bmin = fminf(fminf(p_min, q_min), fminf(neg_lambda, ruv));
            const float bmax = fmaxf(fmaxf(p_max, q_max), fmaxf(neg_lambda, ruv));
            sb = pow2u(muppet_scale_index((unsigned)bwd, bmax, bmin));
        }
        float gp[J], gq[J];
        if (bwd == 8) {
            const float sq_rev = 1 / (sb * sb);
            const int ruv_i = f2i8_sat(roundf(ruv * sb));
            const int lam_i = f2i8_sat(roundf(-1.0f * lambda * sb));
#pragma unroll
            for (int j = 0; j < J; ++j) {
                const int pi = f2i8_sat(roundf(p.v[j] * sb)), qi = f2i8_sat(roundf(q.v[j] * sb));
                gp[j] = (float)(qi * ruv_i + pi * lam_i) * sq_rev;
                gq[j] = (float)(pi * ruv_i + qi * lam_i) * sq_rev;
            }
        } else if (bwd == 32) {
#pragma unroll
            for (int j = 0; j < J; ++j) {
                gp[j] = ruv * q.v[j] - lambda * p.v[j];
                gq[j] = ruv * p.v[j] - lambda * q.v[j];
            }
        } else {
            const float sb_rev = 1 / sb;
            const half_t t_ruv = grid_h(ruv, sb, sb_rev), t_lam = grid_h(-1 * lambda, sb, sb_rev);
#pragma unroll
            for (int j = 0; j < J; ++j) {
                const half_t ph = grid_h(p.v[j], sb, sb_rev), qh = grid_h(q.v[j], sb, sb_rev);
                gp[j] = (float)(half_t)(qh * t_ruv + ph * t_lam);
                gq[j] = (float)(half_t)(ph * t_ruv + qh * t_lam);
            }
        }
#pragma unroll
        for (int e = 0; e < E; ++e) {
            float g = upper ? gp[2 * e + 1] : gp[2 * e];
            float h = upper ? gq[2 * e + 1] : gq[2 * e];
            row.p[e] = row.p[e] + lrate * g;
            row.q[e] = row.q[e] + lrate * h;
        }
        this->store(row, i);
        if (fwd != 32 && bwd != 32 && processed >= first_sample) {
            float np = gp[0] * gp[0] + gp[1] * gp[1];
            float nq = gq[0] * gq[0] + gq[1] * gq[1];
            if constexpr (J == 4) {
                float b = gp[2] * gp[2] + gp[3] * gp[3]; np = np + b;
                float c = gq[2] * gq[2] + gq[3] * gq[3]; nq = nq + c;
            }
            float npq = np + nq;
            npq = tree32(npq, OpAdd());
            sum_norms_reg += npq;
#pragma unroll
            for (int e = 0; e < E; ++e) {
                float g = upper ? gp[2 * e + 1] : gp[2 * e];
                float h = upper ? gq[2 * e + 1] : gq[2 * e];
                grad_acc[e] += g + h;       // flushed once per worker in finish()
            }
        }
    }
    __device__ __forceinline__ void finish(const Params& a, uint32_t wid) const
    {
        if (wid >= a.num_workers) return;
        if (this->lane == 0) a.sum_norms[wid] = sum_norms_reg;
#pragma unroll
        for (int e = 0; e < E; ++e)
            if (grad_acc[e] != 0.f) atomicAdd(a.sum_updated_val + this->lane + 64 * e, grad_acc[e]);
    }
};

// ---- AFP ---------------------------------------------------------------------------------------
struct AfpQ { int r; int n; int itv; float mov_avg_range; };

// get_only_scaling_factor_cvpr, afp_sgd_kernel.h:8-16
__device__ __forceinline__ float afp_scale_index(unsigned bitwidth, float max_v)
{
    if (max_v == 0) return 0;
    const float denom = pow2i((int)bitwidth - 1) - 1;
    return fabsf(ceilf(__builtin_log2f(max_v / denom)));
}
__device__ __forceinline__ float afp_grid(float v, float s, float s_rev) { return roundf(v * s) * s_rev; }
// QPA, afp_sgd_kernel.h:104-125
__device__ __forceinline__ AfpQ afp_qpa(float diff, float range, float prev)
{
    AfpQ q;
    const float threshold = 0.0005f, alpha = 0.04f, beta = 0.1f, delta = 100, gamma = 2;
    if (diff <= threshold) { q.r = f2i_sat(fabsf(ceilf(__builtin_log2f(range / (pow2i(8 - 1) - 1))))); q.n = 8; }
    else { q.r = f2i_sat(fabsf(ceilf(__builtin_log2f(range / (pow2i(16 - 1) - 1))))); q.n = 16; }
    q.mov_avg_range = alpha * range + (1.0f - alpha) * prev;
    float i1 = delta * diff * diff;
    float i2 = fabsf(q.mov_avg_range - prev);
    q.itv = f2i_sat((beta / fmaxf(i1, i2)) - gamma);
    return q;
}
__device__ __forceinline__ int afp_sat8(float t) { return (int)(t > 127.0f ? 127.0f : (t < -128.0f) ? -128.0f : t); }
__device__ __forceinline__ float ufirst(float x) { return from_bits<float>((uint32_t)__builtin_amdgcn_readfirstlane((int)bits(x))); }
__device__ __forceinline__ int ufirst(int x) { return __builtin_amdgcn_readfirstlane(x); }

template <int K, bool COH> struct AfpRule : DenseBase<K, COH> {
    using Base = DenseBase<K, COH>;
    using typename Base::Row;
    using typename Base::Info;
    static constexpr int E = Base::E;
    static constexpr int J = K / 32;
    static constexpr int kAhead = 1, kRing = 4;
    static constexpr bool kSplittable = false;    // the per-worker quantiser state lives for one launch
    struct Params { float* p; float* q; float lrate; float lambda; int afp_epoch; int init_threshold; bool accumulate; };
    float lrate, lambda; int afp_epoch, init_threshold;
    AfpQ uq, iq, bq;
    int upd_u, upd_i, upd_b, cur_iter;
    float sp, sq, sb;
    bool upper;

    __device__ __forceinline__ void init(const Params& a, uint8_t*, int lane_, uint32_t)
    {
        this->P = a.p; this->Q = a.q; this->lane = lane_; lrate = a.lrate; lambda = a.lambda;
        afp_epoch = a.afp_epoch; init_threshold = a.init_threshold;
        uq = AfpQ{0, 0, 0, 0.f}; iq = uq; bq = uq;
        upd_u = upd_i = upd_b = cur_iter = 0; sp = sq = sb = 0.f; upper = lane_ >= 32;
    }
    // QEM / QEM_64, afp_sgd_kernel.h:32-59
    __device__ __forceinline__ float qem(const float* v, float max_v) const
    {
        const float s = pow2u(f2u_sat(afp_scale_index(8, max_v))), s_rev = 1 / s;
        float aq = fabsf(afp_grid(v[0], s, s_rev)), a = fabsf(v[0]);
#pragma unroll
        for (int j = 1; j < J; ++j) { aq = aq + fabsf(afp_grid(v[j], s, s_rev)); a = a + fabsf(v[j]); }
        aq = tree32(aq, OpAdd()); a = tree32(a, OpAdd());
        return __builtin_log2f(fabsf((a - aq) / a) + 1);
    }
    // QEM_BP / QEM_BP_64, afp_sgd_kernel.h:61-102
    __device__ __forceinline__ float qem_bp(const float* p, const float* q, float ruv, float max_v) const
    {
        const float s = pow2u(f2u_sat(afp_scale_index(8, max_v))), s_rev = 1 / s;
        float aq = fabsf(afp_grid(p[0], s, s_rev)), a = fabsf(p[0]);
#pragma unroll
        for (int j = 1; j < J; ++j) { aq = aq + fabsf(afp_grid(p[j], s, s_rev)); a = a + fabsf(p[j]); }
#pragma unroll
        for (int j = 0; j < J; ++j) { aq = aq + fabsf(afp_grid(q[j], s, s_rev)); a = a + fabsf(q[j]); }
        aq = aq + fabsf(afp_grid(lambda, s, s_rev)); a = a + fabsf(lambda);
        aq = aq + fabsf(afp_grid(ruv, s, s_rev)); a = a + fabsf(ruv);
        aq = tree32(aq, OpAdd()); a = tree32(a, OpAdd());
        return __builtin_log2f(fabsf((a - aq) / a) + 1);
    }
    static __device__ __forceinline__ AfpQ uniform(AfpQ q)
    {
        q.r = ufirst(q.r); q.n = ufirst(q.n); q.itv = ufirst(q.itv); q.mov_avg_range = ufirst(q.mov_avg_range);
        return q;
    }
    template <int CLS> __device__ __forceinline__ void update(Row& row, const Info& i, uint32_t)
    {
        Mirror<K> p, q;
        p.build(row.p, upper); q.build(row.q, upper);
        float p_abs = fabsf(p.v[0]), q_abs = fabsf(q.v[0]);
#pragma unroll
        for (int j = 1; j < J; ++j) { p_abs = fmaxf(p_abs, fabsf(p.v[j])); q_abs = fmaxf(q_abs, fabsf(q.v[j])); }
        if (cur_iter == upd_u) {
            const float mx = tree32(p_abs, OpMax());
            const float diff = qem(p.v, mx);
            if (cur_iter == 0) uq.mov_avg_range = mx;
            uq = uniform(afp_qpa(diff, mx, uq.mov_avg_range));
            sp = pow2i(uq.r);
            if (afp_epoch == 0 && cur_iter < init_threshold) uq.itv = 1;
            upd_u += uq.itv;
        }
        if (cur_iter == upd_i) {
            const float mx = tree32(q_abs, OpMax());
            const float diff = qem(q.v, mx);
            if (cur_iter == 0) iq.mov_avg_range = mx;
            iq = uniform(afp_qpa(diff, mx, iq.mov_avg_range));
            sq = pow2i(iq.r);
            if (afp_epoch == 0 && cur_iter < init_threshold) iq.itv = 1;
            upd_i += iq.itv;
        }
        float pred;
        if (uq.n == 8 && iq.n == 8) {
            int acc = 0;
#pragma unroll
            for (int j = 0; j < J; ++j) acc += afp_sat8(roundf(p.v[j] * sp)) * afp_sat8(roundf(q.v[j] * sq));
            acc = tree32(acc, OpAdd());
            pred = acc / (sp * sq);
        } else {
            const float sp_rev = 1 / sp, sq_rev = 1 / sq;
            half2_t t;
            t.x = (half_t)afp_grid(p.v[0], sp, sp_rev) * (half_t)afp_grid(q.v[0], sq, sq_rev);
            t.y = (half_t)afp_grid(p.v[1], sp, sp_rev) * (half_t)afp_grid(q.v[1], sq, sq_rev);
            if constexpr (J == 4) {
                half2_t t2;
                t2.x = (half_t)afp_grid(p.v[2], sp, sp_rev) * (half_t)afp_grid(q.v[2], sq, sq_rev);
                t2.y = (half_t)afp_grid(p.v[3], sp, sp_rev) * (half_t)afp_grid(q.v[3], sq, sq_rev);
                t = t + t2;
            }
            t = tree32(t, OpAdd());
            pred = (float)(half_t)(t.x + t.y);
        }
        const float ruv = i.r - pred;
        if (cur_iter == upd_b) {
            float mx = fmaxf(p_abs, q_abs);
            mx = fmaxf(fmaxf(mx, fabsf(lambda)), fabsf(ruv));
            mx = tree32(mx, OpMax());
            const float diff = qem_bp(p.v, q.v, ruv, mx);
            if (cur_iter == 0) bq.mov_avg_range = mx;
            bq = uniform(afp_qpa(diff, mx, bq.mov_avg_range));
            sb = pow2i(bq.r);
            if (afp_epoch == 0 && cur_iter < init_threshold) bq.itv = 1;
            upd_b += bq.itv;
        }
        float gp[J], gq[J];
        if (bq.n == 8) {
            const int lam_i = afp_sat8(roundf(-1.0f * lambda * sb));
            const int ruv_i = afp_sat8(roundf(ruv * sb));
            const float sq_rev = 1 / (sb * sb);
#pragma unroll
            for (int j = 0; j < J; ++j) {
                const int pi = afp_sat8(roundf(p.v[j] * sb)), qi = afp_sat8(roundf(q.v[j] * sb));
                gp[j] = (float)(qi * ruv_i + pi * lam_i) * sq_rev;
                gq[j] = (float)(pi * ruv_i + qi * lam_i) * sq_rev;
            }
        } else {
            const float sb_rev = 1 / sb;
            const half_t t_ruv = (half_t)afp_grid(ruv, sb, sb_rev), t_lam = (half_t)afp_grid(-1.0f * lambda, sb, sb_rev);
#pragma unroll
            for (int j = 0; j < J; ++j) {
                const half_t ph = (half_t)afp_grid(p.v[j], sb, sb_rev), qh = (half_t)afp_grid(q.v[j], sb, sb_rev);
                gp[j] = (float)(half_t)(qh * t_ruv + ph * t_lam);
                gq[j] = (float)(half_t)(ph * t_ruv + qh * t_lam);
            }
        }
#pragma unroll
        for (int e = 0; e < E; ++e) {
            const float g = upper ? gp[2 * e + 1] : gp[2 * e];
            const float h = upper ? gq[2 * e + 1] : gq[2 * e];
            row.p[e] = row.p[e] + lrate * g;
            row.q[e] = row.q[e] + lrate * h;
        }
        this->store(row, i);
        cur_iter += 1;
    }
    __device__ __forceinline__ void finish(const Params&, uint32_t) const {}
};

}  // namespace mf
