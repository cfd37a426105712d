// Update rules over dense fp32 P/Q: plain SGD and MPT (fp32 master, binary16 arithmetic).
//
// Row layout in registers: lane L holds element L (k = 64) or elements L and L+64 (k = 128); every
// row access is one or two fully coalesced 256-byte loads.  With that ownership the reference's
// summation order -- warp lane l adds elements l, l+32, l+64, l+96 as ((a+b)+(c+d)) and a
// 16,8,4,2,1 tree follows (sgd/sgd_kernel.h:55-63) -- is reproduced exactly by
//   t0 = m[L] + m[L^32]; t1 = m[L+64] + m[(L^32)+64]; s = t0 + t1; tree over 16,8,4,2,1,
// so results are bit-identical to a sequential evaluation in the reference's order.
#pragma once
#include "hogwild.h"

namespace mf {

template <int K> struct DenseRow {
    static constexpr int E = K / 64;
    float p[E], q[E];
};
struct DenseInfo { float r; uint32_t u, v, thin; };
struct NoPrep {};

template <int K, bool COH> struct DenseBase {
    static constexpr int E = K / 64;
    using Row = DenseRow<K>;
    using Info = DenseInfo;
    using Prep = NoPrep;
    static constexpr int kClasses = 1;
    float* P;
    float* Q;
    int lane;

    __device__ __forceinline__ Prep prepare(const Rating&, bool) const { return Prep(); }
    __device__ __forceinline__ int classify(const Prep&, bool) const { return 0; }
    static __device__ __forceinline__ Info no_row() { return Info{0.f, 0xffffffffu, 0xffffffffu, 0u}; }   // matches no rating
    __device__ __forceinline__ Info info(const Rating& my, const Prep&, int j) const
    {
        Info i;
        i.r = bcast(my.r, j);
        i.u = bcast(my.u, j);
        i.v = bcast(my.v, j);
        i.thin = bcast(my.thin, j);
        return i;
    }
    template <int CLS> __device__ __forceinline__ void load(Row& row, const Info& i) const
    {
        const float* pp = P + (size_t)i.u * K + lane;
        const float* qq = Q + (size_t)i.v * K + lane;
#pragma unroll
        for (int e = 0; e < E; ++e) { row.p[e] = row_load(pp + 64 * e); row.q[e] = row_load(qq + 64 * e); }
    }
    // dp, dq: the change of each element (new - old as the rule computes it), added to a hot row
    __device__ __forceinline__ void store(const Row& row, const Info& i, const float* dp, const float* dq) const
    {
        float* pp = P + (size_t)i.u * K + lane;
        float* qq = Q + (size_t)i.v * K + lane;
        if (!(i.thin & 1u)) {
#pragma unroll
            for (int e = 0; e < E; ++e) { if (i.thin & 4u) row_add(pp + 64 * e, dp[e]); else row_store<COH>(pp + 64 * e, row.p[e]); }
        }
        if (!(i.thin & 2u)) {
#pragma unroll
            for (int e = 0; e < E; ++e) { if (i.thin & 8u) row_add(qq + 64 * e, dq[e]); else row_store<COH>(qq + 64 * e, row.q[e]); }
        }
    }
    // rules that keep last-writer-wins on every row
    __device__ __forceinline__ void store(const Row& row, const Info& i) const
    {
        float* pp = P + (size_t)i.u * K + lane;
        float* qq = Q + (size_t)i.v * K + lane;
        if (!(i.thin & 1u)) {
#pragma unroll
            for (int e = 0; e < E; ++e) row_store<COH>(pp + 64 * e, row.p[e]);
        }
        if (!(i.thin & 2u)) {
#pragma unroll
            for (int e = 0; e < E; ++e) row_store<COH>(qq + 64 * e, row.q[e]);
        }
    }
    __device__ __forceinline__ void forward(Row& nxt, const Info& in, const Row& cur, const Info& ic) const
    {
        if (in.u == ic.u) {
#pragma unroll
            for (int e = 0; e < E; ++e) nxt.p[e] = cur.p[e];
        }
        if (in.v == ic.v) {
#pragma unroll
            for (int e = 0; e < E; ++e) nxt.q[e] = cur.q[e];
        }
    }
};

// Sum over the k products in the reference order; T is float or half_t, m[e] the product of element L+64e.
template <int E, class T> __device__ __forceinline__ T dot_reference_order(const T* m)
{
    if constexpr (E == 1) {
        return reduce_wave(m[0], OpAdd());
    } else {
        T t0 = step_xor32(m[0], OpAdd());
        T t1 = step_xor32(m[1], OpAdd());
        T s = t0 + t1;
        return reduce_half_wave(s, OpAdd());
    }
}

// single_sgd_k128/k64_hogwild_kernel, sgd/sgd_kernel.h:55-76.
template <int K, bool COH> struct SgdRule : DenseBase<K, COH> {
    using Base = DenseBase<K, COH>;
    using typename Base::Row;
    using typename Base::Info;
    static constexpr int E = Base::E;
    static constexpr int kAhead = 3, kRing = 8;
    static constexpr bool kSplittable = true;
    struct Params { float* p; float* q; float lrate; float lambda; bool accumulate; };
    float lrate, lambda;

    __device__ __forceinline__ void init(const Params& a, uint8_t*, int lane_, uint32_t)
    {
        this->P = a.p; this->Q = a.q; this->lane = lane_; lrate = a.lrate; lambda = a.lambda;
    }
    template <int CLS> __device__ __forceinline__ void update(Row& row, const Info& i, uint32_t) const
    {
        float m[E];
#pragma unroll
        for (int e = 0; e < E; ++e) m[e] = row.p[e] * row.q[e];
        const float dot = dot_reference_order<E, float>(m);
        const float ruv = i.r - dot;
        float dp[E], dq[E];
#pragma unroll
        for (int e = 0; e < E; ++e) {
            const float pe = row.p[e], qe = row.q[e];
            dp[e] = lrate * (ruv * qe - lambda * pe);
            dq[e] = lrate * (ruv * pe - lambda * qe);
            row.p[e] = (i.thin & 1u) ? pe : pe + dp[e];
            row.q[e] = (i.thin & 2u) ? qe : qe + dq[e];
        }
        this->store(row, i, dp, dq);
    }
    __device__ __forceinline__ void finish(const Params&, uint32_t) const {}
};

// mpt_sgd_k128/k64_hogwild_kernel, mpt/mpt_sgd_kernel.h:15-16,38-91.
template <int K, bool COH> struct MptRule : DenseBase<K, COH> {
    using Base = DenseBase<K, COH>;
    using typename Base::Row;
    using typename Base::Info;
    static constexpr int E = Base::E;
    static constexpr int kAhead = 3, kRing = 8;
    static constexpr bool kSplittable = true;
    struct Params { float* p; float* q; float lrate; uint16_t scaled_lambda_half; float scaling_factor; bool accumulate; };
    float lrate, scaling_factor_rev;
    half_t lambda_h, scaling_factor_h;

    __device__ __forceinline__ void init(const Params& a, uint8_t*, int lane_, uint32_t)
    {
        this->P = a.p; this->Q = a.q; this->lane = lane_; lrate = a.lrate;
        scaling_factor_rev = 1 / a.scaling_factor;
        scaling_factor_h = (half_t)a.scaling_factor;
        lambda_h = from_bits<half_t>(a.scaled_lambda_half);
    }
    template <int CLS> __device__ __forceinline__ void update(Row& row, const Info& i, uint32_t) const
    {
        const half_t r_h = (half_t)i.r;
        half_t ph[E], qh[E], m[E];
#pragma unroll
        for (int e = 0; e < E; ++e) { ph[e] = (half_t)row.p[e]; qh[e] = (half_t)row.q[e]; m[e] = ph[e] * qh[e]; }
        const half_t dot = dot_reference_order<E, half_t>(m);
        const half_t ruv = scaling_factor_h * (r_h - dot);
        float dp[E], dq[E];
#pragma unroll
        for (int e = 0; e < E; ++e) {
            const half_t gp = ruv * qh[e] - lambda_h * ph[e];
            const half_t gq = ruv * ph[e] - lambda_h * qh[e];
            dp[e] = lrate * (scaling_factor_rev * (float)gp);
            dq[e] = lrate * (scaling_factor_rev * (float)gq);
            row.p[e] = (i.thin & 1u) ? row.p[e] : row.p[e] + dp[e];
            row.q[e] = (i.thin & 2u) ? row.q[e] : row.q[e] + dq[e];
        }
        this->store(row, i, dp, dq);
    }
    __device__ __forceinline__ void finish(const Params&, uint32_t) const {}
};

// mem_quant_sgd_k128/k64_hogwild_kernel, sgd/sgd_kernel.h:81-164: dense binary16 P/Q, binary32 arithmetic.  Lane L holds
// elements L and L+64 of a row (two coalesced 128-byte accesses), widened.  The reference's lane l sums its products
// left to right, p1*q1 + p2*q2 + p3*q3 + p4*q4 over elements l, l+32, l+64, l+96: with a = m0[l], b = m0[l+32],
// c = m1[l], d = m1[l+32] (l = L mod 32) that is ((a + b) + c) + d, formed identically in both half-waves.
template <int K, bool COH> struct MemQuantRule {
    static constexpr int E = K / 64;
    using Row = DenseRow<K>;
    using Info = DenseInfo;
    using Prep = NoPrep;
    static constexpr int kClasses = 1;
    static constexpr int kAhead = 3, kRing = 8;
    static constexpr bool kSplittable = true;
    struct Params { uint16_t* p; uint16_t* q; float lrate; float lambda; bool accumulate; };
    uint16_t* P; uint16_t* Q; float lrate, lambda; int lane;

    __device__ __forceinline__ void init(const Params& a, uint8_t*, int lane_, uint32_t) { P = a.p; Q = a.q; lrate = a.lrate; lambda = a.lambda; lane = lane_; }
    __device__ __forceinline__ Prep prepare(const Rating&, bool) const { return Prep(); }
    __device__ __forceinline__ int classify(const Prep&, bool) const { return 0; }
    static __device__ __forceinline__ Info no_row() { return Info{0.f, 0xffffffffu, 0xffffffffu, 0u}; }
    __device__ __forceinline__ Info info(const Rating& my, const Prep&, int j) const
    {
        Info i;
        i.r = bcast(my.r, j); i.u = bcast(my.u, j); i.v = bcast(my.v, j); i.thin = bcast(my.thin, j);
        return i;
    }
    template <int CLS> __device__ __forceinline__ void load(Row& row, const Info& i) const
    {
        const uint16_t* pp = P + (size_t)i.u * K + lane;
        const uint16_t* qq = Q + (size_t)i.v * K + lane;
#pragma unroll
        for (int e = 0; e < E; ++e) {
            row.p[e] = (float)from_bits<half_t>((uint32_t)row_load(pp + 64 * e));
            row.q[e] = (float)from_bits<half_t>((uint32_t)row_load(qq + 64 * e));
        }
    }
    __device__ __forceinline__ void forward(Row& nxt, const Info& in, const Row& cur, const Info& ic) const
    {
        if (in.u == ic.u) {
#pragma unroll
            for (int e = 0; e < E; ++e) nxt.p[e] = cur.p[e];
        }
        if (in.v == ic.v) {
#pragma unroll
            for (int e = 0; e < E; ++e) nxt.q[e] = cur.q[e];
        }
    }
    // store the rounded row, or add the rounded change to a hot row: even lanes add the pair (own, right neighbour)
    __device__ __forceinline__ void write_side(uint16_t* base, const float* now, const float* change, bool hot) const
    {
#pragma unroll
        for (int e = 0; e < E; ++e) {
            if (hot) {
                const uint32_t mine = bits((half_t)change[e]);
                const uint32_t other = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)mine, 0xB1 /* quad_perm 1,0,3,2 */, 0xf, 0xf, false);
                if (!(lane & 1)) row_add(reinterpret_cast<half2_t*>(base + 64 * e), from_bits<half2_t>(mine | (other << 16)));
            } else {
                row_store<COH>(base + 64 * e, (uint16_t)bits((half_t)now[e]));
            }
        }
    }
    template <int CLS> __device__ __forceinline__ void update(Row& row, const Info& i, uint32_t) const
    {
        float dot;
        if constexpr (E == 1) {
            dot = reduce_wave(row.p[0] * row.q[0], OpAdd());                // k = 64: p1*q1 + p2*q2, then the tree
        } else {
            const float m0 = row.p[0] * row.q[0], m1 = row.p[1] * row.q[1];
            const float o0 = lane_xor32(m0), o1 = lane_xor32(m1);
            const bool upper = lane >= 32;
            float s = m0 + o0;                                              // a + b
            s = s + (upper ? o1 : m1);                                      // + c
            s = s + (upper ? m1 : o1);                                      // + d
            dot = reduce_half_wave(s, OpAdd());
        }
        const float ruv = i.r - dot;
        float dp[E], dq[E];
#pragma unroll
        for (int e = 0; e < E; ++e) {
            const float pe = row.p[e], qe = row.q[e];
            dp[e] = lrate * (ruv * qe - lambda * pe);
            dq[e] = lrate * (ruv * pe - lambda * qe);
            // the register copy is what the row holds afterwards: the sum rounded to binary16
            row.p[e] = (i.thin & 1u) ? pe : (float)(half_t)(pe + dp[e]);
            row.q[e] = (i.thin & 2u) ? qe : (float)(half_t)(qe + dq[e]);
        }
        if (!(i.thin & 1u)) write_side(P + (size_t)i.u * K + lane, row.p, dp, i.thin & 4u);
        if (!(i.thin & 2u)) write_side(Q + (size_t)i.v * K + lane, row.q, dq, i.thin & 8u);
    }
    __device__ __forceinline__ void finish(const Params&, uint32_t) const {}
};

}  // namespace mf
