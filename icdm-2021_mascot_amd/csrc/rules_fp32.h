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
// What the dense fp32 rules broadcast per rating: the two rows as addresses (the matrix row, or this XCD's copy of a
// replicated row) and Rating::thin with four more bits, one per store window of the hot-row code (DenseBase::store).
// Addresses and window bits are computed once per chunk across the 64 lanes (DenseBase::prepare); per rating that costs
// two more v_readlane where the scalar unit would otherwise rebuild both addresses from the row ids for the loads and
// again for the stores and derive the four window sizes from thin (about forty scalar instructions per rating).
// Measured at 100M ratings: 7 to 11 % per epoch at k = 64, where these rules are bound by instruction issue, nothing at
// k = 128, where they are bound by the memory side; at 8M and 20M ratings, where a worker's chain of ratings is bound by
// latency, 5 and 13 % at k = 128 and 20 % at k = 64.
struct DenseAddrInfo { float r; uint32_t thin; uint64_t u, v; };
struct DenseAddrPrep { uint64_t pu, pv; uint32_t thin; };

template <int K, bool COH> struct DenseBase {
    static constexpr int E = K / 64;
    using Row = DenseRow<K>;
    using Info = DenseAddrInfo;      // u, v: the addresses of the two rows
    using Prep = DenseAddrPrep;
    // Chunk classes: 1 = no rating of the chunk has an update that is skipped (thinning is opt-in, so every chunk of a
    // default run): its loop carries no selects for it; 0 = the general loop.
    static constexpr int kClasses = 2;
    static constexpr int kK = K;
    template <class Params> static void row_storage(const Params& a, RowStorage& u, RowStorage& v) { u.dense = a.p; v.dense = a.q; }
    float* P;
    float* Q;
    float* RP;      // replica rows (Schedule::slot_u), or null
    float* RQ;
    float rep_scale;   // an update of a replicated row's copy takes a step this many times as long (Params::rep_scale)
    int lane;
    float lrate_rep;   // learning rate x rep_scale, for the rules whose learning rate is one number
    // the step factor of one side of a rating: bit = 16 (user row) or 32 (item row) of Info::thin marks a replicated row.
    // Selects between two wave-uniform numbers: scalar instructions.
    __device__ __forceinline__ float step_of(float lrate, uint32_t thin, uint32_t bit) const { return (thin & bit) ? lrate_rep : lrate; }
    __device__ __forceinline__ float scale_of(uint32_t thin, uint32_t bit) const { return (thin & bit) ? rep_scale : 1.0f; }

    // Bits of Info::thin above Rating::thin's six: the size of a row in bytes, a single bit, shifted left by 0..3 says
    // that the user / item row's window for device-coherent stores and the user / item row's window for cached stores
    // (the copy of a replicated row) is open, so that a window's size is one shift and one mask.
    static constexpr uint32_t kRowBytes = K * 4u;
    static_assert((kRowBytes & (kRowBytes - 1u)) == 0u && kRowBytes > 63u, "the window bits lie above Rating::thin's");
    // first element of a row of the matrix or, for a replicated row, of this XCD's copy
    template <class T> static __device__ __forceinline__ T* row_of(T* matrix, T* replicas, uint32_t row)
    {
        return ((row & kReplicaRow) ? replicas : matrix) + (size_t)(row & ~kReplicaRow) * K;
    }
    // side 0: the user row, 1: the item row.  A row's new value is stored unless the update is thinned or added
    // instead; a replicated row's copy is stored with an ordinary cached store (it stays in this XCD's L2) through a
    // second window with that cache policy.
    static __device__ __forceinline__ bool stores_row(uint32_t thin, int side) { return !((thin & (5u << side)) || (COH && (thin & (16u << side)))); }
    static __device__ __forceinline__ bool stores_copy(uint32_t thin, int side) { return COH && (thin & (20u << side)) == (16u << side); }
    __device__ __forceinline__ Prep prepare(const Rating& my, bool) const
    {
        Prep pr;
        pr.pu = reinterpret_cast<uint64_t>(row_of(P, RP, my.ru));
        pr.pv = reinterpret_cast<uint64_t>(row_of(Q, RQ, my.rv));
        pr.thin = my.thin | (stores_row(my.thin, 0) ? kRowBytes : 0u) | (stores_row(my.thin, 1) ? kRowBytes << 1 : 0u)
                  | (stores_copy(my.thin, 0) ? kRowBytes << 2 : 0u) | (stores_copy(my.thin, 1) ? kRowBytes << 3 : 0u);
        return pr;
    }
    __device__ __forceinline__ int classify(const Rating& my, const Prep&, bool valid) const
    {
        return __builtin_amdgcn_ballot_w64(valid && (my.thin & 3u)) == 0ull ? 1 : 0;
    }
    // bit = 1 (user row) or 2 (item row) of Info::thin: this side's update is skipped
    template <int CLS> static __device__ __forceinline__ bool skips(uint32_t thin, uint32_t bit) { return CLS == 0 && (thin & bit); }
    static __device__ __forceinline__ Info no_row() { return Info{0.f, 0u, 1ull, 1ull}; }   // matches no rating: no row lies at an odd address
    // equal addresses are the same row, which is all forward() needs
    __device__ __forceinline__ Info info(const Rating& my, const Prep& pr, int j) const
    {
        Info i;
        i.r = bcast(my.r, j);
        i.thin = bcast(pr.thin, j);
        i.u = bcast(pr.pu, j);
        i.v = bcast(pr.pv, j);
        return i;
    }
    template <int CLS> __device__ __forceinline__ void load(Row& row, const Info& i) const
    {
        const float* pp = reinterpret_cast<const float*>(i.u) + lane;
        const float* qq = reinterpret_cast<const float*>(i.v) + lane;
#pragma unroll
        for (int e = 0; e < E; ++e) { row.p[e] = row_load(pp + 64 * e); row.q[e] = row_load(qq + 64 * e); }
    }
    // dp, dq: the change of each element (new - old as the rule computes it), added to a hot row.  Kernels with
    // the hot-row code store through a row window (mf_device.h): one store per element and side is always
    // issued, and dropped when the update is thinned or added instead.  (Measured at 100M ratings, k = 128: 3 % faster
    // for these rules, whose epoch is bound by bytes in flight; the binary16 rules are bound by instruction issue,
    // lose more to the dropped stores than the longer look-ahead gives them, and keep their branches.)
    template <bool HOT> __device__ __forceinline__ void store(const Row& row, const Info& i, const float* dp, const float* dq) const
    {
        float* pp = reinterpret_cast<float*>(i.u) + lane;
        float* qq = reinterpret_cast<float*>(i.v) + lane;
        if constexpr (!HOT) {
#pragma unroll
            for (int e = 0; e < E; ++e) { row_store<COH>(pp + 64 * e, row.p[e]); row_store<COH>(qq + 64 * e, row.q[e]); }
        } else {
            const bool add_p = (i.thin & 5u) == 4u, add_q = (i.thin & 10u) == 8u;
            const row_window_t wp = row_window(i.u, i.thin & kRowBytes);
            const row_window_t wq = row_window(i.v, (i.thin >> 1) & kRowBytes);
#pragma unroll
            for (int e = 0; e < E; ++e) {
                window_store<COH>(wp, (uint32_t)(lane + 64 * e) * 4u, bits(row.p[e]));
                window_store<COH>(wq, (uint32_t)(lane + 64 * e) * 4u, bits(row.q[e]));
            }
            if constexpr (COH) {
                const row_window_t rp = row_window(i.u, (i.thin >> 2) & kRowBytes);
                const row_window_t rq = row_window(i.v, (i.thin >> 3) & kRowBytes);
#pragma unroll
                for (int e = 0; e < E; ++e) {
                    window_store<false>(rp, (uint32_t)(lane + 64 * e) * 4u, bits(row.p[e]));
                    window_store<false>(rq, (uint32_t)(lane + 64 * e) * 4u, bits(row.q[e]));
                }
            }
            if (add_p) {
#pragma unroll
                for (int e = 0; e < E; ++e) row_add(pp + 64 * e, dp[e]);
            }
            if (add_q) {
#pragma unroll
                for (int e = 0; e < E; ++e) row_add(qq + 64 * e, dq[e]);
            }
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
    struct Params { float* p; float* q; float lrate; float lambda; bool accumulate; void* rep_p; void* rep_q; float rep_scale; };
    float lrate, lambda;

    __device__ __forceinline__ void init(const Params& a, uint8_t*, int lane_, uint32_t)
    {
        this->P = a.p; this->Q = a.q; this->RP = static_cast<float*>(a.rep_p); this->RQ = static_cast<float*>(a.rep_q);
        this->lane = lane_; lrate = a.lrate; lambda = a.lambda; this->rep_scale = a.rep_scale; this->lrate_rep = a.lrate * a.rep_scale;
    }
    template <int CLS, bool HOT, bool SCALED> __device__ __forceinline__ void update(Row& row, const Info& i, uint32_t) const
    {
        float m[E];
#pragma unroll
        for (int e = 0; e < E; ++e) m[e] = row.p[e] * row.q[e];
        const float dot = dot_reference_order<E, float>(m);
        const float ruv = i.r - dot;
        const float lr_p = SCALED ? this->step_of(lrate, i.thin, 16u) : lrate, lr_q = SCALED ? this->step_of(lrate, i.thin, 32u) : lrate;
        float dp[E], dq[E];
#pragma unroll
        for (int e = 0; e < E; ++e) {
            const float pe = row.p[e], qe = row.q[e];
            dp[e] = lr_p * (ruv * qe - lambda * pe);
            dq[e] = lr_q * (ruv * pe - lambda * qe);
            row.p[e] = Base::template skips<CLS>(i.thin, 1u) ? pe : pe + dp[e];
            row.q[e] = Base::template skips<CLS>(i.thin, 2u) ? qe : qe + dq[e];
        }
        this->template store<HOT>(row, i, dp, dq);
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
    struct Params { float* p; float* q; float lrate; uint16_t scaled_lambda_half; float scaling_factor; bool accumulate; void* rep_p; void* rep_q; float rep_scale; };
    float lrate, scaling_factor_rev;
    half_t lambda_h, scaling_factor_h;

    __device__ __forceinline__ void init(const Params& a, uint8_t*, int lane_, uint32_t)
    {
        this->P = a.p; this->Q = a.q; this->RP = static_cast<float*>(a.rep_p); this->RQ = static_cast<float*>(a.rep_q);
        this->lane = lane_; lrate = a.lrate; this->rep_scale = a.rep_scale; this->lrate_rep = a.lrate * a.rep_scale;
        scaling_factor_rev = 1 / a.scaling_factor;
        scaling_factor_h = (half_t)a.scaling_factor;
        lambda_h = from_bits<half_t>(a.scaled_lambda_half);
    }
    template <int CLS, bool HOT, bool SCALED> __device__ __forceinline__ void update(Row& row, const Info& i, uint32_t) const
    {
        const half_t r_h = (half_t)i.r;
        half_t ph[E], qh[E], m[E];
#pragma unroll
        for (int e = 0; e < E; ++e) { ph[e] = (half_t)row.p[e]; qh[e] = (half_t)row.q[e]; m[e] = ph[e] * qh[e]; }
        const half_t dot = dot_reference_order<E, half_t>(m);
        const half_t ruv = scaling_factor_h * (r_h - dot);
        const float lr_p = SCALED ? this->step_of(lrate, i.thin, 16u) : lrate, lr_q = SCALED ? this->step_of(lrate, i.thin, 32u) : lrate;
        float dp[E], dq[E];
#pragma unroll
        for (int e = 0; e < E; ++e) {
            const half_t gp = ruv * qh[e] - lambda_h * ph[e];
            const half_t gq = ruv * ph[e] - lambda_h * qh[e];
            dp[e] = lr_p * (scaling_factor_rev * (float)gp);
            dq[e] = lr_q * (scaling_factor_rev * (float)gq);
            row.p[e] = Base::template skips<CLS>(i.thin, 1u) ? row.p[e] : row.p[e] + dp[e];
            row.q[e] = Base::template skips<CLS>(i.thin, 2u) ? row.q[e] : row.q[e] + dq[e];
        }
        this->template store<HOT>(row, i, dp, dq);
    }
    __device__ __forceinline__ void finish(const Params&, uint32_t) const {}
};

// mem_quant_sgd_k128/k64_hogwild_kernel, sgd/sgd_kernel.h:81-164: dense binary16 P/Q, binary32 arithmetic.
// k = 64: lane L holds element L.  k = 128: lane L holds the pair of elements 2L, 2L+1 (one 4-byte access per lane and
// side, as in the MASCOT kernel).  The reference's lane l sums its products left to right,
// p1*q1 + p2*q2 + p3*q3 + p4*q4 over elements l, l+32, l+64, l+96, and then runs the 16,8,4,2,1 tree over l.  Element
// l + 32j sits in row j of 16 lanes, position l/2, half l%2: the four rows are summed in order first, the tree's
// steps 16,8,4,2 are rotations by 8,4,2,1 inside a row and its last step adds the two halves.
template <int K, bool COH> struct MemQuantRule {
    static constexpr int E = K / 64;
    struct Row { uint32_t p, q; };      // the binary16 values as loaded (a pair at k = 128): half the registers of widened rows
    using Info = DenseAddrInfo;         // u, v: the addresses of the two rows, computed once per chunk (as for the fp32 rules)
    struct Prep { uint64_t pu, pv; };
    static constexpr int kClasses = 2;      // 1: no update of the chunk is skipped (as for the fp32 rules)
    static constexpr int kAhead = 3, kRing = 8;
    static constexpr bool kSplittable = true;
    struct Params { uint16_t* p; uint16_t* q; float lrate; float lambda; bool accumulate; void* rep_p; void* rep_q; float rep_scale; };
    uint16_t* P; uint16_t* Q; uint16_t* RP; uint16_t* RQ; float lrate, lambda, lrate_rep; int lane;

    __device__ __forceinline__ void init(const Params& a, uint8_t*, int lane_, uint32_t)
    {
        P = a.p; Q = a.q; RP = static_cast<uint16_t*>(a.rep_p); RQ = static_cast<uint16_t*>(a.rep_q); lrate = a.lrate; lambda = a.lambda; lane = lane_;
        lrate_rep = a.lrate * a.rep_scale;
    }
    // a replica slot is k * 4 bytes for every rule; a binary16 row fills its first half
    static __device__ __forceinline__ uint16_t* row_of(uint16_t* matrix, uint16_t* replicas, uint32_t row)
    {
        return (row & kReplicaRow) ? replicas + (size_t)(row & ~kReplicaRow) * (2 * K) : matrix + (size_t)row * K;
    }
    static constexpr int kK = K;
    static void row_storage(const Params& a, RowStorage& u, RowStorage& v) { u.dense = a.p; u.elem_bytes = 2; v.dense = a.q; v.elem_bytes = 2; }
    __device__ __forceinline__ Prep prepare(const Rating& my, bool) const
    {
        return Prep{reinterpret_cast<uint64_t>(row_of(P, RP, my.ru)), reinterpret_cast<uint64_t>(row_of(Q, RQ, my.rv))};
    }
    __device__ __forceinline__ int classify(const Rating& my, const Prep&, bool valid) const
    {
        return __builtin_amdgcn_ballot_w64(valid && (my.thin & 3u)) == 0ull ? 1 : 0;
    }
    static __device__ __forceinline__ Info no_row() { return Info{0.f, 0u, 1ull, 1ull}; }      // no row lies at an odd address
    __device__ __forceinline__ Info info(const Rating& my, const Prep& pr, int j) const
    {
        Info i;
        i.r = bcast(my.r, j); i.thin = bcast(my.thin, j); i.u = bcast(pr.pu, j); i.v = bcast(pr.pv, j);
        return i;
    }
    __device__ __forceinline__ uint32_t load_side(const uint16_t* row) const
    {
        if constexpr (E == 2) return row_load(reinterpret_cast<const uint32_t*>(row) + lane);
        else return (uint32_t)row_load(row + lane);
    }
    template <int CLS> __device__ __forceinline__ void load(Row& row, const Info& i) const
    {
        row.p = load_side(reinterpret_cast<const uint16_t*>(i.u));
        row.q = load_side(reinterpret_cast<const uint16_t*>(i.v));
    }
    __device__ __forceinline__ void forward(Row& nxt, const Info& in, const Row& cur, const Info& ic) const
    {
        if (in.u == ic.u) nxt.p = cur.p;
        if (in.v == ic.v) nxt.q = cur.q;
    }
    static __device__ __forceinline__ void widen(float* f, uint32_t raw)
    {
        if constexpr (E == 2) { const half2_t h = from_bits<half2_t>(raw); f[0] = (float)h.x; f[1] = (float)h.y; }
        else f[0] = (float)from_bits<half_t>(raw);
    }
    static __device__ __forceinline__ uint32_t narrow(const float* f)
    {
        if constexpr (E == 2) { half2_t h; h.x = (half_t)f[0]; h.y = (half_t)f[1]; return bits(h); }
        else return bits((half_t)f[0]);
    }
    // store the rounded row, or add the rounded change to a hot row
    __device__ __forceinline__ void write_side(uint16_t* row, uint32_t now, const float* change, bool hot, bool replicated) const
    {
        if (replicated && !hot) {      // this XCD's copy: an ordinary cached store
            if constexpr (E == 2) row_store<false>(reinterpret_cast<uint32_t*>(row) + lane, now);
            else row_store<false>(row + lane, (uint16_t)now);
            return;
        }
        if constexpr (E == 2) {
            uint32_t* at = reinterpret_cast<uint32_t*>(row) + lane;
            if (hot) row_add(reinterpret_cast<half2_t*>(at), from_bits<half2_t>(narrow(change)));
            else row_store<COH>(at, now);
        } else {
            if (hot) {      // even lanes add the pair (own, right neighbour)
                const uint32_t mine = narrow(change);
                const uint32_t other = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)mine, 0xB1 /* quad_perm 1,0,3,2 */, 0xf, 0xf, false);
                if (!(lane & 1)) row_add(reinterpret_cast<half2_t*>(row + lane), from_bits<half2_t>(mine | (other << 16)));
            } else {
                row_store<COH>(row + lane, (uint16_t)now);
            }
        }
    }
    // The dot product at k = 128 from the products of the even (x) and odd (y) elements of every lane.  Per 16-lane
    // position the four rows are summed in order, ((row 0 + row 1) + row 2) + row 3, x in the lower half-wave and y in
    // the upper one at the same time: v_permlane32_swap(x, y) leaves [x.rows01, y.rows01] and [x.rows23, y.rows23],
    // v_permlane16_swap of each with itself spreads its even and its odd row.  Then the tree inside the rows
    // (rotations by 8, 4, 2, 1) and the last step, even + odd, across the half-waves.
    static __device__ __forceinline__ float dot_rows_in_order(float x, float y)
    {
        auto halves = __builtin_amdgcn_permlane32_swap(bits(x), bits(y), false, false);
        auto lo = __builtin_amdgcn_permlane16_swap(halves[0], halves[0], false, false);      // [0]: rows 0 0 | 0 0 of x | y, [1]: rows 1
        auto hi = __builtin_amdgcn_permlane16_swap(halves[1], halves[1], false, false);      // [0]: rows 2, [1]: rows 3
        float s = from_bits<float>(lo[0]) + from_bits<float>(lo[1]);
        s = s + from_bits<float>(hi[0]);
        s = s + from_bits<float>(hi[1]);
        s = reduce_row16(s, OpAdd());
        return step_xor32(s, OpAdd());
    }
    template <int CLS, bool HOT, bool SCALED> __device__ __forceinline__ void update(Row& row, const Info& i, uint32_t) const
    {
        float pf[E], qf[E];
        widen(pf, row.p); widen(qf, row.q);
        float dot;
        if constexpr (E == 1) {
            dot = reduce_wave(pf[0] * qf[0], OpAdd());                // k = 64: p1*q1 + p2*q2, then the tree
        } else {
            dot = dot_rows_in_order(pf[0] * qf[0], pf[1] * qf[1]);
        }
        const float ruv = i.r - dot;
        // a replicated row's copy takes a longer step (Params::rep_scale)
        const float lr_p = (SCALED && (i.thin & 16u)) ? lrate_rep : lrate, lr_q = (SCALED && (i.thin & 32u)) ? lrate_rep : lrate;
        float dp[E], dq[E], np[E], nq[E];
#pragma unroll
        for (int e = 0; e < E; ++e) {
            dp[e] = lr_p * (ruv * qf[e] - lambda * pf[e]);
            dq[e] = lr_q * (ruv * pf[e] - lambda * qf[e]);
            np[e] = pf[e] + dp[e];
            nq[e] = qf[e] + dq[e];
        }
        // the register copy is what the row holds afterwards: the sum rounded to binary16
        if (!(CLS == 0 && (i.thin & 1u))) { row.p = narrow(np); write_side(reinterpret_cast<uint16_t*>(i.u), row.p, dp, i.thin & 4u, i.thin & 16u); }
        if (!(CLS == 0 && (i.thin & 2u))) { row.q = narrow(nq); write_side(reinterpret_cast<uint16_t*>(i.v), row.q, dq, i.thin & 8u, i.thin & 32u); }
    }
    __device__ __forceinline__ void finish(const Params&, uint32_t) const {}
};

}  // namespace mf
