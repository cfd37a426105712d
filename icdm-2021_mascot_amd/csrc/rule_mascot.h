// MASCOT update rule: P/Q stored per popularity group as binary16 or binary32 rows
// (mascot/mascot_sgd_kernel.h:1-457 and _k64.h of the reference), four precision cases per rating,
// sampled gradient statistics for the g-switching estimator.
//
// Register layout: lane L holds elements 2L, 2L+1 of a row (k = 128; one packed dword for a binary16
// row, one 8-byte load for a binary32 row) or element L (k = 64).  For k = 128 the reference's
// order -- warp lane l sums elements l, l+32, l+64, l+96 as ((a+b)+(c+d)), then a 16,8,4,2,1 tree --
// maps onto packed lanes as: step over lanes L^16 (elements +32), lanes L^32 (+64), then rotates by
// 8,4,2,1 inside a row of 16 lanes (warp lanes +16,+8,+4,+2) and finally low half + high half
// (warp lanes +1).  Every add is a packed v_pk_add_f16, each half rounded separately, so the
// binary16 dot is bit-identical to the reference's sequence of roundings.
//
// The group search of the reference (two 32-wide register compares plus a shared-memory fallback per
// rating, mascot_sgd_kernel.h:104-180) is replaced by one binary search per lane over the end-index
// table in LDS, done once for the 64 ratings of a chunk; the result is the row address, which is
// what the per-rating loop broadcasts.
#pragma once
#include "hogwild.h"

namespace mf {

// SAMPLED = false compiles the sampled-statistics code out: the kernel for launches in which no rating is sampled.
// MIXED = false compiles the straight-line path for chunks of mixed precisions out (such chunks take the general path,
// so the results are the same): the kernel for runs in which every group is still binary16, which then keeps the
// registers of the binary16 path alone and with them one more resident wavefront per SIMD.
template <int K, bool COH, bool SAMPLED, bool MIXED = true> struct MascotRuleT {
    static constexpr int E = K / 64;                        // elements per lane
    static constexpr int kAhead = 3, kRing = 8;
    // chunks of mixed precisions look two ratings ahead (measured at 100M and 250M ratings: three ratings make the states
    // with some groups promoted 1-20 % slower and only the all-promoted state 3 % faster)
    static constexpr int kAheadClass2 = 2;
    // chunk classes: 1 = every rating of the chunk touches two binary16 rows (the state every group starts in): loads
    // and arithmetic without any branching; 2 = any mix of precisions, every rating inside the group tables: every
    // rating loads its rows with the same instructions and branches four ways, on the precisions of its two rows, into
    // arithmetic and stores written for that case, each way issuing one store per side; 0 = anything, including ratings
    // that are skipped (an index outside the tables)
    static constexpr int kClasses = MIXED ? 3 : 2;
    // no register limit is asked for: the build for all-binary16 runs fits six wavefronts per SIMD by itself (80), the
    // build with the mixed path takes 83 (five), and held to 80 it spills and gains nothing (measured)
    static constexpr int kMinWavesPerSimd = 1;
    using HV = typename std::conditional<E == 2, half2_t, half_t>::type;

    struct Params {
        void* const* p; void* const* q;
        const uint32_t* user_end; const uint32_t* item_end;
        const uint8_t* user_prec; const uint8_t* item_prec;
        float* grad_sum_p; float* grad_sum_q; float* norm_sum_p; float* norm_sum_q;
        uint32_t first_sample; uint32_t user_groups; uint32_t item_groups;
        float lrate; float lambda; bool accumulate;
        uint32_t norm_stride;     // columns per group in norm_sum_* (workgroups of an ordinary launch)
        bool lds_stats;           // sampled gradient sums are kept per workgroup in LDS and flushed once
        void* rep_p; void* rep_q; // replica rows (Schedule::slot_u): slots of kReplicaSlotBytes, a binary16 row in the first half
        float rep_scale;          // an update of a replicated row's copy takes a step this many times as long
    };
    static constexpr uint32_t kReplicaSlotBytes = K * 4u;
    static constexpr int kK = K;
    static void row_storage(const Params& a, RowStorage& u, RowStorage& v)
    {
        u.group_ptr = a.p; u.group_end = a.user_end; u.group_prec = a.user_prec; u.groups = a.user_groups;
        v.group_ptr = a.q; v.group_end = a.item_end; v.group_prec = a.item_prec; v.groups = a.item_groups;
    }
    static constexpr bool kSplittable = true;
    // raw row registers: binary16 rows use r[0] only
    struct Row { uint32_t p[E], q[E]; };
    struct Prep { uint64_t pptr, qptr; uint32_t flags; };
    struct Info { float r; uint64_t pptr, qptr; uint32_t flags, thin; };
    // flags: bit0 user row is fp32, bit1 item row is fp32, bit2 rating is skipped (index outside the
    // group table), bits 3..16 user group, bits 17..30 item group
    static constexpr uint32_t kSkip = 4u;

    uint64_t* pptr_s; uint64_t* qptr_s;
    float* unorm_s; float* inorm_s;
    uint32_t* uend_s; uint32_t* iend_s;
    uint8_t* uprec_s; uint8_t* iprec_s;
    float* grad_sum_p; float* grad_sum_q;
    float* ugrad_s; float* igrad_s;      // per-workgroup [groups][K] sums in LDS, or null
    uint32_t* ulock_s; uint32_t* ilock_s; // with them: one lock per group (add_sums_locked)
    uint32_t first_sample, user_groups, item_groups;
    float lrate, lambda, lrate_rep;
    uint32_t lr_h_bits, lr_rep_h_bits;     // the binary16 learning rate in both halves of a dword: ordinary step, step of a replicated row's copy
    uint64_t rep_p, rep_q;
    int lane;
    // Sampled sums of the most popular group of each side (the last one; with Zipf-like data it takes half of all
    // ratings) stay in registers and reach the shared sums once per wavefront: one contended group lock less.
    mutable float top_gp[E], top_gq[E], top_np, top_nq;

    static __host__ __device__ size_t lds_bytes(uint32_t ug, uint32_t ig) { return ((size_t)(ug + ig) * (8 + 4 + 4 + 1) + 31) / 16 * 16; }
    static size_t lds_stats_bytes(uint32_t ug, uint32_t ig) { return (size_t)(ug + ig) * (K + 1) * sizeof(float); }

    __device__ __forceinline__ void init(const Params& a, uint8_t* smem, int lane_, uint32_t)
    {
        lane = lane_;
        user_groups = a.user_groups; item_groups = a.item_groups;
        pptr_s = reinterpret_cast<uint64_t*>(smem);
        qptr_s = pptr_s + user_groups;
        unorm_s = reinterpret_cast<float*>(qptr_s + item_groups);
        inorm_s = unorm_s + user_groups;
        uend_s = reinterpret_cast<uint32_t*>(inorm_s + item_groups);
        iend_s = uend_s + user_groups;
        uprec_s = reinterpret_cast<uint8_t*>(iend_s + item_groups);
        iprec_s = uprec_s + user_groups;
        for (uint32_t g = threadIdx.x; g < user_groups; g += blockDim.x) {
            pptr_s[g] = reinterpret_cast<uint64_t>(a.p[g]); uend_s[g] = a.user_end[g];
            uprec_s[g] = a.user_prec[g]; unorm_s[g] = 0.f;
        }
        for (uint32_t g = threadIdx.x; g < item_groups; g += blockDim.x) {
            qptr_s[g] = reinterpret_cast<uint64_t>(a.q[g]); iend_s[g] = a.item_end[g];
            iprec_s[g] = a.item_prec[g]; inorm_s[g] = 0.f;
        }
        grad_sum_p = a.grad_sum_p; grad_sum_q = a.grad_sum_q;
        first_sample = a.first_sample; lrate = a.lrate; lambda = a.lambda; lrate_rep = a.lrate * a.rep_scale;
        lr_h_bits = bits((half_t)lrate) * 0x10001u; lr_rep_h_bits = bits((half_t)lrate_rep) * 0x10001u;
        rep_p = reinterpret_cast<uint64_t>(a.rep_p); rep_q = reinterpret_cast<uint64_t>(a.rep_q);
        for (int e = 0; e < E; ++e) { top_gp[e] = 0.f; top_gq[e] = 0.f; }
        top_np = 0.f; top_nq = 0.f;
        ugrad_s = nullptr; igrad_s = nullptr; ulock_s = nullptr; ilock_s = nullptr;
        if (a.lds_stats) {
            ugrad_s = reinterpret_cast<float*>(smem + lds_bytes(user_groups, item_groups));
            igrad_s = ugrad_s + (size_t)user_groups * K;
            ulock_s = reinterpret_cast<uint32_t*>(igrad_s + (size_t)item_groups * K);
            ilock_s = ulock_s + user_groups;
            for (uint32_t i = threadIdx.x; i < (user_groups + item_groups) * (K + 1); i += blockDim.x) ugrad_s[i] = 0.f;   // sums and locks
        }
        __syncthreads();
    }

    // min{g : idx <= end[g]}; rows of a group are idx - end[g-1] - 1 (mascot_sgd_kernel.h:104-143).
    static __device__ __forceinline__ uint32_t search(const uint32_t* end, uint32_t groups, uint32_t idx)
    {
        uint32_t lo = 0, hi = groups - 1;
        while (lo < hi) {
            uint32_t mid = (lo + hi) >> 1;
            if (idx <= end[mid]) hi = mid; else lo = mid + 1;
        }
        return lo;
    }
    __device__ __forceinline__ Prep prepare(const Rating& my, bool valid) const
    {
        Prep pr; pr.pptr = 0; pr.qptr = 0; pr.flags = kSkip;
        if (valid) {
            const uint32_t ug = search(uend_s, user_groups, my.u);
            const uint32_t ig = search(iend_s, item_groups, my.v);
            const bool ok = my.u <= uend_s[ug] && my.v <= iend_s[ig];
            const uint32_t urow = ug ? my.u - uend_s[ug - 1] - 1 : my.u;
            const uint32_t irow = ig ? my.v - iend_s[ig - 1] - 1 : my.v;
            const uint32_t up = uprec_s[ug] ? 1u : 0u, ip = iprec_s[ig] ? 1u : 0u;
            // a rating that is skipped carries null pointers: forward() then matches it with no row
            pr.pptr = ok ? pptr_s[ug] + (uint64_t)urow * (K * (up ? 4u : 2u)) : 0ull;
            pr.qptr = ok ? qptr_s[ig] + (uint64_t)irow * (K * (ip ? 4u : 2u)) : 0ull;
            // a replicated row: this XCD's copy, in the precision of the row's group
            if (ok && (my.ru & kReplicaRow)) pr.pptr = rep_p + (uint64_t)(my.ru & ~kReplicaRow) * kReplicaSlotBytes;
            if (ok && (my.rv & kReplicaRow)) pr.qptr = rep_q + (uint64_t)(my.rv & ~kReplicaRow) * kReplicaSlotBytes;
            pr.flags = up | (ip << 1) | (ok ? 0u : kSkip) | (ug << 3) | (ig << 17);
        }
        return pr;
    }
    __device__ __forceinline__ int classify(const Rating& my, const Prep& pr, bool valid) const
    {
        // skipped ratings and thinned updates (opt-in, Schedule::keep_u) leave out memory instructions: general path
        if (__builtin_amdgcn_ballot_w64(valid && ((pr.flags & kSkip) != 0u || (my.thin & 3u) != 0u)) != 0ull) return 0;
        return __builtin_amdgcn_ballot_w64(valid && (pr.flags & 3u) != 0u) == 0ull ? 1 : (MIXED ? 2 : 0);
    }
    static __device__ __forceinline__ Info no_row() { return Info{0.f, 0ull, 0ull, kSkip, 0u}; }      // null pointers: forward() matches no row
    __device__ __forceinline__ Info info(const Rating& my, const Prep& pr, int j) const
    {
        Info i;
        i.r = bcast(my.r, j);
        i.pptr = bcast(pr.pptr, j);
        i.qptr = bcast(pr.qptr, j);
        i.flags = bcast(pr.flags, j);
        i.thin = bcast(my.thin, j);
        return i;
    }

    static __device__ __forceinline__ void load_side(uint32_t* r, uint64_t ptr, bool fp32, int lane)
    {
        if (fp32) {
            if constexpr (E == 2) {
                const uint64_t v = row_load((reinterpret_cast<const uint64_t*>(ptr) + lane));
                r[0] = (uint32_t)v; r[1] = (uint32_t)(v >> 32);
            } else {
                r[0] = row_load((reinterpret_cast<const uint32_t*>(ptr) + lane));
            }
        } else {
            if constexpr (E == 2) r[0] = row_load((reinterpret_cast<const uint32_t*>(ptr) + lane));
            else r[0] = row_load((reinterpret_cast<const uint16_t*>(ptr) + lane));
        }
    }
    // Chunks of mixed precisions (class 2): the same load instruction for a row of either precision, so that a rating
    // takes no branch on its way to the rows and the compiler can count the loads in flight (a branch between two load
    // instructions was measured: the counted waits become waits for everything, 42 instead of 29 ms per epoch on 250M
    // ratings).  The load goes through a window over the row (a buffer resource of the row's size): accesses past its
    // end are dropped by the hardware, dword by dword, and come back zero.
    // k = 128: one 8-byte load serves both precisions.  A binary32 row is read at 8 bytes per lane; a binary16 row at 4
    // bytes per lane, where the load's first dword is the lane's pair of elements and its second the next lane's, which
    // nothing uses (the last lane's second dword lies past the window).
    // k = 64: one 4-byte load.  A binary32 row is read at 4 bytes per lane; of a binary16 row every lane reads the dword
    // that holds its element and its neighbour's, and arrive() keeps the lane's half.
    static __device__ __forceinline__ void load_mixed(uint32_t* r, uint64_t ptr, bool fp32, int lane)
    {
        const row_window_t w = row_window(ptr, fp32 ? K * 4u : K * 2u);
        if constexpr (E == 2) {
            const auto v = __builtin_amdgcn_raw_buffer_load_b64(w, (int)((uint32_t)lane << (fp32 ? 3u : 2u)), 0, 0);
            r[0] = v[0]; r[1] = v[1];
        } else {
            r[0] = __builtin_amdgcn_raw_buffer_load_b32(w, (int)(((uint32_t)lane >> (fp32 ? 0u : 1u)) << 2), 0, 0);
        }
    }
    // hot row (Schedule::keep_u): add the change of this lane's elements to the row in memory
    static __device__ __forceinline__ void add_side_half(uint64_t ptr, HV d, int lane)
    {
        if constexpr (E == 2) {
            row_add((reinterpret_cast<half2_t*>(ptr) + lane), d);
        } else {
            // one element per lane: even lanes add the pair (own, right neighbour)
            const uint32_t mine = (uint32_t)bits(d);
            const uint32_t other = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)mine, 0xB1 /* quad_perm 1,0,3,2 */, 0xf, 0xf, false);
            if (!(lane & 1)) row_add(reinterpret_cast<half2_t*>(reinterpret_cast<uint16_t*>(ptr) + lane), from_bits<half2_t>(mine | (other << 16)));
        }
    }
    // An add to a binary32 row at k = 128 is two instructions.  With the lane's own elements 2L, 2L+1 each of them would
    // touch every other dword of the whole row: twice the 64-byte pieces at the memory side, where the adds are carried
    // out.  One v_permlane32_swap turns the pairs into the row's halves instead: `lower` holds elements 0..63 (the even
    // ones in lanes 0..31, the odd ones in lanes 32..63), `upper` elements 64..127; returns the byte offset of this
    // lane's element of the lower half.
    static __device__ __forceinline__ uint32_t halves_of_row(const float* d, float& lower, float& upper, int lane)
    {
        const auto r = __builtin_amdgcn_permlane32_swap(bits(d[0]), bits(d[1]), false, false);
        lower = from_bits<float>(r[0]); upper = from_bits<float>(r[1]);
        return ((((uint32_t)lane & 31u) << 1) | ((uint32_t)lane >> 5)) * 4u;
    }
    // The general path (class 0: the few chunks that are cut short or hold a skipped or thinned rating) adds the pairs as
    // they are: the rearrangement above would cost the whole kernel four registers, and with them a resident wavefront
    // per SIMD, for chunks that are hardly ever seen.
    static __device__ __forceinline__ void add_side_float(uint64_t ptr, const float* d, int lane)
    {
#pragma unroll
        for (int e = 0; e < E; ++e) row_add((reinterpret_cast<float*>(ptr) + lane * E + e), d[e]);
    }
    template <bool C = COH> static __device__ __forceinline__ void store_side(const uint32_t* r, uint64_t ptr, bool fp32, int lane)
    {
        if (fp32) {
            if constexpr (E == 2) row_store<C>((reinterpret_cast<uint64_t*>(ptr) + lane), (uint64_t)r[0] | ((uint64_t)r[1] << 32));
            else row_store<C>((reinterpret_cast<uint32_t*>(ptr) + lane), r[0]);
        } else {
            if constexpr (E == 2) row_store<C>((reinterpret_cast<uint32_t*>(ptr) + lane), r[0]);
            else row_store<C>((reinterpret_cast<uint16_t*>(ptr) + lane), (uint16_t)r[0]);
        }
    }
    template <int CLS> __device__ __forceinline__ void load(Row& row, const Info& i) const
    {
        if constexpr (CLS == 1) {
            load_side(row.p, i.pptr, false, lane);
            load_side(row.q, i.qptr, false, lane);
        } else if constexpr (CLS == 2) {
            load_mixed(row.p, i.pptr, i.flags & 1u, lane);
            load_mixed(row.q, i.qptr, i.flags & 2u, lane);
        } else {
#pragma unroll
            for (int e = 0; e < E; ++e) { row.p[e] = 0; row.q[e] = 0; }
            if (i.flags & kSkip) return;
            load_side(row.p, i.pptr, i.flags & 1u, lane);
            load_side(row.q, i.qptr, i.flags & 2u, lane);
        }
    }
    // load_mixed at k = 64: a binary16 row arrives as the dword that holds the lane's element and its neighbour's; keep
    // the lane's half in the low bits, the form every other path leaves a binary16 element in (wave-uniform selects)
    template <int CLS> __device__ __forceinline__ void arrive(Row& row, const Info& i) const
    {
        if constexpr (CLS == 2 && E == 1) {
            const uint32_t shift = ((uint32_t)lane & 1u) * 16u;
            row.p[0] = (i.flags & 1u) ? row.p[0] : ((row.p[0] >> shift) & 0xffffu);
            row.q[0] = (i.flags & 2u) ? row.q[0] : ((row.q[0] >> shift) & 0xffffu);
        }
    }
    // selects, no branches: a branch here would sit between the row loads and their first use
    __device__ __forceinline__ void forward(Row& nxt, const Info& in, const Row& cur, const Info& ic) const
    {
        // skipped ratings and empty slots have null pointers; copies between two of those are never used
        const bool same_p = in.pptr == ic.pptr, same_q = in.qptr == ic.qptr;
#pragma unroll
        for (int e = 0; e < E; ++e) {
            nxt.p[e] = same_p ? cur.p[e] : nxt.p[e];
            nxt.q[e] = same_q ? cur.q[e] : nxt.q[e];
        }

    }

    // ---- reductions in the reference order ------------------------------------------------
    static __device__ __forceinline__ half_t dot_half(HV m)
    {
        if constexpr (E == 2) {
            m = step_xor16(m, OpAdd());
            m = step_xor32(m, OpAdd());
            m = reduce_row16(m, OpAdd());
            return m.x + m.y;
        } else {
            return reduce_wave(m, OpAdd());
        }
    }
    static __device__ __forceinline__ float dot_float(const float* m)
    {
        if constexpr (E == 2) {
            // both element sums in one register: v_permlane16_swap(a, b) leaves [a.r0 b.r0 a.r2 b.r2] and
            // [a.r1 b.r1 a.r3 b.r3], whose sum is the lane ^ 16 step of a in rows 0, 2 and of b in rows 1, 3; the
            // lane ^ 32 step and the rotations inside the rows follow as for one value, a + b is the last step
            auto ab = __builtin_amdgcn_permlane16_swap(bits(m[0]), bits(m[1]), false, false);
            float s = from_bits<float>(ab[0]) + from_bits<float>(ab[1]);
            s = step_xor32(s, OpAdd());
            s = reduce_row16(s, OpAdd());
            return step_xor16(s, OpAdd());
        } else {
            return reduce_wave(m[0], OpAdd());
        }
    }
    static __device__ __forceinline__ float widen(HV h, int e)
    {
        if constexpr (E == 2) return (float)(e ? h.y : h.x); else return (float)h;
    }
    static __device__ __forceinline__ HV narrow(const float* f)
    {
        if constexpr (E == 2) { HV h; h.x = (half_t)f[0]; h.y = (half_t)f[1]; return h; } else return (half_t)f[0];
    }
    static __device__ __forceinline__ HV half_pair(uint32_t both)      // a dword with the same binary16 value in both halves
    {
        if constexpr (E == 2) return from_bits<half2_t>(both); else return from_bits<half_t>(both & 0xffffu);
    }
    static __device__ __forceinline__ HV splat(half_t v)
    {
        if constexpr (E == 2) { HV h; h.x = v; h.y = v; return h; } else return v;
    }
    // sampled statistics of one binary16 side: ||g||^2 into the block's LDS slot, g into the workgroup's LDS
    // sums or, without them, into the global sums.  The LDS accesses are spelled in the LDS address space: a
    // pointer that may be either would make them flat instructions, which wait for every outstanding row load.
    typedef __attribute__((address_space(3))) float lds_float;
    typedef __attribute__((address_space(3))) uint32_t lds_u32;
    static __device__ __forceinline__ void lds_add(float* p, float v)
    {
        (void)__hip_atomic_fetch_add((lds_float*)p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
    // Adds to a group's sums in LDS under the group's lock.  A 64-lane ds_add_f32 occupies the LDS of a gfx950 CU
    // for about 190 clocks (a third of a lane per clock, measured), an integer exchange and ordinary reads and
    // writes run at full rate: taking the lock, reading, adding in registers and writing back is ten times
    // faster.  The LDS operations of one wavefront execute in program order, so the release (the last write) is
    // seen after the sums; every access is volatile, which keeps the compiler to that order as well.  The holder
    // releases after a fixed straight-line sequence, so every waiting wavefront gets the lock.
    __device__ __forceinline__ void add_sums_locked(const float* g, float n, uint32_t group, float* norm_s, float* grad_s, uint32_t* lock_s) const
    {
        volatile lds_u32* lock = (volatile lds_u32*)(lock_s + group);
        for (;;) {
            uint32_t held = 1u;
            if (lane == 0) held = __hip_atomic_exchange(lock, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            if (__builtin_amdgcn_readfirstlane(held) == 0u) break;
            __builtin_amdgcn_s_sleep(1);
        }
        // LDS layout [group][e][lane]: consecutive lanes on consecutive banks
        volatile lds_float* sums = (volatile lds_float*)(grad_s + (size_t)group * K + lane);
        volatile lds_float* norm = (volatile lds_float*)(norm_s + group);
        float have[E], have_n = 0.f;
#pragma unroll
        for (int e = 0; e < E; ++e) have[e] = sums[e * kWave];
        if (lane == 0) have_n = *norm;
#pragma unroll
        for (int e = 0; e < E; ++e) sums[e * kWave] = have[e] + g[e];
        if (lane == 0) {
            *norm = have_n + n;
            __hip_atomic_store(lock, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        }
    }
    __device__ __forceinline__ void add_sums(const float* g, float n, uint32_t group, float* norm_s, float* grad_sum, float* grad_s, uint32_t* lock_s) const
    {
        if (grad_s) {
            add_sums_locked(g, n, group, norm_s, grad_s, lock_s);
        } else {
            if (lane == 0) lds_add(&norm_s[group], n);
#pragma unroll
            for (int e = 0; e < E; ++e) atomicAdd(grad_sum + (size_t)group * K + (size_t)lane * E + e, g[e]);
        }
    }
    __device__ __forceinline__ void sample(const float* g, uint32_t group, bool user_side) const
    {
        float n = g[0] * g[0];
        if constexpr (E == 2) n = n + g[1] * g[1];
        n = reduce_wave(n, OpAdd());
        if (user_side) {
            if (group == user_groups - 1) { for (int e = 0; e < E; ++e) top_gp[e] += g[e]; top_np += n; }
            else add_sums(g, n, group, unorm_s, grad_sum_p, ugrad_s, ulock_s);
        } else {
            if (group == item_groups - 1) { for (int e = 0; e < E; ++e) top_gq[e] += g[e]; top_nq += n; }
            else add_sums(g, n, group, inorm_s, grad_sum_q, igrad_s, ilock_s);
        }
    }

    // Writes one side of an update: the new row `r` (raw registers) or, for an added row, its change `d` (binary32; a
    // binary16 row receives it rounded, which is exact when it was computed in binary16).  bits: the side's thin bits
    // shifted down -- 4 the row is added to, 16 the row is this XCD's copy of a replicated row.
    // the same for a binary16 row whose change was computed in binary16 (mascot_sgd_kernel.h:188-278)
    template <int CLS, bool HOT> __device__ __forceinline__ void write_side_half(const uint32_t* r, HV d, uint64_t ptr, uint32_t bits_) const
    {
        if (HOT && (bits_ & 20u) == 16u) store_side<false>(r, ptr, false, lane);
        else if (HOT && (bits_ & 4u)) add_side_half(ptr, d, lane);
        else store_side(r, ptr, false, lane);
    }
    template <int CLS, bool HOT> __device__ __forceinline__ void write_side(const uint32_t* r, const float* d, uint64_t ptr, bool fp32, uint32_t bits_) const
    {
        static_assert(CLS != 2, "chunks of mixed precisions write through write_side_known");
        if (HOT && (bits_ & 20u) == 16u) store_side<false>(r, ptr, fp32, lane);
        else if (HOT && (bits_ & 4u)) { if (fp32) add_side_float(ptr, d, lane); else add_side_half(ptr, narrow(d), lane); }
        else store_side(r, ptr, fp32, lane);
    }
    // The same for a side whose precision is a compile-time constant: one store, or the adds of that precision, through
    // plain global accesses.  Chunks of mixed precisions write this way: their update branches four ways on the precisions
    // of the rating's two rows (wave-uniform), and every way issues one store per side, so the counted waits for the row
    // loads that are in flight hold on all of them.
    template <bool HOT, bool FP32> __device__ __forceinline__ void write_side_known(const uint32_t* r, const float* d, uint64_t ptr, uint32_t bits_) const
    {
        if (HOT && (bits_ & 20u) == 16u) store_side<false>(r, ptr, FP32, lane);
        else if (HOT && (bits_ & 4u)) {
            if constexpr (FP32 && E == 2) {
                float lower, upper;
                const uint32_t at = halves_of_row(d, lower, upper, lane);
                row_add(reinterpret_cast<float*>(ptr + at), lower);
                row_add(reinterpret_cast<float*>(ptr + at + K * 2u), upper);
            } else if constexpr (FP32) add_side_float(ptr, d, lane);
            else add_side_half(ptr, narrow(d), lane);
        }
        else store_side(r, ptr, FP32, lane);
    }
    template <int CLS, bool HOT, bool SCALED> __device__ __forceinline__ void update(Row& row, const Info& i, uint32_t processed) const
    {
        if constexpr (CLS == 2) {
            switch (i.flags & 3u) {
            case 0u: update_case<CLS, HOT, SCALED, 0>(row, i, processed); break;
            case 1u: update_case<CLS, HOT, SCALED, 1>(row, i, processed); break;
            case 2u: update_case<CLS, HOT, SCALED, 2>(row, i, processed); break;
            default: update_case<CLS, HOT, SCALED, 3>(row, i, processed); break;
            }
        } else update_case<CLS, HOT, SCALED, -1>(row, i, processed);
    }
    // CASE: the precisions of the two rows when they are known at compile time (bit 0 the user row is binary32, bit 1 the
    // item row), or -1: read from the rating's flags
    template <int CLS, bool HOT, bool SCALED, int CASE> __device__ __forceinline__ void update_case(Row& row, const Info& i, uint32_t processed) const
    {
        if (CLS == 0 && (i.flags & kSkip)) return;
        const bool up = CASE >= 0 ? (CASE & 1) != 0 : (CLS != 1 && (i.flags & 1u)), ip = CASE >= 0 ? (CASE & 2) != 0 : (CLS != 1 && (i.flags & 2u));
        // thinned updates (only read the row) occur in chunks of class 0 only: classify() sends their chunks there
        const bool skip_p = CLS == 0 && HOT && (i.thin & 1u), skip_q = CLS == 0 && HOT && (i.thin & 2u);
        const bool sampled = SAMPLED && processed >= first_sample;
        const uint32_t ug = (i.flags >> 3) & 0x3fffu, ig = (i.flags >> 17) & 0x3fffu;
        if (!up && !ip) {
            // mascot_sgd_kernel.h:188-278: everything in binary16, one rounding per operation
            const HV lam_h = splat((half_t)lambda);
            // the step of each side: a replicated row's copy (thin bit 4 / 5) takes the longer one
            const HV lr_p = half_pair((SCALED && (i.thin & 16u)) ? lr_rep_h_bits : lr_h_bits), lr_q = half_pair((SCALED && (i.thin & 32u)) ? lr_rep_h_bits : lr_h_bits);
            const half_t r_h = (half_t)i.r;
            const HV P = from_bits<HV>(row.p[0]), Q = from_bits<HV>(row.q[0]);
            const half_t dot = dot_half(P * Q);
            const HV ruv = splat(r_h - dot);
            const HV gp = ruv * Q - lam_h * P;
            const HV gq = ruv * P - lam_h * Q;
            if (!skip_p) {
                row.p[0] = bits(HV(__builtin_elementwise_fma(lr_p, gp, P)));
                write_side_half<(CLS == 2 ? 1 : CLS), HOT>(row.p, lr_p * gp, i.pptr, i.thin);
            }
            if (!skip_q) {
                row.q[0] = bits(HV(__builtin_elementwise_fma(lr_q, gq, Q)));
                write_side_half<(CLS == 2 ? 1 : CLS), HOT>(row.q, lr_q * gq, i.qptr, i.thin >> 1);
            }
            if (sampled) {
                float g[E];
#pragma unroll
                for (int e = 0; e < E; ++e) g[e] = widen(gp, e);
                sample(g, ug, true);
#pragma unroll
                for (int e = 0; e < E; ++e) g[e] = widen(gq, e);
                sample(g, ig, false);
            }
        } else {
            float pf[E], qf[E], m[E];
            {   // selects on wave-uniform flags: a binary16 row's second register holds nothing of the row
                const HV P = from_bits<HV>(row.p[0]), Q = from_bits<HV>(row.q[0]);
#pragma unroll
                for (int e = 0; e < E; ++e) {
                    pf[e] = up ? from_bits<float>(row.p[e]) : widen(P, e);
                    qf[e] = ip ? from_bits<float>(row.q[e]) : widen(Q, e);
                }
            }
#pragma unroll
            for (int e = 0; e < E; ++e) m[e] = pf[e] * qf[e];
            const float ruv = i.r - dot_float(m);
            const float lr_p = (SCALED && (i.thin & 16u)) ? lrate_rep : lrate, lr_q = (SCALED && (i.thin & 32u)) ? lrate_rep : lrate;
            float gp[E], gq[E], np_[E], nq_[E];
#pragma unroll
            for (int e = 0; e < E; ++e) {
                gp[e] = ruv * qf[e] - lambda * pf[e];
                gq[e] = ruv * pf[e] - lambda * qf[e];
                np_[e] = __builtin_fmaf(lr_p, gp[e], pf[e]);
                nq_[e] = __builtin_fmaf(lr_q, gq[e], qf[e]);
            }
            float d[E];
            if (!skip_p) {
                const uint32_t rounded = bits(narrow(np_));
#pragma unroll
                for (int e = 0; e < E; ++e) row.p[e] = up ? bits(np_[e]) : (e == 0 ? rounded : row.p[e]);
                if (HOT && (i.thin & 4u)) { for (int e = 0; e < E; ++e) d[e] = lr_p * gp[e]; }
                if constexpr (CASE >= 0) { if constexpr ((CASE & 1) != 0) write_side_known<HOT, true>(row.p, d, i.pptr, i.thin); else write_side_known<HOT, false>(row.p, d, i.pptr, i.thin); }
                else write_side<CLS, HOT>(row.p, d, i.pptr, up, i.thin);
            }
            if (!skip_q) {
                const uint32_t rounded = bits(narrow(nq_));
#pragma unroll
                for (int e = 0; e < E; ++e) row.q[e] = ip ? bits(nq_[e]) : (e == 0 ? rounded : row.q[e]);
                if (HOT && (i.thin & 8u)) { for (int e = 0; e < E; ++e) d[e] = lr_q * gq[e]; }
                if constexpr (CASE >= 0) { if constexpr ((CASE & 2) != 0) write_side_known<HOT, true>(row.q, d, i.qptr, i.thin >> 1); else write_side_known<HOT, false>(row.q, d, i.qptr, i.thin >> 1); }
                else write_side<CLS, HOT>(row.q, d, i.qptr, ip, i.thin >> 1);
            }
            if (sampled) {
                if (!up) sample(gp, ug, true);
                if (!ip) sample(gq, ig, false);
            }
        }
    }

    // mascot_sgd_kernel.h:448-456: per-block norm sums, layout [group][norm_stride]
    __device__ __forceinline__ void finish(const Params& a, uint32_t) const
    {
        if constexpr (SAMPLED) {
            const float np0 = bcast(top_np, 0), nq0 = bcast(top_nq, 0);
            if (np0 != 0.f) add_sums(top_gp, np0, user_groups - 1, unorm_s, grad_sum_p, ugrad_s, ulock_s);
            if (nq0 != 0.f) add_sums(top_gq, nq0, item_groups - 1, inorm_s, grad_sum_q, igrad_s, ilock_s);
        }
        __syncthreads();
        // a launch that continues an epoch (accumulate) adds to what the earlier launches of the epoch left
        for (uint32_t g = threadIdx.x; g < user_groups; g += blockDim.x) {
            float* dst = &a.norm_sum_p[(size_t)a.norm_stride * g + blockIdx.x];
            *dst = a.accumulate ? *dst + unorm_s[g] : unorm_s[g];
        }
        for (uint32_t g = threadIdx.x; g < item_groups; g += blockDim.x) {
            float* dst = &a.norm_sum_q[(size_t)a.norm_stride * g + blockIdx.x];
            *dst = a.accumulate ? *dst + inorm_s[g] : inorm_s[g];
        }
        if (!a.accumulate) {   // columns no workgroup of this launch owns (a launch of fewer, larger workgroups)
            for (uint32_t col = gridDim.x + blockIdx.x; col < a.norm_stride; col += gridDim.x) {
                for (uint32_t g = threadIdx.x; g < user_groups; g += blockDim.x) a.norm_sum_p[(size_t)a.norm_stride * g + col] = 0.f;
                for (uint32_t g = threadIdx.x; g < item_groups; g += blockDim.x) a.norm_sum_q[(size_t)a.norm_stride * g + col] = 0.f;
            }
        }
        if (ugrad_s) {     // single flush of the workgroup's gradient sums
            // LDS slot [g][e][l] holds element l*E + e of group g
            auto element = [](uint32_t i) { const uint32_t g = i / K, r = i % K; return g * K + (r % kWave) * E + r / kWave; };
            for (uint32_t i = threadIdx.x; i < user_groups * K; i += blockDim.x) { const float v = ugrad_s[i]; if (v != 0.f) atomicAdd(grad_sum_p + element(i), v); }
            for (uint32_t i = threadIdx.x; i < item_groups * K; i += blockDim.x) { const float v = igrad_s[i]; if (v != 0.f) atomicAdd(grad_sum_q + element(i), v); }
        }
    }
};
template <int K, bool COH> using MascotRule = MascotRuleT<K, COH, true>;
template <int K, bool COH> using MascotPlainRule = MascotRuleT<K, COH, false>;
template <int K, bool COH> using MascotBinary16Rule = MascotRuleT<K, COH, false, false>;

}  // namespace mf
