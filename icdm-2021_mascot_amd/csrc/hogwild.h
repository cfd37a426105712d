// The Hogwild driver loop shared by every update kernel (sgd/sgd_kernel.h:14-37 of the
// reference, redesigned for wave64 and for memory-level parallelism):
//   * one wavefront = one worker; it walks update_count windows of update_vector_size ratings;
//   * a window is consumed in chunks of up to 64 ratings: one coalesced streaming load puts rating j
//     of the chunk in lane j (the next chunk's ratings are requested while the current chunk runs),
//     everything that does not need the rows (group search, row addresses) is computed once,
//     vectorised across the 64 lanes, and the per-rating loop broadcasts lane j's scalars with
//     v_readlane;
//   * the per-rating loop is a software pipeline over a ring of kRing register slots: the rows of
//     rating j+kAhead are requested before rating j is reduced, updated and stored, so kAhead+1
//     ratings of a wavefront are in flight and a row's latency hides behind kAhead updates;
//   * a row requested early can be stale if one of the kAhead ratings in between updates the same
//     row.  Row identities are wave-uniform scalars, so that is a scalar compare per older slot; on
//     a match the freshly computed row is forwarded from that slot's registers.  A worker therefore
//     applies its own updates strictly in order (what a bit-exact check needs); different workers
//     still race on P and Q without atomics -- that is Hogwild.
#pragma once
#include "mf_device.h"
#include <type_traits>

namespace mf {

template <int I, int N, class F> __device__ __forceinline__ void static_for(F&& f)
{
    if constexpr (I < N) {
        f(std::integral_constant<int, I>());
        static_for<I + 1, N>(f);
    }
}

// SCALED: this launch gives the copies of replicated rows a longer step (Params::rep_scale != 1); otherwise the rules'
// code for it is compiled out of the loop.
template <class Rule, int CLS, bool HOT, bool SCALED>
__device__ __forceinline__ void process_chunk(Rule& rule, const Rating& my, const typename Rule::Prep& prep, int n, uint32_t processed)
{
    constexpr int A = Rule::kAhead;
    constexpr int S = Rule::kRing;
    static_assert(S >= 2 * A + 1, "ring must keep kAhead finished rows next to kAhead+1 pending ones");
    typename Rule::Row ring[S];
    typename Rule::Info inf[S];
    static_for<0, A>([&](auto D) {
        constexpr int d = decltype(D)::value;
        if (d < n) { inf[d] = rule.info(my, prep, d); rule.template load<CLS>(ring[d], inf[d]); }
    });
    for (int j0 = 0; j0 < n; j0 += S) {
        static_for<0, S>([&](auto D) {
            constexpr int d = decltype(D)::value;
            const int j = j0 + d;
            if (j < n) {
                if (j + A < n) {
                    constexpr int sl = (d + A) % S;
                    inf[sl] = rule.info(my, prep, j + A);
                    rule.template load<CLS>(ring[sl], inf[sl]);
                }
                // rows this rating shares with one of the previous kAhead ratings: newest wins
                static_for<0, A>([&](auto H) {
                    constexpr int h = A - decltype(H)::value;          // A, A-1, ..., 1
                    constexpr int sh = (d - h + 2 * S) % S;
                    if (j >= h) rule.forward(ring[d], inf[d], ring[sh], inf[sh]);
                });
                rule.template update<CLS, HOT, SCALED>(ring[d], inf[d], processed + (uint32_t)j);
            }
        });
    }
}

// A chunk of exactly kWave ratings (the usual case: windows are multiples of 64).  Same pipeline, but every
// memory instruction of the steady state sits on a straight line: loads that are issued under a condition make
// the compiler's wait-count bookkeeping fall back to "wait for everything", which turns the look-ahead into one
// full memory latency per rating.  Ring slots start out with row ids nothing can match, so the first ratings
// need no special case either.
// A rule may look ahead by a different number of ratings in chunks of class 2 (kAheadClass2).
template <class Rule, int CLS, class = void> struct ahead_of { static constexpr int value = Rule::kAhead; };
template <class Rule> struct ahead_of<Rule, 2, std::void_t<decltype(Rule::kAheadClass2)>> { static constexpr int value = Rule::kAheadClass2; };
// A rule may prepare a row whose loads have arrived before it is compared with older rows (arrive<CLS>).
template <int CLS, class Rule, class Row, class Info> __device__ __forceinline__ auto row_arrived(const Rule& rule, Row& row, const Info& i, int) -> decltype(rule.template arrive<CLS>(row, i), void()) { rule.template arrive<CLS>(row, i); }
template <int CLS, class Rule, class Row, class Info> __device__ __forceinline__ void row_arrived(const Rule&, Row&, const Info&, long) {}

template <class Rule, int CLS, bool HOT, bool SCALED>
__device__ __forceinline__ void process_full_chunk(Rule& rule, const Rating& my, const typename Rule::Prep& prep, uint32_t processed)
{
    constexpr int A = ahead_of<Rule, CLS>::value;
    constexpr int S = Rule::kRing;
    static_assert(S >= 2 * A + 1 && kWave % S == 0, "the ring divides a full chunk");
    typename Rule::Row ring[S];
    typename Rule::Info inf[S];
    static_for<0, S>([&](auto D) { inf[decltype(D)::value] = rule.no_row(); });
    auto fetch_rows = [&](auto SL, int j) {
        constexpr int sl = decltype(SL)::value;
        inf[sl] = rule.info(my, prep, j);
        if constexpr (!HOT) inf[sl].thin = 0u;
        rule.template load<CLS>(ring[sl], inf[sl]);
    };
    auto step = [&](auto D, int j) {
        constexpr int d = decltype(D)::value;
        row_arrived<CLS>(rule, ring[d], inf[d], 0);
        static_for<0, A>([&](auto H) {
            constexpr int h = A - decltype(H)::value;          // A, A-1, ..., 1: newest wins
            constexpr int sh = (d - h + 2 * S) % S;
            rule.forward(ring[d], inf[d], ring[sh], inf[sh]);
        });
        rule.template update<CLS, HOT, SCALED>(ring[d], inf[d], processed + (uint32_t)j);
    };
    static_for<0, A>([&](auto D) { fetch_rows(D, decltype(D)::value); });
    for (int j0 = 0; j0 < kWave - S; j0 += S) {
        static_for<0, S>([&](auto D) {
            constexpr int d = decltype(D)::value;
            fetch_rows(std::integral_constant<int, (d + A) % S>(), j0 + d + A);
            step(D, j0 + d);
        });
    }
    static_for<0, S>([&](auto D) {
        constexpr int d = decltype(D)::value;
        if constexpr (d + A < S) fetch_rows(std::integral_constant<int, d + A>(), kWave - S + d + A);
        step(D, kWave - S + d);
    });
}

// A rule may ask for a minimum number of resident wavefronts per SIMD (kMinWavesPerSimd): the compiler then keeps the
// kernel's registers within 512 / that many.  For rules whose natural allocation lands just above a step (85 VGPRs
// is 5 wavefronts per SIMD, 80 is 6) this decides whether all workers of a launch are resident at once.
template <class Rule, class = void> struct min_waves_per_simd { static constexpr int value = 1; };
template <class Rule> struct min_waves_per_simd<Rule, std::void_t<decltype(Rule::kMinWavesPerSimd)>> { static constexpr int value = Rule::kMinWavesPerSimd; };

template <class Rule, bool HOT>
__global__ __launch_bounds__(kMaxBlock) __attribute__((amdgpu_waves_per_eu(min_waves_per_simd<Rule>::value)))
void hogwild_kernel(Schedule s, typename Rule::Params prm)
{
    extern __shared__ __align__(16) uint8_t smem[];
    const int lane = threadIdx.x & (kWave - 1);
    const uint32_t waves_per_block = blockDim.x >> 6;
    const uint32_t total_waves = gridDim.x * waves_per_block;
    const uint32_t first_wid = (uint32_t)__builtin_amdgcn_readfirstlane((int)(blockIdx.x * waves_per_block + (threadIdx.x >> 6)));
    Rule rule;
    rule.init(prm, smem, lane, first_wid);              // may synchronise the workgroup
    const uint32_t xcd = HOT ? xcd_id() : 0u;           // which copy of the replicated rows this wavefront works on
    // a launch normally has one wavefront per worker; a launch with fewer wavefronts (the sampled tail of
    // a MASCOT epoch, which keeps per-workgroup statistics in LDS) lets each wavefront play several workers,
    // and may cut every worker's range into s.pieces parts (on chunk boundaries) to even out the wavefronts' loads
    const uint32_t pieces = s.pieces ? s.pieces : 1u;
    for (uint32_t item = first_wid; item < s.num_workers * pieces && s.range_begin < s.range_end; item += total_waves) {
        const uint32_t wid = item % s.num_workers, piece = item / s.num_workers;
        // this wavefront handles the worker's ratings with processed index in [range_begin, range_end)
        uint32_t range_begin = s.range_begin, range_end = s.range_end;
        if (pieces > 1) {
            auto cut = [&](uint32_t i) -> uint32_t {
                if (i == 0) return s.range_begin;
                if (i == pieces) return s.range_end;
                const uint32_t at = s.range_begin + (uint32_t)((uint64_t)(s.range_end - s.range_begin) * i / pieces);
                const uint32_t down = at - (at % s.update_vector_size) % (uint32_t)kWave;     // a chunk boundary of its window
                return down > s.range_begin ? down : s.range_begin;
            };
            range_begin = cut(piece); range_end = cut(piece + 1);
            if (range_begin >= range_end) continue;
        }
        uint32_t processed = range_begin;
        uint32_t ite = range_begin / s.update_vector_size;
        uint32_t c = range_begin - ite * s.update_vector_size;
        auto window_of = [&](uint32_t it) -> uint32_t {
            uint32_t st;
            if (s.window_start) st = s.window_start[(size_t)it * s.num_workers + wid] % s.nnz;
            else st = window_start_rng(s.epoch_key, wid, it, s.nnz);
            return (uint32_t)__builtin_amdgcn_readfirstlane((int)st);
        };
        auto chunk_len = [&](uint32_t cc, uint32_t pp) -> int {
            uint32_t left = s.update_vector_size - cc;
            if (left > range_end - pp) left = range_end - pp;
            return left < (uint32_t)kWave ? (int)left : kWave;
        };
        auto fetch = [&](uint32_t st, uint32_t cc, int nn) -> Rating {
            Rating x = {0.f, 0u, 0u, 0u, 0u, 0u};
            if (lane < nn) {
                uint32_t off = (cc + (uint32_t)lane) % s.nnz;
                uint32_t idx = st + off;
                if (idx >= s.nnz || idx < st) idx -= s.nnz;
                x = load_rating(s.R, idx);
                if constexpr (HOT) {
                    const uint32_t rnd = (uint32_t)(mix64(s.epoch_key ^ (((uint64_t)idx << 20) ^ (uint64_t)wid ^ 0x7468696eull)) >> 40);
                    const uint32_t ku = s.keep_u[x.u], kv = s.keep_v[x.v];
                    // two independent draws, uniform over 0..254
                    if (ku == kKeepReplicated || ku == kKeepReplicatedAdded) {
                        x.thin |= ku == kKeepReplicated ? 16u : 20u; x.ru = kReplicaRow | (xcd * s.slots_u + s.slot_u[x.u]);
                    } else if (ku != 255u) x.thin |= (((rnd & 0xfffu) * 255u) >> 12) > ku ? 5u : 4u;
                    if (kv == kKeepReplicated || kv == kKeepReplicatedAdded) {
                        x.thin |= kv == kKeepReplicated ? 32u : 40u; x.rv = kReplicaRow | (xcd * s.slots_v + s.slot_v[x.v]);
                    } else if (kv != 255u) x.thin |= (((rnd >> 12) * 255u) >> 12) > kv ? 10u : 8u;
                }
            }
            return x;
        };
        uint32_t start = window_of(ite);
        int n = chunk_len(c, processed);
        Rating my = fetch(start, c, n);
        while (true) {
            // position of the chunk after this one, and its ratings, requested now
            uint32_t nprocessed = processed + (uint32_t)n;
            uint32_t nc = c + (uint32_t)n, nite = ite, nstart = start;
            const bool more = nprocessed < range_end;
            int nn = 0;
            Rating nmy = {0.f, 0u, 0u, 0u, 0u, 0u};
            if (more) {
                if (nc >= s.update_vector_size) { nc = 0; ++nite; nstart = window_of(nite); }
                nn = chunk_len(nc, nprocessed);
                nmy = fetch(nstart, nc, nn);
            }
            const bool valid = lane < n;
            typename Rule::Prep prep = rule.prepare(my, valid);
            const int cls = rule.classify(my, prep, valid);
            // classes (see the rules): 1 and 2 promise ratings that all take the same memory instructions; full
            // chunks of those run the straight-line pipeline, everything else the general one
            auto run = [&](auto Scaled) {
                constexpr bool SC = decltype(Scaled)::value;
                if (Rule::kClasses > 1 && cls == 1) {
                    if (n == kWave) process_full_chunk<Rule, 1, HOT, SC>(rule, my, prep, processed);
                    else process_chunk<Rule, 1, HOT, SC>(rule, my, prep, n, processed);
                } else if (Rule::kClasses > 2 && cls == 2 && n == kWave) {
                    process_full_chunk<Rule, 2, HOT, SC>(rule, my, prep, processed);
                } else if (Rule::kClasses == 1 && n == kWave) {
                    process_full_chunk<Rule, 0, HOT, SC>(rule, my, prep, processed);
                } else {
                    process_chunk<Rule, 0, HOT, SC>(rule, my, prep, n, processed);
                }
            };
            // the few launches with longer steps on replicated rows (the first epoch by default) take their own copy of
            // the loops, so that every other launch pays nothing for them
            if (HOT && prm.rep_scale != 1.0f) run(std::true_type()); else run(std::false_type());
            if (!more) break;
            processed = nprocessed; c = nc; ite = nite; start = nstart; n = nn; my = nmy;
        }
    }
    rule.finish(prm, first_wid);                         // may synchronise the workgroup
}

}  // namespace mf
