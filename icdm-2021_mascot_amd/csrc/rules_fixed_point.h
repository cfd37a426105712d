// MuPPET (block fixed point, muppet/muppet_sgd_kernel.h) and AFP (adaptive fixed point,
// afp/afp_sgd_kernel.h) update rules over dense fp32 P/Q.
//
// Both rules derive per-rating scale factors from warp-wide statistics.  Lane L holds elements L and L+64 of a row
// (k = 64: element L), i.e. the lower half-wave holds what the reference's lane l = L keeps as its 1st and 3rd value
// (elements l, l+64) and the upper half-wave its 2nd and 4th (l+32, l+96).  Minima, maxima and the int8 dot product
// are exact in any order, so they are plain 64-lane reductions.  Where the order of floating-point additions
// matters it is reproduced: the binary16 dot keeps the reference's .x lane sums in the lower half-wave and the .y
// sums in the upper one (two independent 16,8,4,2,1 trees, added at the end); squared norms pair the halves first,
// (x[l]^2 + x[l+32]^2) + (x[l+64]^2 + x[l+96]^2).  Only AFP's occasional error measurement (QEM), whose per-lane
// sums run left to right over all four values, rebuilds the 32-lane view (Mirror) in both half-waves.
#pragma once
#include "rules_fp32.h"

namespace mf {

// roundf (halves away from zero) in three instructions: 0x1.fffffep-2 is the largest binary32 below one half, so the
// sum reaches the next integer exactly when the fraction is at least one half, and for |x| >= 2^23 it rounds back to
// x.  Equal to roundf for every binary32 value, signed zeros included (checked exhaustively on the CPU,
// tests/test_host_io.py); the library's roundf expands to six instructions.
__device__ __forceinline__ float round_half_away(float x) { return __builtin_truncf(x + __builtin_copysignf(0x1.fffffep-2f, x)); }

// Saturating conversions (CUDA's float-to-integer casts saturate and map NaN to 0).  Written without branches:
// the value is clamped first, so the conversion itself is always in range, and selects pick the special cases;
// nested ifs became nested exec-mask regions, a dozen scalar instructions per converted element.
__device__ __forceinline__ uint32_t f2u_sat(float f)
{
    const uint32_t r = (uint32_t)__builtin_amdgcn_fmed3f(f, 0.0f, 4294967040.0f);
    return (f > 0.0f) ? (f >= 4294967296.0f ? 0xffffffffu : r) : 0u;
}
__device__ __forceinline__ int f2i_sat(float f)
{
    const int r = (int)__builtin_amdgcn_fmed3f(f, -2147483648.0f, 2147483520.0f);
    return (f != f) ? 0 : (f >= 2147483648.0f ? 2147483647 : r);
}
// The hardware's own float-to-integer conversions truncate, saturate and map NaN to 0, which is what CUDA's casts do;
// spelled as instructions because an out-of-range cast has no defined value in C++.
// The compiler's hazard bookkeeping does not look inside an asm statement, so each one is self-contained whatever
// produced its input: it starts with the wait state a transcendental's result needs before a VALU instruction may read
// it (s_nop is not a VALU instruction: the other wavefronts of the SIMD issue meanwhile), and a transcendental inside
// is followed by one before its result is read.  Results leave through an ordinary (non-transcendental) conversion.
__device__ __forceinline__ int hw_cvt_i32(float f) { int r; asm("s_nop 0\n\tv_cvt_i32_f32_e32 %0, %1" : "=v"(r) : "v"(f)); return r; }
// (unsigned)floorf(log2f(x)) for x that is not subnormal: the conversion truncates, and negative logarithms and NaN
// give 0 with or without the floor
__device__ __forceinline__ uint32_t floor_log2_u32(float x)
{
    uint32_t r;
    asm("s_nop 0\n\tv_log_f32_e32 %0, %1\n\ts_nop 0\n\tv_cvt_u32_f32_e32 %0, %0" : "=v"(r) : "v"(x));
    return r;
}
// (signed char) of roundf(x), saturating, NaN -> 0: the conversion truncates by itself, so round_half_away's own
// truncation is not needed, and clamping the integer afterwards equals clamping the float before (four instructions
// where rounding, clamping, converting and the NaN select took seven)
__device__ __forceinline__ int round_to_i8(float x)
{
    const int v = hw_cvt_i32(x + __builtin_copysignf(0x1.fffffep-2f, x));
    return v < -128 ? -128 : (v > 127 ? 127 : v);
}
// (signed char) of roundf(x * s) for a scale s = 2^n, n >= 0: the product by a power of two is exact (or infinite), so
// the fused multiply-add rounds exactly as the product followed by the addition does, and the sign of the product is
// the sign of x (0 * inf and NaN give NaN -> 0 either way); the sign constant is shared by every quantisation of x.
__device__ __forceinline__ int round_to_i8_scaled(float x, float s)
{
    const int v = hw_cvt_i32(__builtin_fmaf(x, s, __builtin_copysignf(0x1.fffffep-2f, x)));
    return v < -128 ? -128 : (v > 127 ? 127 : v);
}
// roundf(x * s) for s = 2^n, n >= 0, likewise
__device__ __forceinline__ float round_half_away_scaled(float x, float s) { return __builtin_truncf(__builtin_fmaf(x, s, __builtin_copysignf(0x1.fffffep-2f, x))); }
// 2^n for an integer-valued exponent, exact (exp2f of an integer in the reference).
__device__ __forceinline__ float pow2u(uint32_t n) { return __builtin_ldexpf(1.0f, n > 1000u ? 1000 : (int)n); }
// The same from integer arithmetic on the exponent field (infinity from n = 128 on): for a wave-uniform n these are
// scalar instructions, where ldexp is a vector one.
__device__ __forceinline__ float pow2u_bits(uint32_t n) { return from_bits<float>(((n > 128u ? 128u : n) + 127u) << 23); }
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
__device__ __forceinline__ half_t grid_h(float v, float s, float s_rev) { return (half_t)(round_half_away_scaled(v, s) * s_rev); }
// 1 / 2^n as the reference's division yields it: 2^n is infinite from n = 128 on, and 1 / inf = 0
__device__ __forceinline__ float pow2_reciprocal(uint32_t n) { return n > 127u ? 0.0f : __builtin_ldexpf(1.0f, -(int)n); }
// x / 2^n, likewise: scaling by a power of two is exact (and rounds like the division where the result is subnormal)
__device__ __forceinline__ float div_pow2(float x, uint32_t n) { return n > 127u ? x * 0.0f : __builtin_ldexpf(x, -(int)n); }

// IEEE 754-2019 maximum: equal to fmaxf for numbers, and one v_maximum3_f32 on gfx950 where fmaxf first
// canonicalises both operands (three instructions after every cross-lane move)
struct OpMaximum { __device__ __forceinline__ float operator()(float a, float b) const { return __builtin_elementwise_maximum(a, b); } };
struct OpMinimum { __device__ __forceinline__ float operator()(float a, float b) const { return __builtin_elementwise_minimum(a, b); } };

// Four wave-wide maxima in one reduction.  In: every lane's own a, b, c, d.  Out: the maximum over all lanes of a in
// rows 0 (lanes 0-15), of c in row 1, of b in row 2 and of d in row 3.  v_permlane32_swap(a, b) leaves [a.lower, b.lower]
// and [a.upper, b.upper], whose maximum folds the half-waves of a into the lower half and those of b into the upper
// half; v_permlane16_swap folds the rows the same way; four rotations finish inside the rows.
//
// The maximum is fmaxf's, as in the reference: a NaN operand is dropped (v_max_f32 with the IEEE mode bit set, which
// compute kernels run with; denormals are kept).  Written as instructions because the compiler puts a canonicalising
// v_max_f32 x, x in front of every fmaxf whose operand comes out of a cross-lane move and cannot fold the rotation
// into the maximum then, and the IEEE 754-2019 maximum it can use instead has no form that rotates: 10 vector
// instructions here, 14 with that one.  The wait states that cross-lane reads of a just-written register need are inside
// the block (the compiler does not count instructions in one): the first for whatever produced the inputs, the last
// for whatever reads the result.
__device__ __forceinline__ float max4_by_rows(float a, float b, float c, float d)
{
    asm("s_nop 1\n\t"
        "v_permlane32_swap_b32 %0, %1\n\t"
        "v_permlane32_swap_b32 %2, %3\n\t"
        "v_max_f32 %0, %0, %1\n\t"                                                       // rows 0,1: a   rows 2,3: b
        "v_max_f32 %2, %2, %3\n\t"                                                       // rows 0,1: c   rows 2,3: d
        "s_nop 1\n\t"
        "v_permlane16_swap_b32 %0, %2\n\t"                                               // [x.r0 y.r0 x.r2 y.r2], [x.r1 y.r1 x.r3 y.r3]
        "v_max_f32 %0, %0, %2\n\t"
        "s_nop 1\n\t"
        "v_max_f32_dpp %0, %0, %0 row_ror:8 row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\t"
        "v_max_f32_dpp %0, %0, %0 row_ror:4 row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\t"
        "v_max_f32_dpp %0, %0, %0 row_ror:2 row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\t"
        "v_max_f32_dpp %0, %0, %0 row_ror:1 row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1"
        : "+v"(a), "+v"(b), "+v"(c), "+v"(d));
    return a;
}
// get_only_scaling_factor (muppet_sgd_kernel.h:7-18) for two value ranges at once.  `extreme` holds, by half-wave, the
// largest value (lower) and the negated smallest value (upper) of a range, the same in both rows of a half-wave or a
// different range in each; the result is the scale index of the lane's range.
//
// The reference evaluates (unsigned)floorf(log2f(fminf(|max_val / max|, |min_val / min|))).  floor and log2 are
// monotonic, so that is the smaller of the two sides' floor(log2(bound / |x|)), and each of those follows from the
// bits of x: with bound = t * 2^eb and |x| = m * 2^e (1 <= t, m < 2) it is eb - e when m <= t and eb - e - 1
// otherwise.  The quotient overflows to infinity exactly when that index reaches 128 (index 2^32 - 1 after the
// unsigned conversion, as for x = 0), an infinite or NaN x gives 0, a negative index 0.  Only within a few ulps of
// m = t can the rounding of the division and of the logarithm decide differently (the result of log2f next to an
// integer n rounds to n within about 2^(log2 n - 24) of it: up to 45 ulps of m for indices below 128); those lanes
// take the division and the logarithm, as before (muppet_scale_index_slow).
__device__ __forceinline__ uint32_t muppet_scale_index_slow(unsigned bitwidth, float extreme, bool upper)
{
    const float val = (float)(1 << (bitwidth - 1));
    const float bound = upper ? (-val) - 0.5f : (val - 1) + 0.5f;
    const float ratio = fabsf(bound / extreme);                                        // |min_val / min| = |min_val / -min|
    const float range_best = step_xor32(ratio, OpMinimum());
    const bool both_zero = step_xor32(fabsf(extreme), OpMaximum()) == 0.0f;
    // x is never subnormal (|bound| >= 127.5 over a finite extreme), so the bare v_log_f32 equals log2f
    const uint32_t idx = floor_log2_u32(range_best);
    return both_zero ? 0u : idx;
}
struct OpUMin { __device__ __forceinline__ uint32_t operator()(uint32_t a, uint32_t b) const { return a < b ? a : b; } };
__device__ __forceinline__ uint32_t muppet_scale_index_by_rows(unsigned bitwidth, float extreme, bool upper)
{
    // bound = 2^(b-1) - 0.5 = (2 - 2^-(b-1)) * 2^(b-2) for the maximum, 2^(b-1) + 0.5 = (1 + 2^-b) * 2^(b-1) for the minimum
    const uint32_t eb = upper ? bitwidth - 1u : bitwidth - 2u;
    const uint32_t t_mant = upper ? (0x800000u >> bitwidth) : 0x800000u - (0x800000u >> (bitwidth - 1u));
    const uint32_t xb = bits(extreme);
    const uint32_t mant = xb & 0x7fffffu;
    const uint32_t idx = (eb + 127u) - ((xb >> 23) & 0xffu) - (mant > t_mant ? 1u : 0u);
    // Everything that is not a plain index 0..127 on a side goes the long way: a mantissa within 64 ulps of the
    // threshold, an extreme of zero or below 2^-121 (index 128 and more: the quotient is infinite), one above the
    // bound (negative index), an infinity or a NaN.  None of them occurs on rows of a model that is being trained.
    const bool rare = (mant - t_mant + 64u <= 128u) | (idx >= 128u);
    if (__builtin_amdgcn_ballot_w64(rare) != 0ull) return muppet_scale_index_slow(bitwidth, extreme, upper);
    return step_xor32(idx, OpUMin());
}

// The same without the long way: false when any lane would need it (`both` is then meaningless).
// `side` is the lane's own side's index; the index of a range is the smaller of its two sides' (lanes L and L ^ 32).
__device__ __forceinline__ bool muppet_scale_index_plain(unsigned bitwidth, float extreme, bool upper, uint32_t& side)
{
    const uint32_t eb = upper ? bitwidth - 1u : bitwidth - 2u;
    const uint32_t t_mant = upper ? (0x800000u >> bitwidth) : 0x800000u - (0x800000u >> (bitwidth - 1u));
    const uint32_t near_bias = 64u - t_mant;
    const uint32_t xb = bits(extreme);
    const uint32_t mant = xb & 0x7fffffu;
    side = (eb + 127u) - ((xb >> 23) & 0xffu) - (mant > t_mant ? 1u : 0u);
    const bool rare = (mant + near_bias <= 128u) | (side >= 128u);
    return __builtin_amdgcn_ballot_w64(rare) == 0ull;
}
// (signed char) of roundf(x * 2^n) when |x| is at most the extreme that a plain scale index n was taken from: the
// product then lies inside (-128.5, 127.5) by more than 64 ulps of the extreme, so nothing saturates, x is a number,
// and the conversion is an ordinary truncating cast.  (A NaN element does reach it: the extrema drop NaNs, as fmaxf and
// fminf do in the reference.  The cast compiles to v_cvt_i32_f32, whose result is defined for every input: NaN gives 0,
// which is what the reference's cast gives, and excess saturates.)
__device__ __forceinline__ int round_to_i8_in_range(float x, float s) { return (int)__builtin_fmaf(x, s, __builtin_copysignf(0x1.fffffep-2f, x)); }
// Sum of an int over the 64 lanes as a wave-uniform value: rotations inside the rows, then the four row sums meet on
// the scalar unit (integer addition: any order)
__device__ __forceinline__ int sum_wave_uniform(int x)
{
    x = reduce_row16(x, OpAdd());
    return __builtin_amdgcn_readlane(x, 0) + __builtin_amdgcn_readlane(x, 16) + __builtin_amdgcn_readlane(x, 32) + __builtin_amdgcn_readlane(x, 48);
}

// round_to_i8(x * 2^n) for a wave-uniform x and n on the scalar unit: |x| = m * 2^-c with an integer m < 2^24, so
// roundf(|x| * 2^n) = (m + 2^(sh-1)) >> sh with sh = c - n (halves away from zero), saturated at `bound` (127 for a
// positive x, 128 for a negative one); sh <= 0 means |x| * 2^n >= 2^23, which saturates like sh = 1.
struct UniformI8 {
    uint32_t m; int c; int bound; int sign; bool finite;
    __device__ __forceinline__ void set(float x)
    {
        const uint32_t b = bits(x), e = (b >> 23) & 0xffu, mant = b & 0x7fffffu;
        m = e ? (mant | 0x800000u) : mant;
        c = 150 - (int)(e ? e : 1u);
        sign = (b >> 31) ? -1 : 1;
        bound = (b >> 31) ? 128 : 127;
        finite = e != 0xffu;
    }
    __device__ __forceinline__ int scaled(uint32_t n) const
    {
        const int sh = c - (int)n;
        const uint32_t r = (m + (1u << ((uint32_t)(sh - 1) & 31u))) >> ((uint32_t)sh & 31u);
        const uint32_t mag = sh < 1 ? (uint32_t)bound : (sh > 31 ? 0u : (r > (uint32_t)bound ? (uint32_t)bound : r));
        return sign * (int)mag;
    }
};

template <int K, bool COH> struct MuppetRule : DenseBase<K, COH> {
    using Base = DenseBase<K, COH>;
    using typename Base::Row;
    using typename Base::Info;
    static constexpr int E = Base::E;
    static constexpr int J = K / 32;
    // One rating of look-ahead: the rule is bound by its arithmetic, and three ratings in flight per wavefront measured
    // slower (the longer register ring costs more than the loads' latency, which the other wavefronts already cover).
    static constexpr int kAhead = 1, kRing = 4;
    struct Params {
        float* p; float* q; float lrate; float lambda; uint32_t first_sample;
        float* sum_updated_val; float* sum_norms; uint32_t num_workers; int fwd; int bwd; bool accumulate;
        void* rep_p; void* rep_q; float rep_scale;
    };
    static constexpr bool kSplittable = false;     // per-worker statistics span the whole launch
    float lrate, lambda; uint32_t first_sample; float* sum_updated_val; int fwd, bwd;
    float sum_norms_reg;
    float grad_acc[K / 64];
    // 8-bit backward pass on the short path: -lambda as an integer mantissa and exponent, and the largest scale index
    // for which lrate * 2^(-2 index) is a normal number computed exactly by exponent arithmetic
    UniformI8 neg_lambda_q;
    bool plain_8bit;
    static constexpr uint32_t kShortPathMaxIndex = 48;

    __device__ __forceinline__ void init(const Params& a, uint8_t*, int lane_, uint32_t)
    {
        this->P = a.p; this->Q = a.q; this->RP = static_cast<float*>(a.rep_p); this->RQ = static_cast<float*>(a.rep_q);
        this->lane = lane_; lrate = a.lrate; lambda = a.lambda; this->rep_scale = a.rep_scale;
        first_sample = a.first_sample; sum_updated_val = a.sum_updated_val; fwd = a.fwd; bwd = a.bwd;
        sum_norms_reg = 0.f;
#pragma unroll
        for (int e = 0; e < E; ++e) grad_acc[e] = 0.f;
        neg_lambda_q.set(-1 * lambda);
        // lrate in [2^-20, 2^20]: with 2 * index <= 96 the product lrate * 2^(-2 index) and every float(int) * that stay normal
        const uint32_t le = (bits(lrate) >> 23) & 0x1ffu;
        plain_8bit = fwd == 8 && bwd == 8 && neg_lambda_q.finite && le >= 107u && le <= 147u;
    }
    // sum over the k values x[j]^2 in the reference's order: per lane (x0^2 + x1^2) + (x2^2 + x3^2); sq[e] = own squares
    static __device__ __forceinline__ float lane_sum_of_squares(const float* sq)
    {
        float a = step_xor32(sq[0], OpAdd());
        if constexpr (E == 2) { const float b = step_xor32(sq[1], OpAdd()); a = a + b; }
        return a;
    }
    // The change of a row is lrate * g.  Both gradient functions return g as g_base * g_scale and lrate * g as
    // g_base * d_scale, one rounding each.
    // Every bit width and every input, as the reference computes it.
    __device__ __forceinline__ void gradients(const float* p, const float* q, float r, float* gbp, float* gbq, float& g_scale, float& d_scale) const
    {
        const bool upper = this->lane >= 32;
        // extrema by rows of 16 lanes: max p, max q, -min p, -min q (all 0 when the forward pass is binary32, as in the reference)
        float extrema = 0, sp = 0, sq = 0, pred;
        uint32_t ip = 0, iq = 0;
        if (fwd != 32) {
            float a = p[0], b = -p[0], c = q[0], d = -q[0];
            if constexpr (E == 2) {
                a = OpMaximum()(a, p[1]); b = OpMaximum()(b, -p[1]);
                c = OpMaximum()(c, q[1]); d = OpMaximum()(d, -q[1]);
            }
            extrema = max4_by_rows(a, b, c, d);
            const uint32_t idx = muppet_scale_index_by_rows((unsigned)fwd, extrema, upper);      // rows 0,2: p   rows 1,3: q
            ip = bcast(idx, 0); iq = bcast(idx, 16);
            sp = pow2u_bits(ip); sq = pow2u_bits(iq);
        }
        if (fwd == 8) {
            int acc = 0;
#pragma unroll
            for (int e = 0; e < E; ++e) acc += round_to_i8_scaled(p[e], sp) * round_to_i8_scaled(q[e], sq);
            acc = reduce_wave(acc, OpAdd());
            // acc / (sp * sq): the divisor is a power of two, or infinite from 2^128 on (quotient 0 with the sign of acc,
            // which is what 2^-1000 gives)
            const uint32_t n = (ip > 1000u ? 1000u : ip) + (iq > 1000u ? 1000u : iq);
            pred = __builtin_ldexpf((float)acc, n > 127u ? -1000 : -(int)n);
        } else if (fwd == 32) {
            float m[E];
#pragma unroll
            for (int e = 0; e < E; ++e) m[e] = p[e] * q[e];
            pred = dot_reference_order<E, float>(m);
        } else {
            const float sp_rev = pow2_reciprocal(ip), sq_rev = pow2_reciprocal(iq);
            // the reference's half2 lanes: .x sums elements l, l+64 (lower half-wave here), .y elements l+32, l+96 (upper)
            half_t t = grid_h(p[0], sp, sp_rev) * grid_h(q[0], sq, sq_rev);
            if constexpr (E == 2) t = t + grid_h(p[1], sp, sp_rev) * grid_h(q[1], sq, sq_rev);
            t = reduce_half_wave(t, OpAdd());
            pred = (float)(half_t)step_xor32(t, OpAdd());
        }
        const float ruv = r - pred;
        float sb = 0;
        uint32_t ib = 0;
        if (bwd != 32) {
            // max(p_max, q_max, -lambda, ruv) in the lower half-wave, -min(p_min, q_min, -lambda, ruv) in the upper one
            const uint32_t flip = upper ? 0x80000000u : 0u;
            const float pq = OpMaximum()(step_xor16(extrema, OpMaximum()), from_bits<float>(bits(-1 * lambda) ^ flip));
            ib = bcast(muppet_scale_index_by_rows((unsigned)bwd, OpMaximum()(pq, from_bits<float>(bits(ruv) ^ flip)), upper), 0);
            sb = pow2u_bits(ib);
        }
        g_scale = 1.0f; d_scale = lrate;
        if (bwd == 8) {
            const int ruv_i = round_to_i8_scaled(ruv, sb);
            const float sq_rev = pow2_reciprocal(2u * ib);
            const int lam_i = round_to_i8_scaled(-1.0f * lambda, sb);
#pragma unroll
            for (int e = 0; e < E; ++e) {
                const int pi = round_to_i8_scaled(p[e], sb), qi = round_to_i8_scaled(q[e], sb);
                gbp[e] = (float)(qi * ruv_i + pi * lam_i) * sq_rev;
                gbq[e] = (float)(pi * ruv_i + qi * lam_i) * sq_rev;
            }
        } else if (bwd == 32) {
#pragma unroll
            for (int e = 0; e < E; ++e) {
                gbp[e] = ruv * q[e] - lambda * p[e];
                gbq[e] = ruv * p[e] - lambda * q[e];
            }
        } else {
            const float sb_rev = pow2_reciprocal(ib);
            const half_t t_ruv = grid_h(ruv, sb, sb_rev), t_lam = grid_h(-1 * lambda, sb, sb_rev);
#pragma unroll
            for (int e = 0; e < E; ++e) {
                const half_t ph = grid_h(p[e], sb, sb_rev), qh = grid_h(q[e], sb, sb_rev);
                gbp[e] = (float)(half_t)(qh * t_ruv + ph * t_lam);
                gbq[e] = (float)(half_t)(ph * t_ruv + qh * t_lam);
            }
        }
    }
    // 8-bit forward and backward pass when both scale indices are plain ones and the backward index is small: nothing
    // saturates, the quantised -lambda comes from the scalar unit, and lrate * 2^(-2 index) from exponent arithmetic
    // (g = integer * 2^(-2 index) is exact, so lrate * g = integer * (lrate * 2^(-2 index)) with the same one
    // rounding).  False, with nothing written, when the inputs are not of that kind.
    __device__ __forceinline__ bool gradients_8bit_plain(const float* p, const float* q, float r, float* gbp, float* gbq, float& g_scale, float& d_scale) const
    {
        const bool upper = this->lane >= 32;
        float a = p[0], b = -p[0], c = q[0], d = -q[0];
        if constexpr (E == 2) {
            a = OpMaximum()(a, p[1]); b = OpMaximum()(b, -p[1]);
            c = OpMaximum()(c, q[1]); d = OpMaximum()(d, -q[1]);
        }
        const float extrema = max4_by_rows(a, b, c, d);
        uint32_t idx;
        if (!muppet_scale_index_plain(8u, extrema, upper, idx)) return false;
        // rows 0, 2: the two sides of p; rows 1, 3: of q
        const uint32_t ip0 = bcast(idx, 0), ip1 = bcast(idx, 32), iq0 = bcast(idx, 16), iq1 = bcast(idx, 48);
        const uint32_t ip = ip0 < ip1 ? ip0 : ip1, iq = iq0 < iq1 ? iq0 : iq1;
        const float sp = pow2u_bits(ip), sq = pow2u_bits(iq);
        int acc = 0;
#pragma unroll
        for (int e = 0; e < E; ++e) {
            const int pi = round_to_i8_in_range(p[e], sp), qi = round_to_i8_in_range(q[e], sq);
            acc += pi * qi;
        }
        acc = sum_wave_uniform(acc);
        const uint32_t n = ip + iq;                                            // at most 254
        const float pred = __builtin_ldexpf((float)acc, n > 127u ? -1000 : -(int)n);
        const float ruv = r - pred;
        const uint32_t flip = upper ? 0x80000000u : 0u;
        const float pq = OpMaximum()(step_xor16(extrema, OpMaximum()), from_bits<float>(bits(-1 * lambda) ^ flip));
        uint32_t idx_b;
        if (!muppet_scale_index_plain(8u, OpMaximum()(pq, from_bits<float>(bits(ruv) ^ flip)), upper, idx_b)) return false;
        const uint32_t ib0 = bcast(idx_b, 0), ib1 = bcast(idx_b, 32);
        const uint32_t ib = ib0 < ib1 ? ib0 : ib1;
        if (ib > kShortPathMaxIndex) return false;
        const float sb = pow2u_bits(ib);
        const int ruv_i = round_to_i8_in_range(ruv, sb);
        const int lam_i = neg_lambda_q.scaled(ib);
        g_scale = from_bits<float>((127u - 2u * ib) << 23);
        d_scale = from_bits<float>(bits(lrate) - (ib << 24));
#pragma unroll
        for (int e = 0; e < E; ++e) {
            const int pi = round_to_i8_in_range(p[e], sb), qi = round_to_i8_in_range(q[e], sb);
            gbp[e] = (float)(qi * ruv_i + pi * lam_i);
            gbq[e] = (float)(pi * ruv_i + qi * lam_i);
        }
        return true;
    }
    template <int CLS, bool HOT, bool SCALED> __device__ __forceinline__ void update(Row& row, const Info& i, uint32_t processed)
    {
        float gbp[E], gbq[E], g_scale, d_scale;
        if (!(plain_8bit && gradients_8bit_plain(row.p, row.q, i.r, gbp, gbq, g_scale, d_scale)))
            gradients(row.p, row.q, i.r, gbp, gbq, g_scale, d_scale);
        // d_scale carries the learning rate: a replicated row's copy takes a longer step (DenseBase::rep_scale; the factor
        // is 1 everywhere else, and a product by 1 is exact)
        const float ds_p = SCALED ? d_scale * this->scale_of(i.thin, 16u) : d_scale, ds_q = SCALED ? d_scale * this->scale_of(i.thin, 32u) : d_scale;
        float dp[E], dq[E];
#pragma unroll
        for (int e = 0; e < E; ++e) {
            dp[e] = ds_p * gbp[e];
            dq[e] = ds_q * gbq[e];
            row.p[e] = Base::template skips<CLS>(i.thin, 1u) ? row.p[e] : row.p[e] + dp[e];
            row.q[e] = Base::template skips<CLS>(i.thin, 2u) ? row.q[e] : row.q[e] + dq[e];
        }
        this->template store<HOT>(row, i, dp, dq);
        if (fwd != 32 && bwd != 32 && processed >= first_sample) {
            float gp[E], gq[E], sp2[E], sq2[E];
#pragma unroll
            for (int e = 0; e < E; ++e) { gp[e] = gbp[e] * g_scale; gq[e] = gbq[e] * g_scale; }
#pragma unroll
            for (int e = 0; e < E; ++e) { sp2[e] = gp[e] * gp[e]; sq2[e] = gq[e] * gq[e]; }
            float npq = lane_sum_of_squares(sp2) + lane_sum_of_squares(sq2);
            npq = reduce_half_wave(npq, OpAdd());
            sum_norms_reg += npq;
#pragma unroll
            for (int e = 0; e < E; ++e) grad_acc[e] += gp[e] + gq[e];       // flushed once per worker in finish()
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
__device__ __forceinline__ float afp_grid(float v, float s, float s_rev) { return round_half_away(v * s) * s_rev; }
// the same for a scale s = 2^n, n >= 0 (the product is exact or infinite, so the fused form rounds alike)
__device__ __forceinline__ float afp_grid_pow2(float v, float s, float s_rev) { return round_half_away_scaled(v, s) * s_rev; }
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
__device__ __forceinline__ float ufirst(float x) { return from_bits<float>((uint32_t)__builtin_amdgcn_readfirstlane((int)bits(x))); }
__device__ __forceinline__ int ufirst(int x) { return __builtin_amdgcn_readfirstlane(x); }

template <int K, bool COH> struct AfpRule : DenseBase<K, COH> {
    using Base = DenseBase<K, COH>;
    using typename Base::Row;
    using typename Base::Info;
    static constexpr int E = Base::E;
    static constexpr int J = K / 32;
    static constexpr int kAhead = 1, kRing = 4;    // as for MuPPET: three ratings ahead measured no faster (k = 128) or slower (k = 64)
    static constexpr int kMinWavesPerSimd = 6;     // 24 wavefronts per CU: 6144 workers resident at a time (85 VGPRs otherwise: 5 per SIMD, 5120)
    static constexpr bool kSplittable = false;    // the per-worker quantiser state lives for one launch
    struct Params { float* p; float* q; float lrate; float lambda; int afp_epoch; int init_threshold; bool accumulate; void* rep_p; void* rep_q; float rep_scale; };
    float lrate, lambda; int afp_epoch, init_threshold;
    AfpQ uq, iq, bq;
    int upd_u, upd_i, upd_b, cur_iter;
    float sp, sq, sb;
    bool upper;
    // What follows from the three quantisers alone, computed when one of them is re-measured (wave-uniform, kept in
    // scalar registers): the exponent that turns the int8 dot into the prediction, the reciprocal scales of the 16-bit
    // paths, the quantised -lambda of both backward paths, 2^(-2 r) and, where it is exact, lrate * 2^(-2 r).
    int pred_exp; float sp_rev, sq_rev;
    int lam_i8; float sb_rev2, d_scale8; bool fused8;
    float sb_rev; half_t t_lam16;
    bool lrate_plain;

    __device__ __forceinline__ void init(const Params& a, uint8_t*, int lane_, uint32_t)
    {
        this->P = a.p; this->Q = a.q; this->RP = static_cast<float*>(a.rep_p); this->RQ = static_cast<float*>(a.rep_q);
        this->lane = lane_; lrate = a.lrate; lambda = a.lambda; this->rep_scale = a.rep_scale;
        afp_epoch = a.afp_epoch; init_threshold = a.init_threshold;
        uq = AfpQ{0, 0, 0, 0.f}; iq = uq; bq = uq;
        upd_u = upd_i = upd_b = cur_iter = 0; sp = sq = sb = 0.f; upper = lane_ >= 32;
        pred_exp = 0; sp_rev = sq_rev = sb_rev = sb_rev2 = d_scale8 = 0.f; lam_i8 = 0; fused8 = false; t_lam16 = (half_t)0.f;
        // lrate in [2^-20, 2^20]: with 2 r <= 96, lrate * 2^(-2 r) and every float(int) * that stay normal numbers
        const uint32_t le = (bits(lrate) >> 23) & 0x1ffu;
        lrate_plain = le >= 107u && le <= 147u;
    }
    __device__ __forceinline__ void forward_changed()
    {
        const uint32_t n = (uint32_t)uq.r + (uint32_t)iq.r;                      // r >= 0
        pred_exp = n > 127u ? -1000 : -(int)n;                                   // acc / (sp * sq): 2^-n, or 0 with the sign of acc
        sp_rev = ufirst(pow2_reciprocal((uint32_t)uq.r)); sq_rev = ufirst(pow2_reciprocal((uint32_t)iq.r));
    }
    __device__ __forceinline__ void backward_changed()
    {
        const uint32_t r = (uint32_t)bq.r;
        lam_i8 = ufirst(round_to_i8_scaled(-1.0f * lambda, sb));
        sb_rev2 = ufirst(pow2_reciprocal(2u * r));
        // g = integer * 2^(-2 r) is exact for small r, so lrate * g = integer * (lrate * 2^(-2 r)) with the same one rounding
        fused8 = lrate_plain && r <= 48u;
        d_scale8 = from_bits<float>(bits(lrate) - ((fused8 ? r : 0u) << 24));
        sb_rev = ufirst(pow2_reciprocal(r));
        t_lam16 = from_bits<half_t>((uint32_t)__builtin_amdgcn_readfirstlane((int)bits((half_t)afp_grid_pow2(-1.0f * lambda, sb, sb_rev))));
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
    template <int CLS, bool HOT, bool SCALED> __device__ __forceinline__ void update(Row& row, const Info& i, uint32_t)
    {
        const float* p = row.p; const float* q = row.q;
        float p_abs = fabsf(p[0]), q_abs = fabsf(q[0]);
        if constexpr (E == 2) { p_abs = OpMaximum()(p_abs, fabsf(p[1])); q_abs = OpMaximum()(q_abs, fabsf(q[1])); }
        // the three re-measurements below happen every itv-th update of the worker; they sum their error terms per
        // lane from left to right over all four values, so they work on the 32-lane view
        if (cur_iter == upd_u) {
            Mirror<K> pm; pm.build(row.p, upper);
            const float mx = reduce_wave(p_abs, OpMaximum());
            const float diff = qem(pm.v, mx);
            if (cur_iter == 0) uq.mov_avg_range = mx;
            uq = uniform(afp_qpa(diff, mx, uq.mov_avg_range));
            sp = pow2i(uq.r);
            forward_changed();
            if (afp_epoch == 0 && cur_iter < init_threshold) uq.itv = 1;
            upd_u += uq.itv;
        }
        if (cur_iter == upd_i) {
            Mirror<K> qm; qm.build(row.q, upper);
            const float mx = reduce_wave(q_abs, OpMaximum());
            const float diff = qem(qm.v, mx);
            if (cur_iter == 0) iq.mov_avg_range = mx;
            iq = uniform(afp_qpa(diff, mx, iq.mov_avg_range));
            sq = pow2i(iq.r);
            forward_changed();
            if (afp_epoch == 0 && cur_iter < init_threshold) iq.itv = 1;
            upd_i += iq.itv;
        }
        float pred;
        if (uq.n == 8 && iq.n == 8) {
            int acc = 0;
#pragma unroll
            for (int e = 0; e < E; ++e) acc += round_to_i8_scaled(p[e], sp) * round_to_i8_scaled(q[e], sq);
            acc = reduce_wave(acc, OpAdd());
            pred = __builtin_ldexpf((float)acc, pred_exp);                           // acc / (sp * sq)
        } else {
            // the reference's half2 lanes: .x sums elements l, l+64 (lower half-wave here), .y elements l+32, l+96 (upper)
            half_t t = (half_t)afp_grid_pow2(p[0], sp, sp_rev) * (half_t)afp_grid_pow2(q[0], sq, sq_rev);
            if constexpr (E == 2) t = t + (half_t)afp_grid_pow2(p[1], sp, sp_rev) * (half_t)afp_grid_pow2(q[1], sq, sq_rev);
            t = reduce_half_wave(t, OpAdd());
            pred = (float)(half_t)step_xor32(t, OpAdd());
        }
        const float ruv = i.r - pred;
        if (cur_iter == upd_b) {
            Mirror<K> pm, qm; pm.build(row.p, upper); qm.build(row.q, upper);
            float mx = OpMaximum()(p_abs, q_abs);
            mx = OpMaximum()(OpMaximum()(mx, fabsf(lambda)), fabsf(ruv));
            mx = reduce_wave(mx, OpMaximum());
            const float diff = qem_bp(pm.v, qm.v, ruv, mx);
            if (cur_iter == 0) bq.mov_avg_range = mx;
            bq = uniform(afp_qpa(diff, mx, bq.mov_avg_range));
            sb = pow2i(bq.r);
            backward_changed();
            if (afp_epoch == 0 && cur_iter < init_threshold) bq.itv = 1;
            upd_b += bq.itv;
        }
        // the change of a row is lrate * g = g_base * d_scale
        float gbp[E], gbq[E], d_scale = lrate;
        if (bq.n == 8) {
            const int ruv_i = round_to_i8_scaled(ruv, sb);
#pragma unroll
            for (int e = 0; e < E; ++e) {
                const int pi = round_to_i8_scaled(p[e], sb), qi = round_to_i8_scaled(q[e], sb);
                gbp[e] = (float)(qi * ruv_i + pi * lam_i8);
                gbq[e] = (float)(pi * ruv_i + qi * lam_i8);
            }
            if (fused8) d_scale = d_scale8;
            else {
#pragma unroll
                for (int e = 0; e < E; ++e) { gbp[e] = gbp[e] * sb_rev2; gbq[e] = gbq[e] * sb_rev2; }
            }
        } else {
            const half_t t_ruv = (half_t)afp_grid_pow2(ruv, sb, sb_rev);
#pragma unroll
            for (int e = 0; e < E; ++e) {
                const half_t ph = (half_t)afp_grid_pow2(p[e], sb, sb_rev), qh = (half_t)afp_grid_pow2(q[e], sb, sb_rev);
                gbp[e] = (float)(half_t)(qh * t_ruv + ph * t_lam16);
                gbq[e] = (float)(half_t)(ph * t_ruv + qh * t_lam16);
            }
        }
        // d_scale carries the learning rate: a replicated row's copy takes a longer step (DenseBase::rep_scale; the factor
        // is 1 everywhere else, and a product by 1 is exact)
        const float ds_p = SCALED ? d_scale * this->scale_of(i.thin, 16u) : d_scale, ds_q = SCALED ? d_scale * this->scale_of(i.thin, 32u) : d_scale;
        float dp[E], dq[E];
#pragma unroll
        for (int e = 0; e < E; ++e) {
            dp[e] = ds_p * gbp[e];
            dq[e] = ds_q * gbq[e];
            row.p[e] = Base::template skips<CLS>(i.thin, 1u) ? row.p[e] : row.p[e] + dp[e];
            row.q[e] = Base::template skips<CLS>(i.thin, 2u) ? row.q[e] : row.q[e] + dq[e];
        }
        this->template store<HOT>(row, i, dp, dq);
        cur_iter += 1;
    }
    __device__ __forceinline__ void finish(const Params&, uint32_t) const {}
};

}  // namespace mf
