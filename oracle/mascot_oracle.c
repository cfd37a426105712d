/*
 * TEST INFRASTRUCTURE ONLY -- CPU restatement of the reference's hot path
 * (Yujaeseo/ICDM-2021_MASCOT).  See mascot_oracle.h for the contract and the
 * list of functions whose parity is unpinned.
 *
 * Conventions restated from the reference kernels: one 32-lane warp processes
 * one rating; lane l holds elements l, l+32 (k=64) or l, l+32, l+64, l+96
 * (k=128) of the P row and the Q row (sgd/sgd_kernel.h:42-52).  A "tree" is
 * the shfl_down 16,8,4,2,1 reduction whose lane-0 value is broadcast
 * (sgd/sgd_kernel.h:57-63).  All arithmetic below is written one operation per
 * statement and compiled with -ffp-contract=off so that every intermediate is
 * rounded exactly once, in the order the reference source spells out; where
 * the reference calls fmaf/__hfma explicitly, so does this file.
 */
#include "mascot_oracle.h"
#include "orc_half.h"
#include <stdlib.h>
#include <math.h>
#include <limits.h>
#ifdef _OPENMP
#include <omp.h>
#endif
#if defined(__F16C__) && !defined(ORC_SOFT_HALF)
#include <immintrin.h>
#define ORC_USE_F16C 1
#endif

/* ------------------------------------------------------------------------ */
/* binary16 helpers                                                          */
/* ------------------------------------------------------------------------ */

/* Round a binary32 value to the nearest binary16 value, returned as binary32.
 * With F16C this is the hardware conversion; otherwise the software routine.
 * Both are pinned against each other by tests/test_oracle_half.py. */
static inline float rn16f(float x)
{
#ifdef ORC_USE_F16C
    return _cvtsh_ss(_cvtss_sh(x, _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC));
#else
    return orc_h2f(orc_f2h(x));
#endif
}
/* Half-valued operands carried as binary32: product exact, sum/difference
 * correctly rounded after the second rounding (24 >= 2*11+2 bits). */
static inline float hmulf(float a, float b) { return rn16f(a * b); }
static inline float haddf(float a, float b) { return rn16f(a + b); }
static inline float hsubf(float a, float b) { return rn16f(a - b); }
static inline float hfmaf_(float a, float b, float c) { return orc_h2f(orc_hfma(orc_f2h(a), orc_f2h(b), orc_f2h(c))); }

uint16_t orc_float2half(float f) { return orc_f2h(f); }
float orc_half2float(uint16_t h) { return orc_h2f(h); }
uint16_t orc_double2half(double d) { return orc_d2h(d); }
uint16_t orc_half_add(uint16_t a, uint16_t b) { return orc_hadd(a, b); }
uint16_t orc_half_sub(uint16_t a, uint16_t b) { return orc_hsub(a, b); }
uint16_t orc_half_mul(uint16_t a, uint16_t b) { return orc_hmul(a, b); }
uint16_t orc_half_fma(uint16_t a, uint16_t b, uint16_t c) { return orc_hfma(a, b, c); }
/* transform_float2half / transform_half2float, model_init.cu:85-105 */
void orc_float2half_array(const float* in, uint16_t* out, uint64_t n) { for (uint64_t i = 0; i < n; i++) out[i] = orc_f2h(in[i]); }
void orc_half2float_array(const uint16_t* in, float* out, uint64_t n) { for (uint64_t i = 0; i < n; i++) out[i] = orc_h2f(in[i]); }

/* ------------------------------------------------------------------------ */
/* schedules                                                                 */
/* ------------------------------------------------------------------------ */

/* mf_methods.cu:101: ceil((double)n / (num_workers * update_vector_size)) */
uint32_t orc_update_count(uint32_t n, uint32_t num_workers, uint32_t update_vector_size)
{
    return (uint32_t)ceil((double)n / (double)(num_workers * update_vector_size));
}
/* mf_methods.cu:102: unsigned = (float)(update_count*128) * sample_ratio, truncated */
uint32_t orc_sample_ratings_num(uint32_t update_count, uint32_t update_vector_size, float sample_ratio)
{
    float v = (float)(update_count * update_vector_size) * sample_ratio;
    return (uint32_t)v;
}
/* mf_methods.cu:172: e >= 5 && e % interval == 5 % interval && e != epochs-1 */
int orc_is_error_check_epoch(uint32_t e, uint32_t interval, uint32_t epochs)
{
    const uint32_t start_idx = 5;
    return (e >= start_idx) && (e % interval == (start_idx % interval)) && (epochs - 1 != e);
}
/* mf_methods.cu:170-175 */
uint32_t orc_first_sample_rating_idx(uint32_t e, uint32_t interval, uint32_t epochs,
                                     uint32_t update_count, uint32_t update_vector_size, float sample_ratio)
{
    uint32_t total = update_count * update_vector_size;
    if (orc_is_error_check_epoch(e, interval, epochs))
        return total - orc_sample_ratings_num(update_count, update_vector_size, sample_ratio);
    return total;
}
/* mf_methods.cu:94-97: float = lr / (1.0 + decay * pow(i, 1.5f)), evaluated in double */
float orc_lr_schedule(float lr, float decay, uint32_t e)
{
    return (float)((double)lr / (1.0 + ((double)decay * pow((double)e, 1.5))));
}

static inline uint64_t mix64(uint64_t z)
{
    z += 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

/* Start of a worker's window.  The index mapping restates sgd/sgd_kernel.h:22-26
 * (origin = (unsigned)(u01 * nnz); start = origin % nnz, with u01 in (0,1] built
 * from 32 random bits as x*2^-32 + 2^-33 in binary32); the 32 random bits come
 * from this build's counter-based generator instead of cuRAND XORWOW seeded with
 * clock() (model_init.cu:15).  parity unpinned for the bit stream. */
uint32_t orc_window_start(uint64_t seed, uint32_t epoch, uint32_t wid, uint32_t ite, uint32_t nnz)
{
    uint64_t h = mix64(seed ^ 0x57494E444F575321ull);
    h = mix64(h + (uint64_t)epoch);
    h = mix64(h ^ (((uint64_t)wid << 32) | (uint64_t)ite));
    uint32_t x = (uint32_t)(h >> 32);
    float t = (float)x * 2.3283064365386963e-10f;
    float u01 = t + 1.1641532182693481e-10f;
    float scaled = u01 * (float)nnz;
    uint32_t origin = (scaled >= 4294967296.0f) ? 0xffffffffu : (uint32_t)scaled;
    return origin % nnz;
}

/* ------------------------------------------------------------------------ */
/* preprocessing                                                             */
/* ------------------------------------------------------------------------ */

/* user_item_histogram, preprocess_utils.h:13-19 */
void orc_histogram(const orc_node* R, uint64_t n, uint32_t* user_cnt, uint32_t n_users, uint32_t* item_cnt, uint32_t n_items)
{
    for (uint32_t i = 0; i < n_users; i++) user_cnt[i] = 0;
    for (uint32_t i = 0; i < n_items; i++) item_cnt[i] = 0;
    for (uint64_t i = 0; i < n; i++) { user_cnt[R[i].u]++; item_cnt[R[i].i]++; }
}

/* thrust::sort_by_key(count, id), preprocess_utils.h:87-88: ascending by count,
 * ids of equal count keep their original (ascending id) order -- the order the
 * radix sort behind thrust gives for 32-bit keys. */
void orc_sort_by_count(const uint32_t* cnt, uint32_t n, uint32_t* sorted_cnt, uint32_t* sorted_id)
{
    /* counting sort by key keeps ties stable */
    uint32_t maxc = 0;
    for (uint32_t i = 0; i < n; i++) if (cnt[i] > maxc) maxc = cnt[i];
    uint64_t* start = (uint64_t*)calloc((size_t)maxc + 2, sizeof(uint64_t));
    for (uint32_t i = 0; i < n; i++) start[cnt[i] + 1]++;
    for (uint64_t c = 1; c <= (uint64_t)maxc + 1; c++) start[c] += start[c - 1];
    for (uint32_t i = 0; i < n; i++) {
        uint64_t pos = start[cnt[i]]++;
        sorted_cnt[pos] = cnt[i];
        sorted_id[pos] = i;
    }
    free(start);
}

/* split_group_based_equal_size_not_strict_ret_end_idx, preprocess_utils.h:101-190.
 * sorted_cnt: rating counts ascending.  Returns the actual number of groups and
 * writes the inclusive last sorted position of each group. */
uint32_t orc_grouping(const uint32_t* sorted_cnt, uint32_t n, uint32_t requested_groups, uint32_t* end_idx_out)
{
    uint32_t threshold = (uint32_t)ceil(n / (float)requested_groups);           /* :110 */
    uint32_t max_cnt = sorted_cnt[n - 1];                                        /* :113 */
    uint32_t* last_pos = (uint32_t*)malloc(((size_t)max_cnt + 1) * sizeof(uint32_t));
    for (uint32_t i = 1; i <= max_cnt; i++) last_pos[i] = 0xffffffffu;           /* :124 */
    last_pos[0] = 0xffffffffu;
    for (uint32_t i = 0; i < n; i++) last_pos[sorted_cnt[i]] = i;                /* :127-130 */
    uint32_t groups = 0, acc = 0, prev = 0;
    for (uint32_t c = 1; c <= max_cnt; c++) {                                    /* :139-152 */
        if (last_pos[c] != 0xffffffffu) {
            acc += (last_pos[c] - prev + 1);
            if (acc >= threshold) { end_idx_out[groups++] = last_pos[c]; acc = 0; }
            else if (c == max_cnt) { end_idx_out[groups++] = last_pos[c]; }
            prev = last_pos[c] + 1;
        }
    }
    free(last_pos);
    return groups;
}

/* preprocess_utils.h:171-187 (group of each id) and :223-241 (id -> sorted position, group sizes) */
void orc_reindex_tables(const uint32_t* sorted_id, uint32_t n, const uint32_t* end_idx, uint32_t groups,
                        uint32_t* id2sorted, uint32_t* id2group, uint32_t* group_size)
{
    for (uint32_t g = 0; g < groups; g++) group_size[g] = 0;
    uint32_t end = 0;
    for (uint32_t g = 0; g < groups; g++) {
        uint32_t start = end;
        end = end_idx[g] + 1;
        for (uint32_t pos = start; pos < end; pos++) id2group[sorted_id[pos]] = g;
    }
    for (uint32_t pos = 0; pos < n; pos++) {
        id2sorted[sorted_id[pos]] = pos;
        group_size[id2group[sorted_id[pos]]]++;
    }
}

/* matrix_reconst_gpu_triplet, preprocess_utils.h:28-36 */
void orc_reindex(orc_node* R, uint64_t n, const uint32_t* user2sorted, const uint32_t* item2sorted)
{
    for (uint64_t i = 0; i < n; i++) { R[i].u = user2sorted[R[i].u]; R[i].i = item2sorted[R[i].i]; }
}

/* In-kernel group search, mascot/mascot_sgd_kernel.h:104-143: the group is the one whose
 * (previous end, end] interval holds idx, i.e. min{g : idx <= end_idx[g]}; the row inside
 * the group is idx - end_idx[g-1] - 1 (idx itself for group 0). */
void orc_group_lookup(uint32_t idx, const uint32_t* end_idx, uint32_t groups, uint32_t* group, uint32_t* local_row)
{
    for (uint32_t g = 0; g < groups; g++) {
        if (idx <= end_idx[g]) {
            *group = g;
            *local_row = (g == 0) ? idx : idx - end_idx[g - 1] - 1;
            return;
        }
    }
    *group = 0xffffffffu; *local_row = 0;
}

/* Seeded replacement for srand(time(0)); std::random_shuffle (mf_methods.cu:38-39):
 * rating i gets a 64-bit key; the shuffled order is ascending key (ties by i).
 * parity unpinned (the reference order is unseeded). */
void orc_shuffle_keys(uint64_t seed, uint64_t n, uint64_t* keys)
{
    uint64_t base = mix64(seed ^ 0x53485546464C4521ull);
    for (uint64_t i = 0; i < n; i++) keys[i] = mix64(base ^ i);
}
typedef struct { uint64_t key; uint64_t idx; } key_idx;
static int key_idx_cmp(const void* a, const void* b)
{
    const key_idx* x = (const key_idx*)a; const key_idx* y = (const key_idx*)b;
    if (x->key != y->key) return x->key < y->key ? -1 : 1;
    return x->idx < y->idx ? -1 : (x->idx > y->idx);
}
void orc_shuffle(uint64_t seed, const orc_node* in, orc_node* out, uint64_t n)
{
    key_idx* ki = (key_idx*)malloc(n * sizeof(key_idx));
    uint64_t base = mix64(seed ^ 0x53485546464C4521ull);
    for (uint64_t i = 0; i < n; i++) { ki[i].key = mix64(base ^ i); ki[i].idx = i; }
    qsort(ki, n, sizeof(key_idx), key_idx_cmp);
    for (uint64_t i = 0; i < n; i++) out[i] = in[ki[i].idx];
    free(ki);
}

/* natural log of x in (0,1], built from +,-,*,/ only so that any IEEE machine
 * gives the same bits: x = m*2^e, m in [sqrt(1/2), sqrt(2)), ln m = 2 atanh((m-1)/(m+1)). */
static double det_log(double x)
{
    uint64_t b = orc_f64_bits(x);
    int e = (int)((b >> 52) & 0x7ff) - 1022;                 /* x = m * 2^e, m in [0.5,1) */
    double m = orc_bits_f64((b & 0x000fffffffffffffull) | 0x3fe0000000000000ull);
    if (m < 0.70710678118654752440) { m = m * 2.0; e = e - 1; }
    double s = (m - 1.0) / (m + 1.0);
    double s2 = s * s;
    double acc = 1.0 / 21.0;
    acc = acc * s2 + 1.0 / 19.0;
    acc = acc * s2 + 1.0 / 17.0;
    acc = acc * s2 + 1.0 / 15.0;
    acc = acc * s2 + 1.0 / 13.0;
    acc = acc * s2 + 1.0 / 11.0;
    acc = acc * s2 + 1.0 / 9.0;
    acc = acc * s2 + 1.0 / 7.0;
    acc = acc * s2 + 1.0 / 5.0;
    acc = acc * s2 + 1.0 / 3.0;
    acc = acc * s2 + 1.0;
    double lnm = (2.0 * s) * acc;
    return (double)e * 0.69314718055994530942 + lnm;
}
/* cos(2*pi*t), t in [0,1): quadrant reduction then Taylor polynomials in +,-,* only. */
static double det_cos2pi(double t)
{
    double t4 = t * 4.0;
    int q = (int)t4;
    double f = t4 - (double)q;
    double a = f * 1.57079632679489661923;
    double a2 = a * a;
    /* cos a = sum (-1)^n a^(2n)/(2n)!, n = 0..10 */
    double c = 1.0 / 2432902008176640000.0;
    c = -1.0 / 6402373705728000.0 + a2 * c;
    c = 1.0 / 20922789888000.0 + a2 * c;
    c = -1.0 / 87178291200.0 + a2 * c;
    c = 1.0 / 479001600.0 + a2 * c;
    c = -1.0 / 3628800.0 + a2 * c;
    c = 1.0 / 40320.0 + a2 * c;
    c = -1.0 / 720.0 + a2 * c;
    c = 1.0 / 24.0 + a2 * c;
    c = -1.0 / 2.0 + a2 * c;
    c = 1.0 + a2 * c;
    /* sin a = a * sum (-1)^n a^(2n)/(2n+1)!, n = 0..10 */
    double s = 1.0 / 51090942171709440000.0;
    s = -1.0 / 121645100408832000.0 + a2 * s;
    s = 1.0 / 355687428096000.0 + a2 * s;
    s = -1.0 / 1307674368000.0 + a2 * s;
    s = 1.0 / 6227020800.0 + a2 * s;
    s = -1.0 / 39916800.0 + a2 * s;
    s = 1.0 / 362880.0 + a2 * s;
    s = -1.0 / 5040.0 + a2 * s;
    s = 1.0 / 120.0 + a2 * s;
    s = -1.0 / 6.0 + a2 * s;
    s = 1.0 + a2 * s;
    s = a * s;
    switch (q & 3) { case 0: return c; case 1: return -s; case 2: return -c; default: return s; }
}
/* init_rand_feature_single, model_init.cu:19-28: array[i] = (float)(N(0,1) * 0.01).
 * The normal deviate is a Box-Muller transform of this build's counter-based bits
 * (the reference draws from cuRAND states seeded with clock()).  parity unpinned. */
static double det_normal(uint64_t h)
{
    uint32_t a = (uint32_t)(h >> 32), b = (uint32_t)h;
    double u1 = ((double)a + 1.0) * 2.3283064365386962890625e-10;
    double u2 = (double)b * 2.3283064365386962890625e-10;
    double rad = sqrt(-2.0 * det_log(u1));
    return rad * det_cos2pi(u2);
}
static void normal_array(uint64_t base, double scale, float* out, uint64_t n)
{
    for (uint64_t i = 0; i < n; i++) out[i] = (float)(det_normal(mix64(base ^ i)) * scale);
}
void orc_init_normal(uint64_t seed, uint64_t stream, float* out, uint64_t n)
{
    normal_array(mix64(mix64(seed ^ 0x494E49544E4F524Dull) + stream), 0.01, out, n);
}

/* Seeded synthetic ratings: the CPU twin of this build's generator (the reference has none; its data sets are
 * downloaded).  Users and items from Zipf(alpha) over a seeded permutation of the ids, ratings from a low-rank
 * truth plus noise rounded to the rating grid, or bimodal 0..100 ratings mapped to r * 0.04 + 1.  parity unpinned
 * against the reference by construction; pinned against the distribution it claims (tests/test_oracle_host.py). */
static uint32_t cdf_rank(const double* cdf, uint32_t count, double x)
{
    uint32_t lo = 0, hi = count - 1;
    while (lo < hi) {
        uint32_t mid = (lo + hi) >> 1;
        if (x < cdf[mid]) hi = mid; else lo = mid + 1;
    }
    return lo;
}
static double* zipf_cdf(uint32_t count, float alpha)
{
    double* cdf = (double*)malloc((size_t)count * sizeof(double));
    double sum = 0.0;
    for (uint32_t i = 0; i < count; i++) { sum += pow((double)(i + 1), -(double)alpha); cdf[i] = sum; }
    for (uint32_t i = 0; i < count; i++) cdf[i] = cdf[i] / sum;
    return cdf;
}
static uint32_t* seeded_permutation(uint32_t count, uint64_t base)
{
    uint32_t* p = (uint32_t*)malloc((size_t)count * sizeof(uint32_t));
    for (uint32_t i = 0; i < count; i++) p[i] = i;
    for (uint32_t i = count; i-- > 1;) {
        uint32_t j = (uint32_t)(mix64(base ^ (uint64_t)i) % ((uint64_t)i + 1));
        uint32_t t = p[i]; p[i] = p[j]; p[j] = t;
    }
    return p;
}
void orc_generate_ratings(const orc_synth_config* c, uint64_t seed, uint64_t first, uint64_t count, orc_node* out)
{
    uint64_t key = mix64(seed ^ 0x53594E5448455449ull);
    double* ucdf = zipf_cdf(c->n_users, c->user_alpha);
    double* icdf = zipf_cdf(c->n_items, c->item_alpha);
    uint32_t* uperm = seeded_permutation(c->n_users, mix64(key + 1));
    uint32_t* iperm = seeded_permutation(c->n_items, mix64(key + 2));
    float *U = NULL, *V = NULL;
    if (!c->bimodal) {
        U = (float*)malloc((size_t)c->n_users * c->rank * sizeof(float));
        V = (float*)malloc((size_t)c->n_items * c->rank * sizeof(float));
        normal_array(mix64(key + 3), 0.5, U, (uint64_t)c->n_users * c->rank);
        normal_array(mix64(key + 4), 0.5, V, (uint64_t)c->n_items * c->rank);
    }
    float inv_step = 1.0f / c->step;
    for (uint64_t i = 0; i < count; i++) {
        uint64_t j = first + i;
        double xu = (double)(mix64(key ^ (j * 4 + 0)) >> 11) * 1.1102230246251565404e-16;
        double xi = (double)(mix64(key ^ (j * 4 + 1)) >> 11) * 1.1102230246251565404e-16;
        uint32_t u = uperm[cdf_rank(ucdf, c->n_users, xu)];
        uint32_t v = iperm[cdf_rank(icdf, c->n_items, xi)];
        float nz = (float)(det_normal(mix64(key ^ (j * 4 + 2))) * (double)c->noise);
        float r;
        if (c->bimodal) {
            double xm = (double)(mix64(key ^ (j * 4 + 3)) >> 11) * 1.1102230246251565404e-16;
            float m = xm < 0.5 ? 20.0f : 80.0f;
            r = fminf(fmaxf(roundf(m + nz), c->lo), c->hi) * 0.04f + 1.0f;
        } else {
            float dot = 0.0f;
            for (uint32_t k = 0; k < c->rank; k++) dot = dot + U[(size_t)u * c->rank + k] * V[(size_t)v * c->rank + k];
            float val = (dot + c->mean) + nz;
            r = fminf(fmaxf(roundf(val * inv_step) * c->step, c->lo), c->hi);
        }
        out[i].r = r; out[i].u = u; out[i].i = v;
    }
    free(ucdf); free(icdf); free(uperm); free(iperm); free(U); free(V);
}

/* ------------------------------------------------------------------------ */
/* warp emulation helpers                                                    */
/* ------------------------------------------------------------------------ */
#define LANES 32
static inline float tree_f(float* x)
{
    for (int off = 16; off >= 1; off >>= 1)
        for (int l = 0; l < off; l++) x[l] = x[l] + x[l + off];
    return x[0];
}
static inline float tree_h(float* x)   /* binary16 values carried as binary32 */
{
    for (int off = 16; off >= 1; off >>= 1)
        for (int l = 0; l < off; l++) x[l] = haddf(x[l], x[l + off]);
    return x[0];
}
static inline int tree_i(int* x)
{
    for (int off = 16; off >= 1; off >>= 1)
        for (int l = 0; l < off; l++) x[l] = x[l] + x[l + off];
    return x[0];
}
/* fp32 dot in the reference order: ((p1q1+p2q2)+(p3q3+p4q4)) per lane (k=128) or
 * (p1q1+p2q2) (k=64), then the tree.  sgd/sgd_kernel.h:55-63, sgd_kernel_k64.h:49-57 */
static float dot_f32(int k, const float* p, const float* q)
{
    float x[LANES];
    for (int l = 0; l < LANES; l++) {
        float m0 = p[l] * q[l];
        float m1 = p[l + 32] * q[l + 32];
        float a = m0 + m1;
        if (k == 128) {
            float m2 = p[l + 64] * q[l + 64];
            float m3 = p[l + 96] * q[l + 96];
            float b = m2 + m3;
            a = a + b;
        }
        x[l] = a;
    }
    return tree_f(x);
}
/* binary16 dot, every product and every sum rounded to binary16.
 * mascot/mascot_sgd_kernel.h:202-211, mpt/mpt_sgd_kernel.h:71-80 */
static float dot_f16(int k, const float* p, const float* q)
{
    float x[LANES];
    for (int l = 0; l < LANES; l++) {
        float m0 = hmulf(p[l], q[l]);
        float m1 = hmulf(p[l + 32], q[l + 32]);
        float a = haddf(m0, m1);
        if (k == 128) {
            float m2 = hmulf(p[l + 64], q[l + 64]);
            float m3 = hmulf(p[l + 96], q[l + 96]);
            float b = haddf(m2, m3);
            a = haddf(a, b);
        }
        x[l] = a;
    }
    return tree_h(x);
}
/* sum of squares in the order of mascot_sgd_kernel.h:244-257: per lane ((a+b)+(c+d)), tree in fp32 */
static float sumsq_f32(int k, const float* g)
{
    float x[LANES];
    for (int l = 0; l < LANES; l++) {
        float m0 = g[l] * g[l];
        float m1 = g[l + 32] * g[l + 32];
        float a = m0 + m1;
        if (k == 128) {
            float m2 = g[l + 64] * g[l + 64];
            float m3 = g[l + 96] * g[l + 96];
            float b = m2 + m3;
            a = a + b;
        }
        x[l] = a;
    }
    return tree_f(x);
}

/* ------------------------------------------------------------------------ */
/* single updates                                                            */
/* ------------------------------------------------------------------------ */

/* single_sgd_k128/k64_hogwild_kernel body, sgd/sgd_kernel.h:55-76, sgd_kernel_k64.h:49-64 */
void orc_sgd_update(int k, float* p, float* q, float r, float lr, float lambda)
{
    float dot = dot_f32(k, p, q);
    float ruv = r - dot;
    for (int e = 0; e < k; e++) {
        float pe = p[e], qe = q[e];
        float a = ruv * qe; float b = lambda * pe; float c = a - b; float d = lr * c;
        p[e] = pe + d;
        a = ruv * pe; b = lambda * qe; c = a - b; d = lr * c;
        q[e] = qe + d;
    }
}

/* mem_quant_sgd_k128/k64_hogwild_kernel body, sgd/sgd_kernel.h:126-163 (k = 64: sgd_kernel_k64.h): binary16 storage,
 * binary32 arithmetic.  Per lane the products are summed left to right (p1*q1 + p2*q2 + p3*q3 + p4*q4), then the
 * 16,8,4,2,1 tree; the new values are rounded to binary16 once.  No contraction (nvcc's choice there is unpinned). */
void orc_mem_quant_update(int k, uint16_t* p, uint16_t* q, float r, float lr, float lambda)
{
    float pf[128], qf[128], x[LANES];
    for (int e = 0; e < k; e++) { pf[e] = orc_h2f(p[e]); qf[e] = orc_h2f(q[e]); }
    for (int l = 0; l < LANES; l++) {
        float m0 = pf[l] * qf[l];
        float m1 = pf[l + 32] * qf[l + 32];
        float a = m0 + m1;
        if (k == 128) {
            float m2 = pf[l + 64] * qf[l + 64];
            a = a + m2;
            float m3 = pf[l + 96] * qf[l + 96];
            a = a + m3;
        }
        x[l] = a;
    }
    float ruv = r - tree_f(x);
    for (int e = 0; e < k; e++) {
        float pe = pf[e], qe = qf[e];
        float a = ruv * qe; float b = lambda * pe; float c = a - b; float d = lr * c; float n = pe + d;
        p[e] = orc_f2h(n);
        a = ruv * pe; b = lambda * qe; c = a - b; d = lr * c; n = qe + d;
        q[e] = orc_f2h(n);
    }
}

/* mpt_sgd_k128/k64_hogwild_kernel body, mpt/mpt_sgd_kernel.h:15-16,38-91.
 * scaled_lambda_h = __float2half_rn(lambda * 1000) is formed by the host (mf_methods.cu:764-765). */
void orc_mpt_update(int k, float* p, float* q, float r, float lr, uint16_t scaled_lambda_h, float scaling_factor)
{
    float scaling_factor_rev = 1 / scaling_factor;
    float sf_h = rn16f(scaling_factor);
    float lam = orc_h2f(scaled_lambda_h);
    float r_h = rn16f(r);
    float ph[128], qh[128];
    for (int e = 0; e < k; e++) { ph[e] = rn16f(p[e]); qh[e] = rn16f(q[e]); }
    float dot = dot_f16(k, ph, qh);
    float ruv = hmulf(sf_h, hsubf(r_h, dot));
    for (int e = 0; e < k; e++) {
        float gp = hsubf(hmulf(ruv, qh[e]), hmulf(lam, ph[e]));
        float gq = hsubf(hmulf(ruv, ph[e]), hmulf(lam, qh[e]));
        float a = scaling_factor_rev * gp; float b = lr * a;
        p[e] = p[e] + b;
        a = scaling_factor_rev * gq; b = lr * a;
        q[e] = q[e] + b;
    }
}

/* mascot_sgd_k128/k64_hogwild_kernel, the four precision cases:
 * half/half mascot_sgd_kernel.h:188-278, half/float :279-341, float/half :343-406, float/float :408-443. */
void orc_mascot_update(int k, void* pv, int user_prec, void* qv, int item_prec, float r, float lr, float lambda,
                       float* grad_p, float* grad_q, float* norm_p, float* norm_q)
{
    float pf[128] = {0}, qf[128] = {0}, gp[128], gq[128];
    if (!user_prec && !item_prec) {
        uint16_t* p = (uint16_t*)pv; uint16_t* q = (uint16_t*)qv;
        float lr_h = rn16f(lr), lam_h = rn16f(lambda), r_h = rn16f(r);       /* :79-80,189 */
        for (int e = 0; e < k; e++) { pf[e] = orc_h2f(p[e]); qf[e] = orc_h2f(q[e]); }
        float dot = dot_f16(k, pf, qf);
        float ruv = hsubf(r_h, dot);
        for (int e = 0; e < k; e++) {
            gp[e] = hsubf(hmulf(ruv, qf[e]), hmulf(lam_h, pf[e]));
            gq[e] = hsubf(hmulf(ruv, pf[e]), hmulf(lam_h, qf[e]));
            p[e] = orc_f2h(hfmaf_(lr_h, gp[e], pf[e]));
            q[e] = orc_f2h(hfmaf_(lr_h, gq[e], qf[e]));
        }
        if (grad_p) { for (int e = 0; e < k; e++) grad_p[e] = gp[e]; *norm_p = sumsq_f32(k, gp); }
        if (grad_q) { for (int e = 0; e < k; e++) grad_q[e] = gq[e]; *norm_q = sumsq_f32(k, gq); }
    } else if (!user_prec && item_prec) {
        uint16_t* p = (uint16_t*)pv; float* q = (float*)qv;
        for (int e = 0; e < k; e++) { pf[e] = orc_h2f(p[e]); qf[e] = q[e]; }
        float dot = dot_f32(k, pf, qf);
        float ruv = r - dot;
        for (int e = 0; e < k; e++) {
            float a = ruv * qf[e]; float b = lambda * pf[e]; gp[e] = a - b;
            p[e] = orc_f2h(fmaf(lr, gp[e], pf[e]));
            a = ruv * pf[e]; b = lambda * qf[e]; float c = a - b;
            q[e] = fmaf(lr, c, qf[e]);
        }
        if (grad_p) { for (int e = 0; e < k; e++) grad_p[e] = gp[e]; *norm_p = sumsq_f32(k, gp); }
    } else if (user_prec && !item_prec) {
        float* p = (float*)pv; uint16_t* q = (uint16_t*)qv;
        for (int e = 0; e < k; e++) { pf[e] = p[e]; qf[e] = orc_h2f(q[e]); }
        float dot = dot_f32(k, pf, qf);
        float ruv = r - dot;
        for (int e = 0; e < k; e++) {
            float a = ruv * pf[e]; float b = lambda * qf[e]; gq[e] = a - b;
            a = ruv * qf[e]; b = lambda * pf[e]; float c = a - b;
            p[e] = fmaf(lr, c, pf[e]);
            q[e] = orc_f2h(fmaf(lr, gq[e], qf[e]));
        }
        if (grad_q) { for (int e = 0; e < k; e++) grad_q[e] = gq[e]; *norm_q = sumsq_f32(k, gq); }
    } else {
        float* p = (float*)pv; float* q = (float*)qv;
        float dot = dot_f32(k, p, q);
        float ruv = r - dot;
        for (int e = 0; e < k; e++) {
            float pe = p[e], qe = q[e];
            float a = ruv * qe; float b = lambda * pe; float c = a - b;
            p[e] = fmaf(lr, c, pe);
            a = ruv * pe; b = lambda * qe; c = a - b;
            q[e] = fmaf(lr, c, qe);
        }
    }
}

/* ---- MuPPET ------------------------------------------------------------ */

static inline uint32_t f2u_sat(float f)   /* cvt.rzi.u32.f32: NaN and negatives -> 0, large -> UINT_MAX */
{
    if (!(f > 0.0f)) return 0u;
    if (f >= 4294967296.0f) return 0xffffffffu;
    return (uint32_t)f;
}
static inline int f2i_sat(float f)        /* cvt.rzi.s32.f32 */
{
    if (f != f) return 0;
    if (f >= 2147483648.0f) return INT_MAX;
    if (f <= -2147483648.0f) return INT_MIN;
    return (int)f;
}
static inline int f2i8_sat(float f)       /* float -> signed char; out-of-range values: parity unpinned */
{
    if (f != f) return 0;
    if (f > 127.0f) return 127;
    if (f < -128.0f) return -128;
    return (int)f;
}
/* Deliberate slips, for tests/test_oracle_mutants.py only: a build with -DORC_MUTATE=n (n = 1..8) puts one plausible
 * mistake into this file, and every one of them must make a pin in tests/test_oracle_pins.py fail -- the evidence that
 * the pins tell a right restatement from a nearly right one.  The normal build (ORC_MUTATE undefined) has none. */
#ifndef ORC_MUTATE
#define ORC_MUTATE 0
#endif
/* get_only_scaling_factor, muppet/muppet_sgd_kernel.h:7-18 (result then stored in an unsigned, :71-73,132-133) */
static uint32_t muppet_scale_index(unsigned bitwidth, float max_v, float min_v)
{
    if (max_v == 0 && min_v == 0) return f2u_sat(0.0f);
    float val = (float)(1 << (bitwidth - 1));
    float max_val = (val - 1) + (ORC_MUTATE == 3 ? -0.5f : 0.5f);     /* slip 3: the half step of the upper bound with the wrong sign */
    float min_val = (-val) - (ORC_MUTATE == 4 ? -0.5f : 0.5f);       /* slip 4: the half step of the lower bound with the wrong sign */
    float range_best = fminf(fabsf(max_val / max_v), fabsf(min_val / min_v));
#if ORC_MUTATE == 1
    return f2u_sat(ceilf(log2f(range_best)));                        /* slip 1: ceiling for floor */
#elif ORC_MUTATE == 2
    return f2u_sat(floorf(log2f(range_best)) + 1.0f);                /* slip 2: index one too large */
#else
    return f2u_sat(floorf(log2f(range_best)));
#endif
}
/* round-to-grid then binary16, muppet_sgd_kernel.h:174-181 */
static inline float muppet_grid_h(float v, float s, float s_rev) { float a = v * s; float b = roundf(a); float c = b * s_rev; return rn16f(c); }

/* muppet_sgd_k128/k64_hogwild_kernel body, muppet/muppet_sgd_kernel.h:110-285, _k64.h:60-203.
 * grad_sum (k floats) and norm receive the sampled statistics when non-NULL and both
 * precisions are below 32 bit (:266). */
void orc_muppet_update(int k, float* p, float* q, float r, float lr, float lambda,
                       int forward_bits, int backward_bits, float* grad_sum, float* norm)
{
    const int J = k / 32;
    float p_min = 0, p_max = 0, q_min = 0, q_max = 0, sp = 0, sq = 0, pred;
    if (forward_bits != 32) {
        p_min = p_max = p[0]; q_min = q_max = q[0];
        for (int e = 1; e < k; e++) { p_min = fminf(p_min, p[e]); p_max = fmaxf(p_max, p[e]); q_min = fminf(q_min, q[e]); q_max = fmaxf(q_max, q[e]); }
        sp = exp2f((float)muppet_scale_index((unsigned)forward_bits, p_max, p_min));
        sq = exp2f((float)muppet_scale_index((unsigned)forward_bits, q_max, q_min));
    }
    if (forward_bits == 8) {
        int x[LANES];
        for (int l = 0; l < LANES; l++) {
            int acc = 0;
            for (int j = 0; j < J; j++) acc += f2i8_sat(roundf(p[l + 32 * j] * sp)) * f2i8_sat(roundf(q[l + 32 * j] * sq));
            x[l] = acc;
        }
        int prod = tree_i(x);
        pred = prod / (sp * sq);
    } else if (forward_bits == 32) {
        pred = dot_f32(k, p, q);
    } else {
        float sp_rev = 1 / sp, sq_rev = 1 / sq;
        float x[LANES], y[LANES];
        for (int l = 0; l < LANES; l++) {
            /* half2 lanes: .x holds elements l (and l+64), .y holds l+32 (and l+96); :174-183 */
            float a = hmulf(muppet_grid_h(p[l], sp, sp_rev), muppet_grid_h(q[l], sq, sq_rev));
            float b = hmulf(muppet_grid_h(p[l + 32], sp, sp_rev), muppet_grid_h(q[l + 32], sq, sq_rev));
            if (k == 128) {
                float c = hmulf(muppet_grid_h(p[l + 64], sp, sp_rev), muppet_grid_h(q[l + 64], sq, sq_rev));
                float d = hmulf(muppet_grid_h(p[l + 96], sp, sp_rev), muppet_grid_h(q[l + 96], sq, sq_rev));
                a = haddf(a, c); b = haddf(b, d);
            }
            x[l] = a; y[l] = b;
        }
        float X = tree_h(x), Y = tree_h(y);
        pred = haddf(X, Y);
    }
    float ruv = r - pred;
    float sb = 0;
    if (backward_bits != 32) {
        float neg_lambda = -1 * lambda;
        float bmin = fminf(fminf(p_min, q_min), fminf(neg_lambda, ruv));
        float bmax = fmaxf(fmaxf(p_max, q_max), fmaxf(neg_lambda, ruv));
        sb = exp2f((float)muppet_scale_index((unsigned)backward_bits, bmax, bmin));
    }
    float gp[128], gq[128];
    if (backward_bits == 8) {
        float sq_rev = 1 / (sb * sb);
#if ORC_MUTATE == 5
        int ruv_i = f2i8_sat(ruv * sb);                              /* slip 5: the quantised error truncated, not rounded */
#else
        int ruv_i = f2i8_sat(roundf(ruv * sb));
#endif
        int lam_i = f2i8_sat(roundf(-1.0f * lambda * sb));
        for (int e = 0; e < k; e++) {
            int pi = f2i8_sat(roundf(p[e] * sb)), qi = f2i8_sat(roundf(q[e] * sb));
            gp[e] = (float)(qi * ruv_i + pi * lam_i) * sq_rev;      /* comp_grad_int8(q, p, ...) :20-23 */
            gq[e] = (float)(pi * ruv_i + qi * lam_i) * sq_rev;
        }
    } else if (backward_bits == 32) {
        for (int e = 0; e < k; e++) {
            float a = ruv * q[e]; float b = lambda * p[e]; gp[e] = a - b;
            a = ruv * p[e]; b = lambda * q[e]; gq[e] = a - b;
        }
    } else {
        float sb_rev = 1 / sb;
        float t_ruv = muppet_grid_h(ruv, sb, sb_rev);
        float t_lam = muppet_grid_h(-1 * lambda, sb, sb_rev);
        for (int e = 0; e < k; e++) {
            float ph = muppet_grid_h(p[e], sb, sb_rev), qh = muppet_grid_h(q[e], sb, sb_rev);
            gp[e] = haddf(hmulf(qh, t_ruv), hmulf(ph, t_lam));      /* comp_grad_fp16(q, p, ...) :25-32 */
            gq[e] = haddf(hmulf(ph, t_ruv), hmulf(qh, t_lam));
        }
    }
    for (int e = 0; e < k; e++) {
        float a = lr * gp[e]; float b = lr * gq[e];
        p[e] = p[e] + a; q[e] = q[e] + b;
    }
    if (grad_sum && forward_bits != 32 && backward_bits != 32) {
        /* :266-285: per lane norm_p + norm_q, tree; grad_sum[e] += gp[e] + gq[e] */
        float x[LANES];
        for (int l = 0; l < LANES; l++) {
            float np, nq;
            { float m0 = gp[l] * gp[l], m1 = gp[l + 32] * gp[l + 32]; np = m0 + m1;
              if (k == 128) { float m2 = gp[l + 64] * gp[l + 64], m3 = gp[l + 96] * gp[l + 96]; float b = m2 + m3; np = np + b; } }
            { float m0 = gq[l] * gq[l], m1 = gq[l + 32] * gq[l + 32]; nq = m0 + m1;
              if (k == 128) { float m2 = gq[l + 64] * gq[l + 64], m3 = gq[l + 96] * gq[l + 96]; float b = m2 + m3; nq = nq + b; } }
            x[l] = np + nq;
        }
        *norm += tree_f(x);
        for (int e = 0; e < k; e++) { float s = gp[e] + gq[e]; grad_sum[e] += s; }
    }
}

/* ---- AFP ---------------------------------------------------------------- */

/* get_only_scaling_factor_cvpr, afp/afp_sgd_kernel.h:8-16 */
static float afp_scale_index(unsigned bitwidth, float max_v)
{
    if (max_v == 0) return 0;
    float denom = exp2f((float)(bitwidth - 1)) - 1;
    float ratio = max_v / denom;
#if ORC_MUTATE == 6
    return fabsf(floorf(log2f(ratio)));                              /* slip 6: floor for ceiling */
#else
    return fabsf(ceilf(log2f(ratio)));
#endif
}
static inline float afp_grid(float v, float s, float s_rev) { float a = v * s; float b = roundf(a); return b * s_rev; }

/* QEM / QEM_64, afp_sgd_kernel.h:32-59, _k64.h:41-64: per-lane left-to-right sums, tree. */
static float afp_qem(int k, const float* v, float max_v)
{
    uint32_t idx = f2u_sat(afp_scale_index(8, max_v));
    float s = exp2f((float)idx), s_rev = 1 / s;
    float xq[LANES], x[LANES];
    for (int l = 0; l < LANES; l++) {
        float aq = fabsf(afp_grid(v[l], s, s_rev)); float a = fabsf(v[l]);
        for (int j = 1; j < k / 32; j++) { aq = aq + fabsf(afp_grid(v[l + 32 * j], s, s_rev)); a = a + fabsf(v[l + 32 * j]); }
        xq[l] = aq; x[l] = a;
    }
    float sum_q = tree_f(xq), sum = tree_f(x);
    float d = sum - sum_q; float e = d / sum;
    return log2f(fabsf(e) + 1);
}
/* QEM_BP / QEM_BP_64, afp_sgd_kernel.h:61-102, _k64.h:1-37: p..., q..., lambda, ruv per lane. */
static float afp_qem_bp(int k, const float* p, const float* q, float lambda, float ruv, float max_v)
{
    uint32_t idx = f2u_sat(afp_scale_index(8, max_v));
    float s = exp2f((float)idx), s_rev = 1 / s;
    float xq[LANES], x[LANES];
    for (int l = 0; l < LANES; l++) {
        float aq = fabsf(afp_grid(p[l], s, s_rev)); float a = fabsf(p[l]);
        for (int j = 1; j < k / 32; j++) { aq = aq + fabsf(afp_grid(p[l + 32 * j], s, s_rev)); a = a + fabsf(p[l + 32 * j]); }
        for (int j = 0; j < k / 32; j++) { aq = aq + fabsf(afp_grid(q[l + 32 * j], s, s_rev)); a = a + fabsf(q[l + 32 * j]); }
        aq = aq + fabsf(afp_grid(lambda, s, s_rev)); a = a + fabsf(lambda);
        aq = aq + fabsf(afp_grid(ruv, s, s_rev));    a = a + fabsf(ruv);
        xq[l] = aq; x[l] = a;
    }
    float sum_q = tree_f(xq), sum = tree_f(x);
    float d = sum - sum_q; float e = d / sum;
    return log2f(fabsf(e) + 1);
}
/* QPA, afp_sgd_kernel.h:104-125 */
static orc_afp_qparams afp_qpa(float diff, float range, float prev_mov_avg_range)
{
    orc_afp_qparams params;
    float threshold = 0.0005f, alpha = 0.04f, beta = 0.1f, delta = 100, gamma = 2;
    if (diff <= threshold) { params.r = f2i_sat(fabsf(ceilf(log2f(range / (exp2f((float)(8 - 1)) - 1))))); params.n = 8; }
    else { params.r = f2i_sat(fabsf(ceilf(log2f(range / (exp2f((float)(16 - 1)) - 1))))); params.n = 16; }
    float a = alpha * range; float b = (1.0f - alpha) * prev_mov_avg_range;
    params.mov_avg_range = a + b;
    float i1 = delta * diff; i1 = i1 * diff;
    float i2 = fabsf(params.mov_avg_range - prev_mov_avg_range);
    float t = beta / fmaxf(i1, i2);
    params.itv = f2i_sat(t - gamma);
    return params;
}
void orc_afp_state_init(orc_afp_state* s)
{
    s->user.r = s->user.n = s->user.itv = 0; s->user.mov_avg_range = 0;
    s->item = s->user; s->backward = s->user;
    s->update_user_params_iter = s->update_item_params_iter = s->update_backward_iter = s->cur_iter = 0;
    s->scaling_factor_p = s->scaling_factor_q = s->scaling_factor_back_prop = 0;
}
static inline int afp_sat8(float t) { return (int)(t > 127.0f ? 127.0f : (t < -128.0f) ? -128.0f : t); }

/* afp_sgd_k128/k64_hogwild_kernel body, afp/afp_sgd_kernel.h:180-374, _k64.h:118-275 */
void orc_afp_update(int k, orc_afp_state* st, float* p, float* q, float r, float lr, float lambda,
                    int epoch, int initialization_threshold)
{
    const int J = k / 32;
    float p_abs_max = 0, q_abs_max = 0;
    for (int e = 0; e < k; e++) { p_abs_max = fmaxf(p_abs_max, fabsf(p[e])); q_abs_max = fmaxf(q_abs_max, fabsf(q[e])); }
    if (st->cur_iter == st->update_user_params_iter) {
        float diff = afp_qem(k, p, p_abs_max);
        if (st->cur_iter == 0) st->user.mov_avg_range = p_abs_max;
        st->user = afp_qpa(diff, p_abs_max, st->user.mov_avg_range);
        st->scaling_factor_p = exp2f((float)st->user.r);
        if (epoch == 0 && st->cur_iter < initialization_threshold) st->user.itv = 1;
        st->update_user_params_iter += st->user.itv;
    }
    if (st->cur_iter == st->update_item_params_iter) {
        float diff = afp_qem(k, q, q_abs_max);
        if (st->cur_iter == 0) st->item.mov_avg_range = q_abs_max;
        st->item = afp_qpa(diff, q_abs_max, st->item.mov_avg_range);
        st->scaling_factor_q = exp2f((float)st->item.r);
        if (epoch == 0 && st->cur_iter < initialization_threshold) st->item.itv = 1;
        st->update_item_params_iter += st->item.itv;
    }
    float sp = st->scaling_factor_p, sq = st->scaling_factor_q, pred;
    if (st->user.n == 8 && st->item.n == 8) {
        int x[LANES];
        for (int l = 0; l < LANES; l++) {
            int acc = 0;
            for (int j = 0; j < J; j++) acc += afp_sat8(roundf(p[l + 32 * j] * sp)) * afp_sat8(roundf(q[l + 32 * j] * sq));
            x[l] = acc;
        }
        int prod = tree_i(x);
        pred = prod / (sp * sq);
    } else {
        float sp_rev = 1 / sp, sq_rev = 1 / sq;
        float x[LANES], y[LANES];
        for (int l = 0; l < LANES; l++) {
            float a = hmulf(rn16f(afp_grid(p[l], sp, sp_rev)), rn16f(afp_grid(q[l], sq, sq_rev)));
            float b = hmulf(rn16f(afp_grid(p[l + 32], sp, sp_rev)), rn16f(afp_grid(q[l + 32], sq, sq_rev)));
            if (k == 128) {
                float c = hmulf(rn16f(afp_grid(p[l + 64], sp, sp_rev)), rn16f(afp_grid(q[l + 64], sq, sq_rev)));
                float d = hmulf(rn16f(afp_grid(p[l + 96], sp, sp_rev)), rn16f(afp_grid(q[l + 96], sq, sq_rev)));
                a = haddf(a, c); b = haddf(b, d);
            }
            x[l] = a; y[l] = b;
        }
        float X = tree_h(x), Y = tree_h(y);
        pred = haddf(X, Y);
    }
    float ruv = r - pred;
    if (st->cur_iter == st->update_backward_iter) {
        float pq_max = fmaxf(p_abs_max, q_abs_max);
        pq_max = fmaxf(fmaxf(pq_max, fabsf(lambda)), fabsf(ruv));
        float diff = afp_qem_bp(k, p, q, lambda, ruv, pq_max);
        if (st->cur_iter == 0) st->backward.mov_avg_range = pq_max;
        st->backward = afp_qpa(diff, pq_max, st->backward.mov_avg_range);
        st->scaling_factor_back_prop = exp2f((float)st->backward.r);
        if (epoch == 0 && st->cur_iter < initialization_threshold) st->backward.itv = 1;
        st->update_backward_iter += st->backward.itv;
    }
    float sb = st->scaling_factor_back_prop;
    float gp[128], gq[128];
    if (st->backward.n == 8) {
        int lam_i = afp_sat8(roundf(-1.0f * lambda * sb));
        int ruv_i = afp_sat8(roundf(ruv * sb));
        float sq_rev = 1 / (sb * sb);
        for (int e = 0; e < k; e++) {
            int pi = afp_sat8(roundf(p[e] * sb)), qi = afp_sat8(roundf(q[e] * sb));
            gp[e] = (float)(qi * ruv_i + pi * lam_i) * sq_rev;       /* comp_grad_int8_cvpr(q, p, ...) :18-21 */
            gq[e] = (float)(pi * ruv_i + qi * lam_i) * sq_rev;
        }
    } else {
        float sb_rev = 1 / sb;
        float t_ruv = rn16f(afp_grid(ruv, sb, sb_rev));
        float t_lam = rn16f(afp_grid(-1.0f * lambda, sb, sb_rev));
        for (int e = 0; e < k; e++) {
            float ph = rn16f(afp_grid(p[e], sb, sb_rev)), qh = rn16f(afp_grid(q[e], sb, sb_rev));
            gp[e] = haddf(hmulf(qh, t_ruv), hmulf(ph, t_lam));       /* comp_grad_fp16_cvpr :23-30 */
            gq[e] = haddf(hmulf(ph, t_ruv), hmulf(qh, t_lam));
        }
    }
    for (int e = 0; e < k; e++) {
        float a = lr * gp[e]; float b = lr * gq[e];
        p[e] = p[e] + a; q[e] = q[e] + b;
    }
    st->cur_iter += 1;
}

/* ------------------------------------------------------------------------ */
/* whole launches                                                            */
/* ------------------------------------------------------------------------ */

static inline uint32_t win_start(const uint32_t* window_start, uint64_t seed, uint32_t epoch,
                                 uint32_t num_workers, uint32_t wid, uint32_t ite, uint32_t nnz)
{
    if (window_start) return window_start[(uint64_t)ite * num_workers + wid] % nnz;
    return orc_window_start(seed, epoch, wid, ite, nnz);
}

/* The launch loops below restate sgd/sgd_kernel.h:14-37: every worker (warp) runs
 * update_count windows of update_vector_size consecutive ratings, offset = (start+i) % nnz.
 * threads <= 1: deterministic order, window-major then worker.  threads > 1: workers are
 * spread over OpenMP threads and race on P/Q without locks (Hogwild), as the warps do. */
#define FOR_EACH_UPDATE_SEQ(...)                                                               \
    for (uint32_t ite = 0; ite < update_count; ite++)                                          \
        for (uint32_t wid = 0; wid < num_workers; wid++) {                                     \
            uint32_t start = win_start(window_start, seed, epoch, num_workers, wid, ite, nnz); \
            for (uint32_t i = 0; i < update_vector_size; i++) {                                \
                const orc_node* nd = &R[(uint32_t)(((uint64_t)start + i) % nnz)];              \
                uint32_t processed_cnt = ite * update_vector_size + i; (void)processed_cnt;    \
                __VA_ARGS__                                                                    \
            }                                                                                  \
        }
#define FOR_EACH_UPDATE_PAR(...)                                                               \
    _Pragma("omp parallel for schedule(dynamic, 1) num_threads(threads)")                      \
    for (uint32_t wid = 0; wid < num_workers; wid++)                                           \
        for (uint32_t ite = 0; ite < update_count; ite++) {                                    \
            uint32_t start = win_start(window_start, seed, epoch, num_workers, wid, ite, nnz); \
            for (uint32_t i = 0; i < update_vector_size; i++) {                                \
                const orc_node* nd = &R[(uint32_t)(((uint64_t)start + i) % nnz)];              \
                uint32_t processed_cnt = ite * update_vector_size + i; (void)processed_cnt;    \
                __VA_ARGS__                                                                    \
            }                                                                                  \
        }

void orc_sgd_epoch(int k, const orc_node* R, uint32_t nnz, float* P, float* Q,
                   uint32_t num_workers, uint32_t update_count, uint32_t update_vector_size,
                   float lr, float lambda, uint64_t seed, uint32_t epoch, const uint32_t* window_start, int threads)
{
    if (threads <= 1) { FOR_EACH_UPDATE_SEQ(orc_sgd_update(k, P + (size_t)nd->u * k, Q + (size_t)nd->i * k, nd->r, lr, lambda);) }
    else { FOR_EACH_UPDATE_PAR(orc_sgd_update(k, P + (size_t)nd->u * k, Q + (size_t)nd->i * k, nd->r, lr, lambda);) }
}

void orc_mem_quant_epoch(int k, const orc_node* R, uint32_t nnz, uint16_t* P, uint16_t* Q,
                         uint32_t num_workers, uint32_t update_count, uint32_t update_vector_size,
                         float lr, float lambda, uint64_t seed, uint32_t epoch, const uint32_t* window_start, int threads)
{
    if (threads <= 1) { FOR_EACH_UPDATE_SEQ(orc_mem_quant_update(k, P + (size_t)nd->u * k, Q + (size_t)nd->i * k, nd->r, lr, lambda);) }
    else { FOR_EACH_UPDATE_PAR(orc_mem_quant_update(k, P + (size_t)nd->u * k, Q + (size_t)nd->i * k, nd->r, lr, lambda);) }
}

void orc_mpt_epoch(int k, const orc_node* R, uint32_t nnz, float* P, float* Q,
                   uint32_t num_workers, uint32_t update_count, uint32_t update_vector_size,
                   float lr, float lambda, float scaling_factor, uint64_t seed, uint32_t epoch,
                   const uint32_t* window_start, int threads)
{
    uint16_t lam_h = orc_f2h(lambda * scaling_factor);          /* mf_methods.cu:765 */
    if (threads <= 1) { FOR_EACH_UPDATE_SEQ(orc_mpt_update(k, P + (size_t)nd->u * k, Q + (size_t)nd->i * k, nd->r, lr, lam_h, scaling_factor);) }
    else { FOR_EACH_UPDATE_PAR(orc_mpt_update(k, P + (size_t)nd->u * k, Q + (size_t)nd->i * k, nd->r, lr, lam_h, scaling_factor);) }
}

void orc_muppet_epoch(int k, const orc_node* R, uint32_t nnz, float* P, float* Q,
                      uint32_t num_workers, uint32_t update_count, uint32_t update_vector_size,
                      float lr, float lambda, uint32_t first_sample_rating_idx,
                      float* sum_updated_val, float* sum_norms, int forward_bits, int backward_bits,
                      uint64_t seed, uint32_t epoch, const uint32_t* window_start, int threads)
{
    for (uint32_t w = 0; w < num_workers; w++) sum_norms[w] = 0;     /* sum_norms_reg = 0, muppet_sgd_kernel.h:75,288 */
    if (threads > 1) {
        /* Hogwild over host threads: workers race on the rows; a worker's norm sum is its own, the sampled gradient
         * sums are kept per thread and folded at the end (the kernel adds them with atomics, in any order) */
        #pragma omp parallel num_threads(threads)
        {
            float* mine = (float*)calloc((size_t)k, sizeof(float));
            #pragma omp for schedule(dynamic, 1)
            for (uint32_t wid = 0; wid < num_workers; wid++)
                for (uint32_t ite = 0; ite < update_count; ite++) {
                    uint32_t start = win_start(window_start, seed, epoch, num_workers, wid, ite, nnz);
                    for (uint32_t i = 0; i < update_vector_size; i++) {
                        const orc_node* nd = &R[(uint32_t)(((uint64_t)start + i) % nnz)];
                        int sample = ite * update_vector_size + i >= first_sample_rating_idx;
                        orc_muppet_update(k, P + (size_t)nd->u * k, Q + (size_t)nd->i * k, nd->r, lr, lambda, forward_bits, backward_bits,
                                          sample ? mine : NULL, sample ? &sum_norms[wid] : NULL);
                    }
                }
            #pragma omp critical
            for (int e = 0; e < k; e++) sum_updated_val[e] += mine[e];
            free(mine);
        }
        return;
    }
    FOR_EACH_UPDATE_SEQ(
        int sample = processed_cnt >= first_sample_rating_idx;
        orc_muppet_update(k, P + (size_t)nd->u * k, Q + (size_t)nd->i * k, nd->r, lr, lambda, forward_bits, backward_bits,
                          sample ? sum_updated_val : NULL, sample ? &sum_norms[wid] : NULL);
    )
}

void orc_afp_epoch(int k, const orc_node* R, uint32_t nnz, float* P, float* Q,
                   uint32_t num_workers, uint32_t update_count, uint32_t update_vector_size,
                   float lr, float lambda, int epoch_arg,
                   uint64_t seed, uint32_t epoch, const uint32_t* window_start, int threads)
{
    orc_afp_state* st = (orc_afp_state*)malloc(sizeof(orc_afp_state) * num_workers);
    for (uint32_t w = 0; w < num_workers; w++) orc_afp_state_init(&st[w]);
    int init_thr = f2i_sat((float)(update_count * update_vector_size) / 10.0f);     /* afp_sgd_kernel.h:145 */
    if (threads > 1) {      /* Hogwild over host threads: the quantiser state belongs to the worker, the rows are raced on */
        FOR_EACH_UPDATE_PAR(
            orc_afp_update(k, &st[wid], P + (size_t)nd->u * k, Q + (size_t)nd->i * k, nd->r, lr, lambda, epoch_arg, init_thr);
        )
        free(st);
        return;
    }
    FOR_EACH_UPDATE_SEQ(
        orc_afp_update(k, &st[wid], P + (size_t)nd->u * k, Q + (size_t)nd->i * k, nd->r, lr, lambda, epoch_arg, init_thr);
    )
    free(st);
}

static inline void* group_row(void** group_ptr, const uint32_t* end_idx, const uint8_t* prec, uint32_t groups,
                              uint32_t idx, int k, uint32_t* g_out, int* prec_out)
{
    uint32_t g, row;
    orc_group_lookup(idx, end_idx, groups, &g, &row);
    *g_out = g; *prec_out = prec[g];
    if (prec[g]) return (float*)group_ptr[g] + (size_t)row * k;
    return (uint16_t*)group_ptr[g] + (size_t)row * k;
}

void orc_mascot_epoch(int k, const orc_node* R, uint32_t nnz, void** user_group_ptr, void** item_group_ptr,
                      const uint32_t* user_end_idx, const uint32_t* item_end_idx,
                      const uint8_t* user_prec, const uint8_t* item_prec, uint32_t user_groups, uint32_t item_groups,
                      uint32_t num_workers, uint32_t update_count, uint32_t update_vector_size,
                      float lr, float lambda, uint32_t first_sample_rating_idx,
                      float* grad_sum_norm_p, float* grad_sum_norm_q, float* norm_sum_p, float* norm_sum_q,
                      uint64_t seed, uint32_t epoch, const uint32_t* window_start, int threads)
{
    uint32_t total = update_count * update_vector_size;
    int sampling = first_sample_rating_idx < total && grad_sum_norm_p && grad_sum_norm_q;
    if (threads > 1 && !sampling) {
        FOR_EACH_UPDATE_PAR(
            uint32_t ug; uint32_t ig; int up; int ip;
            void* prow = group_row(user_group_ptr, user_end_idx, user_prec, user_groups, nd->u, k, &ug, &up);
            void* qrow = group_row(item_group_ptr, item_end_idx, item_prec, item_groups, nd->i, k, &ig, &ip);
            orc_mascot_update(k, prow, up, qrow, ip, nd->r, lr, lambda, NULL, NULL, NULL, NULL);
        )
        return;
    }
    double* gsp = NULL; double* gsq = NULL; double* nsp = NULL; double* nsq = NULL;
    if (sampling) {
        gsp = (double*)calloc((size_t)user_groups * k, sizeof(double)); gsq = (double*)calloc((size_t)item_groups * k, sizeof(double));
        nsp = (double*)calloc(user_groups, sizeof(double)); nsq = (double*)calloc(item_groups, sizeof(double));
    }
    if (threads > 1) {
        /* a check epoch as a Hogwild loop: the workers race on the rows as in the plain epochs; the sampled sums are
         * kept per thread in binary64 and folded at the end, so they do not depend on the interleaving beyond the
         * rows the gradients were computed from */
        #pragma omp parallel num_threads(threads)
        {
            double* tgsp = (double*)calloc((size_t)user_groups * k, sizeof(double)); double* tgsq = (double*)calloc((size_t)item_groups * k, sizeof(double));
            double* tnsp = (double*)calloc(user_groups, sizeof(double)); double* tnsq = (double*)calloc(item_groups, sizeof(double));
            float tgp[128], tgq[128];
            #pragma omp for schedule(dynamic, 1)
            for (uint32_t wid = 0; wid < num_workers; wid++)
                for (uint32_t ite = 0; ite < update_count; ite++) {
                    uint32_t start = win_start(window_start, seed, epoch, num_workers, wid, ite, nnz);
                    for (uint32_t i = 0; i < update_vector_size; i++) {
                        const orc_node* nd = &R[(uint32_t)(((uint64_t)start + i) % nnz)];
                        uint32_t processed_cnt = ite * update_vector_size + i;
                        uint32_t ug; uint32_t ig; int up; int ip; float np = 0; float nq = 0;
                        void* prow = group_row(user_group_ptr, user_end_idx, user_prec, user_groups, nd->u, k, &ug, &up);
                        void* qrow = group_row(item_group_ptr, item_end_idx, item_prec, item_groups, nd->i, k, &ig, &ip);
                        int sample = processed_cnt >= first_sample_rating_idx;
                        orc_mascot_update(k, prow, up, qrow, ip, nd->r, lr, lambda, sample ? tgp : NULL, sample ? tgq : NULL, &np, &nq);
                        if (sample) {
                            if (!up) { tnsp[ug] += np; for (int e = 0; e < k; e++) tgsp[(size_t)ug * k + e] += tgp[e]; }
                            if (!ip) { tnsq[ig] += nq; for (int e = 0; e < k; e++) tgsq[(size_t)ig * k + e] += tgq[e]; }
                        }
                    }
                }
            #pragma omp critical
            {
                for (size_t i = 0; i < (size_t)user_groups * k; i++) gsp[i] += tgsp[i];
                for (size_t i = 0; i < (size_t)item_groups * k; i++) gsq[i] += tgsq[i];
                for (uint32_t g = 0; g < user_groups; g++) nsp[g] += tnsp[g];
                for (uint32_t g = 0; g < item_groups; g++) nsq[g] += tnsq[g];
            }
            free(tgsp); free(tgsq); free(tnsp); free(tnsq);
        }
        for (size_t i = 0; i < (size_t)user_groups * k; i++) grad_sum_norm_p[i] += (float)gsp[i];
        for (size_t i = 0; i < (size_t)item_groups * k; i++) grad_sum_norm_q[i] += (float)gsq[i];
        for (uint32_t g = 0; g < user_groups; g++) norm_sum_p[g] += (float)nsp[g];
        for (uint32_t g = 0; g < item_groups; g++) norm_sum_q[g] += (float)nsq[g];
        free(gsp); free(gsq); free(nsp); free(nsq);
        return;
    }
    float gp[128], gq[128];
    FOR_EACH_UPDATE_SEQ(
        uint32_t ug; uint32_t ig; int up; int ip; float np = 0; float nq = 0;
        void* prow = group_row(user_group_ptr, user_end_idx, user_prec, user_groups, nd->u, k, &ug, &up);
        void* qrow = group_row(item_group_ptr, item_end_idx, item_prec, item_groups, nd->i, k, &ig, &ip);
        int sample = sampling && processed_cnt >= first_sample_rating_idx;
        orc_mascot_update(k, prow, up, qrow, ip, nd->r, lr, lambda, sample ? gp : NULL, sample ? gq : NULL, &np, &nq);
        if (sample) {
            if (!up) { nsp[ug] += np; for (int e = 0; e < k; e++) gsp[(size_t)ug * k + e] += gp[e]; }
            if (!ip) { nsq[ig] += nq; for (int e = 0; e < k; e++) gsq[(size_t)ig * k + e] += gq[e]; }
        }
    )
    if (sampling) {
        for (size_t i = 0; i < (size_t)user_groups * k; i++) grad_sum_norm_p[i] += (float)gsp[i];
        for (size_t i = 0; i < (size_t)item_groups * k; i++) grad_sum_norm_q[i] += (float)gsq[i];
        for (uint32_t g = 0; g < user_groups; g++) norm_sum_p[g] += (float)nsp[g];
        for (uint32_t g = 0; g < item_groups; g++) norm_sum_q[g] += (float)nsq[g];
        free(gsp); free(gsq); free(nsp); free(nsq);
    }
}

/* ------------------------------------------------------------------------ */
/* evaluation and g-switching                                                */
/* ------------------------------------------------------------------------ */

/* gpu_test_rmse, rmse.h:57-96,183-188: sqrt(sum (r - p.q)^2 / test_n); evaluated in binary64 here. */
double orc_rmse(int k, const orc_node* test, uint64_t test_n, const float* P, const float* Q)
{
    double sum = 0;
    for (uint64_t i = 0; i < test_n; i++) {
        const float* p = P + (size_t)test[i].u * k; const float* q = Q + (size_t)test[i].i * k;
        double dot = 0;
        for (int e = 0; e < k; e++) dot += (double)p[e] * (double)q[e];
        double d = (double)test[i].r - dot;
        sum += d * d;
    }
    return sqrt(sum / (double)test_n);
}

/* Same figure straight from grouped storage (what mf_methods.cu:249-313 assembles on the
 * host before calling gpu_test_rmse): binary16 rows are widened exactly. */
double orc_rmse_grouped(int k, const orc_node* test, uint64_t test_n, void** user_group_ptr, void** item_group_ptr,
                        const uint32_t* user_end_idx, const uint32_t* item_end_idx,
                        const uint8_t* user_prec, const uint8_t* item_prec, uint32_t user_groups, uint32_t item_groups)
{
    double sum = 0;
    for (uint64_t i = 0; i < test_n; i++) {
        uint32_t ug, ig; int up, ip;
        void* prow = group_row(user_group_ptr, user_end_idx, user_prec, user_groups, test[i].u, k, &ug, &up);
        void* qrow = group_row(item_group_ptr, item_end_idx, item_prec, item_groups, test[i].i, k, &ig, &ip);
        double dot = 0;
        for (int e = 0; e < k; e++) {
            double pe = up ? (double)((float*)prow)[e] : (double)orc_h2f(((uint16_t*)prow)[e]);
            double qe = ip ? (double)((float*)qrow)[e] : (double)orc_h2f(((uint16_t*)qrow)[e]);
            dot += pe * qe;
        }
        double d = (double)test[i].r - dot;
        sum += d * d;
    }
    return sqrt(sum / (double)test_n);
}

/* mf_methods.cu:327-345: error[g] = (sum_k grad_sum[g,k]^2) / (sum_blocks norm_sum[g,b]) / initial[g];
 * -1 for binary32 groups.  norm_sum is [groups][norm_blocks]. */
void orc_group_error(int k, uint32_t groups, const float* grad_sum_norm, const float* norm_sum, uint32_t norm_blocks,
                     const uint8_t* prec, const float* initial_error, float* error_out)
{
    for (uint32_t g = 0; g < groups; g++) {
        if (prec[g] == 0) {
            float acc = 0, nacc = 0;
            for (int e = 0; e < k; e++) acc += powf(grad_sum_norm[(size_t)g * k + e], 2);
            for (uint32_t b = 0; b < norm_blocks; b++) nacc += norm_sum[(size_t)g * norm_blocks + b];
            float err = acc / (float)nacc;
            error_out[g] = err / initial_error[g];
        } else error_out[g] = -1;
    }
}

/* MuPPET precision ladder, mf_methods.cu:659-697.  Arrays hold the per-epoch history up to
 * epoch e inclusive.  Returns 1 when the bit width moves up one rung. */
int orc_muppet_ladder_step(int k, int e, int* switched_epoch, int* precision_idx, float* max_grad_diversity,
                           int* violation_times, const float* sum_norms_epoch, const float* sum_updated_val_epoch)
{
    const int resolution_size = 3, gamma = 1;
    const float alpha = 1.0f, beta = 1.5f, lambda_for_threshold = 0.3f;
    float decaying_threshold = (float)(alpha + (beta * exp(-1 * lambda_for_threshold * (e))));
    if (ORC_MUTATE == 7) decaying_threshold *= 0.9f;                 /* slip 7: a threshold 10 % lower */
    if (e - *switched_epoch >= resolution_size) {
        float sum_norms_resolution = 0, sum_updated_val_norm = 0;
        float acc[128];
        for (int i = 0; i < k; i++) acc[i] = 0;
        for (int wi = e - resolution_size + 1 + (ORC_MUTATE == 8 ? 1 : 0); wi <= e; wi++) {      /* slip 8: a window one epoch short */
            sum_norms_resolution += sum_norms_epoch[wi];
            for (int i = 0; i < k; i++) acc[i] += sum_updated_val_epoch[wi * k + i];
        }
        for (int i = 0; i < k; i++) sum_updated_val_norm += powf(acc[i], 2);
        float div = sum_norms_resolution / sum_updated_val_norm;
        *max_grad_diversity = *max_grad_diversity < div ? div : *max_grad_diversity;
        float ratio = *max_grad_diversity / div;
        if (ratio > decaying_threshold && ++(*violation_times) == gamma) {
            (*precision_idx)++;
            *switched_epoch = e;
            *max_grad_diversity = -1.f;
            *violation_times = 0;
            return 1;
        }
    }
    return 0;
}
