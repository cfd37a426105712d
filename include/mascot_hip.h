/*
 * libmascot_hip -- C ABI of the MI355X (gfx950) matrix-factorization training path.
 *
 * Every entry point below stands in for one kernel launch (or one host driver) of
 * Yujaeseo/ICDM-2021_MASCOT; the comment on each names the reference file:line it
 * replaces (paths relative to the reference checkout).  Conventions:
 *   - plain C types only; all pointers are DEVICE pointers unless a parameter is
 *     documented as host memory; the caller owns every buffer;
 *   - `stream` is a hipStream_t passed as void* (NULL = default stream); launches are
 *     asynchronous, nothing here synchronises unless documented;
 *   - return value: 0 on success, a positive hipError_t when the HIP runtime refused
 *     something, MF_EINVAL (-1) for arguments the kernels cannot take (the call then
 *     launches nothing); mf_last_error() gives the message of the last failure on the
 *     calling thread;
 *   - a "worker" is one 64-lane wavefront processing one rating at a time, the
 *     counterpart of the reference's 32-lane warp (`-wg`); k is 64 or 128.
 *
 * Scheduling.  A launch runs `num_workers` workers; each runs `update_count` windows of
 * `update_vector_size` consecutive ratings (offset = (start + i) % nnz), as
 * sgd/sgd_kernel.h:14-37 does.  The reference draws `start` from cuRAND states seeded
 * with clock() (model_init.cu:12-17); here it is
 *     start = window_start[ite * num_workers + worker] % nnz     if window_start != NULL
 *     start = counter_rng(seed, epoch, worker, ite) * nnz        otherwise
 * so that a run is reproducible and a caller (or a test) can pin the schedule.
 */
#ifndef MASCOT_HIP_H
#define MASCOT_HIP_H
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MF_OK 0
#define MF_EINVAL (-1)

/* COO rating triple, common_struct.h:8-12 (12 bytes, array of structures). */
typedef struct { float r; uint32_t u; uint32_t i; } mf_node;

int mf_version(void);
const char* mf_last_error(void);
/* How the update kernels read and write P/Q rows (process-wide, takes effect at the next launch):
 *   1 (default)  device-coherent: every row store writes through the per-XCD L2 to the memory side and drops the
 *                copies other L2s hold (agent-scope relaxed atomic stores; loads stay ordinary cached loads),
 *                so a worker sees the latest row any other worker stored -- the semantics the reference
 *                gets from a GPU with one L2.  All stores to one row serialise at the memory side, which
 *                bounds the epoch when a single row takes percents of all ratings (see
 *                mf_set_hot_row_thinning for what mf_train does about that).
 *   0            cached: ordinary write-back stores; each of the 8 XCDs works on its own L2-resident copy
 *                of a hot row until it is evicted, copies are merged last-writer-wins.
 * No counterpart in the reference (one L2, nothing to choose).  mf_train picks per run, see there. */
int mf_set_row_coherence(int coherent);
int mf_get_row_coherence(void);
/* Cuts every fp32-SGD / MPT / MASCOT update call into `splits` consecutive kernel launches (each worker's
 * windows are divided evenly).  A kernel boundary writes back and invalidates the per-XCD L2s, so with
 * cached row accesses the XCDs' copies of hot rows are reconciled `splits` times per epoch instead of once.
 * Default 1.  No counterpart in the reference. */
int mf_set_epoch_splits(uint32_t splits);
uint32_t mf_get_epoch_splits(void);
/* Hot rows for the update calls (process-wide, both NULL = off, the default).
 * user_keep[row], item_keep[row] are device arrays of bytes indexed like P and Q rows (for MASCOT: sorted row
 * order).  255 marks an ordinary row.  A row with a smaller value is a hot row, meant for rows that have several
 * updates in flight at any time: (1) a rating updates the row with probability (keep+1)/255 and otherwise only
 * reads it for the other side's update; (2) an update that is carried out adds its change to the row in memory
 * (an atomic add per element) instead of storing the new row, so concurrent updates add up where
 * last-writer-wins would keep one of them.  The sum of C stale gradients is a step C times as long, which is why
 * rows with many updates in flight are thinned.  mf_train builds the tables from the rating counts when
 * mf_params.hot_row_inflight > 0.  No counterpart in the reference.  The tables must
 * stay valid while launches that use them are in flight. */
int mf_set_hot_row_thinning(const uint8_t* user_keep, const uint8_t* item_keep);
/* The table mf_train builds for one side (host arrays): counts[row] ratings of `n` fall on the row; with
 * F = min(num_workers, 8192) * 4 updates in flight on the device a row has about F * counts[row] / n of them.
 * Rows with at most one stay ordinary (255); the others become hot rows, kept with probability
 * min(1, inflight_cap / in flight): table value clip(floor(keep * 255) - 1, 0, 254). */
int mf_hot_row_table(const uint32_t* counts, uint32_t rows, uint32_t n, uint32_t num_workers, float inflight_cap, uint8_t* table);
/* Seeded synthetic ratings (no counterpart in the reference, whose data sets are downloaded): users and items are
 * drawn independently from Zipf(alpha) over a random permutation of the ids; a rating is
 * clamp(round_to_step(U_u . V_i + mean + noise * N(0,1)), lo, hi) with rank-`rank` factors U, V ~ N(0, 0.5^2), or,
 * with bimodal != 0, clamp(round(m + noise * N(0,1)), lo, hi) * 0.04 + 1 with m = 20 or 80 (the 0..100 ratings of
 * BASELINE.json's fifth configuration mapped like the reference maps its 0..100 data set, io_utils.h:75).  Rating j
 * depends on (seed, j) only, so any range [first, first + count) of the stream can be generated on its own; the
 * command line takes the first n_train ratings for training and the next n_test for the test set. */
typedef struct {
    uint32_t n_users, n_items;
    uint64_t n_train, n_test;
    float user_alpha, item_alpha;
    uint32_t rank;
    float noise, mean, step, lo, hi;
    uint32_t bimodal;
} mf_synth_config;
/* The synthetic stand-ins of BASELINE.json's configurations 1..5; MF_EINVAL for any other number. */
int mf_synth_baseline_config(int config, mf_synth_config* out);
/* Writes ratings [first, first + count) of the stream to the device array `out` (ids are dense, 0-based).
 * Builds its tables (two CDFs, two permutations, the factors) on every call and frees them before returning, so it
 * synchronises the stream. */
int mf_generate_ratings(const mf_synth_config* cfg, uint64_t seed, uint64_t first, uint64_t count, mf_node* out, void* stream);
/* The same into a host array (allocates, generates on the default stream, copies back, frees). */
int mf_generate_ratings_host(const mf_synth_config* cfg, uint64_t seed, uint64_t first, uint64_t count, mf_node* host_out);
/* Measurement aid, no counterpart in the reference: the memory traffic of one epoch of updates without the
 * arithmetic.  Worker w (one wavefront) walks ratings [w*ceil(n/W), (w+1)*ceil(n/W)); per rating it reads row u of p
 * and row i of q (row_bytes = 128, 256 or 512 bytes each: k = 64 binary16, k = 128 binary16 / k = 64 binary32,
 * k = 128 binary32) and writes both back unchanged, with the store policy of mf_set_row_coherence's value
 * `coherent`.  With keep tables (as for mf_set_hot_row_thinning; both or neither) a thinned update only reads its
 * row; an update of a hot row that is kept is a store here as well.  p and q keep their contents (writes of other
 * code that race with the probe may be lost).  The time of this launch is what the memory system sustains for the
 * sequence of addresses and the write policy of an epoch; bench.py reports the update kernel's time beside it. */
int mf_row_traffic_probe(const mf_node* R, uint32_t n, void* p, void* q, uint32_t row_bytes, uint32_t num_workers,
                         const uint8_t* user_keep, const uint8_t* item_keep, uint64_t seed, int coherent, void* stream);
/* Number of per-block columns mf_mascot_sgd_hogwild writes into norm_sum_p / norm_sum_q
 * (the reference's `block_num`, mf_methods.cu:109). */
uint32_t mf_mascot_norm_blocks(uint32_t num_workers);
/* Host-side closed forms of the schedule (mf_methods.cu:94-111,170-175). */
uint32_t mf_update_count(uint32_t n, uint32_t num_workers, uint32_t update_vector_size);
/* Worker count mf_train uses for mf_params.num_workers == 0: n / 16384 (about 128 windows per worker), a multiple
 * of 4, between 16 and 6144.  The updates in flight grow with the workers and so does the distance to a sequential
 * run; the reference's fixed default (2048, main.cu:28) suits neither 400k nor 100M ratings on this GPU. */
uint32_t mf_auto_workers(uint32_t n);
uint32_t mf_first_sample_rating_idx(uint32_t e, uint32_t interval, uint32_t epochs, uint32_t update_count,
                                    uint32_t update_vector_size, float sample_ratio);
float mf_lr_schedule(float lr, float decay, uint32_t e);
/* The counter-based window start the kernels use when window_start == NULL (host twin). */
uint32_t mf_window_start(uint64_t seed, uint32_t epoch, uint32_t worker, uint32_t ite, uint32_t nnz);

/* ---- Hogwild SGD update launches ---------------------------------------------------- */

/* single_sgd_k128/k64_hogwild_kernel, sgd/sgd_kernel.h:1-79, sgd/sgd_kernel_k64.h:1-67;
 * launch site mf_methods.cu:879-905.  p: [users][k] fp32, q: [items][k] fp32. */
int mf_single_sgd_hogwild(const mf_node* R, uint32_t nnz, float* p, float* q, int k,
                          uint32_t num_workers, uint32_t update_count, uint32_t update_vector_size,
                          float lrate, float lambda,
                          uint64_t seed, uint32_t epoch, const uint32_t* window_start, void* stream);

/* mem_quant_sgd_k128/k64_hogwild_kernel launch (-v 7, the reference's default version), mf_methods.cu:1345-1372:
 * dense binary16 P [users][k], Q [items][k] (bit patterns), binary32 arithmetic, new values rounded to binary16. */
int mf_mem_quant_sgd_hogwild(const mf_node* R, uint32_t nnz, uint16_t* p, uint16_t* q, int k,
                             uint32_t num_workers, uint32_t update_count, uint32_t update_vector_size,
                             float lrate, float lambda,
                             uint64_t seed, uint32_t epoch, const uint32_t* window_start, void* stream);
/* mpt_sgd_k128/k64_hogwild_kernel, mpt/mpt_sgd_kernel.h:1-93, mpt/mpt_sgd_kernel_k64.h;
 * launch site mf_methods.cu:772-799.  scaled_lambda_half = binary16 bits of lambda*scaling_factor
 * (mf_methods.cu:764-765). */
int mf_mpt_sgd_hogwild(const mf_node* R, uint32_t nnz, float* p, float* q, int k,
                       uint32_t num_workers, uint32_t update_count, uint32_t update_vector_size,
                       float lrate, uint16_t scaled_lambda_half, float scaling_factor,
                       uint64_t seed, uint32_t epoch, const uint32_t* window_start, void* stream);

/* muppet_sgd_k128/k64_hogwild_kernel, muppet/muppet_sgd_kernel.h:50-292, _k64.h; launch site
 * mf_methods.cu:613-647.  sum_updated_val: [k] (+=, caller zeroes, mf_methods.cu:606-607);
 * sum_norms: [num_workers] (overwritten).  Precisions are 8, 12, 14, 16 or 32. */
int mf_muppet_sgd_hogwild(const mf_node* R, uint32_t nnz, float* p, float* q, int k,
                          uint32_t num_workers, uint32_t update_count, uint32_t update_vector_size,
                          float lrate, float lambda, uint32_t first_sample_rating_idx,
                          float* sum_updated_val, float* sum_norms,
                          uint8_t forward_prop_precision, uint8_t backward_prop_precision,
                          uint64_t seed, uint32_t epoch, const uint32_t* window_start, void* stream);

/* afp_sgd_k128/k64_hogwild_kernel, afp/afp_sgd_kernel.h:127-375, _k64.h; launch site
 * mf_methods.cu:480-507.  `afp_epoch` is the kernel's `epoch` argument (first tenth of
 * epoch 0 re-measures every update). */
int mf_afp_sgd_hogwild(const mf_node* R, uint32_t nnz, float* p, float* q, int k,
                       uint32_t num_workers, uint32_t update_count, uint32_t update_vector_size,
                       float lrate, float lambda, int afp_epoch,
                       uint64_t seed, uint32_t epoch, const uint32_t* window_start, void* stream);

/* mascot_sgd_k128/k64_hogwild_kernel, mascot/mascot_sgd_kernel.h:1-457, _k64.h:1-397; launch
 * site mf_methods.cu:189-237.
 *   p, q              device arrays of user_group_num / item_group_num device pointers; group g is
 *                     [group_size][k] binary16 (prec 0) or binary32 (prec 1), rows in sorted order
 *   *_group_end_idx   inclusive last sorted row of each group (preprocess_utils.h:189-213)
 *   *_group_prec_info one byte per group
 *   grad_sum_norm_*   [groups][k] fp32, += of the sampled gradients (caller zeroes on check epochs)
 *   norm_sum_*        [groups][mf_mascot_norm_blocks(num_workers)] fp32, overwritten
 *   ratings with processed index >= first_sample_rating_idx are sampled. */
int mf_mascot_sgd_hogwild(const mf_node* R, uint32_t nnz, void* const* p, void* const* q, int k,
                          uint32_t num_workers, uint32_t update_count, uint32_t update_vector_size,
                          float lrate, float lambda,
                          const uint32_t* user_group_end_idx, const uint32_t* item_group_end_idx,
                          const uint8_t* user_group_prec_info, const uint8_t* item_group_prec_info,
                          float* grad_sum_norm_p, float* grad_sum_norm_q, float* norm_sum_p, float* norm_sum_q,
                          uint32_t first_sample_rating_idx, uint32_t user_group_num, uint32_t item_group_num,
                          uint64_t seed, uint32_t epoch, const uint32_t* window_start, void* stream);

/* ---- m-quantization: conversion and grouped storage ---------------------------------- */

/* transform_float2half, model_init.cu:96-105 (round to nearest even). */
int mf_transform_float2half(const float* in, uint16_t* out, uint64_t n, void* stream);
/* transform_half2float / mem_cpy_fp16tofp32 / mem_cpy_fp162fp32, model_init.cu:85-112,
 * precision_switching.h:1-6 (exact widening; promotes one group on a precision switch). */
int mf_transform_half2float(const uint16_t* in, float* out, uint64_t n, void* stream);
/* cpyparams2grouped_params_for_comparison_indexing(+_k64), model_init.cu:30-83: row e of the dense
 * fp32 matrix -> binary16 row (entity2sorted_idx[e] - first row of its group) of group entity2group[e]. */
int mf_cpyparams2grouped_params(const float* original_params, void* const* converted_params,
                                const uint32_t* group_end_idx, const uint32_t* entity2group,
                                const uint32_t* entity2sorted_idx, int k, uint32_t n, uint32_t group_num, void* stream);
/* The gather the reference does on the host every epoch (mf_methods.cu:249-313): grouped storage
 * -> dense fp32 [n][k] in sorted row order, widening binary16 groups exactly. */
int mf_grouped_params2dense(void* const* group_ptr, const uint32_t* group_end_idx, const uint8_t* group_prec_info,
                            float* dense, int k, uint32_t n, uint32_t group_num, void* stream);

/* ---- g-switching: error estimate and evaluation -------------------------------------- */

/* Per-group error of mf_methods.cu:327-379 on the device:
 *   error[g] = (sum_k grad_sum_norm[g][k]^2) / (sum_b norm_sum[g][b]) / initial_error[g],  -1 for fp32 groups.
 * grad_sum_norm is zeroed afterwards like the host loop does (mf_methods.cu:333). */
int mf_group_error(float* grad_sum_norm, const float* norm_sum, uint32_t norm_blocks, const uint8_t* group_prec_info,
                   const float* initial_error, float* error_out, int k, uint32_t group_num, void* stream);
/* get_test_rmse_coalesced_k128/k64 + host finish, rmse.h:26-189.  Adds sum((r - p.q)^2) over the test
 * ratings into *sum_sq (one device double, caller zeroes); rmse = sqrt(sum_sq / test_n). */
int mf_test_rmse(const mf_node* test, uint32_t test_n, const float* p, const float* q, int k,
                 double* sum_sq, void* stream);
/* gpu_test_rmse, rmse.h:168-189, as the stand-alone evaluator calls it (test_mf/test.cu:68): host pointers in,
 * uploads P [n_users][k], Q [n_items][k] and the test ratings, returns sqrt(sum((r - p.q)^2) / test_n) in *rmse.
 * Unlike the reference it rejects test ratings whose ids lie outside the model. */
int mf_gpu_test_rmse(const mf_node* test, uint32_t test_n, const float* p, const float* q, uint32_t n_users, uint32_t n_items,
                     int k, double* rmse);
/* Same as mf_test_rmse, reading grouped storage directly (no host gather, no H2D of P and Q). */
int mf_test_rmse_grouped(const mf_node* test, uint32_t test_n, void* const* p, void* const* q, int k,
                         const uint32_t* user_group_end_idx, const uint32_t* item_group_end_idx,
                         const uint8_t* user_group_prec_info, const uint8_t* item_group_prec_info,
                         uint32_t user_group_num, uint32_t item_group_num, double* sum_sq, void* stream);

/* ---- model init and preprocessing ----------------------------------------------------- */

/* init_rand_state + init_rand_feature_single, model_init.cu:12-28: array[i] = (float)(N(0,1) * 0.01),
 * from a counter-based generator keyed by (seed, stream_id, i) instead of clock()-seeded cuRAND states. */
int mf_init_rand_feature(float* array, uint64_t n, uint64_t seed, uint64_t stream_id, void* stream);
/* init_idx_arr, preprocess_utils.h:6-11. */
int mf_init_idx_arr(uint32_t* arr, uint32_t n, void* stream);
/* user_item_histogram, preprocess_utils.h:13-19 (caller zeroes the bins). */
int mf_user_item_histogram(const mf_node* R, uint32_t n, uint32_t* user_bin, uint32_t* item_bin, void* stream);
/* thrust::sort_by_key(cnt, idx), preprocess_utils.h:87-88: ascending stable sort of the counts carrying
 * the ids, in place.  Allocates its temporary storage with hipMalloc and synchronises the stream. */
int mf_sort_by_count(uint32_t* cnt, uint32_t* idx, uint32_t n, void* stream);
/* matrix_reconst_gpu_triplet, preprocess_utils.h:28-36 (in place). */
int mf_matrix_reconst_triplet(mf_node* R, const uint32_t* user2sorted_idx, const uint32_t* item2sorted_idx,
                              uint32_t n, void* stream);
/* Seeded replacement for srand(time(0)); std::random_shuffle(R, R+n) (mf_methods.cu:38-39): out = in
 * permuted by ascending 64-bit key(seed, i).  Allocates temporaries with hipMalloc, synchronises. */
int mf_shuffle_ratings(const mf_node* in, mf_node* out, uint32_t n, uint64_t seed, void* stream);

/* ---- host training drivers (the reference's mf_methods.h:4-11 surface) -------------------
 * These take HOST pointers, allocate and free their own device memory with hipMalloc, run on
 * the current device's default stream and block until the run is finished.  One host thread. */

/* Parameter + the run-level fields of Mf_info, common_struct.h:19-35,87-91; defaults main.cu:19-32. */
typedef struct {
    float lambda;             /* -b  */
    float learning_rate;      /* -a  */
    float decay;              /* -d  */
    float sample_ratio;       /* -r / -s */
    float error_threshold;    /* -e  */
    uint32_t interval;        /* -it */
    uint32_t user_group_num;  /* -ug (requested; the grouping may return fewer, preprocess_utils.h:189-190) */
    uint32_t item_group_num;  /* -ig */
    uint32_t k;               /* -k  */
    uint32_t num_workers;     /* -wg; 0 = mf_auto_workers(n) */
    uint32_t epoch;           /* -l  */
    uint32_t thread_block_size; /* -bl: accepted for compatibility; workgroups are always 4 wavefronts here */
    uint32_t version;         /* -v: 1 MASCOT, 2 AFP, 3 MuPPET, 4 MPT, 5 fp32 SGD (0 = alias of 5), 6 MASCOT (the reference's
                                 naive kernel: same arithmetic, runs the MASCOT path), 7 binary16 storage with
                                 binary32 arithmetic, 8 whole-model precision switching */
    uint32_t is_yahoo;        /* MuPPET starts at 12 bit (mf_methods.cu:600) */
    uint64_t seed;            /* replaces time(0) / clock() seeding */
    uint32_t verbose;         /* 1: print the reference's stdout lines (mf_methods.cu:396 etc.) */
    uint32_t cached_rows;     /* 0: device-coherent row stores (default), 1: cached, see mf_set_row_coherence */
    uint32_t epoch_splits;    /* kernel launches per epoch, 0 or 1 = one, see mf_set_epoch_splits */
    float hot_row_inflight;   /* > 0: rows expected to have more than one update in flight become hot rows, thinned
                                 to at most this many updates in flight (see mf_set_hot_row_thinning); 0 = off */
    float hot_row_inflight_early; /* the cap during the first hot_row_early_epochs epochs, while all rows still grow
                                 from their small initial values and popular rows need many updates (default 8 for
                                 2 epochs, then hot_row_inflight = 2; 16 diverges in one run of sixteen at 100M
                                 ratings) */
    uint32_t hot_row_early_epochs;
} mf_params;

/* What a run reports back; every pointer is optional host memory owned by the caller. */
typedef struct {
    double* rmse_per_epoch;        /* [epoch] test RMSE after each epoch (mf_methods.cu:395-396) */
    float* lr_per_epoch;           /* [epoch] */
    float* sgd_ms_per_epoch;       /* [epoch] hipEvent time of the update kernel(s) (mf_methods.cu:187-241) */
    uint32_t* user2sorted_idx;     /* [n_users] MASCOT only: dense id -> popularity-sorted row */
    uint32_t* item2sorted_idx;     /* [n_items] */
    uint32_t* user_group_end_idx;  /* [requested user_group_num] MASCOT only */
    uint32_t* item_group_end_idx;  /* [requested item_group_num] */
    uint8_t* user_group_prec_info; /* [requested user_group_num] final precision per group */
    uint8_t* item_group_prec_info;
    uint32_t user_group_num;       /* actual number of groups (out) */
    uint32_t item_group_num;
    mf_node* test_reconst;         /* [test_n] MASCOT only: the test set in sorted index space (io_utils.h:374-405) */
    double preprocess_ms, switching_ms, error_ms, sgd_ms, total_ms;   /* mf_methods.cu:401-418 */
    uint32_t update_count;
    uint32_t muppet_final_bits;
} mf_report;

void mf_default_params(mf_params* out);
/* init_model_single / init_model_half, model_init.cu:138-173: p [n_users*k], q [n_items*k] on the host,
 * N(0,1)*0.01 from the seeded generator; `half_rounded` != 0 rounds every value through binary16. */
int mf_init_model(float* p, float* q, uint32_t n_users, uint32_t n_items, uint32_t k, uint64_t seed, int half_rounded);
/* mascot_training_mf / adaptive_fixed_point_training_mf / muppet_training_mf / mixed_precision_training_mf /
 * training_single_mf, mf_methods.cu:36-434,436-527,529-711,713-818,820-924, selected by params->version.
 *   R, test        host COO arrays in dense (first-seen) id space; R is shuffled on the device with
 *                  params->seed, the caller's array is left untouched
 *   p, q           host [n_users*k], [n_items*k]: initial model in, trained model out.  For version 1 the
 *                  rows come back in popularity-sorted order (as save_trained_model_reconst expects). */
int mf_train(const mf_params* params, const mf_node* R, uint32_t n, uint32_t n_users, uint32_t n_items,
             const mf_node* test, uint32_t test_n, float* p, float* q, mf_report* report);
/* Host grouping, split_group_based_equal_size_not_strict_ret_end_idx, preprocess_utils.h:101-190:
 * sorted_cnt ascending rating counts; writes inclusive end indices (capacity n) and returns their number. */
uint32_t mf_group_end_indices(const uint32_t* sorted_cnt, uint32_t n, uint32_t requested_groups, uint32_t* end_idx_out);

#ifdef __cplusplus
}
#endif
#endif
