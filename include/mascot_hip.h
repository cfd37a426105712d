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
/* ---- options of the Hogwild update launches --------------------------------------------------
 * Every update entry point below exists in two forms: mf_<rule>_sgd_hogwild(...) with the reference launch's
 * arguments, and mf_<rule>_sgd_hogwild_opt(..., options) with one more pointer to this structure (NULL = defaults,
 * which is what the short form passes).  The structure is read during the call and carries no state between calls;
 * the device arrays it names must stay valid until the launches of the call have finished.  None of it has a
 * counterpart in the reference, which runs on a GPU with one L2 and a few hundred updates in flight.
 *
 * cached_rows   0 (default) device-coherent: every row store writes through the per-XCD L2 to the memory side
 *               (agent-scope relaxed atomic stores; loads stay ordinary cached loads), so a worker sees the latest
 *               row any other worker stored -- the semantics the reference gets from a GPU with one L2.  All
 *               stores to one row serialise at the memory side, which bounds the epoch when a single row takes
 *               percents of all ratings; that is what the hot-row tables are for.
 *               1 cached: ordinary write-back stores; each of the 8 XCDs works on its own L2-resident copy of a
 *               row for as long as it stays cached, copies are merged last-writer-wins.
 * launches      kernel launches the call is cut into (0 or 1 = one; each worker's windows are divided evenly).
 *               A kernel boundary writes back and invalidates the per-XCD L2s; replicated rows are averaged there.
 * user_keep, item_keep   hot-row tables, both or neither: device arrays of bytes indexed like P and Q rows (for
 *               MASCOT: sorted row order).
 *                 255  an ordinary row: the new row is stored (the reference's rule, last writer wins);
 *                 254  a hot row, meant for rows with a few updates in flight at any time: the update adds its
 *                      change to the row in memory (an atomic add per element), so concurrent updates add up where
 *                      last-writer-wins would keep one of them;
 *                 MF_KEEP_REPLICATED (253)  a replicated row, meant for rows with many updates in flight: every XCD
 *                      works on a copy of its own with ordinary cached loads and stores -- the copy lives in that
 *                      XCD's L2, where its workers race on it as the reference's warps race on a row, every update
 *                      carried out -- and after every kernel launch of the call the row and the copies become the
 *                      mean of the copies that changed (mf_replica_sync_dense).  Nothing of such a row serialises at
 *                      the memory side;
 *                 MF_KEEP_REPLICATED_ADDED (252)  a replicated row whose updates are added to the XCD's copy instead of
 *                      stored, meant for rows with a few updates in flight per XCD: they add up inside the XCD as
 *                      added updates do on an unreplicated row;
 *                 0..251  a hot row that is thinned: a rating updates it with probability (value+1)/255 (an added
 *                      update, as for 254) and otherwise only reads it for the other side's update.
 * user_slot, item_slot   [rows] uint16: for a replicated row its slot in the replica blocks (read for those rows only)
 * user_slot_row, item_slot_row   [slots] the row of every slot
 * user_replicas, item_replicas   caller-owned scratch of MF_XCDS * slots * k * 4 bytes, 256-byte aligned; slot s of
 *               XCD x is at (x * slots + s) * k * 4 and holds the row in the precision it is stored in.  Filled from
 *               the rows at the start of every call; nothing is kept in it between calls.
 * user_slots, item_slots   replicated rows per side (at most 65535; 0 = none)
 * replica_step_scale   0 (default): a copy of a replicated row is updated like any row, and the merge takes the mean of
 *               the copies that changed.  >= 1: scaled steps.  A copy sees the ratings of one XCD only, and the mean of X
 *               copies moves by the X-th part of what the copies moved together; so an update of a copy takes a step
 *               replica_step_scale times as long (at most X when X < MF_XCDS) (the learning rate of that side of the rating is multiplied), and
 *               the merge is the mean over the X = min(MF_XCDS, workgroups of the launch) copies in play, untouched ones
 *               counting as the row.  With X = 1 (a launch of one workgroup) nothing changes.  The caller bounds the
 *               factor by what keeps a single step stable: factor x learning rate x |other side's row|^2 well below 2
 *               (mf_replica_step_scale).
 * all_binary16  MASCOT only, a hint: 1 = every group of both sides is binary16 in this call.  The call then launches a
 *               build of the kernel without the fast path for chunks of mixed precisions, which keeps one more
 *               wavefront per SIMD resident (4 % per epoch at 100M ratings).  A wrong hint costs time, not results:
 *               that build takes its general path for any chunk that touches a binary32 group.
 * resident_workers   0 (default): as many workers run at a time as the device keeps resident.  > 0: at most about that
 *               many (rounded down to whole workgroups per compute unit, at least one): the ordinary launches of the call
 *               ask for LDS they do not use, which keeps further workgroups off a compute unit.  Fewer updates in flight
 *               bring a run closer to a sequential one and cost time; mf_train uses it for the first epoch
 *               (mf_params.early_inflight).  The hot-row tables of such a call are the caller's to build for the lower
 *               number of updates in flight.  The sampled launch of a MASCOT check epoch is not affected. */
#define MF_KEEP_ORDINARY 255
#define MF_KEEP_ADDED 254
#define MF_KEEP_REPLICATED 253
#define MF_KEEP_REPLICATED_ADDED 252
#define MF_XCDS 8
typedef struct {
    uint32_t cached_rows;
    uint32_t launches;
    const uint8_t* user_keep;
    const uint8_t* item_keep;
    const uint16_t* user_slot;
    const uint16_t* item_slot;
    const uint32_t* user_slot_row;
    const uint32_t* item_slot_row;
    void* user_replicas;
    void* item_replicas;
    uint32_t user_slots, item_slots;
    float replica_step_scale;
    uint32_t all_binary16;
    uint32_t resident_workers;
} mf_hogwild_options;
/* What the update calls do with replicated rows before and after every kernel launch, for a dense matrix [rows][k] of
 * elem_bytes-wide elements (2: binary16, 4: binary32): merge = 0 copies row slot_row[s] into slot s of every XCD's
 * replica block; merge = 1 sets the row and all its copies to the mean of those copies that differ from the row
 * (summed in binary32 in XCD order, divided by their number, rounded once); a row none of whose copies differs stays. */
int mf_replica_sync_dense(void* matrix, uint32_t elem_bytes, int k, void* replicas, const uint32_t* slot_row, uint32_t slots,
                          int merge, void* stream);
/* The table mf_train builds for one side (host arrays): counts[row] ratings of `n` fall on the row; with
 * `inflight` updates in flight on the device (mf_hogwild_inflight) a row has about inflight * counts[row] / n of them.
 * Rows with at most one stay ordinary (255).  Of the others, rows above replicate_above (> 0) are marked
 * MF_KEEP_REPLICATED -- MF_KEEP_REPLICATED_ADDED instead up to add_within x MF_XCDS in flight (add_within: updates in
 * flight per XCD; 0 = never) -- and numbered in row order (slot[row], slot_row[slot]; slot may be NULL
 * when replicate_above is 0; at most 65535, the rows with the highest counts); rows above thin_above (> 0) are thinned
 * to that many updates in flight: value clip(floor(thin_above / in flight * 255) - 1, 0, 251); the rest are added (254).
 * Returns the number of replicated rows in *slots. */
int mf_hot_row_table(const uint32_t* counts, uint32_t rows, uint32_t n, float inflight, float replicate_above, float thin_above, float add_within,
                     uint8_t* table, uint16_t* slot, uint32_t* slot_row, uint32_t* slots);
/* Updates in flight during a launch of `num_workers` workers of the update rule of mf_params.version (1..8) at this k:
 * min(num_workers, wavefronts the device keeps resident for that kernel) x the ratings a wavefront keeps in flight
 * (4; 2 for MuPPET and AFP).  Asks the HIP runtime for the kernel's occupancy on the current device. */
float mf_hogwild_inflight(uint32_t version, int k, uint32_t num_workers, uint32_t user_groups, uint32_t item_groups);
/* The same for launches with mf_hogwild_options::resident_workers set (0 = not set): what such a launch really keeps
 * in flight -- the cap works in whole workgroups per compute unit and does nothing to a launch that is below it anyway. */
float mf_hogwild_inflight_capped(uint32_t version, int k, uint32_t num_workers, uint32_t user_groups, uint32_t item_groups, uint32_t resident_workers);
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
 * Convenience form: allocates the tables (mf_synth_tables_bytes), builds them, generates and frees them again, so it
 * synchronises the stream. */
int mf_generate_ratings(const mf_synth_config* cfg, uint64_t seed, uint64_t first, uint64_t count, mf_node* out, void* stream);
/* The same in two steps with caller-owned device memory: mf_synth_build_tables fills `workspace` (256-byte aligned, at
 * least mf_synth_tables_bytes(cfg) bytes) with the two CDFs, the two permutations and the factors of (cfg, seed) -- its
 * host-side tables are copied from pageable memory, so this step waits for the stream once -- and
 * mf_generate_ratings_ws then writes any range of the stream from those tables: one kernel launch, nothing allocated,
 * nothing synchronised. */
size_t mf_synth_tables_bytes(const mf_synth_config* cfg);
int mf_synth_build_tables(const mf_synth_config* cfg, uint64_t seed, void* workspace, size_t workspace_bytes, void* stream);
int mf_generate_ratings_ws(const mf_synth_config* cfg, uint64_t seed, const void* tables, uint64_t first, uint64_t count, mf_node* out, void* stream);
/* The same into a host array (allocates, generates on the default stream, copies back, frees). */
int mf_generate_ratings_host(const mf_synth_config* cfg, uint64_t seed, uint64_t first, uint64_t count, mf_node* host_out);
/* Measurement aid, no counterpart in the reference: the memory traffic of one epoch of updates without the
 * arithmetic.  Worker w (one wavefront) walks ratings [w*ceil(n/W), (w+1)*ceil(n/W)); per rating it reads row u of p
 * and row i of q (row_bytes = 128, 256 or 512 bytes each: k = 64 binary16, k = 128 binary16 / k = 64 binary32,
 * k = 128 binary32) and writes both back unchanged, with the store policy, hot-row tables and replicated rows of
 * `options` (NULL = defaults; `launches` is ignored, replica slots are taken as row_bytes wide, so the options' replica
 * arrays must hold MF_XCDS * slots * row_bytes bytes: with the options of an update call at rank k, row_bytes <= 4 k): a thinned update
 * only reads its row, an added update is a store here, a replicated row is read and written in this XCD's copy.
 * p and q keep their contents (writes of other code that race with the probe may be lost).  The time of this launch is
 * what the memory system sustains for the sequence of addresses and the write policy of an epoch; bench.py reports the
 * update kernel's time beside it. */
int mf_row_traffic_probe(const mf_node* R, uint32_t n, void* p, void* q, uint32_t row_bytes, uint32_t num_workers,
                         uint64_t seed, void* stream, const mf_hogwild_options* options);
/* The same with rows of different widths on the two sides (the wider twice the other: a MASCOT epoch after the groups of
 * one side have been promoted to binary32); replica slots are as wide as their side's rows. */
int mf_row_traffic_probe_sides(const mf_node* R, uint32_t n, void* p, void* q, uint32_t user_row_bytes, uint32_t item_row_bytes,
                               uint32_t num_workers, uint64_t seed, void* stream, const mf_hogwild_options* options);
/* Number of per-block columns mf_mascot_sgd_hogwild writes into norm_sum_p / norm_sum_q
 * (the reference's `block_num`, mf_methods.cu:109). */
uint32_t mf_mascot_norm_blocks(uint32_t num_workers);
/* Host-side closed forms of the schedule (mf_methods.cu:94-111,170-175). */
uint32_t mf_update_count(uint32_t n, uint32_t num_workers, uint32_t update_vector_size);
/* Worker count mf_train uses for mf_params.num_workers == 0: n / 16384 (about 128 windows per worker), a multiple
 * of 4, at least 16.  The updates in flight grow with the workers and so does the distance to a sequential run, until
 * the chip is full (6144 resident workers, reached at about 95M ratings); from there on the count is n / 2048 (16
 * windows per worker), which changes nothing in flight and evens out the end of every launch.  The reference's fixed
 * default (2048, main.cu:28) suits neither 400k nor 100M ratings on this GPU. */
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
int mf_single_sgd_hogwild_opt(const mf_node* R, uint32_t nnz, float* p, float* q, int k,
                          uint32_t num_workers, uint32_t update_count, uint32_t update_vector_size,
                          float lrate, float lambda,
                          uint64_t seed, uint32_t epoch, const uint32_t* window_start, void* stream,
        const mf_hogwild_options* options);

/* mem_quant_sgd_k128/k64_hogwild_kernel launch (-v 7, the reference's default version), mf_methods.cu:1345-1372:
 * dense binary16 P [users][k], Q [items][k] (bit patterns), binary32 arithmetic, new values rounded to binary16. */
int mf_mem_quant_sgd_hogwild(const mf_node* R, uint32_t nnz, uint16_t* p, uint16_t* q, int k,
                             uint32_t num_workers, uint32_t update_count, uint32_t update_vector_size,
                             float lrate, float lambda,
                             uint64_t seed, uint32_t epoch, const uint32_t* window_start, void* stream);
int mf_mem_quant_sgd_hogwild_opt(const mf_node* R, uint32_t nnz, uint16_t* p, uint16_t* q, int k,
                             uint32_t num_workers, uint32_t update_count, uint32_t update_vector_size,
                             float lrate, float lambda,
                             uint64_t seed, uint32_t epoch, const uint32_t* window_start, void* stream,
        const mf_hogwild_options* options);
/* mpt_sgd_k128/k64_hogwild_kernel, mpt/mpt_sgd_kernel.h:1-93, mpt/mpt_sgd_kernel_k64.h;
 * launch site mf_methods.cu:772-799.  scaled_lambda_half = binary16 bits of lambda*scaling_factor
 * (mf_methods.cu:764-765). */
int mf_mpt_sgd_hogwild(const mf_node* R, uint32_t nnz, float* p, float* q, int k,
                       uint32_t num_workers, uint32_t update_count, uint32_t update_vector_size,
                       float lrate, uint16_t scaled_lambda_half, float scaling_factor,
                       uint64_t seed, uint32_t epoch, const uint32_t* window_start, void* stream);
int mf_mpt_sgd_hogwild_opt(const mf_node* R, uint32_t nnz, float* p, float* q, int k,
                       uint32_t num_workers, uint32_t update_count, uint32_t update_vector_size,
                       float lrate, uint16_t scaled_lambda_half, float scaling_factor,
                       uint64_t seed, uint32_t epoch, const uint32_t* window_start, void* stream,
        const mf_hogwild_options* options);

/* muppet_sgd_k128/k64_hogwild_kernel, muppet/muppet_sgd_kernel.h:50-292, _k64.h; launch site
 * mf_methods.cu:613-647.  sum_updated_val: [k] (+=, caller zeroes, mf_methods.cu:606-607);
 * sum_norms: [num_workers] (overwritten).  Precisions are 8, 12, 14, 16 or 32. */
int mf_muppet_sgd_hogwild(const mf_node* R, uint32_t nnz, float* p, float* q, int k,
                          uint32_t num_workers, uint32_t update_count, uint32_t update_vector_size,
                          float lrate, float lambda, uint32_t first_sample_rating_idx,
                          float* sum_updated_val, float* sum_norms,
                          uint8_t forward_prop_precision, uint8_t backward_prop_precision,
                          uint64_t seed, uint32_t epoch, const uint32_t* window_start, void* stream);
int mf_muppet_sgd_hogwild_opt(const mf_node* R, uint32_t nnz, float* p, float* q, int k,
                          uint32_t num_workers, uint32_t update_count, uint32_t update_vector_size,
                          float lrate, float lambda, uint32_t first_sample_rating_idx,
                          float* sum_updated_val, float* sum_norms,
                          uint8_t forward_prop_precision, uint8_t backward_prop_precision,
                          uint64_t seed, uint32_t epoch, const uint32_t* window_start, void* stream,
        const mf_hogwild_options* options);

/* afp_sgd_k128/k64_hogwild_kernel, afp/afp_sgd_kernel.h:127-375, _k64.h; launch site
 * mf_methods.cu:480-507.  `afp_epoch` is the kernel's `epoch` argument (first tenth of
 * epoch 0 re-measures every update). */
int mf_afp_sgd_hogwild(const mf_node* R, uint32_t nnz, float* p, float* q, int k,
                       uint32_t num_workers, uint32_t update_count, uint32_t update_vector_size,
                       float lrate, float lambda, int afp_epoch,
                       uint64_t seed, uint32_t epoch, const uint32_t* window_start, void* stream);
int mf_afp_sgd_hogwild_opt(const mf_node* R, uint32_t nnz, float* p, float* q, int k,
                       uint32_t num_workers, uint32_t update_count, uint32_t update_vector_size,
                       float lrate, float lambda, int afp_epoch,
                       uint64_t seed, uint32_t epoch, const uint32_t* window_start, void* stream,
        const mf_hogwild_options* options);

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
int mf_mascot_sgd_hogwild_opt(const mf_node* R, uint32_t nnz, void* const* p, void* const* q, int k,
                          uint32_t num_workers, uint32_t update_count, uint32_t update_vector_size,
                          float lrate, float lambda,
                          const uint32_t* user_group_end_idx, const uint32_t* item_group_end_idx,
                          const uint8_t* user_group_prec_info, const uint8_t* item_group_prec_info,
                          float* grad_sum_norm_p, float* grad_sum_norm_q, float* norm_sum_p, float* norm_sum_q,
                          uint32_t first_sample_rating_idx, uint32_t user_group_num, uint32_t item_group_num,
                          uint64_t seed, uint32_t epoch, const uint32_t* window_start, void* stream,
        const mf_hogwild_options* options);

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
 * the ids, in place.  Convenience form: allocates its workspace with hipMalloc, frees it and therefore
 * synchronises the stream. */
int mf_sort_by_count(uint32_t* cnt, uint32_t* idx, uint32_t n, void* stream);
/* The same with a caller-owned workspace (256-byte aligned device memory of at least
 * mf_sort_by_count_workspace_bytes(n) bytes: the sort's output buffers and rocPRIM's temporary storage): asynchronous
 * on `stream`, allocates nothing, synchronises nothing.  The size query needs a current device (0 on failure). */
size_t mf_sort_by_count_workspace_bytes(uint32_t n);
int mf_sort_by_count_ws(uint32_t* cnt, uint32_t* idx, uint32_t n, void* workspace, size_t workspace_bytes, void* stream);
/* mf_sort_by_count for callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc); no counterpart in the reference.  The sort's workspace is a 20 MiB array in the
 * library's own device image (each GPU the library runs on holds its copy until the process ends), so the call
 * allocates and frees nothing and is asynchronous on `stream`.  At most mf_sort_by_count_static_max() = 1,048,576
 * counts; more are refused with MF_EINVAL.  All calls on one GPU share that array: calls that overlap on one GPU
 * (different streams, different host threads) race -- run them one after another.  Nothing in the array has to
 * start at zero between calls.  The first call on a device asks the runtime for the address of that device's copy of the
 * array (hipGetSymbolAddress, under a mutex): a caller that captures streams into graphs makes one call outside any
 * capture first. */
uint32_t mf_sort_by_count_static_max(void);
int mf_sort_by_count_static(uint32_t* cnt, uint32_t* idx, uint32_t n, void* stream);
/* matrix_reconst_gpu_triplet, preprocess_utils.h:28-36 (in place). */
int mf_matrix_reconst_triplet(mf_node* R, const uint32_t* user2sorted_idx, const uint32_t* item2sorted_idx,
                              uint32_t n, void* stream);
/* Seeded replacement for srand(time(0)); std::random_shuffle(R, R+n) (mf_methods.cu:38-39): out = in
 * permuted by ascending 64-bit key(seed, i).  Convenience form: allocates its workspace, frees it, synchronises. */
int mf_shuffle_ratings(const mf_node* in, mf_node* out, uint32_t n, uint64_t seed, void* stream);
/* The same with a caller-owned workspace (256-byte aligned, mf_shuffle_ratings_workspace_bytes(n) bytes: keys, ids,
 * the permutation and rocPRIM's temporary storage): asynchronous, allocates nothing, synchronises nothing. */
size_t mf_shuffle_ratings_workspace_bytes(uint32_t n);
int mf_shuffle_ratings_ws(const mf_node* in, mf_node* out, uint32_t n, uint64_t seed, void* workspace, size_t workspace_bytes, void* stream);

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
    uint32_t cached_rows;     /* mf_hogwild_options::cached_rows */
    uint32_t epoch_splits;    /* mf_hogwild_options::launches; 0 = one launch, or replica_merges when rows are replicated */
    float hot_row_inflight;   /* > 0: hot rows that are not replicated and have more than this many updates in flight are
                                 thinned to it (mf_hogwild_options, keep values 0..251); 0 (default) = nothing is thinned.
                                 A chunk of 64 ratings with a skipped update takes the kernels' general loop, which
                                 waits for every row it loads: with thinning instead of replication (replicate_inflight
                                 0) nearly every chunk has one, 22.5 ms per MASCOT epoch and 34 per fp32 epoch at 100M
                                 ratings against 11.4 and 20.1 with the defaults */
    float hot_row_inflight_early; /* with thinning: the cap during the first hot_row_early_epochs epochs */
    uint32_t hot_row_early_epochs;
    uint32_t hot_rows;        /* 1 (default): rows expected to have more than one update in flight become hot rows (updates
                                 added in memory, MF_KEEP_ADDED); 0 with replicate_inflight = hot_row_inflight = 0: no tables
                                 at all, every row is stored as the reference does (last writer wins) */
    float replicate_inflight; /* rows expected to have more than this many updates in flight get a copy per XCD
                                 (MF_KEEP_REPLICATED); the expectation is mf_hogwild_inflight() x the row's share of the
                                 ratings.  < 0 (default): mf_replicate_threshold(learning_rate, mean rating); 0 = no replicas */
    uint32_t replica_merges;  /* launches per epoch when rows are replicated: their copies are averaged after each (default 0: n / 25M, between 1 and 4) */
    float replica_add_inflight; /* > 0: replicated rows with at most this many updates in flight per XCD have their updates
                                 added to the XCD's copy (MF_KEEP_REPLICATED_ADDED) instead of stored.  Default 0: at
                                 100M ratings the extra atomic adds cost 9 ms per epoch and gain 0.0007 test RMSE */
    float replica_step_scale; /* mf_hogwild_options::replica_step_scale.  < 0 (default): mf_replica_step_scale(learning_rate,
                                 mean rating), for MuPPET (version 3) 0: its 8-bit passes diverge, at random, at factors
                                 the other rules run at.  0 = off (unscaled steps, mean of the changed copies) */
    uint32_t wg_counts_updates; /* 0 (default): num_workers is the number of workers (wavefronts), each of which keeps four
                                 ratings in flight (two for MuPPET and AFP), so -wg W puts 4 W updates in flight where the
                                 reference's -wg W puts W.  1: num_workers is the reference's figure, the updates in
                                 flight, and the run uses num_workers / 4 (/ 2) workers -- the reading under which the
                                 reference's documented settings (-wg 2048, README.md:33) mean here what they mean there */
    uint32_t replica_step_epochs; /* the first epochs that use replica_step_scale; later ones run unscaled (default 1: the
                                 epoch in which every row grows from its small initial value and a replicated row, which
                                 keeps one of the many updates in flight on a copy, is furthest behind; afterwards the
                                 unscaled mean of eight copies is the less noisy estimate.  0 = every epoch) */
    float early_inflight;     /* runs with hot-row tables: the first early_inflight_epochs epochs run with this fraction of the
                                 updates in flight the device would keep (mf_hogwild_options::resident_workers, and tables
                                 built for that number).  A row keeps one of the updates that are in flight on it at a
                                 time, so while the rows are far from their optimum the distance to a sequential run
                                 grows with the updates in flight: at 100M ratings the test RMSE after the first epoch is
                                 0.049 / 0.024 / 0.023 / 0.015 above the sequential run's with all / half / a third / a
                                 quarter of them, and that epoch takes 15.7 / 19.8 / 20.9 / 33.4 ms.  Between 0 and 1;
                                 0 or 1 = off.  Default 0.5.  The cap works in workgroups per compute unit, so a run with
                                 fewer than 1024 workers is not affected */
    uint32_t early_inflight_epochs; /* default 1 */
    float replicate_inflight_late; /* from epoch replicate_late_from on (counted from 0; default 1: the second epoch) rows above
                                 this many updates in flight get copies: a lower bar than replicate_inflight keeps more
                                 rows in the L2s and adds to fewer at the memory side.  Past the first epoch the mean of
                                 the copies loses nothing measurable (100M ratings: bars 8.68 / 6 / 4 / 3 / 2 from the
                                 second epoch on give 13.5 / 13.0 / 12.2 / 11.7 / 11.3 ms per epoch and the same test RMSE up
                                 to epoch 50 within 0.0005, epochs 3 and 4 ending 0.001 closer to the sequential run with
                                 the lower bars; only with every row above one update in flight replicated do epochs 2
                                 to 8 fall behind, by 0.001), while in the first epoch every averaged row shows (bars
                                 8.68 / 6 / 4 / 3 throughout: 0.023 / 0.027 / 0.030 / 0.032 above the sequential run after
                                 epoch 1).  < 0 (default): a quarter of replicate_inflight's value in runs that keep at
                                 least 4096 updates in flight (1024 workers), the same bar throughout in smaller ones,
                                 whose epochs are bound by the latency of a worker's chain and gain little from more
                                 copies; 0 = the same bar throughout */
    uint32_t replicate_late_from;
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
    uint8_t* muppet_bits_per_epoch; /* [epoch] MuPPET only: the bit width every epoch ran at (mf_methods.cu:596-601,691) */
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
/* The same run with the epochs handed to the caller one at a time (no counterpart in the reference, whose drivers
 * run to the end): mf_session_create does what mf_train does before its first epoch (checks, upload, shuffle,
 * pre-processing, hot-row tables), every mf_session_epoch runs the next epoch exactly as mf_train would -- update
 * launches, error estimate, precision switching, test RMSE -- and returns that epoch's test RMSE and the hipEvent time
 * of its update launches, mf_session_finish copies the model to p, q (and fills the MASCOT tables of the report).
 * `report` is optional, must outlive the session and is filled as in mf_train.  One host thread per session. */
typedef struct mf_session mf_session;
int mf_session_create(const mf_params* params, const mf_node* R, uint32_t n, uint32_t n_users, uint32_t n_items,
                      const mf_node* test, uint32_t test_n, const float* p, const float* q, mf_report* report, mf_session** session);
int mf_session_epoch(mf_session* session, double* test_rmse, float* sgd_ms);
int mf_session_finish(mf_session* session, float* p, float* q);
void mf_session_destroy(mf_session* session);
/* The worker count the session runs (mf_params.num_workers, or mf_auto_workers), and its hot rows: rows replicated per
 * side in the tables most of the run uses (those of the later epochs when the bar for copies is lowered after the first
 * ones, mf_params.replicate_inflight_late) and the updates in flight those tables were built for (0 when the run has no
 * tables). */
uint32_t mf_session_workers(const mf_session* session);
int mf_session_hot_rows(const mf_session* session, uint32_t* user_replicated, uint32_t* item_replicated, float* inflight);
/* The session's training ratings on the device (shuffled; for MASCOT re-indexed to sorted rows) and the launch options
 * its update calls of `epoch` use; both stay owned by the session and valid until mf_session_destroy.  For
 * measurements that replay the session's memory traffic (mf_row_traffic_probe). */
int mf_session_device_state(const mf_session* session, uint32_t epoch, const mf_node** ratings, const mf_hogwild_options** options);
/* The groups of one side of a MASCOT session (side 0: users, 1: items; no counterpart in the reference, which prints
 * its group tables): *groups = their number (0 for the versions without groups), prec[g] = 1 where group g is held in
 * binary32 now (precision_switching.h:8-51 has promoted it), ratings[g] = training ratings that fall on the group's
 * rows.  prec and ratings are optional host arrays of at least the requested group count (mf_params.user_group_num /
 * item_group_num).  An update touches one user row and one item row, so the bytes an epoch moves follow from these
 * two tables: 12 + 2 k (2 or 4) bytes per side and rating. */
int mf_session_groups(const mf_session* session, int side, uint32_t* groups, uint8_t* prec, uint64_t* ratings);
/* Promotes the groups g with mask[g] != 0 of one side to binary32 now, as the precision switching does when a group's
 * error exceeds the threshold (precision_switching.h:8-51: exact widening, pointer and precision tables refreshed);
 * groups that are binary32 already stay.  `groups` must equal the side's group count.  For measurements of epochs
 * after switching; waits for the device. */
int mf_session_promote_groups(mf_session* session, int side, const uint8_t* mask, uint32_t groups);
/* Above how many updates in flight mf_train replicates a row when mf_params.replicate_inflight < 0 (the default):
 * 0.3 / (learning_rate * mean |rating|), between 2 and 16.  Added updates of one row that are in flight together sum
 * gradients taken at the same stale row; the sum stays a contraction while their number x lr x mean rating < 2. */
float mf_replicate_threshold(float learning_rate, float mean_rating);
/* The step factor mf_train gives the copies of replicated rows when mf_params.replica_step_scale < 0 (the default):
 * 0.15 / (learning_rate * mean |rating|), half the bound above, between 1 and MF_XCDS (4.3 for learning rate 0.01 and
 * ratings around 3.5; measured there: 8 still converges, 12 diverges in the first epoch). */
float mf_replica_step_scale(float learning_rate, float mean_rating);
/* Host grouping, split_group_based_equal_size_not_strict_ret_end_idx, preprocess_utils.h:101-190:
 * sorted_cnt ascending rating counts; writes inclusive end indices (capacity n) and returns their number. */
uint32_t mf_group_end_indices(const uint32_t* sorted_cnt, uint32_t n, uint32_t requested_groups, uint32_t* end_idx_out);

#ifdef __cplusplus
}
#endif
#endif
