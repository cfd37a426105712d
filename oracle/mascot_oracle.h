/*
 * TEST INFRASTRUCTURE ONLY -- CPU restatement of the reference's hot path.
 * Nothing that ships may call into this library; it is the checker that the
 * tests, the smoke run and the bench's cpu_baseline leg compare against.
 *
 * Every function cites the reference lines it restates (paths relative to the
 * reference checkout).  Functions whose behaviour no reference fixture, closed
 * form or brute-force check pins say "parity unpinned" here:
 *
 *   - orc_window_start / orc_init_normal / orc_shuffle_keys: the reference is
 *     unseeded (clock()/time(0) seeds, cuRAND XORWOW), so these restate this
 *     build's own seeded generators, not the reference's streams.
 *     parity unpinned (by construction; only the index mapping is closed form).
 *   - orc_generate_ratings: synthetic data has no counterpart in the reference
 *     (its data sets are downloaded); this is the twin of the build's own
 *     generator.  parity unpinned against the reference by construction; the
 *     distribution it claims (Zipf marginals, rating grid, low-rank signal,
 *     range independence) is pinned in tests/test_oracle_host.py.
 *   - MuPPET / AFP: floor/ceil(log2f(x)) for x within one ulp of a power of
 *     two, and float -> int8 conversion of values outside [-128,127], depend on
 *     CUDA's libdevice / cvt behaviour.  parity unpinned for those inputs.
 *   - AFP's error measurement (QEM, afp/afp_sgd_kernel.h:32-59) uses the value
 *     of log2f itself, not its floor: the last bit of the host's log2f, of
 *     CUDA's and of a GPU's v_log_f32 may differ, and the re-measurement
 *     interval computed from it then differs by one now and then.  parity
 *     unpinned for whole AFP trajectories (single epochs on conflict-free
 *     schedules are compared bit for bit with the GPU and agree).
 *   - orc_sgd_update / orc_mem_quant_update: binary32 arithmetic that nvcc may
 *     contract into fma where the source writes a*b - c*d; this restatement
 *     rounds every operation.  parity unpinned for that choice (the update is
 *     pinned as a gradient step within binary32 rounding, the summation order
 *     by a crafted row).
 *   - orc_mascot_epoch, sampled epochs: the order in which the per-group
 *     squared norms and gradient sums of racing warps are added
 *     (mascot/mascot_sgd_kernel.h:259-276: atomics and an unsynchronised +=)
 *     is not fixed by the reference; this restatement adds them in rating
 *     order.  parity unpinned for that order (any order agrees to 1e-5
 *     relative, which is what the tests hold the GPU's sums to).
 *
 * Pinned by tests/test_oracle_pins.py with engines that share no code with this
 * file (numpy.float16, Python integers, math.frexp) and hand-worked rows:
 * orc_mpt_update, orc_muppet_update and its scale index, orc_afp_* (scale,
 * QEM / QEM_BP, QPA, the re-measurement schedule) and the MuPPET ladder
 * (orc_muppet_ladder_step).
 */
#ifndef MASCOT_ORACLE_H
#define MASCOT_ORACLE_H
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct { float r; uint32_t u; uint32_t i; } orc_node;   /* common_struct.h:8-12 */

/* ---- binary16 ---------------------------------------------------------- */
uint16_t orc_float2half(float f);
float    orc_half2float(uint16_t h);
uint16_t orc_double2half(double d);
uint16_t orc_half_add(uint16_t a, uint16_t b);
uint16_t orc_half_sub(uint16_t a, uint16_t b);
uint16_t orc_half_mul(uint16_t a, uint16_t b);
uint16_t orc_half_fma(uint16_t a, uint16_t b, uint16_t c);
void orc_float2half_array(const float* in, uint16_t* out, uint64_t n);
void orc_half2float_array(const uint16_t* in, float* out, uint64_t n);

/* ---- schedules --------------------------------------------------------- */
uint32_t orc_update_count(uint32_t n, uint32_t num_workers, uint32_t update_vector_size);
uint32_t orc_sample_ratings_num(uint32_t update_count, uint32_t update_vector_size, float sample_ratio);
int      orc_is_error_check_epoch(uint32_t e, uint32_t interval, uint32_t epochs);
uint32_t orc_first_sample_rating_idx(uint32_t e, uint32_t interval, uint32_t epochs,
                                     uint32_t update_count, uint32_t update_vector_size, float sample_ratio);
float    orc_lr_schedule(float lr, float decay, uint32_t e);
uint32_t orc_window_start(uint64_t seed, uint32_t epoch, uint32_t wid, uint32_t ite, uint32_t nnz);

/* ---- preprocessing ----------------------------------------------------- */
void orc_histogram(const orc_node* R, uint64_t n, uint32_t* user_cnt, uint32_t n_users,
                   uint32_t* item_cnt, uint32_t n_items);
void orc_sort_by_count(const uint32_t* cnt, uint32_t n, uint32_t* sorted_cnt, uint32_t* sorted_id);
uint32_t orc_grouping(const uint32_t* sorted_cnt, uint32_t n, uint32_t requested_groups,
                      uint32_t* end_idx_out /* capacity n */);
void orc_reindex_tables(const uint32_t* sorted_id, uint32_t n, const uint32_t* end_idx, uint32_t groups,
                        uint32_t* id2sorted, uint32_t* id2group, uint32_t* group_size);
void orc_reindex(orc_node* R, uint64_t n, const uint32_t* user2sorted, const uint32_t* item2sorted);
void orc_group_lookup(uint32_t idx, const uint32_t* end_idx, uint32_t groups, uint32_t* group, uint32_t* local_row);
void orc_shuffle_keys(uint64_t seed, uint64_t n, uint64_t* keys);
void orc_shuffle(uint64_t seed, const orc_node* in, orc_node* out, uint64_t n);
void orc_init_normal(uint64_t seed, uint64_t stream, float* out, uint64_t n);
/* Seeded synthetic ratings, the twin of the build's mf_generate_ratings (same field order as mf_synth_config). */
typedef struct {
    uint32_t n_users, n_items;
    uint64_t n_train, n_test;
    float user_alpha, item_alpha;
    uint32_t rank;
    float noise, mean, step, lo, hi;
    uint32_t bimodal;
} orc_synth_config;
void orc_generate_ratings(const orc_synth_config* c, uint64_t seed, uint64_t first, uint64_t count, orc_node* out);

/* ---- single updates (in place on one P row and one Q row) -------------- */
void orc_sgd_update(int k, float* p, float* q, float r, float lr, float lambda);
/* mem_quant_sgd (-v 7), sgd/sgd_kernel.h:81-164: binary16 rows, binary32 arithmetic */
void orc_mem_quant_update(int k, uint16_t* p, uint16_t* q, float r, float lr, float lambda);
void orc_mpt_update(int k, float* p, float* q, float r, float lr, uint16_t scaled_lambda_h, float scaling_factor);
/* prec: 0 = binary16 row (uint16_t*), 1 = binary32 row (float*).  grad_p/grad_q (k floats)
 * and norm_p/norm_q receive the sampled statistics of the binary16 sides; untouched for
 * binary32 sides.  Pass NULL to skip statistics. */
void orc_mascot_update(int k, void* p, int user_prec, void* q, int item_prec, float r, float lr, float lambda,
                       float* grad_p, float* grad_q, float* norm_p, float* norm_q);
void orc_muppet_update(int k, float* p, float* q, float r, float lr, float lambda,
                       int forward_bits, int backward_bits, float* grad_sum /* k, += */, float* norm /* += */);

typedef struct { int r; int n; int itv; float mov_avg_range; } orc_afp_qparams;   /* afp_sgd_kernel.h:1-6 */
typedef struct {
    orc_afp_qparams user, item, backward;
    int update_user_params_iter, update_item_params_iter, update_backward_iter, cur_iter;
    float scaling_factor_p, scaling_factor_q, scaling_factor_back_prop;
} orc_afp_state;
void orc_afp_state_init(orc_afp_state* s);
void orc_afp_update(int k, orc_afp_state* s, float* p, float* q, float r, float lr, float lambda,
                    int epoch, int initialization_threshold);

/* ---- whole-launch restatements (sequential: ite-major, then worker) ---- */
/* window_start may be NULL (then orc_window_start(seed, epoch, wid, ite, nnz) is used). */
void orc_mem_quant_epoch(int k, const orc_node* R, uint32_t nnz, uint16_t* P, uint16_t* Q,
                         uint32_t num_workers, uint32_t update_count, uint32_t update_vector_size,
                         float lr, float lambda, uint64_t seed, uint32_t epoch, const uint32_t* window_start, int threads);
void orc_sgd_epoch(int k, const orc_node* R, uint32_t nnz, float* P, float* Q,
                   uint32_t num_workers, uint32_t update_count, uint32_t update_vector_size,
                   float lr, float lambda, uint64_t seed, uint32_t epoch, const uint32_t* window_start, int threads);
void orc_mpt_epoch(int k, const orc_node* R, uint32_t nnz, float* P, float* Q,
                   uint32_t num_workers, uint32_t update_count, uint32_t update_vector_size,
                   float lr, float lambda, float scaling_factor, uint64_t seed, uint32_t epoch,
                   const uint32_t* window_start, int threads);
void orc_muppet_epoch(int k, const orc_node* R, uint32_t nnz, float* P, float* Q,
                      uint32_t num_workers, uint32_t update_count, uint32_t update_vector_size,
                      float lr, float lambda, uint32_t first_sample_rating_idx,
                      float* sum_updated_val /* k */, float* sum_norms /* num_workers */,
                      int forward_bits, int backward_bits,
                      uint64_t seed, uint32_t epoch, const uint32_t* window_start, int threads);
void orc_afp_epoch(int k, const orc_node* R, uint32_t nnz, float* P, float* Q,
                   uint32_t num_workers, uint32_t update_count, uint32_t update_vector_size,
                   float lr, float lambda, int epoch_arg,
                   uint64_t seed, uint32_t epoch, const uint32_t* window_start, int threads);
/* grouped storage: user_group_ptr[g] is a uint16_t* (prec 0) or float* (prec 1) array of group_size*k.
 * grad_sum_norm_{p,q}: [groups*k] (+=); norm_sum_{p,q}: [groups] (+=, all workers folded). */
void orc_mascot_epoch(int k, const orc_node* R, uint32_t nnz, void** user_group_ptr, void** item_group_ptr,
                      const uint32_t* user_end_idx, const uint32_t* item_end_idx,
                      const uint8_t* user_prec, const uint8_t* item_prec, uint32_t user_groups, uint32_t item_groups,
                      uint32_t num_workers, uint32_t update_count, uint32_t update_vector_size,
                      float lr, float lambda, uint32_t first_sample_rating_idx,
                      float* grad_sum_norm_p, float* grad_sum_norm_q, float* norm_sum_p, float* norm_sum_q,
                      uint64_t seed, uint32_t epoch, const uint32_t* window_start, int threads);

/* ---- evaluation and g-switching --------------------------------------- */
double orc_rmse(int k, const orc_node* test, uint64_t test_n, const float* P, const float* Q);
double orc_rmse_grouped(int k, const orc_node* test, uint64_t test_n, void** user_group_ptr, void** item_group_ptr,
                        const uint32_t* user_end_idx, const uint32_t* item_end_idx,
                        const uint8_t* user_prec, const uint8_t* item_prec, uint32_t user_groups, uint32_t item_groups);
void orc_group_error(int k, uint32_t groups, const float* grad_sum_norm, const float* norm_sum, uint32_t norm_blocks,
                     const uint8_t* prec, const float* initial_error, float* error_out);
int orc_muppet_ladder_step(int k, int e, int* switched_epoch, int* precision_idx, float* max_grad_diversity,
                           int* violation_times, const float* sum_norms_epoch, const float* sum_updated_val_epoch);

#ifdef __cplusplus
}
#endif
#endif
