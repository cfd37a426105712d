// extern "C" launchers of the Hogwild update kernels: process-wide settings, closed forms of the schedule, and the
// fp32 SGD and MPT entry points (the other rules' entry points sit in launch_*.hip).
#include "hogwild_launch.h"
#include "rules_fp32.h"

namespace mf {

static thread_local char g_error[512] = "";
void set_error(const char* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof g_error, fmt, ap);
    va_end(ap);
}


// ---- replicated rows: copy out, average back -------------------------------------------------------------------
// One wavefront per replicated row.  merge = 0: every XCD's copy := the row.  merge = 1: the row and every copy := the
// mean of the copies that differ from the row (an XCD that did not touch its copy -- no workgroup of the launch ran
// there, or none of its ratings fell on the row -- has nothing to contribute), summed in binary32 in XCD order and
// rounded once to the row's precision; if no copy differs the row stays as it is.  With in_play > 0 the mean is taken
// over that many copies, the ones that do not differ counting as the row: the sum of the changed copies plus
// (in_play - changed) times the row, divided by in_play.
struct SyncSide { RowStorage rows; uint8_t* replicas; const uint32_t* slot_row; uint32_t slots; };
template <int K>
__global__ __launch_bounds__(kWave) void replica_sync_kernel(SyncSide user, SyncSide item, int merge, uint32_t in_play)
{
    constexpr int E = K / kWave;
    const bool is_item = blockIdx.x >= user.slots;
    const SyncSide& side = is_item ? item : user;
    const uint32_t slot = is_item ? blockIdx.x - user.slots : blockIdx.x;
    const uint32_t row = side.slot_row[slot];
    uint8_t* master; bool wide;
    if (side.rows.dense) {
        wide = side.rows.elem_bytes == 4;
        master = static_cast<uint8_t*>(side.rows.dense) + (size_t)row * K * side.rows.elem_bytes;
    } else {
        uint32_t lo = 0, hi = side.rows.groups - 1;            // min{g : row <= end[g]}
        while (lo < hi) { const uint32_t mid = (lo + hi) >> 1; if (row <= side.rows.group_end[mid]) hi = mid; else lo = mid + 1; }
        const uint32_t local = lo ? row - side.rows.group_end[lo - 1] - 1 : row;
        wide = side.rows.group_prec[lo] != 0;
        master = static_cast<uint8_t*>(side.rows.group_ptr[lo]) + (size_t)local * K * (wide ? 4u : 2u);
    }
    const size_t slot_bytes = (size_t)K * 4u;
    auto copy_of = [&](uint32_t x) { return side.replicas + ((size_t)x * side.slots + slot) * slot_bytes; };
    auto load = [&](const uint8_t* at, int e) { return wide ? reinterpret_cast<const float*>(at)[e] : (float)reinterpret_cast<const half_t*>(at)[e]; };
    auto store = [&](uint8_t* at, int e, float v) { if (wide) reinterpret_cast<float*>(at)[e] = v; else reinterpret_cast<half_t*>(at)[e] = (half_t)v; };
    float base[E], out[E];
#pragma unroll
    for (int j = 0; j < E; ++j) { base[j] = load(master, (int)threadIdx.x + j * kWave); out[j] = base[j]; }
    if (merge) {
        float sum[E];
#pragma unroll
        for (int j = 0; j < E; ++j) sum[j] = 0.f;
        uint32_t changed = 0;
        for (uint32_t x = 0; x < kXcds; ++x) {
            float v[E]; bool differs = false;
#pragma unroll
            for (int j = 0; j < E; ++j) { v[j] = load(copy_of(x), (int)threadIdx.x + j * kWave); differs |= bits(v[j]) != bits(base[j]); }
            if (__builtin_amdgcn_ballot_w64(differs) != 0ull) {        // wave-uniform: the whole copy counts or does not
                ++changed;
#pragma unroll
                for (int j = 0; j < E; ++j) sum[j] += v[j];
            }
        }
        if (changed) {
            const uint32_t copies = in_play > changed ? in_play : changed;
#pragma unroll
            for (int j = 0; j < E; ++j) {
                if (copies > changed) sum[j] += (float)(copies - changed) * base[j];
                out[j] = sum[j] / (float)copies; store(master, (int)threadIdx.x + j * kWave, out[j]);
            }
        }
    }
    for (uint32_t x = 0; x < kXcds; ++x) {
#pragma unroll
        for (int j = 0; j < E; ++j) store(copy_of(x), (int)threadIdx.x + j * kWave, out[j]);
    }
}
int replica_sync(const ReplicaSide& user, const ReplicaSide& item, int k, bool merge, void* stream, uint32_t in_play)
{
    const uint32_t blocks = user.slots + item.slots;
    if (blocks == 0) return MF_OK;
    const SyncSide u{user.rows, user.replicas, user.slot_row, user.slots}, v{item.rows, item.replicas, item.slot_row, item.slots};
    if (k == 128) hipLaunchKernelGGL(replica_sync_kernel<128>, dim3(blocks), dim3(kWave), 0, as_stream(stream), u, v, merge ? 1 : 0, in_play);
    else hipLaunchKernelGGL(replica_sync_kernel<64>, dim3(blocks), dim3(kWave), 0, as_stream(stream), u, v, merge ? 1 : 0, in_play);
    return launch_status("replica_sync");
}

float inflight_sgd(int k, uint32_t num_workers, uint32_t cap) { return inflight_updates<SgdRule>(k, num_workers, 0, cap); }
float inflight_mpt(int k, uint32_t num_workers, uint32_t cap) { return inflight_updates<MptRule>(k, num_workers, 0, cap); }

}  // namespace mf

using namespace mf;

extern "C" {


int mf_version(void) { return 1; }
const char* mf_last_error(void) { return g_error; }
int mf_replica_sync_dense(void* matrix, uint32_t elem_bytes, int k, void* replicas, const uint32_t* slot_row, uint32_t slots, int merge, void* stream)
{
    if (k != 64 && k != 128) return invalid("mf_replica_sync_dense: k must be 64 or 128 (got %d)", k);
    if (elem_bytes != 2 && elem_bytes != 4) return invalid("mf_replica_sync_dense: elem_bytes is 2 (binary16) or 4 (binary32)");
    if (slots == 0) return MF_OK;
    if (!matrix || !replicas || !slot_row) return invalid("mf_replica_sync_dense: null pointer");
    ReplicaSide side, none;
    side.rows.dense = matrix; side.rows.elem_bytes = elem_bytes; side.replicas = static_cast<uint8_t*>(replicas); side.slot_row = slot_row; side.slots = slots;
    return replica_sync(side, none, k, merge != 0, stream);
}
float mf_hogwild_inflight_capped(uint32_t version, int k, uint32_t num_workers, uint32_t user_groups, uint32_t item_groups, uint32_t resident_workers)
{
    if (k != 64 && k != 128) return 0.f;
    const uint32_t cap = resident_workers;
    switch (version) {
    case 0: case 5: return inflight_sgd(k, num_workers, cap);
    case 4: return inflight_mpt(k, num_workers, cap);
    case 3: return inflight_muppet(k, num_workers, cap);
    case 2: return inflight_afp(k, num_workers, cap);
    case 7: return inflight_mem_quant(k, num_workers, cap);
    case 8: return inflight_mascot(k, num_workers, 1, 1, cap);
    case 1: case 6: return inflight_mascot(k, num_workers, user_groups ? user_groups : 1, item_groups ? item_groups : 1, cap);
    default: return 0.f;
    }
}
float mf_hogwild_inflight(uint32_t version, int k, uint32_t num_workers, uint32_t user_groups, uint32_t item_groups)
{
    return mf_hogwild_inflight_capped(version, k, num_workers, user_groups, item_groups, 0);
}
uint32_t mf_mascot_norm_blocks(uint32_t num_workers) { return grid_for(num_workers); }

uint32_t mf_update_count(uint32_t n, uint32_t num_workers, uint32_t update_vector_size)
{
    if (num_workers == 0 || update_vector_size == 0) return 0;
    return (uint32_t)std::ceil((double)n / (double)((uint64_t)num_workers * update_vector_size));
}
uint32_t mf_first_sample_rating_idx(uint32_t e, uint32_t interval, uint32_t epochs, uint32_t update_count,
                                    uint32_t update_vector_size, float sample_ratio)
{
    const uint32_t start_idx = 5;
    const uint32_t total = update_count * update_vector_size;
    if (interval == 0) return total;
    const bool check = (e >= start_idx) && (e % interval == (start_idx % interval)) && (epochs - 1 != e);
    if (!check) return total;
    const uint32_t sample_ratings_num = (uint32_t)((float)total * sample_ratio);
    return total - sample_ratings_num;
}
float mf_lr_schedule(float lr, float decay, uint32_t e)
{
    return (float)((double)lr / (1.0 + ((double)decay * std::pow((double)e, 1.5))));
}
uint32_t mf_window_start(uint64_t seed, uint32_t epoch, uint32_t worker, uint32_t ite, uint32_t nnz)
{
    if (nnz == 0) return 0;
    return window_start_rng(window_epoch_key(seed, epoch), worker, ite, nnz);
}

int mf_single_sgd_hogwild_opt(const mf_node* R, uint32_t nnz, float* p, float* q, int k,
                              uint32_t num_workers, uint32_t update_count, uint32_t update_vector_size,
                              float lrate, float lambda,
                              uint64_t seed, uint32_t epoch, const uint32_t* window_start, void* stream, const mf_hogwild_options* options)
{
    if (int rc = check_schedule("mf_single_sgd_hogwild", R, nnz, k, num_workers, update_count, update_vector_size, options)) return rc;
    if (!p || !q) return invalid("mf_single_sgd_hogwild: null model pointer");
    const Call c = make_call(R, nnz, num_workers, update_count, update_vector_size, seed, epoch, window_start, options);
    return launch_k_coh<SgdRule>("mf_single_sgd_hogwild", k, c, [&](auto a) { a.p = p; a.q = q; a.lrate = lrate; a.lambda = lambda; return a; }, 0, stream, whole_epoch(c));
}
int mf_single_sgd_hogwild(const mf_node* R, uint32_t nnz, float* p, float* q, int k,
                          uint32_t num_workers, uint32_t update_count, uint32_t update_vector_size,
                          float lrate, float lambda,
                          uint64_t seed, uint32_t epoch, const uint32_t* window_start, void* stream)
{
    return mf_single_sgd_hogwild_opt(R, nnz, p, q, k, num_workers, update_count, update_vector_size, lrate, lambda, seed, epoch, window_start, stream, nullptr);
}

int mf_mpt_sgd_hogwild_opt(const mf_node* R, uint32_t nnz, float* p, float* q, int k,
                           uint32_t num_workers, uint32_t update_count, uint32_t update_vector_size,
                           float lrate, uint16_t scaled_lambda_half, float scaling_factor,
                           uint64_t seed, uint32_t epoch, const uint32_t* window_start, void* stream, const mf_hogwild_options* options)
{
    if (int rc = check_schedule("mf_mpt_sgd_hogwild", R, nnz, k, num_workers, update_count, update_vector_size, options)) return rc;
    if (!p || !q) return invalid("mf_mpt_sgd_hogwild: null model pointer");
    if (!(scaling_factor > 0)) return invalid("mf_mpt_sgd_hogwild: scaling_factor must be positive");
    const Call c = make_call(R, nnz, num_workers, update_count, update_vector_size, seed, epoch, window_start, options);
    return launch_k_coh<MptRule>("mf_mpt_sgd_hogwild", k, c, [&](auto a) {
        a.p = p; a.q = q; a.lrate = lrate; a.scaled_lambda_half = scaled_lambda_half; a.scaling_factor = scaling_factor; return a; }, 0, stream, whole_epoch(c));
}
int mf_mpt_sgd_hogwild(const mf_node* R, uint32_t nnz, float* p, float* q, int k,
                       uint32_t num_workers, uint32_t update_count, uint32_t update_vector_size,
                       float lrate, uint16_t scaled_lambda_half, float scaling_factor,
                       uint64_t seed, uint32_t epoch, const uint32_t* window_start, void* stream)
{
    return mf_mpt_sgd_hogwild_opt(R, nnz, p, q, k, num_workers, update_count, update_vector_size, lrate, scaled_lambda_half, scaling_factor, seed, epoch, window_start, stream, nullptr);
}

}  // extern "C"
