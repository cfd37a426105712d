// Host training drivers: the five variants of mf_methods.cu (mascot_training_mf :36-434,
// adaptive_fixed_point_training_mf :436-527, muppet_training_mf :529-711,
// mixed_precision_training_mf :713-818, training_single_mf :820-924) behind one entry point.
//
// What changed against the reference's drivers: the model never leaves the device during training
// (the reference copies every group to the host and the dense model back for the RMSE each epoch,
// mf_methods.cu:249-313, rmse.h:170-171); the test RMSE reads the grouped storage directly; the
// per-group error is finished on the device; grouped storage is one binary16 arena and one binary32
// arena per side instead of one cudaMalloc per group and per switch (precision_switching.h:13-24);
// shuffle, histogram, sort and re-indexing run on the device; every random choice is seeded.
#include <hip/hip_runtime_api.h>
#include <algorithm>
#include <chrono>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>
#include "mf_host.h"

namespace {

using mf::check_hip;
using mf::invalid;

struct DevBuf {
    void* p = nullptr;
    size_t bytes = 0;
    DevBuf() = default;
    DevBuf(const DevBuf&) = delete;
    DevBuf& operator=(const DevBuf&) = delete;
    ~DevBuf() { if (p) (void)hipFree(p); }
    int alloc(size_t n, const char* what)
    {
        bytes = n;
        return check_hip(hipMalloc(&p, n ? n : 4), what);
    }
    template <class T> T* as() const { return static_cast<T*>(p); }
};

struct Timer {
    hipEvent_t a = nullptr, b = nullptr;
    Timer() { (void)hipEventCreate(&a); (void)hipEventCreate(&b); }
    ~Timer() { if (a) (void)hipEventDestroy(a); if (b) (void)hipEventDestroy(b); }
    void start() { (void)hipEventRecord(a, nullptr); }
    float stop() { (void)hipEventRecord(b, nullptr); (void)hipEventSynchronize(b); float ms = 0; (void)hipEventElapsedTime(&ms, a, b); return ms; }
};

double now_ms()
{
    return std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now().time_since_epoch()).count();
}

#define MF_TRY(expr) do { int rc_ = (expr); if (rc_ != 0) return rc_; } while (0)
#define HIP_TRY(expr, what) do { int rc_ = check_hip((expr), what); if (rc_ != 0) return rc_; } while (0)

struct Common {
    const mf_params* prm;
    uint32_t n, n_users, n_items, test_n, k;
    uint32_t update_vector_size = 128;       // hard-coded in every driver (mf_methods.cu:100,858)
    uint32_t update_count;
    DevBuf d_R, d_test, d_sum_sq;
    std::vector<float> lr;
    mf_report* rep;
};

// The kernels index P and Q with the ids in the ratings and cannot know the row counts: check them here, on the
// host, where a bad id is an error message and not an out-of-bounds access on the device.
int check_ids(const char* what, const mf_node* R, uint32_t n, uint32_t n_users, uint32_t n_items)
{
    for (uint32_t i = 0; i < n; ++i)
        if (R[i].u >= n_users || R[i].i >= n_items)
            return invalid("mf_train: %s rating %u names user %u / item %u, the model has %u users and %u items", what, i, R[i].u, R[i].i, n_users, n_items);
    return 0;
}

int upload_and_shuffle(Common& c, const mf_node* R, const mf_node* test)
{
    MF_TRY(check_ids("training", R, c.n, c.n_users, c.n_items));
    MF_TRY(check_ids("test", test, c.test_n, c.n_users, c.n_items));
    DevBuf staging;
    MF_TRY(staging.alloc((size_t)c.n * sizeof(mf_node), "hipMalloc(ratings staging)"));
    MF_TRY(c.d_R.alloc((size_t)c.n * sizeof(mf_node), "hipMalloc(ratings)"));
    HIP_TRY(hipMemcpy(staging.p, R, (size_t)c.n * sizeof(mf_node), hipMemcpyHostToDevice), "H2D ratings");
    // srand(time(0)); random_shuffle(R, R+n)  (mf_methods.cu:38-39) -> seeded device shuffle
    MF_TRY(mf_shuffle_ratings(staging.as<mf_node>(), c.d_R.as<mf_node>(), c.n, c.prm->seed, nullptr));
    MF_TRY(c.d_test.alloc((size_t)c.test_n * sizeof(mf_node), "hipMalloc(test)"));
    if (c.test_n) HIP_TRY(hipMemcpy(c.d_test.p, test, (size_t)c.test_n * sizeof(mf_node), hipMemcpyHostToDevice), "H2D test");
    MF_TRY(c.d_sum_sq.alloc(sizeof(double), "hipMalloc(rmse accumulator)"));
    return 0;
}

void fill_schedule(Common& c)
{
    const mf_params& p = *c.prm;
    c.update_count = mf_update_count(c.n, p.num_workers, c.update_vector_size);
    c.lr.resize(p.epoch);
    for (uint32_t e = 0; e < p.epoch; ++e) c.lr[e] = mf_lr_schedule(p.learning_rate, p.decay, e);
    if (c.rep) {
        c.rep->update_count = c.update_count;
        if (c.rep->lr_per_epoch) std::copy(c.lr.begin(), c.lr.end(), c.rep->lr_per_epoch);
    }
}

int report_epoch(Common& c, uint32_t e, double rmse, float sgd_ms)
{
    if (c.rep) {
        if (c.rep->rmse_per_epoch) c.rep->rmse_per_epoch[e] = rmse;
        if (c.rep->sgd_ms_per_epoch) c.rep->sgd_ms_per_epoch[e] = sgd_ms;
        c.rep->sgd_ms += sgd_ms;
    }
    if (c.prm->verbose) { std::printf("%u %g %g\n", e + 1, (double)c.lr[e], rmse); std::fflush(stdout); }   // mf_methods.cu:396
    if (c.test_n && !std::isfinite(rmse))
        return invalid("mf_train: the model diverged in epoch %u (the test RMSE is not finite); lower the learning rate, or the "
                       "hot-row caps (hot_row_inflight_early, hot_row_inflight) if hot rows are on", e + 1);
    return 0;
}

int finish_rmse(Common& c, double* out)
{
    double sum = 0;
    HIP_TRY(hipMemcpy(&sum, c.d_sum_sq.p, sizeof(double), hipMemcpyDeviceToHost), "D2H rmse accumulator");
    *out = c.test_n ? std::sqrt(sum / (double)c.test_n) : 0.0;      // rmse.h:188
    return 0;
}

int dense_rmse(Common& c, const float* d_p, const float* d_q, double* out)
{
    HIP_TRY(hipMemsetAsync(c.d_sum_sq.p, 0, sizeof(double), nullptr), "memset rmse accumulator");
    MF_TRY(mf_test_rmse(c.d_test.as<mf_node>(), c.test_n, d_p, d_q, (int)c.k, c.d_sum_sq.as<double>(), nullptr));
    return finish_rmse(c, out);
}

// Hot-row table from rating counts (see mf_set_hot_row_thinning): a row with count c has about F*c/n updates in
// flight (F = resident workers x ratings a worker keeps in flight).  Rows with more than one are hot rows (their
// updates are added); of those, rows above inflight_cap are thinned to inflight_cap updates in flight.
std::vector<uint8_t> keep_table(const uint32_t* cnt, uint32_t rows, uint32_t n, uint32_t num_workers, float inflight_cap)
{
    const double resident = num_workers < 8192u ? num_workers : 8192u;      // 256 CUs x 32 wavefronts
    const double F = resident * 4.0;                                         // three ratings of look-ahead
    std::vector<uint8_t> t(rows);
    for (uint32_t r = 0; r < rows; ++r) {
        const double inflight = F * (double)cnt[r] / (double)n;
        if (inflight <= 1.0) { t[r] = 255; continue; }
        const double keep = inflight > inflight_cap ? inflight_cap / inflight : 1.0;
        const int v = (int)std::floor(keep * 255.0) - 1;
        t[r] = (uint8_t)(v < 0 ? 0 : (v > 254 ? 254 : v));
    }
    return t;
}

// The two pairs of hot-row tables of a run: the early cap for the first epochs, while every row still grows from its
// small initial value and the popular rows need many updates, and the steady cap afterwards.
struct HotRows {
    DevBuf early_u, early_v, steady_u, steady_v;
    bool active = false;
    uint32_t early_epochs = 0;
    ~HotRows() { if (active) (void)mf_set_hot_row_thinning(nullptr, nullptr); }
    static int upload(DevBuf& d, const std::vector<uint8_t>& t)
    {
        MF_TRY(d.alloc(t.size(), "hipMalloc(hot-row table)"));
        HIP_TRY(hipMemcpy(d.p, t.data(), t.size(), hipMemcpyHostToDevice), "H2D hot-row table");
        return 0;
    }
    int install(const mf_params& prm, const uint32_t* ucnt, uint32_t n_users, const uint32_t* icnt, uint32_t n_items, uint32_t n)
    {
        if (!(prm.hot_row_inflight > 0)) return 0;
        early_epochs = prm.hot_row_inflight_early > prm.hot_row_inflight ? prm.hot_row_early_epochs : 0;
        MF_TRY(upload(steady_u, keep_table(ucnt, n_users, n, prm.num_workers, prm.hot_row_inflight)));
        MF_TRY(upload(steady_v, keep_table(icnt, n_items, n, prm.num_workers, prm.hot_row_inflight)));
        if (early_epochs) {
            MF_TRY(upload(early_u, keep_table(ucnt, n_users, n, prm.num_workers, prm.hot_row_inflight_early)));
            MF_TRY(upload(early_v, keep_table(icnt, n_items, n, prm.num_workers, prm.hot_row_inflight_early)));
        }
        active = true;
        return 0;
    }
    // tables for the launches of epoch e (a launch takes the pointers with it, so switching between launches is safe)
    int select(uint32_t e)
    {
        if (!active) return 0;
        const bool early = e < early_epochs;
        return mf_set_hot_row_thinning((early ? early_u : steady_u).as<uint8_t>(), (early ? early_v : steady_v).as<uint8_t>());
    }
};

// Whole-model precision switching (-v 8, training_switching_only, mf_methods.cu:1396-1562): the MASCOT kernel with
// one group per side that holds every row in its original order (the arithmetic of switching_only_sgd_k128/k64 is
// the binary16 / binary32 case of the MASCOT kernel, sgd/sgd_kernel.h:166-344), the sampled statistics of both sides
// added together, and both sides promoted at once.
struct WholeModel {
    DevBuf hp, hq, ptr_p, ptr_q, end_u, end_i, prec, gsp, gsq, nsp, nsq;
    uint32_t norm_blocks = 0;
    bool is_float = false;
    float initial_error = 1.f;
    int init(Common& c, const float* d_p, const float* d_q, uint32_t num_workers)
    {
        const size_t pn = (size_t)c.n_users * c.k, qn = (size_t)c.n_items * c.k;
        MF_TRY(hp.alloc(pn * 2, "hipMalloc(binary16 P)"));
        MF_TRY(hq.alloc(qn * 2, "hipMalloc(binary16 Q)"));
        MF_TRY(mf_transform_float2half(d_p, hp.as<uint16_t>(), pn, nullptr));
        MF_TRY(mf_transform_float2half(d_q, hq.as<uint16_t>(), qn, nullptr));
        norm_blocks = mf_mascot_norm_blocks(num_workers);
        MF_TRY(ptr_p.alloc(8, "hipMalloc")); MF_TRY(ptr_q.alloc(8, "hipMalloc")); MF_TRY(end_u.alloc(4, "hipMalloc")); MF_TRY(end_i.alloc(4, "hipMalloc"));
        MF_TRY(prec.alloc(1, "hipMalloc")); MF_TRY(gsp.alloc(c.k * 4, "hipMalloc")); MF_TRY(gsq.alloc(c.k * 4, "hipMalloc"));
        MF_TRY(nsp.alloc((size_t)norm_blocks * 4, "hipMalloc")); MF_TRY(nsq.alloc((size_t)norm_blocks * 4, "hipMalloc"));
        const uint32_t eu = c.n_users - 1, ei = c.n_items - 1;
        HIP_TRY(hipMemcpy(end_u.p, &eu, 4, hipMemcpyHostToDevice), "H2D"); HIP_TRY(hipMemcpy(end_i.p, &ei, 4, hipMemcpyHostToDevice), "H2D");
        return point_at(hp.p, hq.p, 0);
    }
    int point_at(void* p, void* q, uint8_t precision)
    {
        HIP_TRY(hipMemcpy(ptr_p.p, &p, 8, hipMemcpyHostToDevice), "H2D"); HIP_TRY(hipMemcpy(ptr_q.p, &q, 8, hipMemcpyHostToDevice), "H2D");
        HIP_TRY(hipMemcpy(prec.p, &precision, 1, hipMemcpyHostToDevice), "H2D");
        is_float = precision != 0;
        return 0;
    }
};

// ---- variants over dense P/Q (versions 2..5, 7, 8) ----------------------------------------------
int train_dense(Common& c, float* p, float* q)
{
    const mf_params& prm = *c.prm;
    const uint32_t version = prm.version == 0 ? 5 : prm.version;
    const size_t pn = (size_t)c.n_users * c.k, qn = (size_t)c.n_items * c.k;
    DevBuf d_p, d_q, d_sum_updated, d_sum_norms;
    MF_TRY(d_p.alloc(pn * 4, "hipMalloc(P)"));
    MF_TRY(d_q.alloc(qn * 4, "hipMalloc(Q)"));
    HIP_TRY(hipMemcpy(d_p.p, p, pn * 4, hipMemcpyHostToDevice), "H2D P");
    HIP_TRY(hipMemcpy(d_q.p, q, qn * 4, hipMemcpyHostToDevice), "H2D Q");

    // MPT: loss scale 1000, lambda*1000 rounded to binary16 on the host (mf_methods.cu:764-765)
    const float scaling_factor = 1000;
    uint16_t scaled_lambda_h = 0;
    if (version == 4) {
        DevBuf tmp_f, tmp_h;
        MF_TRY(tmp_f.alloc(8, "hipMalloc")); MF_TRY(tmp_h.alloc(8, "hipMalloc"));
        const float v[2] = {prm.lambda * scaling_factor, 0.f};
        HIP_TRY(hipMemcpy(tmp_f.p, v, 8, hipMemcpyHostToDevice), "H2D");
        MF_TRY(mf_transform_float2half(tmp_f.as<float>(), tmp_h.as<uint16_t>(), 2, nullptr));
        uint16_t hb[2];
        HIP_TRY(hipMemcpy(hb, tmp_h.p, 4, hipMemcpyDeviceToHost), "D2H");
        scaled_lambda_h = hb[0];
    }
    // MuPPET ladder state (mf_methods.cu:586-601)
    const unsigned char bit_width_set[5] = {8, 12, 14, 16, 32};
    int precision_idx = prm.is_yahoo ? 1 : 0, switched_epoch = -1, violation_times = 0;
    float max_grad_diversity = -1.f;
    const int resolution_size = 3, gamma = 1;
    std::vector<float> sum_norms_epoch(prm.epoch, 0.f), sum_updated_val_epoch((size_t)prm.epoch * c.k, 0.f), sum_norms(prm.num_workers), sum_updated(c.k);
    uint32_t muppet_first_sample = 0;
    if (version == 3) {
        MF_TRY(d_sum_updated.alloc(c.k * 4, "hipMalloc(sum_updated_val)"));
        MF_TRY(d_sum_norms.alloc((size_t)prm.num_workers * 4, "hipMalloc(sum_norms)"));
        const int sample_ratings_num = (int)((float)(c.update_count * c.update_vector_size) * prm.sample_ratio);   // :563
        muppet_first_sample = c.update_count * c.update_vector_size - (uint32_t)sample_ratings_num;
    }

    // -v 7: dense binary16 storage next to the fp32 buffers, which then only serve the RMSE and the result
    DevBuf d_hp, d_hq;
    if (version == 7) {
        MF_TRY(d_hp.alloc(pn * 2, "hipMalloc(binary16 P)"));
        MF_TRY(d_hq.alloc(qn * 2, "hipMalloc(binary16 Q)"));
        MF_TRY(mf_transform_float2half(d_p.as<float>(), d_hp.as<uint16_t>(), pn, nullptr));
        MF_TRY(mf_transform_float2half(d_q.as<float>(), d_hq.as<uint16_t>(), qn, nullptr));
    }
    WholeModel whole;
    const uint32_t total = c.update_count * c.update_vector_size;
    const uint32_t whole_sample_num = (uint32_t)(int)((float)total * prm.sample_ratio);       // mf_methods.cu:1425
    if (version == 8) MF_TRY(whole.init(c, d_p.as<float>(), d_q.as<float>(), prm.num_workers));

    HotRows hot;
    if (prm.hot_row_inflight > 0) {
        DevBuf d_ucnt, d_icnt;
        MF_TRY(d_ucnt.alloc((size_t)c.n_users * 4, "hipMalloc(user counts)"));
        MF_TRY(d_icnt.alloc((size_t)c.n_items * 4, "hipMalloc(item counts)"));
        HIP_TRY(hipMemset(d_ucnt.p, 0, (size_t)c.n_users * 4), "memset");
        HIP_TRY(hipMemset(d_icnt.p, 0, (size_t)c.n_items * 4), "memset");
        MF_TRY(mf_user_item_histogram(c.d_R.as<mf_node>(), c.n, d_ucnt.as<uint32_t>(), d_icnt.as<uint32_t>(), nullptr));
        std::vector<uint32_t> ucnt(c.n_users), icnt(c.n_items);
        HIP_TRY(hipMemcpy(ucnt.data(), d_ucnt.p, (size_t)c.n_users * 4, hipMemcpyDeviceToHost), "D2H user counts");
        HIP_TRY(hipMemcpy(icnt.data(), d_icnt.p, (size_t)c.n_items * 4, hipMemcpyDeviceToHost), "D2H item counts");
        MF_TRY(hot.install(prm, ucnt.data(), c.n_users, icnt.data(), c.n_items, c.n));
    }
    Timer t;
    const mf_node* R = c.d_R.as<mf_node>();
    for (uint32_t e = 0; e < prm.epoch; ++e) {
        MF_TRY(hot.select(e));
        bool whole_check = false;
        const double err0 = now_ms();
        if (version == 3) HIP_TRY(hipMemsetAsync(d_sum_updated.p, 0, c.k * 4, nullptr), "memset sum_updated_val");
        double err_ms = now_ms() - err0;
        t.start();
        switch (version) {
        case 5: MF_TRY(mf_single_sgd_hogwild(R, c.n, d_p.as<float>(), d_q.as<float>(), (int)c.k, prm.num_workers, c.update_count, c.update_vector_size,
                                             c.lr[e], prm.lambda, prm.seed, e, nullptr, nullptr)); break;
        case 4: MF_TRY(mf_mpt_sgd_hogwild(R, c.n, d_p.as<float>(), d_q.as<float>(), (int)c.k, prm.num_workers, c.update_count, c.update_vector_size,
                                          c.lr[e], scaled_lambda_h, scaling_factor, prm.seed, e, nullptr, nullptr)); break;
        case 3: {
            const int idx = precision_idx > 4 ? 4 : precision_idx;      // the reference indexes past the table once at 32 bit (mf_methods.cu:691)
            MF_TRY(mf_muppet_sgd_hogwild(R, c.n, d_p.as<float>(), d_q.as<float>(), (int)c.k, prm.num_workers, c.update_count, c.update_vector_size,
                                         c.lr[e], prm.lambda, muppet_first_sample, d_sum_updated.as<float>(), d_sum_norms.as<float>(),
                                         bit_width_set[idx], bit_width_set[idx], prm.seed, e, nullptr, nullptr));
            break;
        }
        case 2: MF_TRY(mf_afp_sgd_hogwild(R, c.n, d_p.as<float>(), d_q.as<float>(), (int)c.k, prm.num_workers, c.update_count, c.update_vector_size,
                                          c.lr[e], prm.lambda, (int)e, prm.seed, e, nullptr, nullptr)); break;
        case 7: MF_TRY(mf_mem_quant_sgd_hogwild(R, c.n, d_hp.as<uint16_t>(), d_hq.as<uint16_t>(), (int)c.k, prm.num_workers, c.update_count,
                                                c.update_vector_size, c.lr[e], prm.lambda, prm.seed, e, nullptr, nullptr)); break;
        case 8: {
            // mf_methods.cu:1460-1466: sampled only while the model is binary16
            whole_check = !whole.is_float && prm.interval && e >= 5 && (e % prm.interval == 5 % prm.interval) && prm.epoch - 1 != e;
            if (whole_check) {
                t.stop();
                const double e0 = now_ms();
                HIP_TRY(hipMemsetAsync(whole.gsp.p, 0, c.k * 4, nullptr), "memset"); HIP_TRY(hipMemsetAsync(whole.gsq.p, 0, c.k * 4, nullptr), "memset");
                err_ms += now_ms() - e0;
                t.start();
            }
            MF_TRY(mf_mascot_sgd_hogwild(R, c.n, whole.ptr_p.as<void*>(), whole.ptr_q.as<void*>(), (int)c.k, prm.num_workers, c.update_count,
                                         c.update_vector_size, c.lr[e], prm.lambda, whole.end_u.as<uint32_t>(), whole.end_i.as<uint32_t>(),
                                         whole.prec.as<uint8_t>(), whole.prec.as<uint8_t>(), whole.gsp.as<float>(), whole.gsq.as<float>(),
                                         whole.nsp.as<float>(), whole.nsq.as<float>(), whole_check ? total - whole_sample_num : total, 1, 1,
                                         prm.seed, e, nullptr, nullptr));
            break;
        }
        default: return invalid("mf_train: version %u is not a dense variant", version);
        }
        const float sgd_ms = t.stop();
        if (version == 7 || (version == 8 && !whole.is_float)) {      // the fp32 copy the RMSE kernel and the caller read
            MF_TRY(mf_transform_half2float((version == 7 ? d_hp : whole.hp).as<uint16_t>(), d_p.as<float>(), pn, nullptr));
            MF_TRY(mf_transform_half2float((version == 7 ? d_hq : whole.hq).as<uint16_t>(), d_q.as<float>(), qn, nullptr));
        }
        if (version == 8 && whole_check) {      // mf_methods.cu:1506-1536
            const double e0 = now_ms();
            std::vector<float> gs(2 * c.k), ns(2 * (size_t)whole.norm_blocks);
            HIP_TRY(hipMemcpy(gs.data(), whole.gsp.p, c.k * 4, hipMemcpyDeviceToHost), "D2H"); HIP_TRY(hipMemcpy(gs.data() + c.k, whole.gsq.p, c.k * 4, hipMemcpyDeviceToHost), "D2H");
            HIP_TRY(hipMemcpy(ns.data(), whole.nsp.p, (size_t)whole.norm_blocks * 4, hipMemcpyDeviceToHost), "D2H");
            HIP_TRY(hipMemcpy(ns.data() + whole.norm_blocks, whole.nsq.p, (size_t)whole.norm_blocks * 4, hipMemcpyDeviceToHost), "D2H");
            float norm_acc = 0, sum_norms_acc = 0;
            for (float v : ns) norm_acc += v;
            for (uint32_t i = 0; i < c.k; ++i) sum_norms_acc += std::pow(gs[i] + gs[c.k + i], 2.0f);
            float quantization_error = sum_norms_acc / norm_acc;
            quantization_error = quantization_error / whole.initial_error;
            if (prm.verbose) { std::printf("Quantization error : %g\n", (double)quantization_error); std::fflush(stdout); }
            if (e == 5) whole.initial_error = quantization_error;
            if (e > 5 && quantization_error > prm.error_threshold) {      // both sides to binary32 (d_p, d_q were just widened)
                MF_TRY(whole.point_at(d_p.p, d_q.p, 1));
                if (c.rep) c.rep->switching_ms += now_ms() - e0;
            }
            err_ms += now_ms() - e0;
        }
        double rmse = 0;
        MF_TRY(dense_rmse(c, d_p.as<float>(), d_q.as<float>(), &rmse));
        MF_TRY(report_epoch(c, e, rmse, sgd_ms));

        if (version == 3) {      // mf_methods.cu:659-697
            const double e0 = now_ms();
            HIP_TRY(hipMemcpy(sum_norms.data(), d_sum_norms.p, (size_t)prm.num_workers * 4, hipMemcpyDeviceToHost), "D2H sum_norms");
            HIP_TRY(hipMemcpy(sum_updated.data(), d_sum_updated.p, c.k * 4, hipMemcpyDeviceToHost), "D2H sum_updated_val");
            float norm_acc = 0;
            for (uint32_t w = 0; w < prm.num_workers; ++w) norm_acc += sum_norms[w];
            sum_norms_epoch[e] = norm_acc;
            for (uint32_t i = 0; i < c.k; ++i) sum_updated_val_epoch[(size_t)e * c.k + i] = sum_updated[i];
            const float decaying_threshold = (float)(1.0f + (1.5f * std::exp(-1 * 0.3f * (float)(int)e)));
            if ((int)e - switched_epoch >= resolution_size) {
                float sum_norms_resolution = 0, sum_updated_val_norm = 0;
                std::vector<float> acc(c.k, 0.f);
                for (int wi = (int)e - resolution_size + 1; wi <= (int)e; ++wi) {
                    sum_norms_resolution += sum_norms_epoch[wi];
                    for (uint32_t i = 0; i < c.k; ++i) acc[i] += sum_updated_val_epoch[(size_t)wi * c.k + i];
                }
                for (uint32_t i = 0; i < c.k; ++i) sum_updated_val_norm += std::pow(acc[i], 2.0f);
                const float div = sum_norms_resolution / sum_updated_val_norm;
                max_grad_diversity = max_grad_diversity < div ? div : max_grad_diversity;
                const float ratio = max_grad_diversity / div;
                if (ratio > decaying_threshold && ++violation_times == gamma) {
                    precision_idx++;
                    switched_epoch = (int)e;
                    max_grad_diversity = -1.f;
                    violation_times = 0;
                }
            }
            err_ms += now_ms() - e0;
        }
        if (c.rep) c.rep->error_ms += err_ms;
    }
    if (c.rep) c.rep->muppet_final_bits = version == 3 ? bit_width_set[precision_idx > 4 ? 4 : precision_idx] : 0;
    HIP_TRY(hipMemcpy(p, d_p.p, pn * 4, hipMemcpyDeviceToHost), "D2H P");
    HIP_TRY(hipMemcpy(q, d_q.p, qn * 4, hipMemcpyDeviceToHost), "D2H Q");
    return 0;
}

// ---- MASCOT (version 1) --------------------------------------------------------------------------
struct Side {
    uint32_t n = 0, groups = 0, k = 0;
    std::vector<uint32_t> sorted_cnt, sorted_id, end_idx, id2sorted, id2group, group_size;
    std::vector<uint8_t> prec;
    std::vector<uint64_t> ptr;          // device address of every group
    std::vector<float> error, initial_error;
    DevBuf half_arena, float_arena, d_ptr, d_end, d_prec, d_grad_sum, d_norm_sum, d_error, d_initial;
    std::vector<size_t> half_off, float_off;
};

// histogram -> sort -> grouping -> re-index tables for one side (preprocess_utils.h:54-241)
int build_side(Side& s, const DevBuf& d_cnt_in, uint32_t n, uint32_t requested_groups, uint32_t k)
{
    s.n = n; s.k = k;
    DevBuf d_idx;
    MF_TRY(d_idx.alloc((size_t)n * 4, "hipMalloc(sort ids)"));
    MF_TRY(mf_init_idx_arr(d_idx.as<uint32_t>(), n, nullptr));
    MF_TRY(mf_sort_by_count(d_cnt_in.as<uint32_t>(), d_idx.as<uint32_t>(), n, nullptr));
    s.sorted_cnt.resize(n); s.sorted_id.resize(n);
    HIP_TRY(hipMemcpy(s.sorted_cnt.data(), d_cnt_in.p, (size_t)n * 4, hipMemcpyDeviceToHost), "D2H sorted counts");
    HIP_TRY(hipMemcpy(s.sorted_id.data(), d_idx.p, (size_t)n * 4, hipMemcpyDeviceToHost), "D2H sorted ids");
    s.end_idx.resize(n);
    s.groups = mf_group_end_indices(s.sorted_cnt.data(), n, requested_groups, s.end_idx.data());
    if (s.groups == 0) return invalid("mf_train: grouping produced no group (no rated rows)");
    s.end_idx.resize(s.groups);
    s.id2sorted.resize(n); s.id2group.resize(n); s.group_size.assign(s.groups, 0);
    uint32_t end = 0;
    for (uint32_t g = 0; g < s.groups; ++g) {                      // preprocess_utils.h:171-187
        const uint32_t start = end;
        end = s.end_idx[g] + 1;
        for (uint32_t pos = start; pos < end; ++pos) s.id2group[s.sorted_id[pos]] = g;
    }
    for (uint32_t pos = 0; pos < n; ++pos) {                       // :223-241
        s.id2sorted[s.sorted_id[pos]] = pos;
        s.group_size[s.id2group[s.sorted_id[pos]]]++;
    }
    return 0;
}

int alloc_side_storage(Side& s, uint32_t norm_blocks)
{
    const size_t align = 256;
    s.half_off.resize(s.groups); s.float_off.resize(s.groups);
    size_t hb = 0, fb = 0;
    for (uint32_t g = 0; g < s.groups; ++g) {
        s.half_off[g] = hb; hb += ((size_t)s.group_size[g] * s.k * 2 + align - 1) / align * align;
        s.float_off[g] = fb; fb += ((size_t)s.group_size[g] * s.k * 4 + align - 1) / align * align;
    }
    MF_TRY(s.half_arena.alloc(hb, "hipMalloc(binary16 arena)"));
    MF_TRY(s.float_arena.alloc(fb, "hipMalloc(binary32 arena)"));
    s.prec.assign(s.groups, 0);
    s.ptr.resize(s.groups);
    for (uint32_t g = 0; g < s.groups; ++g) s.ptr[g] = reinterpret_cast<uint64_t>(s.half_arena.p) + s.half_off[g];
    MF_TRY(s.d_ptr.alloc((size_t)s.groups * 8, "hipMalloc(group pointers)"));
    MF_TRY(s.d_end.alloc((size_t)s.groups * 4, "hipMalloc(group end idx)"));
    MF_TRY(s.d_prec.alloc(s.groups, "hipMalloc(group prec)"));
    MF_TRY(s.d_grad_sum.alloc((size_t)s.groups * s.k * 4, "hipMalloc(grad_sum_norm)"));
    MF_TRY(s.d_norm_sum.alloc((size_t)s.groups * norm_blocks * 4, "hipMalloc(norm_sum)"));
    MF_TRY(s.d_error.alloc((size_t)s.groups * 4, "hipMalloc(group error)"));
    MF_TRY(s.d_initial.alloc((size_t)s.groups * 4, "hipMalloc(initial error)"));
    HIP_TRY(hipMemcpy(s.d_ptr.p, s.ptr.data(), (size_t)s.groups * 8, hipMemcpyHostToDevice), "H2D group pointers");
    HIP_TRY(hipMemcpy(s.d_end.p, s.end_idx.data(), (size_t)s.groups * 4, hipMemcpyHostToDevice), "H2D group end idx");
    HIP_TRY(hipMemset(s.d_prec.p, 0, s.groups), "memset group prec");
    HIP_TRY(hipMemset(s.d_grad_sum.p, 0, (size_t)s.groups * s.k * 4), "memset grad_sum_norm");
    s.error.assign(s.groups, 0.f);
    s.initial_error.assign(s.groups, 1.0f);                        // mf_methods.cu:149-150
    HIP_TRY(hipMemcpy(s.d_initial.p, s.initial_error.data(), (size_t)s.groups * 4, hipMemcpyHostToDevice), "H2D initial error");
    return 0;
}

// precision_switching_by_groups_grad_diversity, precision_switching.h:8-51, for one side
int switch_side(Side& s, float threshold)
{
    bool changed = false;
    for (uint32_t g = 0; g < s.groups; ++g) {
        if (s.error[g] > threshold && s.prec[g] == 0) {
            float* dst = reinterpret_cast<float*>(static_cast<char*>(s.float_arena.p) + s.float_off[g]);
            const uint16_t* src = reinterpret_cast<const uint16_t*>(s.ptr[g]);
            MF_TRY(mf_transform_half2float(src, dst, (uint64_t)s.group_size[g] * s.k, nullptr));
            s.ptr[g] = reinterpret_cast<uint64_t>(dst);
            s.prec[g] = 1;
            changed = true;
        }
    }
    if (changed) {
        HIP_TRY(hipMemcpy(s.d_prec.p, s.prec.data(), s.groups, hipMemcpyHostToDevice), "H2D group prec");
        HIP_TRY(hipMemcpy(s.d_ptr.p, s.ptr.data(), (size_t)s.groups * 8, hipMemcpyHostToDevice), "H2D group pointers");
    }
    return 0;
}

void print_errors(const char* title, const Side& s)
{
    std::printf("\n%s\n", title);
    for (uint32_t g = 0; g < s.groups; ++g) {
        if (s.error[g] == -1) std::printf("-1 "); else std::printf("%g ", (double)s.error[g]);
    }
}

int train_mascot(Common& c, float* p, float* q)
{
    const mf_params& prm = *c.prm;
    const size_t pn = (size_t)c.n_users * c.k, qn = (size_t)c.n_items * c.k;
    Side U, I;
    const double pre0 = now_ms();
    {   // histogram (train only), sort, grouping, re-index of train and test (mf_methods.cu:54-66)
        DevBuf d_ucnt, d_icnt;
        MF_TRY(d_ucnt.alloc((size_t)c.n_users * 4, "hipMalloc(user counts)"));
        MF_TRY(d_icnt.alloc((size_t)c.n_items * 4, "hipMalloc(item counts)"));
        HIP_TRY(hipMemset(d_ucnt.p, 0, (size_t)c.n_users * 4), "memset");
        HIP_TRY(hipMemset(d_icnt.p, 0, (size_t)c.n_items * 4), "memset");
        MF_TRY(mf_user_item_histogram(c.d_R.as<mf_node>(), c.n, d_ucnt.as<uint32_t>(), d_icnt.as<uint32_t>(), nullptr));
        MF_TRY(build_side(U, d_ucnt, c.n_users, prm.user_group_num, c.k));
        MF_TRY(build_side(I, d_icnt, c.n_items, prm.item_group_num, c.k));
    }
    if (prm.verbose) {      // preprocess_utils.h:192-206
        std::printf("The number of user groups   : %u\nThe number of item groups   : %u\n", U.groups, I.groups);
        for (uint32_t g = 0; g < U.groups; ++g) std::printf("%u ", U.end_idx[g]);
        std::printf("\n\n");
        for (uint32_t g = 0; g < I.groups; ++g) std::printf("%u ", I.end_idx[g]);
        std::printf("\n");      // the reference leaves the line open, so its first epoch line lands on it
        std::fflush(stdout);
    }
    DevBuf d_u2s, d_i2s;
    MF_TRY(d_u2s.alloc((size_t)c.n_users * 4, "hipMalloc(user2sorted)"));
    MF_TRY(d_i2s.alloc((size_t)c.n_items * 4, "hipMalloc(item2sorted)"));
    HIP_TRY(hipMemcpy(d_u2s.p, U.id2sorted.data(), (size_t)c.n_users * 4, hipMemcpyHostToDevice), "H2D user2sorted");
    HIP_TRY(hipMemcpy(d_i2s.p, I.id2sorted.data(), (size_t)c.n_items * 4, hipMemcpyHostToDevice), "H2D item2sorted");
    MF_TRY(mf_matrix_reconst_triplet(c.d_R.as<mf_node>(), d_u2s.as<uint32_t>(), d_i2s.as<uint32_t>(), c.n, nullptr));
    MF_TRY(mf_matrix_reconst_triplet(c.d_test.as<mf_node>(), d_u2s.as<uint32_t>(), d_i2s.as<uint32_t>(), c.test_n, nullptr));

    const uint32_t norm_blocks = mf_mascot_norm_blocks(prm.num_workers);
    MF_TRY(alloc_side_storage(U, norm_blocks));
    MF_TRY(alloc_side_storage(I, norm_blocks));
    {   // cpy2grouped_parameters_gpu_for_comparison_indexing, model_init.cu:175-222
        DevBuf d_dense, d_id2group;
        MF_TRY(d_dense.alloc(std::max(pn, qn) * 4, "hipMalloc(dense init)"));
        MF_TRY(d_id2group.alloc((size_t)std::max(c.n_users, c.n_items) * 4, "hipMalloc(id2group)"));
        HIP_TRY(hipMemcpy(d_dense.p, p, pn * 4, hipMemcpyHostToDevice), "H2D P");
        HIP_TRY(hipMemcpy(d_id2group.p, U.id2group.data(), (size_t)c.n_users * 4, hipMemcpyHostToDevice), "H2D user2group");
        MF_TRY(mf_cpyparams2grouped_params(d_dense.as<float>(), U.d_ptr.as<void*>(), U.d_end.as<uint32_t>(), d_id2group.as<uint32_t>(),
                                           d_u2s.as<uint32_t>(), (int)c.k, c.n_users, U.groups, nullptr));
        HIP_TRY(hipDeviceSynchronize(), "synchronize");
        HIP_TRY(hipMemcpy(d_dense.p, q, qn * 4, hipMemcpyHostToDevice), "H2D Q");
        HIP_TRY(hipMemcpy(d_id2group.p, I.id2group.data(), (size_t)c.n_items * 4, hipMemcpyHostToDevice), "H2D item2group");
        MF_TRY(mf_cpyparams2grouped_params(d_dense.as<float>(), I.d_ptr.as<void*>(), I.d_end.as<uint32_t>(), d_id2group.as<uint32_t>(),
                                           d_i2s.as<uint32_t>(), (int)c.k, c.n_items, I.groups, nullptr));
        HIP_TRY(hipDeviceSynchronize(), "synchronize");
    }
    HotRows hot;      // rows are in popularity-sorted order: the sorted counts index them directly
    MF_TRY(hot.install(prm, U.sorted_cnt.data(), c.n_users, I.sorted_cnt.data(), c.n_items, c.n));
    if (c.rep) c.rep->preprocess_ms = now_ms() - pre0;

    const uint32_t start_idx = 5;                                   // mf_methods.cu:110
    const uint32_t total = c.update_count * c.update_vector_size;
    Timer t;
    for (uint32_t e = 0; e < prm.epoch; ++e) {
        MF_TRY(hot.select(e));
        const uint32_t first_sample = mf_first_sample_rating_idx(e, prm.interval, prm.epoch, c.update_count, c.update_vector_size, prm.sample_ratio);
        const bool error_check = first_sample < total || (prm.interval && e >= start_idx && (e % prm.interval == start_idx % prm.interval) && prm.epoch - 1 != e);
        double err_ms = 0;
        if (error_check) {          // mf_methods.cu:178-182
            const double e0 = now_ms();
            HIP_TRY(hipMemsetAsync(U.d_grad_sum.p, 0, (size_t)U.groups * c.k * 4, nullptr), "memset grad_sum_norm_p");
            HIP_TRY(hipMemsetAsync(I.d_grad_sum.p, 0, (size_t)I.groups * c.k * 4, nullptr), "memset grad_sum_norm_q");
            err_ms += now_ms() - e0;
        }
        t.start();
        MF_TRY(mf_mascot_sgd_hogwild(c.d_R.as<mf_node>(), c.n, U.d_ptr.as<void*>(), I.d_ptr.as<void*>(), (int)c.k,
                                     prm.num_workers, c.update_count, c.update_vector_size, c.lr[e], prm.lambda,
                                     U.d_end.as<uint32_t>(), I.d_end.as<uint32_t>(), U.d_prec.as<uint8_t>(), I.d_prec.as<uint8_t>(),
                                     U.d_grad_sum.as<float>(), I.d_grad_sum.as<float>(), U.d_norm_sum.as<float>(), I.d_norm_sum.as<float>(),
                                     first_sample, U.groups, I.groups, prm.seed, e, nullptr, nullptr));
        const float sgd_ms = t.stop();
        if (error_check) {          // mf_methods.cu:316-389
            const double e0 = now_ms();
            MF_TRY(mf_group_error(U.d_grad_sum.as<float>(), U.d_norm_sum.as<float>(), norm_blocks, U.d_prec.as<uint8_t>(), U.d_initial.as<float>(),
                                  U.d_error.as<float>(), (int)c.k, U.groups, nullptr));
            MF_TRY(mf_group_error(I.d_grad_sum.as<float>(), I.d_norm_sum.as<float>(), norm_blocks, I.d_prec.as<uint8_t>(), I.d_initial.as<float>(),
                                  I.d_error.as<float>(), (int)c.k, I.groups, nullptr));
            HIP_TRY(hipMemcpy(U.error.data(), U.d_error.p, (size_t)U.groups * 4, hipMemcpyDeviceToHost), "D2H user group error");
            HIP_TRY(hipMemcpy(I.error.data(), I.d_error.p, (size_t)I.groups * 4, hipMemcpyDeviceToHost), "D2H item group error");
            if (prm.verbose) { print_errors("<User groups>", U); print_errors("<Item groups>", I); std::printf("\n"); }
            if (e == start_idx) {   // :381-388
                U.initial_error = U.error; I.initial_error = I.error;
                HIP_TRY(hipMemcpy(U.d_initial.p, U.initial_error.data(), (size_t)U.groups * 4, hipMemcpyHostToDevice), "H2D initial error");
                HIP_TRY(hipMemcpy(I.d_initial.p, I.initial_error.data(), (size_t)I.groups * 4, hipMemcpyHostToDevice), "H2D initial error");
            }
            err_ms += now_ms() - e0;
            if (e > start_idx) {    // :392
                const double s0 = now_ms();
                MF_TRY(switch_side(U, prm.error_threshold));
                MF_TRY(switch_side(I, prm.error_threshold));
                HIP_TRY(hipDeviceSynchronize(), "synchronize");
                if (c.rep) c.rep->switching_ms += now_ms() - s0;
            }
        }
        if (c.rep) c.rep->error_ms += err_ms;
        HIP_TRY(hipMemsetAsync(c.d_sum_sq.p, 0, sizeof(double), nullptr), "memset rmse accumulator");
        MF_TRY(mf_test_rmse_grouped(c.d_test.as<mf_node>(), c.test_n, U.d_ptr.as<void*>(), I.d_ptr.as<void*>(), (int)c.k,
                                    U.d_end.as<uint32_t>(), I.d_end.as<uint32_t>(), U.d_prec.as<uint8_t>(), I.d_prec.as<uint8_t>(),
                                    U.groups, I.groups, c.d_sum_sq.as<double>(), nullptr));
        double rmse = 0;
        MF_TRY(finish_rmse(c, &rmse));
        MF_TRY(report_epoch(c, e, rmse, sgd_ms));
    }

    {   // trained model back to the host in sorted row order (what save_trained_model_reconst writes)
        DevBuf d_dense;
        MF_TRY(d_dense.alloc(std::max(pn, qn) * 4, "hipMalloc(dense out)"));
        MF_TRY(mf_grouped_params2dense(U.d_ptr.as<void*>(), U.d_end.as<uint32_t>(), U.d_prec.as<uint8_t>(), d_dense.as<float>(), (int)c.k, c.n_users, U.groups, nullptr));
        HIP_TRY(hipMemcpy(p, d_dense.p, pn * 4, hipMemcpyDeviceToHost), "D2H P");
        MF_TRY(mf_grouped_params2dense(I.d_ptr.as<void*>(), I.d_end.as<uint32_t>(), I.d_prec.as<uint8_t>(), d_dense.as<float>(), (int)c.k, c.n_items, I.groups, nullptr));
        HIP_TRY(hipMemcpy(q, d_dense.p, qn * 4, hipMemcpyDeviceToHost), "D2H Q");
    }
    if (c.rep) {
        mf_report& r = *c.rep;
        r.user_group_num = U.groups; r.item_group_num = I.groups;
        if (r.user2sorted_idx) std::copy(U.id2sorted.begin(), U.id2sorted.end(), r.user2sorted_idx);
        if (r.item2sorted_idx) std::copy(I.id2sorted.begin(), I.id2sorted.end(), r.item2sorted_idx);
        if (r.user_group_end_idx) std::copy(U.end_idx.begin(), U.end_idx.end(), r.user_group_end_idx);
        if (r.item_group_end_idx) std::copy(I.end_idx.begin(), I.end_idx.end(), r.item_group_end_idx);
        if (r.user_group_prec_info) std::copy(U.prec.begin(), U.prec.end(), r.user_group_prec_info);
        if (r.item_group_prec_info) std::copy(I.prec.begin(), I.prec.end(), r.item_group_prec_info);
        if (r.test_reconst && c.test_n) HIP_TRY(hipMemcpy(r.test_reconst, c.d_test.p, (size_t)c.test_n * sizeof(mf_node), hipMemcpyDeviceToHost), "D2H test");   // mf_methods.cu:399
    }
    return 0;
}

}  // namespace

extern "C" {

void mf_default_params(mf_params* out)       // main.cu:19-32
{
    std::memset(out, 0, sizeof *out);
    out->lambda = 0.015f; out->learning_rate = 0.01f; out->decay = 0.1f; out->sample_ratio = 0.01f; out->error_threshold = 0.001f;
    out->k = 128; out->epoch = 50; out->num_workers = 2048; out->thread_block_size = 128;
    out->user_group_num = 10; out->item_group_num = 10; out->version = 7; out->interval = 1; out->seed = 1;
    out->hot_row_inflight = 2.0f; out->hot_row_inflight_early = 8.0f; out->hot_row_early_epochs = 2;   // no reference counterpart: see mf_set_hot_row_thinning
}

uint32_t mf_group_end_indices(const uint32_t* sorted_cnt, uint32_t n, uint32_t requested_groups, uint32_t* end_idx_out)
{
    if (!sorted_cnt || !end_idx_out || n == 0 || requested_groups == 0) return 0;
    const uint32_t threshold = (uint32_t)std::ceil(n / (float)requested_groups);
    const uint32_t max_cnt = sorted_cnt[n - 1];
    std::vector<uint32_t> last_pos((size_t)max_cnt + 1, 0xffffffffu);
    for (uint32_t i = 0; i < n; ++i) last_pos[sorted_cnt[i]] = i;
    uint32_t groups = 0, acc = 0, prev = 0;
    for (uint32_t cnt = 1; cnt <= max_cnt; ++cnt) {
        if (last_pos[cnt] == 0xffffffffu) continue;
        acc += last_pos[cnt] - prev + 1;
        if (acc >= threshold) { end_idx_out[groups++] = last_pos[cnt]; acc = 0; }
        else if (cnt == max_cnt) { end_idx_out[groups++] = last_pos[cnt]; }
        prev = last_pos[cnt] + 1;
    }
    return groups;
}

int mf_init_model(float* p, float* q, uint32_t n_users, uint32_t n_items, uint32_t k, uint64_t seed, int half_rounded)
{
    if (!p || !q) return invalid("mf_init_model: null pointer");
    if (k != 64 && k != 128) return invalid("mf_init_model: k must be 64 or 128 (got %u)", k);
    const size_t pn = (size_t)n_users * k, qn = (size_t)n_items * k;
    DevBuf d, dh;
    MF_TRY(d.alloc(std::max(pn, qn) * 4 + 8, "hipMalloc(init)"));
    if (half_rounded) MF_TRY(dh.alloc(std::max(pn, qn) * 2 + 8, "hipMalloc(init half)"));
    for (int side = 0; side < 2; ++side) {
        const size_t cnt = side ? qn : pn;
        MF_TRY(mf_init_rand_feature(d.as<float>(), cnt, seed, (uint64_t)side, nullptr));
        if (half_rounded) {     // conversion_features_half + transform_feature_vector_half2float (model_init.cu:224-264)
            MF_TRY(mf_transform_float2half(d.as<float>(), dh.as<uint16_t>(), cnt, nullptr));
            MF_TRY(mf_transform_half2float(dh.as<uint16_t>(), d.as<float>(), cnt, nullptr));
        }
        HIP_TRY(hipMemcpy(side ? q : p, d.p, cnt * 4, hipMemcpyDeviceToHost), "D2H init");
    }
    return 0;
}

int mf_gpu_test_rmse(const mf_node* test, uint32_t test_n, const float* p, const float* q, uint32_t n_users, uint32_t n_items, int k, double* rmse)
{
    if (!rmse) return invalid("mf_gpu_test_rmse: null result pointer");
    *rmse = 0;
    if (test_n == 0) return invalid("mf_gpu_test_rmse: empty test set");
    if (!test || !p || !q) return invalid("mf_gpu_test_rmse: null pointer");
    if (k != 64 && k != 128) return invalid("mf_gpu_test_rmse: k must be 64 or 128 (got %d)", k);
    for (uint32_t i = 0; i < test_n; ++i)        // the kernel indexes P and Q with these
        if (test[i].u >= n_users || test[i].i >= n_items)
            return invalid("mf_gpu_test_rmse: test rating %u names user %u / item %u, the model has %u users and %u items", i, test[i].u, test[i].i, n_users, n_items);
    DevBuf d_test, d_p, d_q, d_sum;
    MF_TRY(d_test.alloc((size_t)test_n * sizeof(mf_node), "hipMalloc(test set)"));
    MF_TRY(d_p.alloc((size_t)n_users * k * 4, "hipMalloc(P)"));
    MF_TRY(d_q.alloc((size_t)n_items * k * 4, "hipMalloc(Q)"));
    MF_TRY(d_sum.alloc(8, "hipMalloc(sum)"));
    HIP_TRY(hipMemcpy(d_test.p, test, (size_t)test_n * sizeof(mf_node), hipMemcpyHostToDevice), "H2D test set");
    HIP_TRY(hipMemcpy(d_p.p, p, (size_t)n_users * k * 4, hipMemcpyHostToDevice), "H2D P");
    HIP_TRY(hipMemcpy(d_q.p, q, (size_t)n_items * k * 4, hipMemcpyHostToDevice), "H2D Q");
    HIP_TRY(hipMemset(d_sum.p, 0, 8), "memset sum");
    MF_TRY(mf_test_rmse(d_test.as<mf_node>(), test_n, d_p.as<float>(), d_q.as<float>(), k, d_sum.as<double>(), nullptr));
    double sum = 0;
    HIP_TRY(hipMemcpy(&sum, d_sum.p, 8, hipMemcpyDeviceToHost), "D2H sum");
    *rmse = std::sqrt(sum / (double)test_n);
    return MF_OK;
}

int mf_hot_row_table(const uint32_t* counts, uint32_t rows, uint32_t n, uint32_t num_workers, float inflight_cap, uint8_t* table)
{
    if (rows == 0) return MF_OK;
    if (!counts || !table) return invalid("mf_hot_row_table: null pointer");
    if (n == 0 || num_workers == 0) return invalid("mf_hot_row_table: no ratings or no workers");
    if (!(inflight_cap > 0)) return invalid("mf_hot_row_table: the cap must be positive");
    const std::vector<uint8_t> t = keep_table(counts, rows, n, num_workers, inflight_cap);
    std::memcpy(table, t.data(), rows);
    return MF_OK;
}

uint32_t mf_auto_workers(uint32_t n)
{
    // about 128 windows of 128 ratings per worker: the ratio at which the runs on 8M and on 100M ratings stay
    // within 0.005 test RMSE of the reference rule run on the CPU; at most 24 wavefronts on each of the 256 CUs
    uint32_t w = (n / 16384u + 3u) / 4u * 4u;
    return w < 16u ? 16u : (w > 6144u ? 6144u : w);
}

int mf_train(const mf_params* params, const mf_node* R, uint32_t n, uint32_t n_users, uint32_t n_items,
             const mf_node* test, uint32_t test_n, float* p, float* q, mf_report* report)
{
    if (!params || !R || !p || !q) return invalid("mf_train: null pointer");
    if (test_n && !test) return invalid("mf_train: null test set");
    if (params->k != 64 && params->k != 128) return invalid("mf_train: k must be 64 or 128 (got %u)", params->k);
    if (n == 0 || n_users == 0 || n_items == 0) return invalid("mf_train: empty problem");
    mf_params with_workers = *params;
    if (with_workers.num_workers == 0) with_workers.num_workers = mf_auto_workers(n);
    params = &with_workers;
    const uint32_t version = params->version == 0 ? 5 : params->version;
    if (version < 1 || version > 8) return invalid("mf_train: version %u does not exist (1 MASCOT, 2 AFP, 3 MuPPET, 4 MPT, 5 fp32 SGD, 6 MASCOT, 7 binary16 storage, 8 whole-model switching)", params->version);
    Common c;
    c.prm = params; c.n = n; c.n_users = n_users; c.n_items = n_items; c.test_n = test_n; c.k = params->k; c.rep = report;
    if (report) { report->preprocess_ms = report->switching_ms = report->error_ms = report->sgd_ms = report->total_ms = 0; report->muppet_final_bits = 0; }
    const double t0 = now_ms();
    const int saved_coherence = mf_get_row_coherence();
    const uint32_t saved_splits = mf_get_epoch_splits();
    MF_TRY(mf_set_row_coherence(params->cached_rows ? 0 : 1));
    MF_TRY(mf_set_epoch_splits(params->epoch_splits ? params->epoch_splits : 1));
    struct Restore { int c; uint32_t s; ~Restore() { (void)mf_set_row_coherence(c); (void)mf_set_epoch_splits(s); } } restore{saved_coherence, saved_splits};
    fill_schedule(c);
    MF_TRY(upload_and_shuffle(c, R, test));
    // -v 6 (mascot_training_mf_naive, mf_methods.cu:926-1301) is MASCOT with the group search done from global memory
    // and shifted end-index tables: the same schedule, arithmetic and epoch logic, so it runs the MASCOT path
    const int rc = (version == 1 || version == 6) ? train_mascot(c, p, q) : train_dense(c, p, q);
    if (rc == 0 && report) report->total_ms = now_ms() - t0;
    return rc;
}

}  // extern "C"
