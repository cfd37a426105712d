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
#include <functional>
#include <memory>
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
    float mean_rating = 0.f;                 // mean |rating| of the training set
    DevBuf d_R, d_test, d_sum_sq;
    std::vector<float> lr;
    std::vector<double> rmse_hist;           // per epoch, whether or not the caller passed a report
    std::vector<float> ms_hist;
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
    c.lr.resize(p.epoch); c.rmse_hist.assign(p.epoch, 0.0); c.ms_hist.assign(p.epoch, 0.f);
    for (uint32_t e = 0; e < p.epoch; ++e) c.lr[e] = mf_lr_schedule(p.learning_rate, p.decay, e);
    if (c.rep) {
        c.rep->update_count = c.update_count;
        if (c.rep->lr_per_epoch) std::copy(c.lr.begin(), c.lr.end(), c.rep->lr_per_epoch);
    }
}

int report_epoch(Common& c, uint32_t e, double rmse, float sgd_ms)
{
    c.rmse_hist[e] = rmse; c.ms_hist[e] = sgd_ms;
    if (c.rep) {
        if (c.rep->rmse_per_epoch) c.rep->rmse_per_epoch[e] = rmse;
        if (c.rep->sgd_ms_per_epoch) c.rep->sgd_ms_per_epoch[e] = sgd_ms;
        c.rep->sgd_ms += sgd_ms;
    }
    if (c.prm->verbose) { std::printf("%u %g %g\n", e + 1, (double)c.lr[e], rmse); std::fflush(stdout); }   // mf_methods.cu:396
    if (c.test_n && !std::isfinite(rmse))
        return invalid("mf_train: the model diverged in epoch %u (the test RMSE is not finite); lower the learning rate, or the "
                       "number of updates in flight up to which a popular row is added to (replicate_inflight; the thinning caps "
                       "hot_row_inflight_early and hot_row_inflight if thinning is on)", e + 1);
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

// Hot-row table of one side from its rating counts (mf_hogwild_options::user_keep): a row with count c has about
// inflight * c / n updates in flight.  Rows with more than one are hot rows: above replicate_above they get a copy per
// XCD (numbered in row order; at most 65535, the most popular ones; updates are stored in the copy, or added to it
// while the XCD's share of them is within add_within), above thin_above they are thinned to that many updates in
// flight, the rest have their updates added.
struct KeepTable { std::vector<uint8_t> keep; std::vector<uint16_t> slot; std::vector<uint32_t> slot_row; };
KeepTable keep_table(const uint32_t* cnt, uint32_t rows, uint32_t n, double inflight, double replicate_above, double thin_above, double add_within = 0)
{
    KeepTable t;
    t.keep.resize(rows); t.slot.assign(rows, 0);
    // the 65535 slots go to the highest counts: raise the bar to the count of the 65536th candidate
    double min_replicated = replicate_above > 0 ? replicate_above : 1e300;
    if (replicate_above > 0) {
        std::vector<uint32_t> cand;
        for (uint32_t r = 0; r < rows; ++r) if (inflight * (double)cnt[r] / (double)n > replicate_above) cand.push_back(cnt[r]);
        if (cand.size() > 65535u) {
            std::nth_element(cand.begin(), cand.begin() + 65535, cand.end(), std::greater<uint32_t>());
            min_replicated = inflight * (double)cand[65535] / (double)n;      // strictly above this one
        }
    }
    for (uint32_t r = 0; r < rows; ++r) {
        const double fly = inflight * (double)cnt[r] / (double)n;
        if (fly <= 1.0) { t.keep[r] = MF_KEEP_ORDINARY; continue; }
        if (fly > min_replicated && t.slot_row.size() < 65535u) {
            // each XCD's copy sees an eighth of the row's updates: a caller may have those added to the copy while they
            // are few (add_within per XCD); otherwise, and above, they are stored (last writer wins inside the XCD)
            t.keep[r] = fly <= add_within * MF_XCDS ? MF_KEEP_REPLICATED_ADDED : MF_KEEP_REPLICATED;
            t.slot[r] = (uint16_t)t.slot_row.size(); t.slot_row.push_back(r);
            continue;
        }
        if (thin_above > 0 && fly > thin_above) {
            const int v = (int)std::floor(thin_above / fly * 255.0) - 1;
            t.keep[r] = (uint8_t)(v < 0 ? 0 : (v > 251 ? 251 : v));
            continue;
        }
        t.keep[r] = MF_KEEP_ADDED;
    }
    return t;
}

// The launch options of a run (mf_hogwild_options) and the device arrays they name: the hot-row tables of both sides
// -- two pairs when rows are thinned, an early cap for the first epochs, while every row still grows from its small
// initial value and the popular rows need many updates, and the steady cap afterwards -- and the replica arrays.
struct HotRows {
    // One set of tables: a keep byte per row, and the numbering of the replicated rows.  A run has up to three sets:
    // `low` for the first epochs when those run with fewer updates in flight (mf_params::early_inflight: fewer rows are
    // hot then), `steady` up to epoch late_from, and `late` from there on, with a lower bar for replication
    // (mf_params::replicate_inflight_late).  The copies of all sets share one array per side, sized for the most slots.
    struct TableSet {
        DevBuf keep, slot, slot_row; uint32_t slots = 0;
        int upload_from(const KeepTable& t, uint32_t rows)
        {
            slots = (uint32_t)t.slot_row.size();
            MF_TRY(upload(keep, t.keep.data(), rows, "hot-row table"));
            if (slots) {
                MF_TRY(upload(slot, t.slot.data(), (size_t)rows * 2, "replica slots"));
                MF_TRY(upload(slot_row, t.slot_row.data(), (size_t)slots * 4, "replica rows"));
            }
            return 0;
        }
    };
    struct SideTables { TableSet steady, low, late; DevBuf early, replicas; };
    SideTables u, v;
    mf_hogwild_options opt_early{}, opt_steady{}, opt_low{}, opt_late{};
    uint32_t low_epochs = 0, late_from = 0xffffffffu;
    mutable mf_hogwild_options opt_current{};
    uint32_t early_epochs = 0;
    float step_scale = 0.f; uint32_t step_epochs = 0;      // scaled steps on replicated rows during the first step_epochs epochs (0: all)
    double inflight = 0, replicate_above = 0, replicate_above_late = 0;
    static constexpr double kLateBarMinInflight = 4096.0;
    static bool wanted(const mf_params& prm) { return prm.hot_rows || prm.hot_row_inflight > 0 || prm.replicate_inflight > 0; }
    static int upload(DevBuf& d, const void* src, size_t bytes, const char* what)
    {
        MF_TRY(d.alloc(bytes, what));
        if (bytes) HIP_TRY(hipMemcpy(d.p, src, bytes, hipMemcpyHostToDevice), what);
        return 0;
    }
    static void point_at(mf_hogwild_options& o, const TableSet& us, const TableSet& vs)
    {
        o.user_keep = us.keep.as<uint8_t>(); o.item_keep = vs.keep.as<uint8_t>();
        o.user_slot = us.slot.as<uint16_t>(); o.item_slot = vs.slot.as<uint16_t>();
        o.user_slot_row = us.slot_row.as<uint32_t>(); o.item_slot_row = vs.slot_row.as<uint32_t>();
        o.user_slots = us.slots; o.item_slots = vs.slots;
    }
    int install(const mf_params& prm, const uint32_t* ucnt, uint32_t n_users, const uint32_t* icnt, uint32_t n_items, uint32_t n,
                uint32_t user_groups, uint32_t item_groups, float mean_rating)
    {
        opt_steady = mf_hogwild_options{};
        opt_steady.cached_rows = prm.cached_rows ? 1u : 0u;
        opt_steady.launches = prm.epoch_splits ? prm.epoch_splits : 1u;
        opt_early = opt_steady;
        low_epochs = 0; late_from = 0xffffffffu;
        if (!wanted(prm)) return 0;
        step_scale = prm.replica_step_scale < 0 ? mf_replica_step_scale(prm.learning_rate, mean_rating) : prm.replica_step_scale;
        // MuPPET takes no longer steps by default.  Measured at 100M ratings, learning rate 0.01, first epoch with half the
        // updates in flight: the other rules run at factors 4.3 (their default) and 6 and diverge at 7 or 8; MuPPET with its
        // 8-bit passes left rows of the order of 1e7 in 6 of 6 runs at 4.3 and in 4 of 12 at 2, at random, and none in 16
        // unscaled runs (test RMSE after the epoch 1.091-1.101 at k = 128; scaled and with all updates in flight:
        // 1.098-1.105 in 10 of 10 runs, 10 ms sooner).
        if (prm.replica_step_scale < 0 && prm.version == 3) step_scale = 0.f;
        step_epochs = prm.replica_step_epochs;
        inflight = mf_hogwild_inflight(prm.version, (int)prm.k, prm.num_workers, user_groups, item_groups);
        if (!(inflight > 0)) return invalid("mf_train: cannot determine the number of updates in flight (%s)", mf_last_error());
        replicate_above = prm.replicate_inflight > 0 ? prm.replicate_inflight : (prm.replicate_inflight < 0 ? mf_replicate_threshold(prm.learning_rate, mean_rating) : 0.0);
        const bool early = prm.hot_row_inflight > 0 && prm.hot_row_inflight_early > prm.hot_row_inflight && prm.hot_row_early_epochs > 0;
        early_epochs = early ? prm.hot_row_early_epochs : 0;
        const uint32_t* cnt[2] = {ucnt, icnt};
        const uint32_t rows[2] = {n_users, n_items};
        SideTables* side[2] = {&u, &v};
        for (int s = 0; s < 2; ++s) {
            MF_TRY(side[s]->steady.upload_from(keep_table(cnt[s], rows[s], n, inflight, replicate_above, prm.hot_row_inflight, prm.replica_add_inflight), rows[s]));
            if (early) {
                const KeepTable e = keep_table(cnt[s], rows[s], n, inflight, replicate_above, prm.hot_row_inflight_early, prm.replica_add_inflight);
                MF_TRY(upload(side[s]->early, e.keep.data(), rows[s], "hot-row table"));
            }
        }
        mf_hogwild_options& o = opt_steady;
        point_at(o, u.steady, v.steady);
        // The first epochs with fewer updates in flight: resident workers capped, tables for that many updates in flight.
        // resident = inflight / ratings a worker keeps in flight, which mf_hogwild_inflight folds in: ask it for one worker.
        double low_inflight = 0; uint32_t capped = 0;
        if (prm.early_inflight > 0.f && prm.early_inflight < 1.f && prm.early_inflight_epochs > 0) {
            const double per_worker = mf_hogwild_inflight(prm.version, (int)prm.k, 1, user_groups, item_groups);
            const uint32_t resident = per_worker > 0 ? (uint32_t)(inflight / per_worker + 0.5) : 0;
            capped = (uint32_t)(resident * (double)prm.early_inflight);
            // what a launch held to that many workers really keeps in flight (whole workgroups per compute unit)
            low_inflight = capped >= 1 ? mf_hogwild_inflight_capped(prm.version, (int)prm.k, prm.num_workers, user_groups, item_groups, capped) : 0.0;
            if (!(low_inflight > 0 && low_inflight < inflight)) low_inflight = 0;
        }
        if (low_inflight > 0) {
            const double thin = prm.hot_row_inflight_early > 0 ? prm.hot_row_inflight_early : prm.hot_row_inflight;
            for (int s = 0; s < 2; ++s)
                MF_TRY(side[s]->low.upload_from(keep_table(cnt[s], rows[s], n, low_inflight, replicate_above, thin, prm.replica_add_inflight), rows[s]));
        }
        // Later epochs with a lower bar for replication (more rows kept as copies in the L2s, fewer added to at the memory side)
        replicate_above_late = prm.replicate_inflight_late > 0 ? prm.replicate_inflight_late : (prm.replicate_inflight_late < 0 ? replicate_above / 4.0 : 0.0);
        // (the default only for runs that keep at least kLateBarMinInflight updates in flight: below that an epoch is bound
        // by the latency of a worker's chain of ratings, not by the memory side, so more copies buy little, and at 2M
        // ratings with 124 workers they cost 0.0017 test RMSE after 12 epochs)
        if (prm.replicate_inflight_late < 0 && inflight < kLateBarMinInflight) replicate_above_late = 0.0;
        const bool late = replicate_above > 0 && replicate_above_late > 0 && replicate_above_late < replicate_above && prm.replicate_late_from < prm.epoch;
        if (late) {
            for (int s = 0; s < 2; ++s)
                MF_TRY(side[s]->late.upload_from(keep_table(cnt[s], rows[s], n, inflight, replicate_above_late, prm.hot_row_inflight, prm.replica_add_inflight), rows[s]));
        }
        for (int s = 0; s < 2; ++s) {
            const uint32_t most = std::max(side[s]->steady.slots, std::max(side[s]->low.slots, side[s]->late.slots));
            if (most) MF_TRY(side[s]->replicas.alloc((size_t)MF_XCDS * most * prm.k * 4, "hipMalloc(row replicas)"));
        }
        o.user_replicas = u.replicas.p; o.item_replicas = v.replicas.p;
        const bool any_slots = u.steady.slots || v.steady.slots || u.late.slots || v.late.slots;
        if (any_slots && prm.epoch_splits == 0) {
            // replica_merges = 0: a launch of at least 25M ratings, at most four launches (the end of a launch, where the
            // last workers run alone, costs a short epoch 13 % per extra launch and a 100M-rating one 0.1 %)
            const uint32_t by_size = n / 25000000u;
            o.launches = prm.replica_merges ? prm.replica_merges : (by_size < 1u ? 1u : (by_size > 4u ? 4u : by_size));
        }
        opt_early = o;
        if (early) { opt_early.user_keep = u.early.as<uint8_t>(); opt_early.item_keep = v.early.as<uint8_t>(); }
        if (low_inflight > 0) {
            opt_low = o;
            opt_low.resident_workers = capped;
            point_at(opt_low, u.low, v.low);
            low_epochs = prm.early_inflight_epochs;
        }
        if (late) {
            opt_late = o;
            point_at(opt_late, u.late, v.late);
            late_from = prm.replicate_late_from;
        }
        return 0;
    }
    // options of the launches of epoch e (valid until the next call)
    bool all_binary16 = false;      // MASCOT runs: no group has been promoted yet
    const mf_hogwild_options* options(uint32_t e) const
    {
        opt_current = e < low_epochs ? opt_low : (e >= late_from ? opt_late : (e < early_epochs ? opt_early : opt_steady));
        opt_current.replica_step_scale = (step_epochs == 0 || e < step_epochs) ? step_scale : 0.f;
        opt_current.all_binary16 = all_binary16 ? 1u : 0u;
        return &opt_current;
    }
    // replicated rows per side in the tables most of the run uses
    uint32_t replicated(int side_index) const
    {
        const SideTables& t = side_index ? v : u;
        return late_from != 0xffffffffu ? t.late.slots : t.steady.slots;
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

// A training run as an object: setup() uploads and prepares, epoch(e) runs epoch e (update launches, error estimate,
// switching, test RMSE), download() brings the model back.  mf_train runs all epochs; the mf_session_* entry points
// hand the epochs to the caller one at a time.
struct Run {
    Common c;
    mf_params prm;
    HotRows hot;
    uint32_t next_epoch = 0;
    virtual ~Run() {}
    virtual int setup(const mf_node* R, const mf_node* test, const float* p, const float* q) = 0;
    virtual int epoch(uint32_t e) = 0;
    virtual int download(float* p, float* q) = 0;
    // grouped runs: the groups of one side (0 users, 1 items), and promotion of chosen groups to binary32
    virtual int groups(int, uint32_t* count, uint8_t*, uint64_t*) const { *count = 0; return 0; }
    virtual int promote(int, const uint8_t*, uint32_t) { return invalid("mf_session_promote_groups: this run keeps no groups (version 1 or 6 only)"); }
};

// ---- variants over dense P/Q (versions 2..5, 7, 8) ----------------------------------------------
struct DenseRun : Run {
    uint32_t version = 5;
    size_t pn = 0, qn = 0;
    DevBuf d_p, d_q, d_sum_updated, d_sum_norms, d_hp, d_hq;
    // MPT: loss scale 1000, lambda*1000 rounded to binary16 (mf_methods.cu:764-765)
    const float scaling_factor = 1000;
    uint16_t scaled_lambda_h = 0;
    // MuPPET ladder state (mf_methods.cu:586-601)
    const unsigned char bit_width_set[5] = {8, 12, 14, 16, 32};
    int precision_idx = 0, switched_epoch = -1, violation_times = 0;
    float max_grad_diversity = -1.f;
    const int resolution_size = 3, gamma = 1;
    std::vector<float> sum_norms_epoch, sum_updated_val_epoch, sum_norms, sum_updated;
    uint32_t muppet_first_sample = 0;
    WholeModel whole;
    uint32_t total = 0, whole_sample_num = 0;
    Timer t;

    int setup(const mf_node* R, const mf_node* test, const float* p, const float* q) override
    {
        version = prm.version == 0 ? 5 : prm.version;
        pn = (size_t)c.n_users * c.k; qn = (size_t)c.n_items * c.k;
        MF_TRY(upload_and_shuffle(c, R, test));
        MF_TRY(d_p.alloc(pn * 4, "hipMalloc(P)"));
        MF_TRY(d_q.alloc(qn * 4, "hipMalloc(Q)"));
        HIP_TRY(hipMemcpy(d_p.p, p, pn * 4, hipMemcpyHostToDevice), "H2D P");
        HIP_TRY(hipMemcpy(d_q.p, q, qn * 4, hipMemcpyHostToDevice), "H2D Q");
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
        precision_idx = prm.is_yahoo ? 1 : 0;
        sum_norms_epoch.assign(prm.epoch, 0.f); sum_updated_val_epoch.assign((size_t)prm.epoch * c.k, 0.f);
        sum_norms.resize(prm.num_workers); sum_updated.resize(c.k);
        if (version == 3) {
            MF_TRY(d_sum_updated.alloc(c.k * 4, "hipMalloc(sum_updated_val)"));
            MF_TRY(d_sum_norms.alloc((size_t)prm.num_workers * 4, "hipMalloc(sum_norms)"));
            const int sample_ratings_num = (int)((float)(c.update_count * c.update_vector_size) * prm.sample_ratio);   // :563
            muppet_first_sample = c.update_count * c.update_vector_size - (uint32_t)sample_ratings_num;
        }
        // -v 7: dense binary16 storage next to the fp32 buffers, which then only serve the RMSE and the result
        if (version == 7) {
            MF_TRY(d_hp.alloc(pn * 2, "hipMalloc(binary16 P)"));
            MF_TRY(d_hq.alloc(qn * 2, "hipMalloc(binary16 Q)"));
            MF_TRY(mf_transform_float2half(d_p.as<float>(), d_hp.as<uint16_t>(), pn, nullptr));
            MF_TRY(mf_transform_float2half(d_q.as<float>(), d_hq.as<uint16_t>(), qn, nullptr));
        }
        total = c.update_count * c.update_vector_size;
        whole_sample_num = (uint32_t)(int)((float)total * prm.sample_ratio);       // mf_methods.cu:1425
        if (version == 8) MF_TRY(whole.init(c, d_p.as<float>(), d_q.as<float>(), prm.num_workers));

        std::vector<uint32_t> ucnt, icnt;
        if (HotRows::wanted(prm)) {
            DevBuf d_ucnt, d_icnt;
            MF_TRY(d_ucnt.alloc((size_t)c.n_users * 4, "hipMalloc(user counts)"));
            MF_TRY(d_icnt.alloc((size_t)c.n_items * 4, "hipMalloc(item counts)"));
            HIP_TRY(hipMemset(d_ucnt.p, 0, (size_t)c.n_users * 4), "memset");
            HIP_TRY(hipMemset(d_icnt.p, 0, (size_t)c.n_items * 4), "memset");
            MF_TRY(mf_user_item_histogram(c.d_R.as<mf_node>(), c.n, d_ucnt.as<uint32_t>(), d_icnt.as<uint32_t>(), nullptr));
            ucnt.resize(c.n_users); icnt.resize(c.n_items);
            HIP_TRY(hipMemcpy(ucnt.data(), d_ucnt.p, (size_t)c.n_users * 4, hipMemcpyDeviceToHost), "D2H user counts");
            HIP_TRY(hipMemcpy(icnt.data(), d_icnt.p, (size_t)c.n_items * 4, hipMemcpyDeviceToHost), "D2H item counts");
        }
        return hot.install(prm, ucnt.data(), c.n_users, icnt.data(), c.n_items, c.n, 1, 1, c.mean_rating);
    }

    int epoch(uint32_t e) override
    {
        const mf_node* R = c.d_R.as<mf_node>();
        hot.all_binary16 = version == 8 && !whole.is_float;
        const mf_hogwild_options* opt = hot.options(e);
        bool whole_check = false;
        const double err0 = now_ms();
        if (version == 3) HIP_TRY(hipMemsetAsync(d_sum_updated.p, 0, c.k * 4, nullptr), "memset sum_updated_val");
        double err_ms = now_ms() - err0;
        t.start();
        switch (version) {
        case 5: MF_TRY(mf_single_sgd_hogwild_opt(R, c.n, d_p.as<float>(), d_q.as<float>(), (int)c.k, prm.num_workers, c.update_count, c.update_vector_size,
                                                 c.lr[e], prm.lambda, prm.seed, e, nullptr, nullptr, opt)); break;
        case 4: MF_TRY(mf_mpt_sgd_hogwild_opt(R, c.n, d_p.as<float>(), d_q.as<float>(), (int)c.k, prm.num_workers, c.update_count, c.update_vector_size,
                                              c.lr[e], scaled_lambda_h, scaling_factor, prm.seed, e, nullptr, nullptr, opt)); break;
        case 3: {
            const int idx = precision_idx > 4 ? 4 : precision_idx;      // the reference indexes past the table once at 32 bit (mf_methods.cu:691)
            if (c.rep && c.rep->muppet_bits_per_epoch) c.rep->muppet_bits_per_epoch[e] = bit_width_set[idx];
            MF_TRY(mf_muppet_sgd_hogwild_opt(R, c.n, d_p.as<float>(), d_q.as<float>(), (int)c.k, prm.num_workers, c.update_count, c.update_vector_size,
                                             c.lr[e], prm.lambda, muppet_first_sample, d_sum_updated.as<float>(), d_sum_norms.as<float>(),
                                             bit_width_set[idx], bit_width_set[idx], prm.seed, e, nullptr, nullptr, opt));
            break;
        }
        case 2: MF_TRY(mf_afp_sgd_hogwild_opt(R, c.n, d_p.as<float>(), d_q.as<float>(), (int)c.k, prm.num_workers, c.update_count, c.update_vector_size,
                                              c.lr[e], prm.lambda, (int)e, prm.seed, e, nullptr, nullptr, opt)); break;
        case 7: MF_TRY(mf_mem_quant_sgd_hogwild_opt(R, c.n, d_hp.as<uint16_t>(), d_hq.as<uint16_t>(), (int)c.k, prm.num_workers, c.update_count,
                                                    c.update_vector_size, c.lr[e], prm.lambda, prm.seed, e, nullptr, nullptr, opt)); break;
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
            MF_TRY(mf_mascot_sgd_hogwild_opt(R, c.n, whole.ptr_p.as<void*>(), whole.ptr_q.as<void*>(), (int)c.k, prm.num_workers, c.update_count,
                                             c.update_vector_size, c.lr[e], prm.lambda, whole.end_u.as<uint32_t>(), whole.end_i.as<uint32_t>(),
                                             whole.prec.as<uint8_t>(), whole.prec.as<uint8_t>(), whole.gsp.as<float>(), whole.gsq.as<float>(),
                                             whole.nsp.as<float>(), whole.nsq.as<float>(), whole_check ? total - whole_sample_num : total, 1, 1,
                                             prm.seed, e, nullptr, nullptr, opt));
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
        if (c.rep) {
            c.rep->error_ms += err_ms;
            c.rep->muppet_final_bits = version == 3 ? bit_width_set[precision_idx > 4 ? 4 : precision_idx] : 0;
        }
        return 0;
    }

    int download(float* p, float* q) override
    {
        HIP_TRY(hipMemcpy(p, d_p.p, pn * 4, hipMemcpyDeviceToHost), "D2H P");
        HIP_TRY(hipMemcpy(q, d_q.p, qn * 4, hipMemcpyDeviceToHost), "D2H Q");
        return 0;
    }
};

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

// precision_switching_by_groups_grad_diversity, precision_switching.h:8-51, for one side: the groups whose error
// exceeds the threshold or, with a mask, the groups the mask names
int switch_side(Side& s, float threshold, const uint8_t* mask = nullptr)
{
    bool changed = false;
    for (uint32_t g = 0; g < s.groups; ++g) {
        if ((mask ? mask[g] != 0 : s.error[g] > threshold) && s.prec[g] == 0) {
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

struct MascotRun : Run {
    size_t pn = 0, qn = 0;
    Side U, I;
    uint32_t norm_blocks = 0, total = 0;
    const uint32_t start_idx = 5;                                   // mf_methods.cu:110
    Timer t;

    int setup(const mf_node* R, const mf_node* test, const float* p, const float* q) override
    {
        pn = (size_t)c.n_users * c.k; qn = (size_t)c.n_items * c.k;
        MF_TRY(upload_and_shuffle(c, R, test));
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

        norm_blocks = mf_mascot_norm_blocks(prm.num_workers);
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
        // rows are in popularity-sorted order: the sorted counts index them directly
        MF_TRY(hot.install(prm, U.sorted_cnt.data(), c.n_users, I.sorted_cnt.data(), c.n_items, c.n, U.groups, I.groups, c.mean_rating));
        if (c.rep) c.rep->preprocess_ms = now_ms() - pre0;
        total = c.update_count * c.update_vector_size;
        return 0;
    }

    int epoch(uint32_t e) override
    {
        const uint32_t first_sample = mf_first_sample_rating_idx(e, prm.interval, prm.epoch, c.update_count, c.update_vector_size, prm.sample_ratio);
        const bool error_check = first_sample < total || (prm.interval && e >= start_idx && (e % prm.interval == start_idx % prm.interval) && prm.epoch - 1 != e);
        double err_ms = 0;
        if (error_check) {          // mf_methods.cu:178-182
            const double e0 = now_ms();
            HIP_TRY(hipMemsetAsync(U.d_grad_sum.p, 0, (size_t)U.groups * c.k * 4, nullptr), "memset grad_sum_norm_p");
            HIP_TRY(hipMemsetAsync(I.d_grad_sum.p, 0, (size_t)I.groups * c.k * 4, nullptr), "memset grad_sum_norm_q");
            err_ms += now_ms() - e0;
        }
        hot.all_binary16 = std::none_of(U.prec.begin(), U.prec.end(), [](uint8_t v) { return v != 0; }) &&
                           std::none_of(I.prec.begin(), I.prec.end(), [](uint8_t v) { return v != 0; });
        t.start();
        MF_TRY(mf_mascot_sgd_hogwild_opt(c.d_R.as<mf_node>(), c.n, U.d_ptr.as<void*>(), I.d_ptr.as<void*>(), (int)c.k,
                                         prm.num_workers, c.update_count, c.update_vector_size, c.lr[e], prm.lambda,
                                         U.d_end.as<uint32_t>(), I.d_end.as<uint32_t>(), U.d_prec.as<uint8_t>(), I.d_prec.as<uint8_t>(),
                                         U.d_grad_sum.as<float>(), I.d_grad_sum.as<float>(), U.d_norm_sum.as<float>(), I.d_norm_sum.as<float>(),
                                         first_sample, U.groups, I.groups, prm.seed, e, nullptr, nullptr, hot.options(e)));
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
        return report_epoch(c, e, rmse, sgd_ms);
    }

    int groups(int side, uint32_t* count, uint8_t* prec, uint64_t* ratings) const override
    {
        const Side& s = side ? I : U;
        *count = s.groups;
        if (prec) std::copy(s.prec.begin(), s.prec.end(), prec);
        if (ratings) {      // rows are in sorted order: group g holds rows (end[g-1], end[g]]
            uint32_t row = 0;
            for (uint32_t g = 0; g < s.groups; ++g) {
                uint64_t sum = 0;
                for (; row <= s.end_idx[g]; ++row) sum += s.sorted_cnt[row];
                ratings[g] = sum;
            }
        }
        return 0;
    }
    int promote(int side, const uint8_t* mask, uint32_t count) override
    {
        Side& s = side ? I : U;
        if (count != s.groups) return invalid("mf_session_promote_groups: the side has %u groups, the mask %u entries", s.groups, count);
        MF_TRY(switch_side(s, 0.f, mask));
        HIP_TRY(hipDeviceSynchronize(), "synchronize");
        return 0;
    }

    int download(float* p, float* q) override
    {
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
};

// Checks the arguments of a run and builds its object (nothing touches the device yet).
int make_run(const mf_params* params, const mf_node* R, uint32_t n, uint32_t n_users, uint32_t n_items,
             const mf_node* test, uint32_t test_n, const float* p, const float* q, mf_report* report, Run** out)
{
    if (!params || !R || !p || !q) return invalid("mf_train: null pointer");
    if (test_n && !test) return invalid("mf_train: null test set");
    if (params->k != 64 && params->k != 128) return invalid("mf_train: k must be 64 or 128 (got %u)", params->k);
    if (n == 0 || n_users == 0 || n_items == 0) return invalid("mf_train: empty problem");
    const uint32_t version = params->version == 0 ? 5 : params->version;
    if (version < 1 || version > 8) return invalid("mf_train: version %u does not exist (1 MASCOT, 2 AFP, 3 MuPPET, 4 MPT, 5 fp32 SGD, 6 MASCOT, 7 binary16 storage, 8 whole-model switching)", params->version);
    // -v 6 (mascot_training_mf_naive, mf_methods.cu:926-1301) is MASCOT with the group search done from global memory
    // and shifted end-index tables: the same schedule, arithmetic and epoch logic, so it runs the MASCOT path
    Run* run = (version == 1 || version == 6) ? static_cast<Run*>(new MascotRun) : static_cast<Run*>(new DenseRun);
    run->prm = *params;
    if (run->prm.num_workers == 0) run->prm.num_workers = mf_auto_workers(n);
    else if (run->prm.wg_counts_updates) {
        // -wg as the reference counts it: updates in flight.  A worker here keeps four ratings in flight (two for the
        // fixed-point rules, whose pipeline looks one rating ahead).
        const uint32_t per_worker = (version == 2 || version == 3) ? 2u : 4u;
        run->prm.num_workers = run->prm.num_workers / per_worker ? run->prm.num_workers / per_worker : 1u;
    }
    Common& c = run->c;
    c.prm = &run->prm; c.n = n; c.n_users = n_users; c.n_items = n_items; c.test_n = test_n; c.k = params->k; c.rep = report;
    if (report) { report->preprocess_ms = report->switching_ms = report->error_ms = report->sgd_ms = report->total_ms = 0; report->muppet_final_bits = 0; }
    double sum = 0;
    for (uint32_t i = 0; i < n; ++i) sum += std::fabs((double)R[i].r);
    c.mean_rating = (float)(sum / (double)n);
    fill_schedule(c);
    *out = run;
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
    // no reference counterpart (mf_hogwild_options): rows with more updates in flight than added updates can safely
    // sum (mf_replicate_threshold) get a copy per XCD, averaged four times per epoch; rows with more than one have
    // their updates added; nothing is thinned
    out->hot_rows = 1; out->replicate_inflight = -1.0f; out->replica_merges = 0;
    out->hot_row_inflight = 0.0f; out->hot_row_inflight_early = 0.0f; out->hot_row_early_epochs = 0;
    out->replica_step_scale = -1.0f; out->replica_step_epochs = 1;
    out->early_inflight = 0.5f; out->early_inflight_epochs = 1;
    out->replicate_inflight_late = -1.0f; out->replicate_late_from = 1;
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

int mf_hot_row_table(const uint32_t* counts, uint32_t rows, uint32_t n, float inflight, float replicate_above, float thin_above, float add_within,
                     uint8_t* table, uint16_t* slot, uint32_t* slot_row, uint32_t* slots)
{
    if (slots) *slots = 0;
    if (rows == 0) return MF_OK;
    if (!counts || !table) return invalid("mf_hot_row_table: null pointer");
    if (n == 0 || !(inflight > 0)) return invalid("mf_hot_row_table: no ratings or no updates in flight");
    if (replicate_above > 0 && (!slot || !slot_row || !slots)) return invalid("mf_hot_row_table: replicated rows need slot, slot_row and slots");
    const KeepTable t = keep_table(counts, rows, n, inflight, replicate_above, thin_above, add_within);
    std::memcpy(table, t.keep.data(), rows);
    if (slot) std::memcpy(slot, t.slot.data(), (size_t)rows * 2);
    if (slot_row && !t.slot_row.empty()) std::memcpy(slot_row, t.slot_row.data(), t.slot_row.size() * 4);
    if (slots) *slots = (uint32_t)t.slot_row.size();
    return MF_OK;
}

float mf_replicate_threshold(float learning_rate, float mean_rating)
{
    // C updates of one row in flight add C gradients taken at the same stale row: a step C times as long.  Along the
    // direction of the other side's mean row the curvature of the objective is about |row|^2, which at convergence is
    // about the mean rating (row . row' = rating with both factors alike), so the summed step stays a contraction while
    // C * lr * mean_rating < 2.  A sixth of that bound leaves room for the first epochs, when every row still
    // moves: 0.3 / (lr * mean_rating), between 2 and 16 (8.3 for lr 0.01 and ratings around 3.6).
    if (!(learning_rate > 0) || !(mean_rating > 0)) return 8.0f;
    const float t = 0.3f / (learning_rate * mean_rating);
    return t < 2.0f ? 2.0f : (t > 16.0f ? 16.0f : t);
}

float mf_replica_step_scale(float learning_rate, float mean_rating)
{
    // Half the bound of mf_replicate_threshold: the copies' longer steps meet the summed updates of the added rows on
    // the other side of the same ratings.  Measured at 100M ratings, learning rate 0.01, mean rating 3.46 (factor 4.3):
    // factors 2 / 4 / 6 / 8 for the first epoch leave the test RMSE 1.158 / 1.132 / 1.128 / 1.138 after it (1.199
    // without, 1.080 for a sequential run), 12 and 16 diverge in the first epoch.
    if (!(learning_rate > 0) || !(mean_rating > 0)) return 1.0f;
    const float t = 0.15f / (learning_rate * mean_rating);
    return t < 1.0f ? 1.0f : (t > (float)MF_XCDS ? (float)MF_XCDS : t);
}


uint32_t mf_auto_workers(uint32_t n)
{
    // About 128 windows of 128 ratings per worker: the ratio at which the runs on 8M and on 100M ratings stay
    // within 0.005 test RMSE of the reference rule run on the CPU.  From about 95M ratings on that count fills the chip
    // (24 wavefronts on each of the 256 CUs = 6144 resident workers): the updates in flight, which decide the distance
    // to a sequential run, no longer grow with the worker count, and workers with 16 windows each, eight times as many
    // as are resident, even out the end of every launch (4 % of the epoch at 100M ratings).
    const uint32_t w = (n / 16384u + 3u) / 4u * 4u;
    if (w < 16u) return 16u;
    if (w < 5800u) return w;
    return (uint32_t)((((uint64_t)n + 2047u) / 2048u + 3u) / 4u * 4u);
}

int mf_train(const mf_params* params, const mf_node* R, uint32_t n, uint32_t n_users, uint32_t n_items,
             const mf_node* test, uint32_t test_n, float* p, float* q, mf_report* report)
{
    const double t0 = now_ms();
    Run* raw = nullptr;
    MF_TRY(make_run(params, R, n, n_users, n_items, test, test_n, p, q, report, &raw));
    std::unique_ptr<Run> run(raw);
    MF_TRY(run->setup(R, test, p, q));
    for (uint32_t e = 0; e < run->prm.epoch; ++e) MF_TRY(run->epoch(e));
    MF_TRY(run->download(p, q));
    if (report) report->total_ms = now_ms() - t0;
    return 0;
}

struct mf_session { std::unique_ptr<Run> run; };

int mf_session_create(const mf_params* params, const mf_node* R, uint32_t n, uint32_t n_users, uint32_t n_items,
                      const mf_node* test, uint32_t test_n, const float* p, const float* q, mf_report* report, mf_session** session)
{
    if (!session) return invalid("mf_session_create: null session pointer");
    *session = nullptr;
    Run* raw = nullptr;
    MF_TRY(make_run(params, R, n, n_users, n_items, test, test_n, p, q, report, &raw));
    std::unique_ptr<Run> run(raw);
    MF_TRY(run->setup(R, test, p, q));
    *session = new mf_session{std::move(run)};
    return 0;
}
int mf_session_epoch(mf_session* session, double* test_rmse, float* sgd_ms)
{
    if (!session || !session->run) return invalid("mf_session_epoch: null session");
    Run& run = *session->run;
    if (run.next_epoch >= run.prm.epoch) return invalid("mf_session_epoch: all %u epochs of the run are done", run.prm.epoch);
    const uint32_t e = run.next_epoch;
    const int rc = run.epoch(e);
    const double rmse = rc == 0 ? run.c.rmse_hist[e] : 0.0;
    const float ms = rc == 0 ? run.c.ms_hist[e] : 0.f;
    if (rc) return rc;
    run.next_epoch = e + 1;
    if (test_rmse) *test_rmse = rmse;
    if (sgd_ms) *sgd_ms = ms;
    return 0;
}
uint32_t mf_session_workers(const mf_session* session) { return session && session->run ? session->run->prm.num_workers : 0; }
int mf_session_hot_rows(const mf_session* session, uint32_t* user_replicated, uint32_t* item_replicated, float* inflight)
{
    if (!session || !session->run) return invalid("mf_session_hot_rows: null session");
    if (user_replicated) *user_replicated = session->run->hot.replicated(0);
    if (item_replicated) *item_replicated = session->run->hot.replicated(1);
    if (inflight) *inflight = (float)session->run->hot.inflight;
    return 0;
}
int mf_session_device_state(const mf_session* session, uint32_t epoch, const mf_node** ratings, const mf_hogwild_options** options)
{
    if (!session || !session->run) return invalid("mf_session_device_state: null session");
    if (ratings) *ratings = session->run->c.d_R.as<mf_node>();
    if (options) *options = session->run->hot.options(epoch);
    return 0;
}
int mf_session_groups(const mf_session* session, int side, uint32_t* groups, uint8_t* prec, uint64_t* ratings)
{
    if (!session || !session->run || !groups) return invalid("mf_session_groups: null pointer");
    if (side != 0 && side != 1) return invalid("mf_session_groups: side is 0 (users) or 1 (items)");
    return session->run->groups(side, groups, prec, ratings);
}
int mf_session_promote_groups(mf_session* session, int side, const uint8_t* mask, uint32_t groups)
{
    if (!session || !session->run || !mask) return invalid("mf_session_promote_groups: null pointer");
    if (side != 0 && side != 1) return invalid("mf_session_promote_groups: side is 0 (users) or 1 (items)");
    return session->run->promote(side, mask, groups);
}
int mf_session_finish(mf_session* session, float* p, float* q)
{
    if (!session || !session->run) return invalid("mf_session_finish: null session");
    if (!p || !q) return invalid("mf_session_finish: null model pointer");
    return session->run->download(p, q);
}
void mf_session_destroy(mf_session* session) { delete session; }

}  // extern "C"
