// quantized_mf: the reference's command line (main.cu:15-175) over libmascot_hip.
// Same flags, the reference's stdout lines (plus two in the parameter echo, "Seed" and "Hot rows", for the two things
// the reference does not have), same model files.  Additions: `-seed <n>` (the reference seeds from
// time(0) and clock(), so two of its runs never agree; here the default seed is fixed), `-compat <0|1>` (1: `-wg`
// counts updates in flight as it does in the reference, where a worker has one; a worker here keeps four, so the run
// uses a quarter as many workers: mf_params.wg_counts_updates), `-cached <0|1>`
// and `-split <n>` (row access policy and kernel launches per epoch, see include/mascot_hip.h), `-hot <0|1>`,
// `-replicate <t>[,<merges>[,<late t>[,<from epoch>]]]` and `-thin <cap>[,<early cap>,<epochs>]` (how rows with several updates in flight are
// treated: mf_params.hot_rows, replicate_inflight, hot_row_inflight; `-hot 0` is the reference's race semantics),
// `-early <fraction>[,<epochs>]` (the first epochs run with that fraction of the updates in flight:
// mf_params.early_inflight), `-synth <c>[,<n>]`
// (no input files: the seeded synthetic stand-in of BASELINE configuration c, optionally with n training ratings
// and the test set scaled alike, generated on the device; mf_generate_ratings).
#include <sys/stat.h>
#include <cstdlib>
#include <cstdio>
#include <iostream>
#include <string>
#include <vector>
#include "io_utils.h"

static bool exists(const std::string& name) { struct stat b; return stat(name.c_str(), &b) == 0; }

int main(int argc, const char* argv[])
{
    std::string infile, outfile, testfile = "None";
    mf_params prm;
    mf_default_params(&prm);
    unsigned reconst_save = 0;
    int use_cache = 0;                                // -cache 1: keep the parsed ratings in <input>.mfcache
    int synth = 0; unsigned long long synth_train = 0;  // -synth <config>[,<training ratings>]
    const char* usage = " [-t <threads> -p <predictions/user> -o <output-tsv>] <input-tsv>";
    if (argc < 2) { std::cout << argv[0] << usage << std::endl; return 0; }
    if (argc == 2) infile = argv[1];
    else {
        for (int i = 0; i < argc; ++i) {
            const std::string a = argv[i];
            const bool has = i < argc - 1;
            if (a == "-i" && has) infile = argv[i + 1];
            if (a == "-o" && has) outfile = argv[i + 1];
            if (a == "-y" && has) testfile = argv[i + 1];
            if (a == "-l" && has) prm.epoch = std::atoi(argv[i + 1]);
            if (a == "-k" && has) prm.k = std::atoi(argv[i + 1]);
            if (a == "-b" && has) prm.lambda = std::atof(argv[i + 1]);
            if (a == "-a" && has) prm.learning_rate = std::atof(argv[i + 1]);
            if (a == "-wg" && has) prm.num_workers = std::atoi(argv[i + 1]);
            if (a == "-d" && has) prm.decay = std::atof(argv[i + 1]);
            if (a == "-bl" && has) prm.thread_block_size = std::atoi(argv[i + 1]);
            if (a == "-v" && has) prm.version = std::atoi(argv[i + 1]);
            if (a == "-r" && has) prm.sample_ratio = std::atof(argv[i + 1]);
            if (a == "-ug" && has) prm.user_group_num = std::atoi(argv[i + 1]);
            if (a == "-ig" && has) prm.item_group_num = std::atoi(argv[i + 1]);
            if (a == "-e" && has) prm.error_threshold = std::atof(argv[i + 1]);
            if (a == "-s" && has) prm.sample_ratio = std::atof(argv[i + 1]);
            if (a == "-it" && has) prm.interval = std::atoi(argv[i + 1]);
            if (a == "-rc" && has) reconst_save = std::atoi(argv[i + 1]);
            if (a == "-seed" && has) prm.seed = std::strtoull(argv[i + 1], nullptr, 10);
            if (a == "-compat" && has) prm.wg_counts_updates = std::atoi(argv[i + 1]) != 0;      // -wg counts updates in flight, as in the reference
            if (a == "-cached" && has) prm.cached_rows = std::atoi(argv[i + 1]);
            if (a == "-split" && has) prm.epoch_splits = std::atoi(argv[i + 1]);
            if (a == "-hot" && has) {            // 0: no hot rows at all, every row stored as the reference does; 1 (default): hot rows
                prm.hot_rows = std::atoi(argv[i + 1]) != 0;
                if (!prm.hot_rows) { prm.replicate_inflight = 0; prm.hot_row_inflight = 0; }
            }
            if (a == "-replicate" && has) {      // <updates in flight above which a row gets a copy per XCD; 0 = none>[,<merges per epoch>[,<the bar in later epochs; 0 = the same>[,<from epoch>]]]
                float above = 0, late = 0; unsigned merges = 0, from = 0;
                const int got = std::sscanf(argv[i + 1], "%f,%u,%f,%u", &above, &merges, &late, &from);
                if (got >= 1) prm.replicate_inflight = above;
                if (got >= 2) prm.replica_merges = merges;
                if (got >= 3) prm.replicate_inflight_late = late;
                if (got >= 4) prm.replicate_late_from = from;
            }
            if (a == "-early" && has) {          // <fraction of the updates in flight during the first epochs; 0 or 1 = off>[,<epochs>]
                float fraction = 0; unsigned ep = 0;
                const int got = std::sscanf(argv[i + 1], "%f,%u", &fraction, &ep);
                if (got >= 1) prm.early_inflight = fraction;
                if (got >= 2) prm.early_inflight_epochs = ep;
            }
            if (a == "-thin" && has) {           // opt-in thinning of hot rows: <steady cap>[,<early cap>,<early epochs>]
                float steady = 0, early = 0; unsigned ep = 0;
                const int got = std::sscanf(argv[i + 1], "%f,%f,%u", &steady, &early, &ep);
                if (got >= 1) prm.hot_row_inflight = steady;
                if (got >= 2) prm.hot_row_inflight_early = early;
                if (got >= 3) prm.hot_row_early_epochs = ep;
            }
            if (a == "-cache" && has) use_cache = std::atoi(argv[i + 1]);
            if (a == "-synth" && has) std::sscanf(argv[i + 1], "%d,%llu", &synth, &synth_train);
            if (a == "-h") { std::cout << argv[0] << usage << std::endl; return 0; }
        }
    }
    mf_synth_config sc = {};
    if (synth) {
        if (int rc = mf_synth_baseline_config(synth, &sc)) { std::cerr << "quantized_mf: " << mf_last_error() << std::endl; return rc > 0 ? rc : 1; }
        if (synth_train && synth_train < sc.n_train) {
            sc.n_test = (uint64_t)((double)sc.n_test * (double)synth_train / (double)sc.n_train);
            sc.n_train = synth_train;
        }
        infile = "synthetic configuration " + std::to_string(synth);
        if (synth == 5) prm.is_yahoo = 1;               // 0..100 ratings, rescaled like the reference's Yahoo set
    } else if (!exists(infile)) { std::cout << infile << " doesn't exist!" << std::endl; return 0; }

    std::cout << std::endl;
    std::cout << "Input file                  : " << infile << std::endl;
    std::cout << "Test file                   : " << testfile << std::endl;
    std::cout << "Output file                 : " << outfile << std::endl;
    std::cout << "Latent features             : " << prm.k << std::endl;
    std::cout << "Learning rate               : " << prm.learning_rate << std::endl;
    std::cout << "Decay                       : " << prm.decay << std::endl;
    std::cout << "Lambda                      : " << prm.lambda << std::endl;
    std::cout << "Iteration                   : " << prm.epoch << std::endl;
    std::cout << "Num of workers              : " << prm.num_workers << (prm.num_workers ? (prm.wg_counts_updates ? " (updates in flight, as the reference counts)" : "") : " (chosen from the number of ratings)") << std::endl;
    std::cout << "Thread block size           : " << prm.thread_block_size << std::endl;
    std::cout << "Sample ratio                : " << prm.sample_ratio << std::endl;
    std::cout << "Error threshold             : " << prm.error_threshold << std::endl;
    std::cout << "Interval                    : " << prm.interval << std::endl;
    std::cout << "Seed                        : " << prm.seed << std::endl;
    std::cout << "Hot rows                    : ";
    if (!prm.hot_rows && !(prm.replicate_inflight != 0) && !(prm.hot_row_inflight > 0)) std::cout << "off (every row stored as the reference does; -hot 0)";
    else {
        std::cout << "updates of rows with more than one update in flight are added";
        if (prm.replicate_inflight < 0) std::cout << "; rows above 0.3 / (learning rate x mean rating) in flight are replicated per XCD";
        else if (prm.replicate_inflight > 0) std::cout << "; rows above " << prm.replicate_inflight << " in flight are replicated per XCD";
        if (prm.replicate_inflight != 0 && prm.replica_merges) std::cout << ", merged " << prm.replica_merges << " times per epoch";
        if (prm.replicate_inflight != 0 && prm.replicate_inflight_late < 0) std::cout << " (above a quarter of that from epoch " << prm.replicate_late_from + 1 << " on)";
        else if (prm.replicate_inflight != 0 && prm.replicate_inflight_late > 0) std::cout << " (above " << prm.replicate_inflight_late << " from epoch " << prm.replicate_late_from + 1 << " on)";
        if (prm.hot_row_inflight > 0) std::cout << "; rows above " << prm.hot_row_inflight << " in flight are thinned";
    }
    std::cout << std::endl;

    Dataset d;
    bool from_cache = false;
    if (synth) {
        std::vector<mf_node> all(sc.n_train + sc.n_test);
        if (int rc = mf_generate_ratings_host(&sc, prm.seed, 0, all.size(), all.data())) { std::cerr << "quantized_mf: " << mf_last_error() << std::endl; return rc > 0 ? rc : 1; }
        std::vector<mf_node> test(all.begin() + (std::ptrdiff_t)sc.n_train, all.end());
        all.resize(sc.n_train);
        dataset_from_ratings(d, std::move(all), test, sc.n_users, sc.n_items);
        std::cout << "Missing the number of ratings : " << d.test_missing << std::endl;
    } else {
        load_dataset(d, infile, testfile, use_cache != 0, &from_cache);
    }
    if (from_cache) std::cout << "Ratings loaded from " << infile << ".mfcache" << std::endl;
    std::cout << "The number of nonzeros      : " << d.R.size() << std::endl;
    std::cout << "The number of users         : " << d.max_user << std::endl;
    std::cout << "The number of items         : " << d.max_item << std::endl;
    std::cout << "The number of test nonzeros : " << d.test.size() << std::endl;

    if (!synth) prm.is_yahoo = infile.find("Yahoo") != std::string::npos;
    prm.verbose = 1;
    if (prm.version == 0) prm.version = 5;          // "-v 0" is accepted as plain fp32 SGD
    const size_t pn = (size_t)d.max_user * prm.k, qn = (size_t)d.max_item * prm.k;
    std::vector<float> p(pn), q(qn);
    // init_model_half for the variants that start from binary16-representable values (main.cu:152-153)
    const int half_init = prm.version == 4 || prm.version == 7 || prm.version == 8;
    if (int rc = mf_init_model(p.data(), q.data(), d.max_user, d.max_item, prm.k, prm.seed, half_init)) {
        std::cerr << "quantized_mf: " << mf_last_error() << std::endl;
        return rc > 0 ? rc : 1;
    }
    mf_report rep = {};
    std::vector<float> ms(prm.epoch);
    std::vector<mf_node> test_reconst(d.test.size());
    rep.sgd_ms_per_epoch = ms.data();
    rep.test_reconst = test_reconst.data();
    if (int rc = mf_train(&prm, d.R.data(), (uint32_t)d.R.size(), d.max_user, d.max_item, d.test.data(), (uint32_t)d.test.size(),
                          p.data(), q.data(), &rep)) {
        std::cerr << "quantized_mf: " << mf_last_error() << std::endl;
        return rc > 0 ? rc : 1;
    }
    // timing summary in the reference's units (micro seconds unless stated), mf_methods.cu:401-418
    if (prm.version == 1 || prm.version == 6) {
        std::cout << "\n<Preprocessing time (micro sec)>" << std::endl;
        std::cout << "Total preprocessing time         : " << rep.preprocess_ms * 1000 << std::endl;
        std::cout << "\n<User & item parameter copy exec time (micro sec)>" << std::endl;
        std::cout << "Precision switching              : " << rep.switching_ms * 1000 / prm.epoch << std::endl;
        std::cout << "Total precision switching time   : " << rep.switching_ms * 1000 << std::endl;
        std::cout << "\n<User & item group error comp exec time (micro sec)>" << std::endl;
        std::cout << "Error computation time           : " << rep.error_ms * 1000 / prm.epoch << std::endl;
        std::cout << "Total error computation time     : " << rep.error_ms * 1000 << std::endl;
        std::cout << "\n<User & item parameter update exec time (micro sec)>" << std::endl;
    }
    std::cout << "Parameters update per epoch      : " << rep.sgd_ms * 1000 / prm.epoch << std::endl;
    std::cout << "Total parameters update          : " << rep.sgd_ms * 1000 << std::endl;
    std::cout << "Total MF time(ms)                : " << (rep.preprocess_ms + rep.switching_ms + rep.error_ms + rep.sgd_ms) << std::endl;
    std::cout << "Ratings per second (update kernel): " << (double)d.R.size() * prm.epoch / (rep.sgd_ms / 1000.0) << std::endl;

    if (!outfile.empty()) {
        // -v 6 trains in the same re-indexed row order as -v 1, so its model is written in that layout as well
        if (prm.version == 1 || prm.version == 6) save_trained_model_reconst(d.max_user, d.max_item, p.data(), q.data(), prm.k, outfile);
        else save_trained_model(d, p.data(), q.data(), prm.k, outfile);
    }
    if ((prm.version == 1 || prm.version == 6) && reconst_save == 1 && !synth) save_reconst_testset(test_reconst, testfile);
    return 0;
}
