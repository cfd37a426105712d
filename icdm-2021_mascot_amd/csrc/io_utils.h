// Host I/O of the quantized_mf command line: rating readers and model writers with the file layouts
// of the reference's io_utils.h.
#pragma once
#include <cstdint>
#include <map>
#include <string>
#include <unordered_map>
#include <vector>
#include "../../include/mascot_hip.h"

struct Dataset {
    std::vector<mf_node> R;                       // training ratings, dense first-seen ids
    std::vector<mf_node> test;                    // test ratings ordered by (user, item), duplicates folded
    std::unordered_map<uint32_t, uint32_t> user_map, item_map;   // original id -> dense id
    std::vector<uint32_t> user_orig, item_orig;   // dense id -> original id
    uint32_t max_user = 0, max_item = 0;          // number of distinct users / items
    uint32_t test_lines_kept = 0;                 // the reference's test_n (counts duplicates, io_utils.h:187)
    uint32_t test_missing = 0;                    // test ratings dropped for an unseen user or item
    std::vector<uint32_t> remove_user, remove_item;   // their original ids, as written to remove_user.txt / remove_item.txt
};

// read_training_dataset, io_utils.h:30-120
bool read_training_dataset(Dataset& d, const std::string& path);
// read_test_dataset, io_utils.h:122-240 (also writes remove_user.txt / remove_item.txt next to the file)
bool read_test_dataset(Dataset& d, const std::string& path);
// Both readers behind a binary cache of what they produce (no counterpart in the reference, whose parse of a
// 100M-line file through getline/stoi/std::map takes minutes).  With use_cache the parsed and re-mapped ratings
// are kept in <train path>.mfcache; a later call with the same two files (same paths, sizes and modification
// times) loads that instead of parsing, prints the same "Missing the number of ratings" line and rewrites the two
// remove_*.txt files.  Without use_cache this is read_training_dataset followed by read_test_dataset.
bool load_dataset(Dataset& d, const std::string& train_path, const std::string& test_path, bool use_cache, bool* from_cache = nullptr);
// A data set from ratings that are already in memory with dense ids (the synthetic generator): `train` is taken as
// it is; `test` goes through the test-set rules of read_test_dataset (ratings of users or items without a training
// rating are dropped and counted, one rating per (user, item) with the later one winning, ordered by user then
// item).  Original ids are the dense ids; no remove_*.txt files are written.
void dataset_from_ratings(Dataset& d, std::vector<mf_node>&& train, const std::vector<mf_node>& test, uint32_t n_users, uint32_t n_items);
// save_trained_model, io_utils.h:242-303: <out>.txt, rows by original id, zero rows for absent ids
bool save_trained_model(const Dataset& d, const float* p, const float* q, uint32_t k, const std::string& outfile);
// save_trained_model_reconst, io_utils.h:305-332: <out>_reconst.txt, rows in the order given
bool save_trained_model_reconst(uint32_t n_users, uint32_t n_items, const float* p, const float* q, uint32_t k, const std::string& outfile);
// save_reconst_testset, io_utils.h:374-405: reconst_<testfile> next to the test file
bool save_reconst_testset(const std::vector<mf_node>& test, const std::string& testfile);

// ---- the stand-alone evaluator (test_mf/test.cu) -------------------------------------------------------------
struct TrainedModel { uint32_t n_users = 0, n_items = 0, k = 0; std::vector<float> p, q; };
// read_trained_model, io_utils.h:334-372: header "users items k", then users*k and items*k numbers
bool read_trained_model(TrainedModel& m, const std::string& path);
// read_testset_pretrained_model, io_utils.h:407-457: raw ids as they stand in the file (no re-mapping)
std::vector<mf_node> read_testset_pretrained_model(const std::string& path);
// remove_elements, io_utils.h:459-514: for version != 1 drops the users / items listed in remove_user.txt /
// remove_item.txt next to the test file; false when one of the two files cannot be opened
bool remove_elements(std::vector<mf_node>& test, unsigned version, const std::string& test_path);
