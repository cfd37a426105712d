// Test driver for the command line's host I/O layer (csrc/io_utils.cpp), built by tests/test_host_io.py with g++.
// usage: host_io_check <train.tsv> <test.tsv> <out prefix> <k>
// Loads the two files as quantized_mf does, fills P and Q with values that depend only on (dense id, column), writes
// both model-file layouts, reads them back with the evaluator's reader and prints what it found.
#include "../icdm-2021_mascot_amd/csrc/io_utils.h"
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <limits>

static float value_of(uint32_t side, uint32_t row, uint32_t col)
{
    // a few values that exercise the number formatting, then a smooth pattern
    const float special[] = {0.0f, -0.0f, 1.0f, -1.5f, 1e-5f, 123456.0f, 1234567.0f, 1e10f, 3.14159274f, 1.17549435e-38f, 1e-45f,
                             0.1f, 0.0001f, 0.00001f, 999999.5f, 65504.0f, -2.5e-7f, std::numeric_limits<float>::infinity()};
    const uint32_t idx = row * 7 + col + side * 3;
    if (idx % 5 == 0) return special[(idx / 5) % (sizeof special / sizeof special[0])];
    return std::sin((float)(idx + 1)) * std::pow(10.0f, (float)((int)(idx % 13) - 6));
}

int main(int argc, char** argv)
{
    if (argc != 5) return 2;
    const std::string train = argv[1], test = argv[2], out = argv[3];
    const uint32_t k = (uint32_t)std::atoi(argv[4]);
    Dataset d;
    if (!load_dataset(d, train, test, false)) return 3;
    std::printf("users %u items %u train %zu test %zu kept_lines %u missing %u\n", d.max_user, d.max_item, d.R.size(), d.test.size(), d.test_lines_kept, d.test_missing);
    for (uint32_t i = 0; i < d.max_user; ++i) std::printf("user %u orig %u\n", i, d.user_orig[i]);
    for (uint32_t i = 0; i < d.max_item; ++i) std::printf("item %u orig %u\n", i, d.item_orig[i]);
    for (const mf_node& t : d.R) std::printf("train %u %u %.9g\n", t.u, t.i, t.r);
    for (const mf_node& t : d.test) std::printf("test %u %u %.9g\n", t.u, t.i, t.r);
    std::vector<float> p((size_t)d.max_user * k), q((size_t)d.max_item * k);
    for (uint32_t r = 0; r < d.max_user; ++r) for (uint32_t c = 0; c < k; ++c) p[(size_t)r * k + c] = value_of(0, r, c);
    for (uint32_t r = 0; r < d.max_item; ++r) for (uint32_t c = 0; c < k; ++c) q[(size_t)r * k + c] = value_of(1, r, c);
    if (!save_trained_model(d, p.data(), q.data(), k, out)) return 4;
    if (!save_trained_model_reconst(d.max_user, d.max_item, p.data(), q.data(), k, out)) return 5;
    if (!save_reconst_testset(d.test, test)) return 6;
    // the evaluator's reader; a model that holds "inf" does not read back (stream extraction stops there, as in the reference)
    TrainedModel m;
    if (read_trained_model(m, out + "_reconst.txt")) std::printf("reread users %u items %u k %u p %zu q %zu\n", m.n_users, m.n_items, m.k, m.p.size(), m.q.size());
    else std::printf("reread failed\n");
    // binary dump of what was written, for the byte-exact comparison on the Python side
    FILE* f = std::fopen((out + ".values").c_str(), "wb");
    if (!f) return 8;
    std::fwrite(p.data(), 4, p.size(), f); std::fwrite(q.data(), 4, q.size(), f);
    std::fclose(f);
    return 0;
}
