// test_mf: the stand-alone evaluator (test_mf/test.cu of the reference).  Reloads a model file written by
// quantized_mf (<out>.txt for -v != 1, <out>_reconst.txt together with reconst_<testfile> for -v 1), reads the
// test ratings with the ids as they stand in the file, and prints the test RMSE computed on the device.
#include <iostream>
#include <string>
#include <sys/stat.h>
#include "io_utils.h"

static bool exists(const std::string& name) { struct stat st; return stat(name.c_str(), &st) == 0; }

int main(int argc, const char* argv[])
{
    std::string infile, testfile = "None";
    unsigned version = 1;
    const char* usage = " [-t <threads> -p <predictions/user> -o <output-tsv>] <input-tsv>";
    if (argc < 2) { std::cout << argv[0] << usage << std::endl; return 0; }
    if (argc == 2) infile = argv[1];
    else {
        for (int i = 0; i < argc; ++i) {
            const std::string a = argv[i];
            const bool has = i < argc - 1;
            if (a == "-i" && has) infile = argv[i + 1];
            if (a == "-y" && has) testfile = argv[i + 1];
            if (a == "-v" && has) version = (unsigned)std::stoi(argv[i + 1]);
            if (a == "-h") { std::cout << argv[0] << usage << std::endl; return 0; }
        }
    }
    if (!exists(infile)) { std::cout << infile << " doesn't exist!" << std::endl; return 0; }
    std::cout << std::endl;
    std::cout << "Input file                  : " << infile << std::endl;
    std::cout << "Test file                   : " << testfile << std::endl;
    std::cout << "Version                     : " << version << std::endl;

    std::vector<mf_node> test = read_testset_pretrained_model(testfile);
    TrainedModel m;
    if (!read_trained_model(m, infile)) { std::cerr << "test_mf: cannot parse the model file " << infile << std::endl; return 1; }
    if (!remove_elements(test, version, testfile)) return 0;          // the reference returns silently here as well
    double rmse = 0;
    if (int rc = mf_gpu_test_rmse(test.data(), (uint32_t)test.size(), m.p.data(), m.q.data(), m.n_users, m.n_items, (int)m.k, &rmse)) {
        std::cerr << "test_mf: " << mf_last_error() << std::endl;
        return rc > 0 ? rc : 1;
    }
    std::cout << "RMSE : " << rmse << std::endl;
    return 0;
}
