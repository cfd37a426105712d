#include "io_utils.h"
#include <algorithm>
#include <cerrno>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <iostream>
#include <sstream>
#include <sys/stat.h>
#include <thread>

namespace {

std::vector<std::string> split(const std::string& s, char delim)
{
    std::vector<std::string> out;
    std::stringstream ss(s);
    std::string item;
    while (std::getline(ss, item, delim)) out.push_back(item);
    return out;
}
// column order from substrings of the path (io_utils.h:40-47)
void column_order(const std::string& path, int& user_idx, int& item_idx)
{
    if (path.find("netflix") != std::string::npos || path.find("25M") != std::string::npos) { user_idx = 1; item_idx = 0; }
    else { user_idx = 0; item_idx = 1; }
}
uint32_t dense_id(std::unordered_map<uint32_t, uint32_t>& map, std::vector<uint32_t>& orig, uint32_t& count, uint32_t id)
{
    auto it = map.find(id);
    if (it != map.end()) return it->second;
    map.emplace(id, count);
    orig.push_back(id);
    return count++;
}
float parse_rating(std::string s)
{
    s.erase(s.find_last_not_of(" \n\r\t") + 1);
    return (float)std::atof(s.c_str());
}
std::string parent_dir(const std::string& path)
{
    const size_t pos = path.find_last_of('/');
    return pos == std::string::npos ? std::string() : path.substr(0, pos);
}
std::string file_name(const std::string& path)
{
    const size_t pos = path.find_last_of('/');
    return pos == std::string::npos ? path : path.substr(pos + 1);
}

}  // namespace

namespace {
// the stdout line and the two side-effect files of read_test_dataset (io_utils.h:200-238)
void report_missing_and_write_remove_files(const Dataset& d, const std::string& test_path)
{
    std::cout << "Missing the number of ratings : " << d.test_missing << std::endl;
    const std::string dir = parent_dir(test_path);
    for (int which = 0; which < 2; ++which) {
        const std::string out = dir + (which ? "/remove_item.txt" : "/remove_user.txt");
        std::ofstream f(out);
        if (f.fail()) { std::cout << "fail to write file named " << out << std::endl; return; }
        for (uint32_t v : (which ? d.remove_item : d.remove_user)) f << v << std::endl;
    }
}
}  // namespace

bool read_training_dataset(Dataset& d, const std::string& path)
{
    std::ifstream file(path);
    if (!file) return false;
    int user_idx, item_idx;
    column_order(path, user_idx, item_idx);
    std::string line;
    if (path.find("Yahoo") != std::string::npos) {           // io_utils.h:49-79: "user|count" then count lines "item\trating"
        while (std::getline(file, line)) {
            std::vector<std::string> head = split(line, '|');
            if (head.size() < 2) continue;
            const uint32_t user = (uint32_t)std::stoi(head[0]);
            const uint32_t cnt = (uint32_t)std::stoi(head[1]);
            const uint32_t u = dense_id(d.user_map, d.user_orig, d.max_user, user);
            for (uint32_t i = 0; i < cnt; ++i) {
                if (!std::getline(file, line)) break;
                std::vector<std::string> tok = split(line, '\t');
                if (tok.size() < 2) continue;
                const uint32_t it = dense_id(d.item_map, d.item_orig, d.max_item, (uint32_t)std::stoi(tok[0]));
                const float rating = (float)std::atof(tok[1].c_str());
                d.R.push_back({(rating / 25.f) + 1.0f, u, it});
            }
        }
    } else {
        while (std::getline(file, line)) {
            std::vector<std::string> tok = split(line, '\t');
            if (tok.size() != 3) continue;
            const uint32_t user = (uint32_t)std::stoi(tok[user_idx]);
            const uint32_t item = (uint32_t)std::stoi(tok[item_idx]);
            const float rating = parse_rating(tok[2]);
            const uint32_t u = dense_id(d.user_map, d.user_orig, d.max_user, user);
            const uint32_t it = dense_id(d.item_map, d.item_orig, d.max_item, item);
            d.R.push_back({rating, u, it});
        }
    }
    return true;
}

bool read_test_dataset(Dataset& d, const std::string& path)
{
    std::vector<uint32_t>& remove_user = d.remove_user;
    std::vector<uint32_t>& remove_item = d.remove_item;
    uint32_t& missing = d.test_missing;
    if (d.user_map.empty()) for (uint32_t i = 0; i < d.user_orig.size(); ++i) d.user_map.emplace(d.user_orig[i], i);
    if (d.item_map.empty()) for (uint32_t i = 0; i < d.item_orig.size(); ++i) d.item_map.emplace(d.item_orig[i], i);
    std::ifstream file(path);
    int user_idx, item_idx;
    column_order(path, user_idx, item_idx);
    // test_R[user][item] = rating: later duplicates overwrite earlier ones (io_utils.h:186)
    std::vector<std::map<uint32_t, float>> test_R(d.max_user);
    std::string line;
    if (file) {
        if (path.find("Yahoo") != std::string::npos) {
            while (std::getline(file, line)) {
                std::vector<std::string> head = split(line, '|');
                if (head.size() < 2) continue;
                const uint32_t cnt = (uint32_t)std::stoi(head[1]);
                auto itu = d.user_map.find((uint32_t)std::stoi(head[0]));
                if (itu == d.user_map.end()) {
                    // the reference counts the block as missing and moves on without consuming its lines
                    // (io_utils.h:153-156); consume them here so the following blocks parse
                    missing += cnt;
                    for (uint32_t i = 0; i < cnt; ++i) std::getline(file, line);
                    continue;
                }
                for (uint32_t i = 0; i < cnt; ++i) {
                    if (!std::getline(file, line)) break;
                    std::vector<std::string> tok = split(line, '\t');
                    if (tok.size() < 2) continue;
                    auto iti = d.item_map.find((uint32_t)std::stoi(tok[0]));
                    if (iti == d.item_map.end()) { missing += 1; continue; }
                    test_R[itu->second][iti->second] = ((float)std::atof(tok[1].c_str()) / 25.f) + 1.0f;
                    d.test_lines_kept++;
                }
            }
        } else {
            while (std::getline(file, line)) {
                std::vector<std::string> tok = split(line, '\t');
                if (tok.size() != 3) continue;
                const uint32_t user = (uint32_t)std::stoi(tok[user_idx]);
                const uint32_t item = (uint32_t)std::stoi(tok[item_idx]);
                const float rating = parse_rating(tok[2]);
                auto itu = d.user_map.find(user);
                auto iti = d.item_map.find(item);
                if (itu != d.user_map.end() && iti != d.item_map.end()) { test_R[itu->second][iti->second] = rating; d.test_lines_kept++; }
                else if (itu == d.user_map.end()) { missing++; remove_user.push_back(user); }
                else { missing++; remove_item.push_back(item); }
            }
        }
    }
    // test_set_preprocess, preprocess_utils.h:38-52: users ascending (dense id), items ascending within a user
    for (uint32_t u = 0; u < d.max_user; ++u)
        for (const auto& kv : test_R[u]) d.test.push_back({kv.second, u, kv.first});
    report_missing_and_write_remove_files(d, path);
    return true;
}

void dataset_from_ratings(Dataset& d, std::vector<mf_node>&& train, const std::vector<mf_node>& test, uint32_t n_users, uint32_t n_items)
{
    d = Dataset();
    d.R = std::move(train);
    d.max_user = n_users; d.max_item = n_items;
    d.user_orig.resize(n_users); d.item_orig.resize(n_items);
    for (uint32_t i = 0; i < n_users; ++i) d.user_orig[i] = i;
    for (uint32_t i = 0; i < n_items; ++i) d.item_orig[i] = i;
    std::vector<uint8_t> user_seen(n_users, 0), item_seen(n_items, 0);
    for (const mf_node& t : d.R) { user_seen[t.u] = 1; item_seen[t.i] = 1; }
    std::vector<std::map<uint32_t, float>> test_R(n_users);
    for (const mf_node& t : test) {
        if (t.u < n_users && t.i < n_items && user_seen[t.u] && item_seen[t.i]) { test_R[t.u][t.i] = t.r; d.test_lines_kept++; }
        else if (t.u >= n_users || !user_seen[t.u]) { d.test_missing++; d.remove_user.push_back(t.u); }
        else { d.test_missing++; d.remove_item.push_back(t.i); }
    }
    for (uint32_t u = 0; u < n_users; ++u)
        for (const auto& kv : test_R[u]) d.test.push_back({kv.second, u, kv.first});
}

// The text of `rows` model rows: row r is k numbers from row(r), or k zeros where row(r) is null, each followed by a
// blank -- what `f << value << " "` writes with the stream's default formatting (%g, six significant digits; the
// reference's writers, io_utils.h:276-297,320-330).  A model of config 4 holds 64M numbers, so blocks of rows are
// formatted by all hardware threads into their own buffers and written in order.
template <class RowOf>
static bool write_rows(std::ofstream& f, size_t rows, uint32_t k, RowOf row)
{
    const unsigned threads = std::max(1u, std::min(16u, std::thread::hardware_concurrency()));
    const size_t block = 2048;                                   // rows per thread and round
    std::vector<std::string> text(threads);
    for (size_t base = 0; base < rows; base += block * threads) {
        auto format = [&](unsigned t) {
            std::string& out = text[t];
            out.clear();
            const size_t lo = std::min(rows, base + block * t), hi = std::min(rows, lo + block);
            out.reserve((hi - lo) * k * 13);
            char buf[40];
            for (size_t r = lo; r < hi; ++r) {
                const float* v = row(r);
                if (!v) { for (uint32_t j = 0; j < k; ++j) out.append("0 ", 2); continue; }
                for (uint32_t j = 0; j < k; ++j) out.append(buf, (size_t)std::snprintf(buf, sizeof buf, "%g ", (double)v[j]));
            }
        };
        std::vector<std::thread> pool;
        for (unsigned t = 1; t < threads; ++t) pool.emplace_back(format, t);
        format(0);
        for (auto& th : pool) th.join();
        for (unsigned t = 0; t < threads; ++t) f.write(text[t].data(), (std::streamsize)text[t].size());
        if (!f) return false;
    }
    return true;
}

bool save_trained_model(const Dataset& d, const float* p, const float* q, uint32_t k, const std::string& outfile)
{
    std::cout << "Save trained model..." << std::endl;
    const std::string outpath = outfile + ".txt";
    std::ofstream f(outpath);
    if (f.fail()) { std::cout << "fail to write file named " << outpath << std::endl; std::cerr << "Error: " << std::strerror(errno); return false; }
    // rows are indexed by original id up to the largest one; ids that never occurred have no row (zeros in the file)
    auto sorted_by_orig = [](const std::vector<uint32_t>& orig) {       // (original id, dense id), ascending original id
        std::vector<std::pair<uint32_t, uint32_t>> v(orig.size());
        for (uint32_t i = 0; i < orig.size(); ++i) v[i] = {orig[i], i};
        std::sort(v.begin(), v.end());
        return v;
    };
    const auto users = sorted_by_orig(d.user_orig), items = sorted_by_orig(d.item_orig);
    auto row_of = [k](const std::vector<std::pair<uint32_t, uint32_t>>& ids, const float* m, size_t orig) -> const float* {
        auto it = std::lower_bound(ids.begin(), ids.end(), std::make_pair((uint32_t)orig, 0u));
        return it != ids.end() && it->first == orig ? m + (size_t)it->second * k : nullptr;
    };
    const size_t user_rows = users.empty() ? 0 : (size_t)users.back().first + 1, item_rows = items.empty() ? 0 : (size_t)items.back().first + 1;
    f << user_rows << " " << item_rows << " " << k << std::endl;
    bool ok = write_rows(f, user_rows, k, [&](size_t r) { return row_of(users, p, r); });
    f << std::endl;
    ok = ok && write_rows(f, item_rows, k, [&](size_t r) { return row_of(items, q, r); });
    return ok && (bool)f;
}

bool save_trained_model_reconst(uint32_t n_users, uint32_t n_items, const float* p, const float* q, uint32_t k, const std::string& outfile)
{
    std::cout << "Save trained reconst model..." << std::endl;
    const std::string outpath = outfile + "_reconst.txt";
    std::ofstream f(outpath);
    if (f.fail()) { std::cout << "fail to write file named " << outpath << std::endl; std::cerr << "Error: " << std::strerror(errno); return false; }
    f << n_users << " " << n_items << " " << k << std::endl;
    bool ok = write_rows(f, n_users, k, [&](size_t r) { return p + r * k; });
    f << std::endl;
    ok = ok && write_rows(f, n_items, k, [&](size_t r) { return q + r * k; });
    return ok && (bool)f;
}

bool save_reconst_testset(const std::vector<mf_node>& test, const std::string& testfile)
{
    std::cout << "Save reconst mat.." << std::endl;
    const std::string out = parent_dir(testfile) + "/reconst_" + file_name(testfile);
    std::ofstream f(out);
    if (f.fail()) { std::cout << "fail to write file named " << out << std::endl; return false; }
    const bool user_first = !(out.find("netflix") != std::string::npos || out.find("25M") != std::string::npos);
    for (const mf_node& t : test) {
        if (user_first) f << t.u << "\t" << t.i << "\t" << t.r << std::endl;
        else f << t.i << "\t" << t.u << "\t" << t.r << std::endl;
    }
    return true;
}

bool read_trained_model(TrainedModel& m, const std::string& path)
{
    std::ifstream f(path);
    if (!f) return false;
    std::string line;
    if (!std::getline(f, line)) return false;
    const std::vector<std::string> tok = split(line, ' ');
    if (tok.size() < 3) return false;
    m.n_users = (uint32_t)std::stoul(tok[0]);
    m.n_items = (uint32_t)std::stoul(tok[1]);
    m.k = (uint32_t)std::atoi(tok[2].c_str());
    m.p.assign((size_t)m.n_users * m.k, 0.f);
    m.q.assign((size_t)m.n_items * m.k, 0.f);
    for (float& v : m.p) if (!(f >> v)) return false;
    for (float& v : m.q) if (!(f >> v)) return false;
    return true;
}

std::vector<mf_node> read_testset_pretrained_model(const std::string& path)
{
    std::vector<mf_node> test;
    std::ifstream f(path);
    if (!f) return test;
    int user_idx, item_idx;
    column_order(path, user_idx, item_idx);
    std::string line;
    if (path.find("Yahoo") != std::string::npos && path.find("reconst") == std::string::npos) {
        while (std::getline(f, line)) {
            const std::vector<std::string> head = split(line, '|');
            if (head.size() < 2) continue;
            const uint32_t u = (uint32_t)std::stoi(head[0]);
            const uint32_t cnt = (uint32_t)std::stoi(head[1]);
            for (uint32_t j = 0; j < cnt; ++j) {
                if (!std::getline(f, line)) break;
                const std::vector<std::string> tok = split(line, '\t');
                if (tok.size() < 2) continue;
                test.push_back({((float)std::atof(tok[1].c_str()) / 25.f) + 1.0f, u, (uint32_t)std::stoi(tok[0])});
            }
        }
    } else {
        while (std::getline(f, line)) {
            const std::vector<std::string> tok = split(line, '\t');
            if (tok.size() != 3) continue;
            test.push_back({parse_rating(tok[2]), (uint32_t)std::stoi(tok[user_idx]), (uint32_t)std::stoi(tok[item_idx])});
        }
    }
    return test;
}

bool remove_elements(std::vector<mf_node>& test, unsigned version, const std::string& test_path)
{
    if (version == 1) return true;
    std::vector<uint32_t> gone[2];
    const std::string dir = parent_dir(test_path);
    for (int which = 0; which < 2; ++which) {
        const std::string path = dir + (which ? "/remove_item.txt" : "/remove_user.txt");
        std::ifstream f(path);
        if (f.fail()) { std::cout << "fail to write file named " << path << std::endl; return false; }   // the reference's wording
        std::string line;
        while (std::getline(f, line)) {
            line.erase(line.find_last_not_of(" \n\r\t") + 1);
            if (!line.empty()) gone[which].push_back((uint32_t)std::stoi(line));
        }
        std::sort(gone[which].begin(), gone[which].end());
    }
    auto listed = [](const std::vector<uint32_t>& v, uint32_t id) { return std::binary_search(v.begin(), v.end(), id); };
    test.erase(std::remove_if(test.begin(), test.end(), [&](const mf_node& t) { return listed(gone[0], t.u) || listed(gone[1], t.i); }), test.end());
    return true;
}

// ---- binary cache of the parsed data set ----------------------------------------------------------------------
namespace {
struct FileId { uint64_t size = 0; int64_t mtime_s = 0, mtime_ns = 0; bool ok = false; };
FileId file_id(const std::string& path)
{
    FileId id;
    struct stat st;
    if (stat(path.c_str(), &st) == 0) { id.size = (uint64_t)st.st_size; id.mtime_s = (int64_t)st.st_mtim.tv_sec; id.mtime_ns = (int64_t)st.st_mtim.tv_nsec; id.ok = true; }
    return id;
}
struct CacheHeader {
    char magic[8];                 // "MFCACHE1"
    uint64_t train_size, test_size;
    int64_t train_mtime_s, train_mtime_ns, test_mtime_s, test_mtime_ns;
    uint64_t test_path_hash;
    uint64_t n_train, n_test, n_remove_user, n_remove_item;
    uint32_t n_users, n_items, test_lines_kept, test_missing;
};
uint64_t fnv1a(const std::string& s)
{
    uint64_t h = 1469598103934665603ull;
    for (unsigned char c : s) { h ^= c; h *= 1099511628211ull; }
    return h;
}
template <class T> bool write_vec(std::ofstream& f, const std::vector<T>& v) { if (!v.empty()) f.write(reinterpret_cast<const char*>(v.data()), (std::streamsize)(v.size() * sizeof(T))); return (bool)f; }
template <class T> bool read_vec(std::ifstream& f, std::vector<T>& v, uint64_t n) { v.resize(n); if (n) f.read(reinterpret_cast<char*>(v.data()), (std::streamsize)(n * sizeof(T))); return (bool)f; }
}  // namespace

bool load_dataset(Dataset& d, const std::string& train_path, const std::string& test_path, bool use_cache, bool* from_cache)
{
    if (from_cache) *from_cache = false;
    const std::string cache_path = train_path + ".mfcache";
    const FileId tr = file_id(train_path), te = file_id(test_path);
    if (use_cache && tr.ok) {
        std::ifstream f(cache_path, std::ios::binary);
        CacheHeader h;
        if (f && f.read(reinterpret_cast<char*>(&h), sizeof h) && std::memcmp(h.magic, "MFCACHE1", 8) == 0 &&
            h.train_size == tr.size && h.train_mtime_s == tr.mtime_s && h.train_mtime_ns == tr.mtime_ns &&
            h.test_size == (te.ok ? te.size : 0) && h.test_mtime_s == te.mtime_s && h.test_mtime_ns == te.mtime_ns &&
            h.test_path_hash == fnv1a(test_path)) {
            Dataset c;
            c.max_user = h.n_users; c.max_item = h.n_items; c.test_lines_kept = h.test_lines_kept; c.test_missing = h.test_missing;
            if (read_vec(f, c.R, h.n_train) && read_vec(f, c.test, h.n_test) && read_vec(f, c.user_orig, h.n_users) &&
                read_vec(f, c.item_orig, h.n_items) && read_vec(f, c.remove_user, h.n_remove_user) && read_vec(f, c.remove_item, h.n_remove_item)) {
                d = std::move(c);
                report_missing_and_write_remove_files(d, test_path);
                if (from_cache) *from_cache = true;
                return true;
            }
        }
    }
    if (!read_training_dataset(d, train_path)) return false;
    read_test_dataset(d, test_path);
    if (use_cache) {
        const std::string tmp = cache_path + ".tmp";
        std::ofstream f(tmp, std::ios::binary);
        CacheHeader h = {};
        std::memcpy(h.magic, "MFCACHE1", 8);
        h.train_size = tr.size; h.train_mtime_s = tr.mtime_s; h.train_mtime_ns = tr.mtime_ns;
        h.test_size = te.ok ? te.size : 0; h.test_mtime_s = te.mtime_s; h.test_mtime_ns = te.mtime_ns;
        h.test_path_hash = fnv1a(test_path);
        h.n_train = d.R.size(); h.n_test = d.test.size(); h.n_remove_user = d.remove_user.size(); h.n_remove_item = d.remove_item.size();
        h.n_users = d.max_user; h.n_items = d.max_item; h.test_lines_kept = d.test_lines_kept; h.test_missing = d.test_missing;
        bool ok = f && f.write(reinterpret_cast<const char*>(&h), sizeof h);
        ok = ok && write_vec(f, d.R) && write_vec(f, d.test) && write_vec(f, d.user_orig) && write_vec(f, d.item_orig) &&
             write_vec(f, d.remove_user) && write_vec(f, d.remove_item);
        f.close();
        if (ok && f) std::rename(tmp.c_str(), cache_path.c_str());
        else { std::remove(tmp.c_str()); std::cout << "could not write " << cache_path << " (continuing without the cache)" << std::endl; }
    }
    return true;
}
