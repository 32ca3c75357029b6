// Host-side I/O: logging, CSR ingestion with label grouping, LIBSVM text loading, key=value
// parameter parsing and the raw binary model file. No device code here.
#include <algorithm>
#include <cstring>
#include <fstream>
#include <iterator>
#include <thread>
#include <map>
#include <sstream>

#include "host.h"

namespace tgbm {

int g_verbose = 1;

void log_info(const char *fmt, ...) {
    if (g_verbose < 1) return;
    va_list ap;
    va_start(ap, fmt);
    std::fputs("INFO  ", stdout);
    std::vprintf(fmt, ap);
    std::fputc('\n', stdout);
    std::fflush(stdout);
    va_end(ap);
}

void log_debug(const char *fmt, ...) {
    if (g_verbose < 2) return;
    va_list ap;
    va_start(ap, fmt);
    std::fputs("DEBUG ", stdout);
    std::vprintf(fmt, ap);
    std::fputc('\n', stdout);
    std::fflush(stdout);
    va_end(ap);
}

void fatal(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    std::fputs("FATAL ", stderr);
    std::vfprintf(stderr, fmt, ap);
    std::fputc('\n', stderr);
    std::fflush(stderr);
    va_end(ap);
    std::abort();
}

bool objective_needs_group_label(const std::string &o) {
    return o == "multi:softprob" || o == "multi:softmax" || o == "binary:logistic";
}

// ObjectiveFunction::need_load_group_file (src/thundergbm/objective/objective_function.cu:23-25)
bool objective_needs_groups(const std::string &o) { return o == "rank:pairwise" || o == "rank:ndcg"; }

bool objective_supported(const std::string &o) {
    return o == "reg:linear" || o == "reg:logistic" || o == "binary:logistic" || o == "multi:softprob" ||
           o == "multi:softmax" || objective_needs_groups(o);
}

void DataSet::load_from_sparse(int n_rows, const float *val, const int *row_ptr, const int *col_idx,
                               const float *labels, const int *grp, int num_group, GBMParam &param,
                               bool count_features) {
    n_features_ = 0;
    y.clear();
    label.clear();
    group.clear();
    TGBM_CHECK(n_rows >= 0 && row_ptr != nullptr, "CSR input: %d rows", n_rows);
    TGBM_CHECK(row_ptr[0] == 0, "CSR input: row_ptr[0] is %d, expected 0", row_ptr[0]);
    for (int i = 0; i < n_rows; ++i)
        TGBM_CHECK(row_ptr[i + 1] >= row_ptr[i], "CSR input: row_ptr decreases at row %d (%d -> %d)", i, row_ptr[i],
                   row_ptr[i + 1]);
    const int nnz = row_ptr[n_rows];
    y.assign(n_rows, 0.f);
    if (labels != nullptr) std::copy(labels, labels + n_rows, y.begin());
    this->val = val;
    this->row_ptr = row_ptr;
    this->col_idx = col_idx;
    this->nnz = nnz;
    features_counted = count_features;
    if (count_features) {
        // largest column index, on a few threads when the matrix is large
        const int n_thr = nnz > (1 << 22) ? (int)std::min(8u, std::max(1u, std::thread::hardware_concurrency())) : 1;
        std::vector<int> part_max(n_thr, 0), part_min(n_thr, 0);
        auto scan = [&](int t) {
            const long b = (long)nnz * t / n_thr, e = (long)nnz * (t + 1) / n_thr;
            int m = 0, lo = 0;
            for (long i = b; i < e; ++i) {
                m = std::max(m, col_idx[i]);
                lo = std::min(lo, col_idx[i]);
            }
            part_max[t] = m;
            part_min[t] = lo;
        };
        std::vector<std::thread> pool;
        for (int t = 1; t < n_thr; ++t) pool.emplace_back(scan, t);
        scan(0);
        for (auto &th : pool) th.join();
        int max_col = 0;
        for (int m : part_max) max_col = std::max(max_col, m);
        for (int lo : part_min) TGBM_CHECK(lo >= 0, "CSR input: negative column index %d", lo);
        TGBM_CHECK(max_col < 2147483647, "CSR input: column index %d leaves no room for the feature count", max_col);
        n_features_ = (size_t)max_col + 1;
        log_info("#instances = %zu, #features = %zu", n_instances(), n_features());
    }
    if (labels != nullptr && objective_needs_group_label(param.objective)) {
        group_label();
        param.num_class = (int)label.size();
    }
    // query group sizes of the ranking objectives (dataset.cpp:64-68)
    if (objective_needs_groups(param.objective)) {
        for (int i = 0; i < num_group; ++i) group.push_back(grp[i]);
        log_info("#groups = %zu", group.size());
    }
}

// dataset.cpp:71-81: one group size per whitespace-separated token
void DataSet::load_group_file(const std::string &file_name) {
    log_info("loading group info from file \"%s\"", file_name.c_str());
    group.clear();
    std::ifstream ifs(file_name);
    TGBM_CHECK(ifs.is_open(), "ranking objective needs a group file, but file %s not found", file_name.c_str());
    int group_size;
    while (ifs >> group_size) group.push_back(group_size);
    log_info("#groups = %zu", group.size());
}

void DataSet::group_label() {
    // labels are truncated to int for the label set; the set is small, so every thread keeps a sorted set of
    // its part while scanning (no sort of all rows) and the sets are merged
    const int n_thr = y.size() > (1u << 22) ? (int)std::min(8u, std::max(1u, std::thread::hardware_concurrency())) : 1;
    std::vector<std::vector<int>> part(n_thr);
    auto collect = [&](int t) {
        const size_t b = y.size() * t / n_thr, e = y.size() * (t + 1) / n_thr;
        std::vector<int> &set = part[t];
        bool have_last = false;
        int last = 0;
        for (size_t i = b; i < e; ++i) {
            const int iv = (int)y[i];
            if (have_last && iv == last) continue;
            have_last = true;
            last = iv;
            auto it = std::lower_bound(set.begin(), set.end(), iv);
            if (it == set.end() || *it != iv) set.insert(it, iv);
        }
    };
    {
        std::vector<std::thread> pool;
        for (int t = 1; t < n_thr; ++t) pool.emplace_back(collect, t);
        collect(0);
        for (auto &th : pool) th.join();
    }
    std::vector<int> distinct;
    for (const std::vector<int> &set : part) {
        std::vector<int> merged;
        std::set_union(distinct.begin(), distinct.end(), set.begin(), set.end(), std::back_inserter(merged));
        distinct.swap(merged);
    }
    label.assign(distinct.begin(), distinct.end());
    // a row's class is the position of its label in the set; labels that are not in it (non-integers)
    // read as class 0, like a failed lookup in the reference's map
    auto remap = [&](int t) {
        const size_t b = y.size() * t / n_thr, e = y.size() * (t + 1) / n_thr;
        for (size_t i = b; i < e; ++i) {
            auto it = std::lower_bound(label.begin(), label.end(), y[i]);
            y[i] = (it != label.end() && *it == y[i]) ? (float)(it - label.begin()) : 0.f;
        }
    };
    std::vector<std::thread> pool;
    for (int t = 1; t < n_thr; ++t) pool.emplace_back(remap, t);
    remap(0);
    for (auto &th : pool) th.join();
}

// One chunk of LIBSVM text: whole lines in [b, e). strtof / strtol never run past a line end because a
// newline is not part of a number and is never skipped as leading white space here.
namespace {
struct LibsvmChunk {
    std::vector<float> y, val;
    std::vector<int> col, row_len;
    size_t max_fid = 0;
    size_t lines = 0;       // text lines of the chunk (data rows, comments and blank lines)
    size_t bad_line = 0;    // 1-based line of the chunk that holds a feature id outside 1 .. 2^31 - 1 (0: none)
    long bad_fid = 0;
};

void parse_libsvm_chunk(const char *b, const char *e, LibsvmChunk &out) {
    const char *line = b;
    while (line < e) {
        const char *eol = static_cast<const char *>(std::memchr(line, '\n', (size_t)(e - line)));
        if (eol == nullptr) eol = e;
        const char *p = line;
        line = eol + 1;
        ++out.lines;
        while (p < eol && (*p == ' ' || *p == '\t')) ++p;
        if (p >= eol || *p == '#' || *p == '\r') continue;
        char *end = nullptr;
        float lab = std::strtof(p, &end);
        if (end == p) continue;
        out.y.push_back(lab);
        p = end;
        int len = 0;
        for (;;) {
            while (p < eol && (*p == ' ' || *p == '\t' || *p == '\r')) ++p;
            if (p >= eol || *p == '#') break;
            long fid = std::strtol(p, &end, 10);
            if (end == p || *end != ':') break;
            p = end + 1;
            if (p >= eol) break;
            float v = std::strtof(p, &end);
            if (end == p) break;
            p = end;
            // LIBSVM feature ids are 1-based (dataset.cpp:243 stores fid - 1): a 0-based file would index column -1
            if ((fid < 1 || fid > 2147483647l) && out.bad_line == 0) {
                out.bad_line = out.lines;
                out.bad_fid = fid;
            }
            out.col.push_back((int)fid - 1);
            out.val.push_back(v);
            ++len;
            if ((size_t)fid > out.max_fid) out.max_fid = (size_t)fid;
        }
        out.row_len.push_back(len);
    }
}
}  // namespace

void DataSet::load_from_file(const std::string &file_name, GBMParam &param) {
    log_info("loading LIBSVM dataset from file ## %s ##", file_name.c_str());
    std::ifstream ifs(file_name, std::ifstream::binary | std::ifstream::ate);
    TGBM_CHECK(ifs.is_open(), "file ## %s ## not found. ", file_name.c_str());
    const size_t bytes = (size_t)ifs.tellg();
    ifs.seekg(0);
    std::string text(bytes + 1, '\0');  // one terminating NUL: the number parsers stop there
    ifs.read(&text[0], (std::streamsize)bytes);
    // chunks of whole lines, parsed by a few threads (the reference's loader splits the file the same way,
    // src/thundergbm/dataset.cpp:170-320), then concatenated in file order
    const int n_thr = bytes > (1u << 22) ? (int)std::min(16u, std::max(1u, std::thread::hardware_concurrency())) : 1;
    std::vector<size_t> cut(n_thr + 1, bytes);
    cut[0] = 0;
    for (int t = 1; t < n_thr; ++t) {
        size_t pos = std::max(cut[t - 1], bytes * t / n_thr);
        const char *nl = pos < bytes ? static_cast<const char *>(std::memchr(text.data() + pos, '\n', bytes - pos)) : nullptr;
        cut[t] = nl ? (size_t)(nl - text.data()) + 1 : bytes;
    }
    std::vector<LibsvmChunk> chunks(n_thr);
    {
        std::vector<std::thread> pool;
        for (int t = 1; t < n_thr; ++t)
            pool.emplace_back([&, t] { parse_libsvm_chunk(text.data() + cut[t], text.data() + cut[t + 1], chunks[t]); });
        parse_libsvm_chunk(text.data() + cut[0], text.data() + cut[1], chunks[0]);
        for (auto &th : pool) th.join();
    }
    y.clear();
    label.clear();
    csr_val.clear();
    csr_col_idx.clear();
    csr_row_ptr.assign(1, 0);
    n_features_ = 0;
    size_t rows = 0, entries = 0, lines_before = 0;
    for (const LibsvmChunk &c : chunks) {
        TGBM_CHECK(c.bad_line == 0,
                   "%s line %zu: feature id %ld is outside 1 .. 2^31 - 1 (LIBSVM feature ids are 1-based)",
                   file_name.c_str(), lines_before + c.bad_line, c.bad_fid);
        lines_before += c.lines;
        rows += c.y.size();
        entries += c.val.size();
    }
    TGBM_CHECK(entries < ((size_t)1 << 31), "more than 2^31 stored values");
    y.reserve(rows);
    csr_val.reserve(entries);
    csr_col_idx.reserve(entries);
    csr_row_ptr.reserve(rows + 1);
    for (const LibsvmChunk &c : chunks) {
        y.insert(y.end(), c.y.begin(), c.y.end());
        csr_val.insert(csr_val.end(), c.val.begin(), c.val.end());
        csr_col_idx.insert(csr_col_idx.end(), c.col.begin(), c.col.end());
        for (int len : c.row_len) csr_row_ptr.push_back(csr_row_ptr.back() + len);
        n_features_ = std::max(n_features_, c.max_fid);
    }
    val = csr_val.data();
    row_ptr = csr_row_ptr.data();
    col_idx = csr_col_idx.data();
    nnz = (long)csr_val.size();
    label = y;  // the reference keeps a copy of all labels here (dataset.cpp:290-291) ...
    log_info("#instances = %zu, #features = %zu", n_instances(), n_features());
    if (objective_needs_groups(param.objective)) load_group_file(file_name + ".group");  // dataset.cpp:302
    if (objective_needs_group_label(param.objective)) {
        group_label();  // ... which grouping replaces by the distinct ones
        param.num_class = (int)label.size();
    }
}

// ---------------------------------------------------------------------------------------------
void Parser::parse_param(GBMParam &p, int argc, char **argv) {
    p = GBMParam();  // defaults of src/thundergbm/parser.cpp:10-28
    if (argc < 2) {
        std::printf("Usage: <config>\n");
        std::exit(0);
    }
    auto parse_value = [&](const char *name_val) {
        char name[256], val[256];
        if (std::sscanf(name_val, "%255[^=]=%255s", name, val) == 2) {
            std::string k(name);
            if (k == "max_depth" || k == "depth") p.depth = std::atoi(val);
            else if (k == "num_round" || k == "n_trees") p.n_trees = std::atoi(val);
            else if (k == "n_gpus") p.n_device = std::atoi(val);
            else if (k == "verbosity" || k == "verbose") p.verbose = std::atoi(val);
            else if (k == "profiling") p.profiling = std::atoi(val);
            else if (k == "data") p.path = val;
            else if (k == "max_bin" || k == "max_num_bin") p.max_num_bin = std::atoi(val);
            else if (k == "colsample" || k == "column_sampling_rate") p.column_sampling_rate = (float)std::atof(val);
            else if (k == "bagging") p.bagging = std::atoi(val);
            else if (k == "num_parallel_tree" || k == "n_parallel_trees") p.n_parallel_trees = std::atoi(val);
            else if (k == "eta" || k == "learning_rate") p.learning_rate = (float)std::atof(val);
            else if (k == "objective") p.objective = val;
            else if (k == "num_class") p.num_class = std::atoi(val);
            else if (k == "min_child_weight") p.min_child_weight = (float)std::atoi(val);  // atoi, as parser.cpp:67
            else if (k == "lambda" || k == "lambda_tgbm") p.lambda = (float)std::atof(val);
            else if (k == "gamma" || k == "min_split_loss") p.gamma = (float)std::atof(val);
            else if (k == "tree_method") p.tree_method = val;
            else log_info("\"%s\" is unknown option!", name);
        } else if (std::string(name_val) == "-help") {
            std::printf("please refer to \"docs/parameters.md\" in the GitHub repository for more information "
                        "about setting the options\n");
            std::exit(0);
        }
    };
    std::ifstream conf(argv[1]);
    std::string line;
    while (std::getline(conf, line)) parse_value(line.c_str());
    for (int i = 0; i < argc; ++i) parse_value(argv[i]);
}

// Model file (src/thundergbm/parser.cpp:102-171), little endian, no header:
// i32 len | objective | f32 lr | i32 num_class | i32 n_trees | f32 base_score | i32 n_label |
// f32 label[] | i32 n_iter | per iter { i32 n_trees_in_iter | per tree { u64 n_nodes | TreeNode[] } }
void Parser::save_model(const std::string &path, const GBMParam &param, const std::vector<std::vector<Tree>> &model,
                        const DataSet &dataset) {
    std::ofstream out(path, std::ios::binary);
    TGBM_CHECK(out.is_open(), "cannot open %s for writing", path.c_str());
    auto put = [&](const void *p, size_t n) { out.write(static_cast<const char *>(p), (std::streamsize)n); };
    int len = (int)param.objective.size();
    put(&len, 4);
    put(param.objective.data(), (size_t)len);
    put(&param.learning_rate, 4);
    put(&param.num_class, 4);
    put(&param.n_trees, 4);
    put(&param.base_score, 4);
    int n_label = (int)dataset.label.size();
    put(&n_label, 4);
    put(dataset.label.data(), sizeof(float) * (size_t)n_label);
    int n_iter = (int)model.size();
    put(&n_iter, 4);
    for (const auto &iter : model) {
        int n_in = (int)iter.size();
        put(&n_in, 4);
        for (const Tree &t : iter) {
            uint64_t n_nodes = t.nodes.size();
            put(&n_nodes, 8);
            put(t.nodes.data(), sizeof(TreeNode) * t.nodes.size());
        }
    }
}

void Parser::load_model(const std::string &path, GBMParam &param, std::vector<std::vector<Tree>> &model,
                        DataSet &dataset) {
    std::ifstream in(path, std::ios::binary);
    TGBM_CHECK(in.is_open(), "cannot open model file %s", path.c_str());
    auto get = [&](void *p, size_t n) {
        in.read(static_cast<char *>(p), (std::streamsize)n);
        TGBM_CHECK((size_t)in.gcount() == n, "model file %s is truncated", path.c_str());
    };
    int len = 0;
    get(&len, 4);
    TGBM_CHECK(len >= 0 && len < 4096, "model file %s: bad objective length", path.c_str());
    std::string obj((size_t)len, '\0');
    get(&obj[0], (size_t)len);
    param.objective = obj;
    get(&param.learning_rate, 4);
    get(&param.num_class, 4);
    get(&param.n_trees, 4);
    get(&param.base_score, 4);
    int n_label = 0;
    get(&n_label, 4);
    TGBM_CHECK(n_label >= 0, "model file %s: bad label count", path.c_str());
    dataset.label.assign((size_t)n_label, 0.f);
    get(dataset.label.data(), sizeof(float) * (size_t)n_label);
    int n_iter = 0;
    get(&n_iter, 4);
    model.clear();
    for (int i = 0; i < n_iter; ++i) {
        int n_in = 0;
        get(&n_in, 4);
        std::vector<Tree> iter((size_t)n_in);
        for (Tree &t : iter) {
            uint64_t n_nodes = 0;
            get(&n_nodes, 8);
            TGBM_CHECK(n_nodes < (1ull << 28), "model file %s: bad node count", path.c_str());
            t.nodes.resize((size_t)n_nodes);
            get(t.nodes.data(), sizeof(TreeNode) * (size_t)n_nodes);
        }
        model.push_back(std::move(iter));
    }
}

}  // namespace tgbm
