// TEST INFRASTRUCTURE ONLY.
//
// CPU restatement of ThunderGBM's single-GPU histogram trainer ("hist_single") and predictor.
// It is the parity checker for the HIP library and the same-box CPU baseline of the benchmark.
// Nothing in the shipped library links, loads or calls this file.
//
// The reference has no CPU training path (docs/faq.md:10-11) and is CUDA-only, so it cannot be
// compiled here; every function below restates the algorithm of the cited reference lines.
// Paths are relative to the reference checkout.
//
// What pins each function (tests/test_oracle_*.py):
//   cut points      closed-form rule on hand inputs, invariants, the a1a fixture (one cut = 1.0 per feature)
//   bin ids         brute force min(#cuts<=v, k-1) against numpy searchsorted
//   gradients       float64 closed forms
//   base score      mean(y) for reg:linear, the logit closed form for binary:logistic, 0 for softmax / ranking
//   histogram       brute-force float64 accumulation; bin counts for squared loss (the oracle itself
//                   accumulates in float64 and rounds once: the reference's float atomics have no defined
//                   order, so their result is only defined up to float round-off)
//   split finding   brute-force enumeration of (feature, bin, direction) in numpy float64
//   update/partition row counts equal hessian sums for squared loss; raw-value threshold consistency
//   prune           hand-built 7-node trees
//   predictor       equality with the training-time prediction on the training rows
//   metrics         reference KATs src/test/test_metrics.cpp:70,84,96; tree size src/test/test_tree.cpp:68
//   bagging         the draws against vectors produced by the thrust headers this image ships (rocThrust;
//                   tests/golden/bagging_thrust_vectors.hip), the engine is libstdc++'s std::minstd_rand
//   ranking         LambdaRank gradients: two-row groups (closed form), pair bookkeeping by brute force over the
//                   group (every drawing position pairs with a position outside its run of equal labels, the
//                   lambdas of a pair cancel), |delta NDCG| = the change of DCG when the two positions swap;
//                   MAP / NDCG: hand-computed lists, a perfect ranking scores 1
// Parity unpinned (no run of the reference is possible): the association order of the reference's
// fp32 sums (atomics, thrust scan/reduce), device expf ulps, ordering of +0.0/-0.0 duplicates in
// the cut-point sort; for the ranking objectives the tie order of std::sort and the std::mt19937 partner
// draws seeded from rand() inside an OpenMP loop (both unspecified in the reference: ties keep row order here
// and draws are a function of (round seed, position)).
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <new>
#include <random>
#include <string>
#include <vector>
#ifdef _OPENMP
#include <omp.h>
#endif

namespace {

struct GH {
    float g, h;
};

// Layout of Tree::TreeNode, include/thundergbm/tree.h:14-30 (48 bytes).
struct Node {
    int final_id, lch, rch, parent;
    float gain, base_weight;
    int split_fid;
    float split_value;
    unsigned char split_bid;
    bool default_right, is_leaf, is_valid, is_pruned;
    GH sum;
};
static_assert(sizeof(Node) == 48, "TreeNode must be 48 bytes");

// Per-node best split, the information of SplitPoint in include/thundergbm/builder/shard.h:23-47
// laid out for the tests (fixed 48 bytes).
struct Split {
    float gain;
    GH missing;
    GH lch_sum;
    int default_right;
    int nid;
    int fid;
    float fval;
    int bid;         // local bin id (split_bid, truncated to unsigned char like the reference)
    int best_index;  // global bin index of the winning candidate
    int pad;
};
static_assert(sizeof(Split) == 48, "Split must be 48 bytes");

inline float calc_weight(GH s, float lambda) { return -s.g / (s.h + lambda); }

// compute_gain lambda, src/thundergbm/builder/hist_tree_builder_single.cu:282-289
inline float compute_gain(GH f, GH l, GH r, float mcw, float lambda) {
    if (l.h >= mcw && r.h >= mcw)
        return (l.g * l.g) / (l.h + lambda) + (r.g * r.g) / (r.h + lambda) - (f.g * f.g) / (f.h + lambda);
    return 0.f;
}

// A level's histograms (nodes x bins): memory that is never touched by one thread alone. A wide sparse configuration
// needs gigabytes per level, and a std::vector would fault its pages in and fill them sequentially.
template <typename T>
struct ZeroedBuffer {
    T *p = nullptr;
    size_t cap = 0, n = 0;
    ZeroedBuffer() = default;
    ZeroedBuffer(const ZeroedBuffer &) = delete;
    ZeroedBuffer &operator=(const ZeroedBuffer &) = delete;
    ~ZeroedBuffer() { std::free(p); }
    T *data() { return p; }
    const T *data() const { return p; }
    size_t size() const { return n; }
    void assign_zero(size_t count) {
        if (count > cap) {
            std::free(p);
            p = (T *)std::malloc(std::max<size_t>(count, 1) * sizeof(T));
            if (!p) throw std::bad_alloc();
            cap = count;
        }
        n = count;
        T *q = p;
#pragma omp parallel for schedule(static) if (count > 200000)
        for (long i = 0; i < (long)count; ++i) q[i] = T{};
    }
    void swap(ZeroedBuffer &o) {
        std::swap(p, o.p);
        std::swap(cap, o.cap);
        std::swap(n, o.n);
    }
};

struct ProbeResult {
    float score;         // signed gain of the probed candidate (0 when the node was not evaluated)
    float dir_gap;       // its gain(missing -> left) - gain(missing -> right)
    float best;          // |gain| of the node's best candidate
    float best_dir_gap;  // gain(missing -> left) - gain(missing -> right) of the best candidate
};

struct Oracle {
    float column_sampling_rate = 1.f;
    bool bagging = false;
    std::vector<char> ignored;  // per feature, this round (empty: none)
    // data (DataSet, src/thundergbm/dataset.cpp:20-63)
    int n = 0, F = 0;
    long nnz = 0;
    std::vector<float> val;
    std::vector<int> col, row_ptr;
    std::vector<float> y;      // mapped to class index for classification
    std::vector<float> label;  // distinct labels
    std::vector<int> group;    // query group sizes (ranking objectives, dataset.cpp:64-68)
    // params (GBMParam, include/thundergbm/common.h:86-111)
    int depth = 6, n_trees = 40, max_num_bin = 255, num_class = 1, tree_per_rounds = 1;
    float mcw = 1, lambda = 1, gamma = 1, rt_eps = 1e-6f, lr = 1, base_score = 0;
    std::string objective = "reg:linear";
    // cuts (HistCut)
    std::vector<float> cut_val;
    std::vector<int> cut_row_ptr, cut_fid;
    int n_bins = 0;
    std::vector<int> bin_id;  // global bin id per nnz
    // training state
    std::vector<float> y_pred;  // class-major
    std::vector<GH> gh;         // class-major
    std::vector<int> nid;
    std::vector<Node> nodes;
    std::vector<Split> sp;
    int cur_class = 0;
    int cur_level = -1;
    bool keep_debug = false;
    bool shadow64 = false;
    // raw (unscanned) histograms of the current and previous level, node-major
    ZeroedBuffer<GH> hist_cur, hist_prev;
    ZeroedBuffer<double> hist64_cur, hist64_prev;  // g,h interleaved
    std::vector<double> hist_scratch;             // build_hist: one fp64 histogram per thread
    std::vector<GH> eval_pre, eval_miss;          // evaluate_node: prefix sums per bin, missing sums per feature
    // debug: per node of the whole tree
    std::vector<float> dbg_score;   // [n_nodes][n_bins], signed gain of every candidate
    std::vector<float> dbg_dir_gap; // [n_nodes][n_bins], gain(missing -> left) - gain(missing -> right) of every candidate
    std::vector<GH> dbg_hist;       // [n_nodes][n_bins], raw hist
    std::vector<double> dbg_hist64; // [n_nodes][n_bins][2]
    std::vector<int> dbg_built;     // [n_nodes] 1 if built from rows, 0 if by subtraction
    // Probes: the debug arrays above need n_nodes x n_bins floats, gigabytes for wide data. A probe names one
    // candidate (global bin index, -1 = none) per node whose signed gain is recorded next to the node's best.
    std::vector<int> probe;              // [n_nodes]
    std::vector<ProbeResult> probe_out;  // [n_nodes]
    std::vector<std::vector<Node>> model;  // iteration-major, class inside
    std::vector<float> metric_log;
    long rows_built_total = 0;      // rows visited by histogram builds (for byte accounting)
    std::vector<long> rows_built_level;
};

// ---------------------------------------------------------------------------------------------
// a1  HistCut::get_cut_points_single, src/thundergbm/hist_cut.cu:232-286 (sort/unique :205-228,
// comparator :196-203, stride selection :259-265 with interval = n_unique / max_num_bins from
// include/thundergbm/util/device_lambda.cuh:33-42).
int cut_points(int F, long nnz, const float *val, const int *col, int max_bin, std::vector<float> &cut_val,
               std::vector<int> &cut_row_ptr, std::vector<int> &cut_fid) {
    std::vector<long> cnt(F + 1, 0);
    for (long i = 0; i < nnz; ++i) cnt[col[i] + 1]++;
    for (int f = 0; f < F; ++f) cnt[f + 1] += cnt[f];
    std::vector<float> byf(nnz);
    {
        std::vector<long> pos(cnt.begin(), cnt.end() - 1);
        for (long i = 0; i < nnz; ++i) byf[pos[col[i]]++] = val[i];
    }
    std::vector<std::vector<float>> per(F);
#pragma omp parallel for schedule(dynamic, 1)
    for (int f = 0; f < F; ++f) {
        float *b = byf.data() + cnt[f], *e = byf.data() + cnt[f + 1];
        if (b == e) continue;
        std::sort(b, e);
        e = std::unique(b, e);  // distinct by ==
        long m = e - b;
        long step = m / max_bin;
        std::vector<float> &out = per[f];
        if (step == 0) {
            out.assign(b, e);
        } else {
            out.reserve(max_bin);
            for (long j = 0; j < max_bin; ++j) out.push_back(b[j * step]);
        }
    }
    cut_val.clear();
    cut_fid.clear();
    cut_row_ptr.assign(F + 1, 0);
    for (int f = 0; f < F; ++f) {
        cut_row_ptr[f] = (int)cut_val.size();
        for (float v : per[f]) {
            cut_val.push_back(v);
            cut_fid.push_back(f);
        }
    }
    cut_row_ptr[F] = (int)cut_val.size();
    return (int)cut_val.size();
}

// a2  HistTreeBuilder_single::get_bin_ids, hist_tree_builder_single.cu:81-119: upper bound with
// the right end clamped to the feature's last cut, plus the feature's global offset.
inline int bin_of(const float *cut_val, const int *cut_row_ptr, int fid, float v) {
    const float *begin = cut_val + cut_row_ptr[fid];
    const float *end = cut_val + cut_row_ptr[fid + 1];
    const float *left = begin, *right = end - 1;
    while (left < right) {
        const float *mid = left + (right - left) / 2;
        if (*mid <= v)
            left = mid + 1;
        else
            right = mid;
    }
    return (int)(left - begin) + cut_row_ptr[fid];
}

// a3  gradients. SquareLoss include/thundergbm/objective/regression_obj.h:130-134, LogisticLoss
// :145-154, Softmax src/thundergbm/objective/multiclass_obj.cu:6-35.
void gradient(const std::string &obj, int n, int num_class, const float *y, const float *yp, GH *gh) {
    if (obj == "reg:linear") {
#pragma omp parallel for
        for (int i = 0; i < n; ++i) gh[i] = GH{yp[i] - y[i], 1.f};
    } else if (obj == "binary:logistic" || obj == "reg:logistic") {
#pragma omp parallel for
        for (int i = 0; i < n; ++i) {
            float p = 1 / (1 + expf(-yp[i]));
            gh[i] = GH{p - y[i], fmaxf(p * (1 - p), 1e-16f)};
        }
    } else {  // multi:softmax / multi:softprob
#pragma omp parallel for
        for (int i = 0; i < n; ++i) {
            float mx = yp[i];
            for (int k = 1; k < num_class; ++k) mx = fmaxf(mx, yp[(long)k * n + i]);
            float sum = 0;
            for (int k = 0; k < num_class; ++k) sum += expf(yp[(long)k * n + i] - mx);
            for (int k = 0; k < num_class; ++k) {
                float p = expf(yp[(long)k * n + i] - mx) / sum;
                float g = (k == y[i]) ? (p - 1) : (p - 0);
                float h = fmaxf(2 * p * (1 - p), 1e-16f);
                gh[(long)k * n + i] = GH{g, h};
            }
        }
    }
}

// DataSet::group_label, src/thundergbm/dataset.cpp:83-101: distinct int-truncated labels in
// ascending order; y is looked up by its exact float value, unknown keys map to 0.
void group_label(std::vector<float> &y, std::vector<float> &label) {
    std::vector<int> t(y.begin(), y.end());
    std::sort(t.begin(), t.end());
    t.erase(std::unique(t.begin(), t.end()), t.end());
    std::map<float, int> m;
    label.clear();
    for (int v : t) {
        m[(float)v] = (int)label.size();
        label.push_back((float)v);
    }
    for (float &v : y) v = (float)m[v];
}


// fp32 sum of (g,h) in a tree order: 256-element sequential leaves, then pairwise. The reference uses
// thrust::reduce (src/thundergbm/tree.cu:31, regression_obj.h:41,101), whose order is unspecified
// but tree-shaped; a long sequential float32 sum of near-constant hessians would drift by more than
// the comparison tolerance.
GH sum_gh(const GH *g, long n) {
    const long CH = 256;
    long nch = (n + CH - 1) / CH;
    std::vector<GH> part((size_t)std::max<long>(nch, 1), GH{0, 0});
#pragma omp parallel for
    for (long c = 0; c < nch; ++c) {
        float a = 0, b = 0;
        long e = std::min<long>(n, (c + 1) * CH);
        for (long i = c * CH; i < e; ++i) {
            a += g[i].g;
            b += g[i].h;
        }
        part[c] = GH{a, b};
    }
    for (long m = nch; m > 1;) {
        long half = (m + 1) / 2;
        for (long i = 0; i + half < m; ++i) {
            part[i].g += part[i + half].g;
            part[i].h += part[i + half].h;
        }
        m = half;
    }
    return part[0];
}

// a4  Tree::init2, src/thundergbm/tree.cu:8-39
void tree_init(Oracle &o, int k) {
    o.cur_class = k;
    int n_max = (1 << (o.depth + 1)) - 1;
    o.nodes.assign(n_max, Node{});
    for (int i = 0; i < n_max; ++i) {
        Node &nd = o.nodes[i];
        std::memset(&nd, 0, sizeof(Node));
        nd.final_id = i;
        nd.split_fid = -1;
        nd.is_valid = false;
        nd.parent = i == 0 ? -1 : (i - 1) / 2;
        if (i < n_max / 2) {
            nd.is_leaf = false;
            nd.lch = 2 * i + 1;
            nd.rch = 2 * i + 2;
        } else {
            nd.is_leaf = true;
            nd.lch = nd.rch = -1;
        }
    }
    const GH rs = sum_gh(o.gh.data() + (long)k * o.n, o.n);
    const float fg = rs.g, fh = rs.h;
    Node &root = o.nodes[0];
    root.sum = GH{fg, fh};
    root.is_valid = true;
    root.base_weight = calc_weight(root.sum, o.lambda);
    std::fill(o.nid.begin(), o.nid.end(), 0);  // ins2node_id.resize(n) zero-fills, tree_builder.cu:156
    o.cur_level = -1;
    if (o.keep_debug) {
        o.dbg_score.assign((size_t)n_max * o.n_bins, 0.f);
        o.dbg_dir_gap.assign((size_t)n_max * o.n_bins, 0.f);
        o.dbg_hist.assign((size_t)n_max * o.n_bins, GH{0, 0});
        if (o.shadow64) o.dbg_hist64.assign((size_t)n_max * o.n_bins * 2, 0.0);
        o.dbg_built.assign(n_max, -1);
    }
}

// Histogram of one node from a list of rows (root: rows == nullptr means 0..cnt-1).
// hist_tree_builder_single.cu:203-216 (root) and :485-505 (node): hist[global_bin] += (g,h) for every
// stored entry of every row; zero g / zero h contributions are skipped (no effect on the sum).
void build_hist(Oracle &o, const int *rows, long cnt, GH *out, double *out64) {
    const int B = o.n_bins;
    const GH *gh = o.gh.data() + (long)o.cur_class * o.n;
    int nt = 1;
#ifdef _OPENMP
    nt = omp_get_max_threads();
#endif
    if (cnt < 4096) nt = 1;
    // (a private histogram per thread is only worth its clearing and adding up when the node's stored entries
    // outnumber the bins: wide sparse data has millions of bins and deep nodes of a few thousand rows)
    const double entries = (double)cnt * (double)o.row_ptr[o.n] / (double)std::max(1, o.n);
    nt = (int)std::max(1.0, std::min((double)nt, entries / (0.5 * (double)std::max(1, B))));
    // The reference adds with float atomics in no defined order, so its own result varies from run to run
    // by float round-off that grows with the number of rows per bin. The oracle accumulates in fp64 and
    // rounds once: the centre of those possible results, and what the 1e-5 parity tolerance refers to.
    std::vector<double> &priv64 = o.hist_scratch;
    if (priv64.size() < (size_t)nt * B * 2) priv64.resize((size_t)nt * B * 2);
#pragma omp parallel for schedule(static) if ((size_t)nt * B > 200000)
    for (long i = 0; i < (long)nt * B * 2; ++i) priv64[i] = 0.0;
#pragma omp parallel num_threads(nt)
    {
        int t = 0;
#ifdef _OPENMP
        t = omp_get_thread_num();
#endif
        double *h64 = priv64.data() + (size_t)t * B * 2;
        long b = cnt * t / nt, e = cnt * (t + 1) / nt;
        for (long r = b; r < e; ++r) {
            int i = rows ? rows[r] : (int)r;
            GH s = gh[i];
            for (int j = o.row_ptr[i]; j < o.row_ptr[i + 1]; ++j) {
                int bid = o.bin_id[j];
                h64[2 * bid] += (double)s.g;
                h64[2 * bid + 1] += (double)s.h;
            }
        }
    }
#pragma omp parallel for schedule(static) if (B > 100000)
    for (int b = 0; b < B; ++b) {
        double g = 0, h = 0;
        for (int t = 0; t < nt; ++t) {
            g += priv64[(size_t)t * B * 2 + 2 * b];
            h += priv64[(size_t)t * B * 2 + 2 * b + 1];
        }
        out[b] = GH{(float)g, (float)h};
        if (out64) {
            out64[2 * b] = g;
            out64[2 * b + 1] = h;
        }
    }
    o.rows_built_total += cnt;
}

// Scan + missing + gain + argmax + record for one node given its raw histogram.
// hist_tree_builder_single.cu:257-390 (root) / :614-752 (pair member).
// Shard::column_sampling, src/thundergbm/builder/shard.cu:8-22, called once per boosting round
// (builder/tree_builder.cu:150-152): shuffle 0..F-1 with std::random_shuffle (process-wide rand()) and mark
// the first max(1, int(F * rate)) columns as *ignored* for the round (the array is re-created, i.e. zeroed,
// by every call: syncarray.h:103-113, syncmem.cpp:76-120). The oracle calls the very library routine the
// reference calls.
void sample_columns(Oracle &o) {
    if (!(o.column_sampling_rate < 1)) return;
    std::vector<int> idx(o.F);
    for (int i = 0; i < o.F; ++i) idx[i] = i;
    std::random_shuffle(idx.begin(), idx.end());
    int sample_count = std::max(1, int(o.F * o.column_sampling_rate));
    o.ignored.assign(o.F, 0);
    for (int i = 0; i < sample_count; ++i) o.ignored[idx[i]] = 1;
}

void evaluate_node(Oracle &o, int node, const GH *raw, Split &s) {
    const int B = o.n_bins, F = o.F;
    const Node &nd = o.nodes[node];
    if (!nd.is_valid) {
        std::memset(&s, 0, sizeof(Split));
        s.fid = -1;
        s.nid = -1;
        return;
    }
    std::vector<GH> &pre = o.eval_pre;
    std::vector<GH> &miss = o.eval_miss;
    pre.resize(B);
    miss.assign(F, GH{0, 0});
    const GH S = nd.sum;
    // (wide data: features in parallel; every feature's scan and every candidate's gain is computed exactly as in the
    // sequential loop, and the arg-max below combines the threads' ranges in ascending order of their bins)
    const bool par = B > 100000;
    // inclusive_scan_by_key over cut_fid (:257, :614): fp32 running sums restarting per feature
#pragma omp parallel for schedule(static) if (par)
    for (int f = 0; f < F; ++f) {
        float g = 0, h = 0;
        for (int b = o.cut_row_ptr[f]; b < o.cut_row_ptr[f + 1]; ++b) {
            g += raw[b].g;
            h += raw[b].h;
            pre[b] = GH{g, h};
        }
        // missing_gh (:265-274): only for splittable nodes and features with at least one cut
        if (!nd.is_leaf && o.cut_row_ptr[f + 1] != o.cut_row_ptr[f]) {
            GH last = pre[o.cut_row_ptr[f + 1] - 1];
            miss[f] = GH{S.g - last.g, S.h - last.h};
        }
    }
    int best = 0;
    float best_score = 0;
    bool first = true;
    float *dbg = o.keep_debug ? o.dbg_score.data() + (size_t)node * B : nullptr;
    int n_parts = 1;
#ifdef _OPENMP
    if (par) n_parts = omp_get_max_threads();
#endif
    std::vector<int> part_best(n_parts, -1);
    std::vector<float> part_score(n_parts, 0.f);
#pragma omp parallel for schedule(static, 1) if (par)
    for (int part = 0; part < n_parts; ++part) {
        const int b_lo = (int)((long)B * part / n_parts), b_hi = (int)((long)B * (part + 1) / n_parts);
        int pb = -1;
        float ps = 0;
        for (int b = b_lo; b < b_hi; ++b) {
            int f = o.cut_fid[b];
            GH l = GH{0, 0};
            if (o.cut_row_ptr[f] != b) l = pre[b - 1];
            GH r = GH{S.g - l.g, S.h - l.h};
            float gr = fmaxf(0.f, compute_gain(S, l, r, o.mcw, o.lambda));
            GH l2 = GH{l.g + miss[f].g, l.h + miss[f].h};
            GH r2 = GH{S.g - l2.g, S.h - l2.h};
            float gl = fmaxf(0.f, compute_gain(S, l2, r2, o.mcw, o.lambda));
            float score = (gl > gr) ? gl : -gr;
            if (!o.ignored.empty() && o.ignored[f]) score = 0;  // :304 / :663: an ignored column's gain is 0
            if (dbg) {
                dbg[b] = score;
                o.dbg_dir_gap[(size_t)node * B + b] = gl - gr;
            }
            if (!o.probe.empty() && (size_t)node < o.probe.size() && o.probe[node] == b)
                o.probe_out[node] = ProbeResult{score, gl - gr, 0.f, 0.f};
            // arg_abs_max (:330-335): larger |gain| wins, ties keep the smaller index
            if (pb < 0 || fabsf(score) > fabsf(ps)) {
                pb = b;
                ps = score;
            }
        }
        part_best[part] = pb;
        part_score[part] = ps;
    }
    for (int part = 0; part < n_parts; ++part) {
        if (part_best[part] < 0) continue;
        if (first || fabsf(part_score[part]) > fabsf(best_score)) {
            best = part_best[part];
            best_score = part_score[part];
            first = false;
        }
    }
    if (!o.probe.empty() && (size_t)node < o.probe.size() && B > 0) {
        // the chosen candidate's two direction gains once more, for the probe record
        int f = o.cut_fid[best];
        GH l = GH{0, 0};
        if (o.cut_row_ptr[f] != best) l = pre[best - 1];
        GH r = GH{S.g - l.g, S.h - l.h};
        float gr = fmaxf(0.f, compute_gain(S, l, r, o.mcw, o.lambda));
        GH l2 = GH{l.g + miss[f].g, l.h + miss[f].h};
        GH r2 = GH{S.g - l2.g, S.h - l2.h};
        float gl = fmaxf(0.f, compute_gain(S, l2, r2, o.mcw, o.lambda));
        o.probe_out[node].best = fabsf(best_score);
        o.probe_out[node].best_dir_gap = gl - gr;
    }
    std::memset(&s, 0, sizeof(Split));
    if (B == 0) {  // no candidate at all: behaves as a zero-gain split point
        s.nid = node;
        s.fid = -1;
        return;
    }
    int f = o.cut_fid[best];
    s.fid = f;
    s.nid = node;
    s.gain = fabsf(best_score);
    s.bid = (int)(unsigned char)(best - o.cut_row_ptr[f]);
    s.missing = miss[f];
    s.default_right = best_score < 0;
    s.lch_sum = GH{0, 0};
    float c0 = o.cut_val[o.cut_row_ptr[f]];
    s.fval = (float)((double)(c0 - fabsf(c0)) - 1e-5);  // :383
    if (best != o.cut_row_ptr[f]) {
        s.lch_sum = pre[best - 1];
        s.fval = o.cut_val[best - 1];
    }
    s.best_index = best;
}

void stash_debug(Oracle &o, int node, const GH *raw, const double *raw64, int built) {
    if (!o.keep_debug) return;
    std::copy(raw, raw + o.n_bins, o.dbg_hist.begin() + (size_t)node * o.n_bins);
    if (o.shadow64 && raw64)
        std::copy(raw64, raw64 + 2 * o.n_bins, o.dbg_hist64.begin() + (size_t)node * o.n_bins * 2);
    o.dbg_built[node] = built;
}

// a5/a6  HistTreeBuilder_single::find_split, hist_tree_builder_single.cu:132-780
void find_split(Oracle &o, int level) {
    const int B = o.n_bins;
    const int n_level = 1 << level;
    const int off = n_level - 1;
    o.sp.assign(n_level, Split{});
    o.hist_cur.swap(o.hist_prev);
    o.hist64_cur.swap(o.hist64_prev);
    o.hist_cur.assign_zero((size_t)n_level * B);
    if (o.shadow64) o.hist64_cur.assign_zero((size_t)n_level * B * 2);
    long built_rows_before = o.rows_built_total;
    if (level == 0) {
        build_hist(o, nullptr, o.n, o.hist_cur.data(), o.shadow64 ? o.hist64_cur.data() : nullptr);
        stash_debug(o, 0, o.hist_cur.data(), o.shadow64 ? o.hist64_cur.data() : nullptr, 1);
        evaluate_node(o, 0, o.hist_cur.data(), o.sp[0]);
    } else {
        // rows of every node of this level in ascending row order (stable radix sort by node id,
        // :401-412)
        std::vector<int> ptr(n_level + 1, 0);
        for (int i = 0; i < o.n; ++i) {
            int x = o.nid[i] - off;
            if (x >= 0 && x < n_level) ptr[x + 1]++;
        }
        for (int x = 0; x < n_level; ++x) ptr[x + 1] += ptr[x];
        std::vector<int> idx(ptr[n_level]);
        {
            std::vector<int> pos(ptr.begin(), ptr.end() - 1);
            for (int i = 0; i < o.n; ++i) {
                int x = o.nid[i] - off;
                if (x >= 0 && x < n_level) idx[pos[x]++] = i;
            }
        }
        for (int p = 0; p < n_level / 2; ++p) {
            int a = 2 * p, b = 2 * p + 1;  // compute a, subtract b
            int nl = ptr[a + 1] - ptr[a], nr = ptr[b + 1] - ptr[b];
            if (std::max(nl, nr) == 0) {
                // :454-465. Both siblings empty: invalid nodes are flagged. A valid pair without rows
                // cannot occur (a split with an empty side has zero gain); instead of reproducing the
                // reference's zero-initialised SplitPoint (which would address node 0) such a node is
                // evaluated on an all-zero histogram and therefore becomes a leaf.
                for (int j = 0; j < 2; ++j)
                    evaluate_node(o, off + 2 * p + j, o.hist_cur.data() + (size_t)(2 * p + j) * B, o.sp[2 * p + j]);
                continue;
            }
            if (nl > nr) std::swap(a, b);  // build the one with fewer rows, ties build the left one
            GH *ha = o.hist_cur.data() + (size_t)a * B;
            GH *hb = o.hist_cur.data() + (size_t)b * B;
            double *ha64 = o.shadow64 ? o.hist64_cur.data() + (size_t)a * B * 2 : nullptr;
            double *hb64 = o.shadow64 ? o.hist64_cur.data() + (size_t)b * B * 2 : nullptr;
            build_hist(o, idx.data() + ptr[a], ptr[a + 1] - ptr[a], ha, ha64);
            const GH *par = o.hist_prev.data() + (size_t)p * B;  // raw parent histogram (:526-540)
#pragma omp parallel for schedule(static) if (B > 100000)
            for (int i = 0; i < B; ++i) hb[i] = GH{par[i].g - ha[i].g, par[i].h - ha[i].h};
            if (o.shadow64) {
                const double *par64 = o.hist64_prev.data() + (size_t)p * B * 2;
                for (int i = 0; i < 2 * B; ++i) hb64[i] = par64[i] - ha64[i];
            }
            stash_debug(o, off + a, ha, ha64, 1);
            stash_debug(o, off + b, hb, hb64, 0);
            evaluate_node(o, off + 2 * p, o.hist_cur.data() + (size_t)(2 * p) * B, o.sp[2 * p]);
            evaluate_node(o, off + 2 * p + 1, o.hist_cur.data() + (size_t)(2 * p + 1) * B, o.sp[2 * p + 1]);
        }
    }
    if ((int)o.rows_built_level.size() <= level) o.rows_built_level.resize(level + 1, 0);
    o.rows_built_level[level] += o.rows_built_total - built_rows_before;
    o.cur_level = level;
}

// a7  HistTreeBuilder_single::update_tree, hist_tree_builder_single.cu:847-902
void update_tree(Oracle &o) {
    for (size_t i = 0; i < o.sp.size(); ++i) {
        const Split &s = o.sp[i];
        if (s.gain > o.rt_eps) {
            if (s.nid == -1) continue;
            Node &nd = o.nodes[s.nid];
            nd.gain = s.gain;
            Node &l = o.nodes[nd.lch];
            Node &r = o.nodes[nd.rch];
            l.is_valid = true;
            r.is_valid = true;
            nd.split_fid = s.fid;
            nd.split_value = s.fval;
            nd.split_bid = (unsigned char)s.bid;
            l.sum = s.lch_sum;
            if (!s.default_right) {
                l.sum = GH{l.sum.g + s.missing.g, l.sum.h + s.missing.h};
                nd.default_right = false;
            } else {
                nd.default_right = true;
            }
            r.sum = GH{nd.sum.g - l.sum.g, nd.sum.h - l.sum.h};
            l.base_weight = calc_weight(l.sum, o.lambda);
            r.base_weight = calc_weight(r.sum, o.lambda);
        } else {
            if (s.nid == -1) continue;
            Node &nd = o.nodes[s.nid];
            nd.is_leaf = true;
            o.nodes[nd.lch].is_valid = false;
            o.nodes[nd.rch].is_valid = false;
        }
    }
}

// a8  HistTreeBuilder_single::update_ins2node_id, hist_tree_builder_single.cu:908-1020. The
// reference's bounded binary search (:941-966) finds the row's stored bin that lies in the split
// feature's bin range; rows must have ascending column indices.
int update_ins2node(Oracle &o) {
    int has_split = 0;
#pragma omp parallel for reduction(| : has_split)
    for (int i = 0; i < o.n; ++i) {
        int x = o.nid[i];
        const Node &nd = o.nodes[x];
        int f = nd.split_fid;
        if (!nd.is_leaf && nd.is_valid && f >= 0 && f < o.F) {
            has_split |= 1;
            int cb = o.cut_row_ptr[f], ce = o.cut_row_ptr[f + 1];
            int split_bid = (int)nd.split_bid + cb;
            long lo = o.row_ptr[i], hi = o.row_ptr[i + 1];
            int bid = -1;
            long prev = -1;
            while (lo != hi) {
                long mid = lo + (hi - lo) / 2;
                if (mid == prev) break;
                prev = mid;
                int t = o.bin_id[mid];
                if (t >= cb && t < ce) {
                    bid = t;
                    break;
                } else if (t < cb)
                    lo = mid;
                else
                    hi = mid;
            }
            bool to_left = true;
            if ((bid == -1 && nd.default_right) || (bid >= split_bid && bid >= 0)) to_left = false;
            o.nid[i] = to_left ? nd.lch : nd.rch;
        }
    }
    return has_split;
}

// a9  Tree::prune_self, src/thundergbm/tree.cu:85-128
int try_prune_leaf(std::vector<Node> &nodes, int x, int np, float gamma, std::vector<int> &cnt) {
    int p = nodes[x].parent;
    if (p == -1) return np;
    Node &pn = nodes[p];
    Node &l = nodes[pn.lch];
    Node &r = nodes[pn.rch];
    cnt[p]++;
    if (cnt[p] >= 2 && pn.gain < gamma) {
        l.is_pruned = true;
        r.is_pruned = true;
        pn.is_leaf = true;
        return try_prune_leaf(nodes, p, np + 2, gamma, cnt);
    }
    return np;
}

int prune(std::vector<Node> &nodes, float gamma) {
    std::vector<int> cnt(nodes.size(), 0);
    int np = 0;
    for (size_t i = 0; i < nodes.size(); ++i)
        if (nodes[i].is_leaf && nodes[i].is_valid) np = try_prune_leaf(nodes, (int)i, np, gamma, cnt);
    int id = 0;
    for (size_t i = 0; i < nodes.size(); ++i)
        if (nodes[i].is_valid && !nodes[i].is_pruned) nodes[i].final_id = id++;
    return np;
}

// a10  TreeBuilder::predict_in_training, src/thundergbm/builder/tree_builder.cu:62-74
void predict_in_training(Oracle &o, int k) {
    float *yp = o.y_pred.data() + (long)k * o.n;
#pragma omp parallel for
    for (int i = 0; i < o.n; ++i) {
        int x = o.nid[i];
        while (x != -1 && o.nodes[x].is_pruned) x = o.nodes[x].parent;
        yp[i] += o.lr * o.nodes[x].base_weight;
    }
}

// ---------------------------------------------------------------------------------------------
// Ranking objectives. NDCG::discounted_gain, include/thundergbm/metric/ranking_metric.h:43-45.
inline float discounted_gain(int label, int rank) { return ((1 << label) - 1) / log2f(rank + 1 + 1); }

// NDCG::get_IDCG, src/thundergbm/metric/rank_metric.cpp:106-123
std::vector<float> get_idcg(const std::vector<int> &gptr, const float *y) {
    const int n_group = (int)gptr.size() - 1;
    std::vector<float> idcg(n_group, 0.f);
    for (int k = 0; k < n_group; ++k) {
        std::vector<float> sorted_label(y + gptr[k], y + gptr[k + 1]);
        std::sort(sorted_label.begin(), sorted_label.end(), std::greater<float>());
        for (size_t i = 0; i < sorted_label.size(); ++i) idcg[k] += discounted_gain((int)sorted_label[i], (int)i);
    }
    return idcg;
}

// RankListMetric::configure_gptr, rank_metric.cpp:39-44
std::vector<int> make_gptr(const std::vector<int> &group) {
    std::vector<int> gptr(group.size() + 1, 0);
    for (size_t i = 1; i < gptr.size(); ++i) gptr[i] = gptr[i - 1] + group[i - 1];
    return gptr;
}

// The partner draw that stands in for std::uniform_int_distribution over std::mt19937(std::rand()): a pure
// function of the round's seed and the drawing row's position in the dataset-wide (group, label order) list.
inline unsigned rank_draw(unsigned seed, unsigned pos, unsigned range) {
    unsigned long long x = ((unsigned long long)seed << 32) | pos;
    x += 0x9E3779B97F4A7C15ull;
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
    x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
    x ^= x >> 31;
    return (unsigned)(((x >> 32) * (unsigned long long)range) >> 32);
}

// LambdaRank::get_gradient, src/thundergbm/objective/ranking_obj.cpp:20-96, with get_delta_z of LambdaRank
// (ranking_obj.h:32) or LambdaRankNDCG (ranking_obj.cpp:105-113). The sums per row are kept in double and
// rounded once. order_out (optional): row at every position of the (label, score) order; pair_out (optional):
// per position the partner's position or -1.
void rank_gradient(bool ndcg, int n, const float *y, const float *score0, const std::vector<int> &group, unsigned seed,
                   GH *gh, int *order_out, int *pair_out) {
    const std::vector<int> gptr = make_gptr(group);
    std::vector<float> idcg;
    if (ndcg) idcg = get_idcg(gptr, y);
    std::vector<double> acc(2 * (size_t)n, 0.0);
    if (pair_out)
        for (int i = 0; i < n; ++i) pair_out[i] = -1;
    const int n_group = (int)group.size();
    for (int k = 0; k < n_group; ++k) {
        const int group_start = gptr[k];
        const int len = gptr[k + 1] - group_start;
        const float *score = score0 + group_start;
        const float *label_data = y + group_start;
        std::vector<int> idx(len);
        for (int i = 0; i < len; ++i) idx[i] = i;
        std::stable_sort(idx.begin(), idx.end(), [=](int a, int b) { return score[a] > score[b]; });
        std::vector<std::pair<float, int>> label_idx(len);
        for (int i = 0; i < len; ++i) {
            label_idx[i].first = label_data[idx[i]];
            label_idx[i].second = idx[i];
        }
        std::stable_sort(label_idx.begin(), label_idx.end(),
                         [](const std::pair<float, int> &a, const std::pair<float, int> &b) { return a.first > b.first; });
        if (order_out)
            for (int i = 0; i < len; ++i) order_out[group_start + i] = group_start + label_idx[i].second;
        for (int i = 0; i < len; ++i) {
            int j = i + 1;
            while (j < len && label_idx[i].first == label_idx[j].first) j++;
            const int nleft = i;
            const int nright = len - j;
            if (nleft + nright != 0) {
                for (int l = i; l < j; ++l) {
                    const int m = (int)rank_draw(seed, (unsigned)(group_start + l), (unsigned)(nleft + nright));
                    int high = 0, low = 0;
                    if (m < nleft) {
                        high = m;
                        low = l;
                    } else {
                        high = l;
                        low = m + j - i;
                    }
                    if (pair_out) pair_out[group_start + l] = group_start + (m < nleft ? high : low);
                    const float high_label = label_idx[high].first;
                    const float low_label = label_idx[low].first;
                    const int high_idx = label_idx[high].second;
                    const int low_idx = label_idx[low].second;
                    float delta_z = 1;
                    if (ndcg) {
                        if (idcg[k] == 0) {
                            delta_z = 0;
                        } else {
                            const float dgI1 = discounted_gain((int)high_label, high);
                            const float dgJ1 = discounted_gain((int)low_label, low);
                            const float dgI2 = discounted_gain((int)high_label, low);
                            const float dgJ2 = discounted_gain((int)low_label, high);
                            delta_z = (dgI1 + dgJ1 - dgI2 - dgJ2) / idcg[k];
                        }
                    }
                    const float abs_delta_z = fabsf(delta_z);
                    const float rhoIJ = 1 / (1 + expf((score[high_idx] - score[low_idx])));
                    const float lambda = -abs_delta_z * rhoIJ;
                    const float hessian = 2 * fmaxf(abs_delta_z * rhoIJ * (1 - rhoIJ), 1e-16f);
                    acc[2 * (size_t)(group_start + high_idx)] += lambda;
                    acc[2 * (size_t)(group_start + high_idx) + 1] += hessian;
                    acc[2 * (size_t)(group_start + low_idx)] -= lambda;
                    acc[2 * (size_t)(group_start + low_idx) + 1] += hessian;
                }
            }
            i = j;  // and the loop header adds one more: the first position of the next run is stepped over
        }
    }
    for (int i = 0; i < n; ++i) gh[i] = GH{(float)acc[2 * (size_t)i], (float)acc[2 * (size_t)i + 1]};
}

// RankListMetric::get_score with MAP::eval_query_group / NDCG::eval_query_group, rank_metric.cpp:9-104
// (topn = INT_MAX). Ties between equal scores keep row order.
float rank_metric(bool ndcg, int n, const float *y, const float *yp, const std::vector<int> &group) {
    const std::vector<int> gptr = make_gptr(group);
    std::vector<float> idcg;
    if (ndcg) idcg = get_idcg(gptr, y);
    const int n_group = (int)group.size();
    float sum_score = 0;
    for (int k = 0; k < n_group; ++k) {
        const int len = gptr[k + 1] - gptr[k];
        const float *label = y + gptr[k];
        const float *score = yp + gptr[k];
        std::vector<int> idx(len);
        for (int i = 0; i < len; ++i) idx[i] = i;
        std::stable_sort(idx.begin(), idx.end(), [=](int a, int b) { return score[a] > score[b]; });
        if (ndcg) {
            if (idcg[k] == 0) {
                sum_score += 1;
                continue;
            }
            float dcg = 0;
            for (int i = 0; i < len; ++i) dcg += discounted_gain((int)label[idx[i]], i);
            sum_score += dcg / idcg[k];
        } else {
            int nhits = 0;
            double sum_ap = 0;
            for (int i = 0; i < len; ++i) {
                if (label[idx[i]] != 0) {
                    nhits++;
                    sum_ap += (double)nhits / (i + 1);
                }
            }
            sum_score += nhits != 0 ? (float)(sum_ap / nhits) : 1.f;
        }
    }
    (void)n;
    return sum_score / n_group;
}

// RowSampler::do_bagging, src/thundergbm/row_sampler.cu:9-38. The reference draws with thrust (a dependency
// from the CUDA toolkit, not part of its checkout): thrust::default_random_engine is minstd_rand, the same
// generator as std::minstd_rand (x <- 48271 x mod 2^31 - 1); thrust::uniform_int_distribution<int>(a, b) maps
// one engine output u through uniform_real_distribution<double>(a, b + 1):
// (u - min) / (1 + (max - min)) * ((b + 1) - a) + a, truncated
// (thrust/random/detail/uniform_int_distribution.inl, uniform_real_distribution.inl).
// Entry i takes the output that follows discard(i), i.e. output i + 1 of one engine seeded once: the draws
// of all entries are the engine's outputs in order.
void bagging_draws(int seed, int N, int count, int *out) {
    std::minstd_rand rng((unsigned)seed);
    const double a = 0.0, b = (double)(N - 1) + 1.0;
    for (int i = 0; i < count; ++i) {
        double result = (double)(rng() - std::minstd_rand::min());
        result /= 1.0 + (double)(std::minstd_rand::max() - std::minstd_rand::min());
        out[i] = (int)(result * (b - a) + a);
    }
}

void do_bagging(std::vector<GH> &gh, int seed) {
    const int N = (int)gh.size();
    std::vector<int> idx(N), ins_count(N, 0);
    bagging_draws(seed, N, N, idx.data());
    for (int i = 0; i < N; ++i) ins_count[idx[i]] += 1;
    for (int i = 0; i < N; ++i) {
        gh[i].g = gh[i].g * ins_count[i];
        gh[i].h = gh[i].h * ins_count[i];
    }
}

bool is_rank(const std::string &obj) { return obj == "rank:pairwise" || obj == "rank:ndcg"; }

// a12  metrics: RMSE src/thundergbm/metric/pointwise_metric.cu:8-22, accuracy / error
// src/thundergbm/metric/multiclass_metric.cu:9-46
float metric(const std::string &obj, int n, int num_class, const float *y, const float *yp) {
    if (obj == "reg:linear" || obj == "reg:logistic") {
        float s = 0;
        for (int i = 0; i < n; ++i) {
            float e = yp[i] - y[i];
            s += e * e;
        }
        return sqrtf(s / n);
    }
    if (obj == "binary:logistic") {
        int t = 0;
        for (int i = 0; i < n; ++i) {
            int k = (1 / (1 + exp(-(double)yp[i])) > 0.5) ? 1 : 0;
            t += (k == y[i]);
        }
        float acc = t / (float)n;
        return 1 - acc;
    }
    int t = 0;
    for (int i = 0; i < n; ++i) {
        int mk = 0;
        float mp = yp[i];
        for (int k = 1; k < num_class; ++k)
            if (yp[(long)k * n + i] > mp) {
                mp = yp[(long)k * n + i];
                mk = k;
            }
        t += (mk == y[i]);
    }
    return t / (float)n;
}

// a3b  init_base_score, regression_obj.h:35-53 / :95-114, called from booster.h:66-73
void init_base_score(Oracle &o) {
    if (o.objective == "reg:linear" || o.objective == "reg:logistic" || o.objective == "binary:logistic") {
        gradient(o.objective, o.n, o.num_class, o.y.data(), o.y_pred.data(), o.gh.data());
        const GH bs = sum_gh(o.gh.data(), o.n);
        const float sg = bs.g, sh = bs.h;
        float w = (float)(-sg / fmax((double)sh, 1e-6));
        if (o.objective == "binary:logistic") {
            w = 1 / (1 + expf(-w));
            o.base_score = -logf(1.0f / w - 1.0f);
        } else {
            o.base_score = w;
        }
        std::fill(o.y_pred.begin(), o.y_pred.end(), o.base_score);
    } else {
        o.base_score = 0;  // objective_function.h:21-24: not implemented for softmax
    }
}

// a11  TreeBuilder::build_approximate, tree_builder.cu:147-194
void build_tree(Oracle &o, int k) {
    tree_init(o, k);
    for (int level = 0; level < o.depth; ++level) {
        find_split(o, level);
        update_tree(o);
        if (!update_ins2node(o)) break;
    }
    prune(o.nodes, o.gamma);
    predict_in_training(o, k);
}

// Booster::boost, include/thundergbm/booster.h:76-93
void boost_round(Oracle &o) {
    if (is_rank(o.objective))
        rank_gradient(o.objective == "rank:ndcg", o.n, o.y.data(), o.y_pred.data(), o.group, (unsigned)std::rand(),
                      o.gh.data(), nullptr, nullptr);
    else
        gradient(o.objective, o.n, o.num_class, o.y.data(), o.y_pred.data(), o.gh.data());
    if (o.bagging) do_bagging(o.gh, std::rand());  // booster.h:84
    sample_columns(o);  // first step of build_approximate, tree_builder.cu:150-152
    std::vector<Node> round_trees;
    for (int k = 0; k < o.tree_per_rounds; ++k) {
        build_tree(o, k);
        round_trees.insert(round_trees.end(), o.nodes.begin(), o.nodes.end());
    }
    o.model.push_back(round_trees);
    if (is_rank(o.objective))
        o.metric_log.push_back(rank_metric(o.objective == "rank:ndcg", o.n, o.y.data(), o.y_pred.data(), o.group));
    else
        o.metric_log.push_back(metric(o.objective, o.n, o.num_class, o.y.data(), o.y_pred.data()));
}

// a13  Predictor::predict_raw, src/thundergbm/predictor.cu:32-189. double accumulation when the
// dense shared-memory path would be taken (n_features * 128 * 4 <= 48 KB), float otherwise.
void predict_raw(int n, int F, const float *val, const int *row_ptr, const int *col, const Node *model, int n_iter,
                 int n_class_trees, int n_nodes, float lr, float base_score, float *out) {
    if (n_class_trees > 1) base_score = 0;
    bool dense_path = (size_t)F * 128 * sizeof(float) <= 48 * 1024;
#pragma omp parallel for
    for (int i = 0; i < n; ++i) {
        const int *ci = col + row_ptr[i];
        const float *cv = val + row_ptr[i];
        int len = row_ptr[i + 1] - row_ptr[i];
        for (int t = 0; t < n_class_trees; ++t) {
            double sd = base_score;
            float sf = base_score;
            for (int it = 0; it < n_iter; ++it) {
                const Node *nd = model + ((size_t)it * n_class_trees + t) * n_nodes;
                int cur = 0;
                while (!nd[cur].is_leaf) {
                    int f = nd[cur].split_fid;
                    const int *p = std::lower_bound(ci, ci + len, f);
                    // (the shared-memory path marks a missing value with +inf in the row's dense vector and tests
                    // `fval < INFINITY`, predictor.cu:96-118: a stored +inf or NaN takes the default direction there)
                    if (p != ci + len && *p == f && (!dense_path || cv[p - ci] < INFINITY)) {
                        float v = cv[p - ci];
                        cur = v < nd[cur].split_value ? nd[cur].lch : nd[cur].rch;
                    } else {
                        cur = nd[cur].default_right ? nd[cur].rch : nd[cur].lch;
                    }
                }
                sd += lr * nd[cur].base_weight;  // float product promoted to double (:126)
                sf += lr * nd[cur].base_weight;
            }
            out[(size_t)t * n + i] += dense_path ? (float)sd : sf;
        }
    }
}

// a14  predict_transform: regression_obj.h:27-32 / :76-92, multiclass_obj.cu:44-88.
// Returns the number of outputs.
long predict_transform(const std::string &obj, int n, int num_class, const float *label, float *y) {
    if (obj == "binary:logistic") {
        for (int i = 0; i < n; ++i) y[i] = label[y[i] > 0 ? 1 : 0];
        return n;
    }
    if (obj == "multi:softmax") {
        int nc = num_class == 2 ? 1 : num_class;
        for (int i = 0; i < n; ++i) {
            int mk = 0;
            float mp = y[i];
            for (int k = 1; k < nc; ++k)
                if (mp < y[(long)k * n + i]) {
                    mp = y[(long)k * n + i];
                    mk = k;
                }
            y[i] = label[mk];
        }
        return n;
    }
    if (obj == "multi:softprob") {
        for (int i = 0; i < n; ++i) {
            float mx = y[i];
            for (int k = 1; k < num_class; ++k) mx = fmaxf(mx, y[(long)k * n + i]);
            float sum = 0;
            for (int k = 0; k < num_class; ++k) {
                y[(long)k * n + i] = expf(y[(long)k * n + i] - mx);
                sum += y[(long)k * n + i];
            }
            for (int k = 0; k < num_class; ++k) y[(long)k * n + i] /= sum;
        }
        return (long)n * num_class;
    }
    if (obj == "reg:logistic") {
        for (int i = 0; i < n; ++i) y[i] = 1 / (1 + expf(-y[i]));
        return n;
    }
    return n;  // reg:linear identity
}

}  // namespace

// ---------------------------------------------------------------------------------------------
extern "C" {

// DataSet::load_from_sparse (dataset.cpp:20-63) + the class bookkeeping of TreeTrainer::train
// (trainer.cu:24-37).
void *orc_create(int n, const float *val, const int *row_ptr, const int *col, const float *y, int depth, int n_trees,
                 float min_child_weight, float lambda, float gamma, int max_num_bin, float learning_rate,
                 const char *objective, int num_class) {
    Oracle *o = new Oracle;
    o->n = n;
    o->nnz = row_ptr[n];
    o->val.assign(val, val + o->nnz);
    o->col.assign(col, col + o->nnz);
    o->row_ptr.assign(row_ptr, row_ptr + n + 1);
    o->y.assign(y, y + n);
    int mx = 0;
    for (long i = 0; i < o->nnz; ++i) mx = std::max(mx, col[i]);
    o->F = mx + 1;
    o->depth = depth;
    o->n_trees = n_trees;
    o->mcw = min_child_weight;
    o->lambda = lambda;
    o->gamma = gamma;
    o->max_num_bin = max_num_bin;
    o->lr = learning_rate;
    o->objective = objective;
    o->num_class = num_class;
    o->tree_per_rounds = 1;
    bool grouped = o->objective == "multi:softprob" || o->objective == "multi:softmax" ||
                   o->objective == "binary:logistic";
    if (grouped) {
        group_label(o->y, o->label);
        o->num_class = (int)o->label.size();
        if (o->num_class > 2) o->tree_per_rounds = o->num_class;
    } else if (o->objective.find("reg:") != std::string::npos) {
        o->num_class = 1;
    }
    return o;
}

void orc_destroy(void *h) { delete (Oracle *)h; }

void orc_set_debug(void *h, int keep_debug, int shadow64) {
    Oracle *o = (Oracle *)h;
    o->keep_debug = keep_debug;
    o->shadow64 = shadow64;
}

// HistTreeBuilder_single::init (:783-844) + Booster::init (booster.h:36-74)
void orc_prepare(void *h) {
    Oracle &o = *(Oracle *)h;
    o.n_bins = cut_points(o.F, o.nnz, o.val.data(), o.col.data(), o.max_num_bin, o.cut_val, o.cut_row_ptr, o.cut_fid);
    o.bin_id.resize(o.nnz);
#pragma omp parallel for
    for (long i = 0; i < o.nnz; ++i) o.bin_id[i] = bin_of(o.cut_val.data(), o.cut_row_ptr.data(), o.col[i], o.val[i]);
    long n_out = (long)o.num_class * o.n;
    if (o.num_class == 2) n_out = o.n;
    o.y_pred.assign(n_out, 0.f);
    o.gh.assign((long)o.num_class * o.n, GH{0, 0});
    o.nid.assign(o.n, 0);
    init_base_score(o);
}

void orc_set_bagging(void *h, int on) { ((Oracle *)h)->bagging = on != 0; }
// idx_i of RowSampler::do_bagging for i = 0..count-1
void orc_bagging_draws(int seed, int N, int count, int *out) { bagging_draws(seed, N, count, out); }
void orc_set_groups(void *h, const int *group, int num_group) {
    ((Oracle *)h)->group.assign(group, group + num_group);
}
// one LambdaRank gradient pass; order_out / pair_out may be null
void orc_rank_gradient(int ndcg, int n, const float *y, const float *score, const int *group, int num_group,
                       unsigned seed, float *gh, int *order_out, int *pair_out) {
    rank_gradient(ndcg != 0, n, y, score, std::vector<int>(group, group + num_group), seed, (GH *)gh, order_out,
                  pair_out);
}
float orc_rank_metric(int ndcg, int n, const float *y, const float *score, const int *group, int num_group) {
    return rank_metric(ndcg != 0, n, y, score, std::vector<int>(group, group + num_group));
}
void orc_set_column_sampling_rate(void *h, float rate) { ((Oracle *)h)->column_sampling_rate = rate; }
void orc_sample_columns(void *h) { sample_columns(*(Oracle *)h); }
void orc_boost(void *h, int rounds) {
    Oracle &o = *(Oracle *)h;
    for (int r = 0; r < rounds; ++r) boost_round(o);
}

// step-wise driving for lock-step tests
void orc_compute_gradient(void *h) {
    Oracle &o = *(Oracle *)h;
    if (is_rank(o.objective))
        rank_gradient(o.objective == "rank:ndcg", o.n, o.y.data(), o.y_pred.data(), o.group, (unsigned)std::rand(),
                      o.gh.data(), nullptr, nullptr);
    else
        gradient(o.objective, o.n, o.num_class, o.y.data(), o.y_pred.data(), o.gh.data());
    if (o.bagging) do_bagging(o.gh, std::rand());
}
void orc_tree_init(void *h, int k) { tree_init(*(Oracle *)h, k); }
void orc_find_split(void *h, int level) { find_split(*(Oracle *)h, level); }
void orc_update_tree(void *h) { update_tree(*(Oracle *)h); }
int orc_update_ins2node(void *h) { return update_ins2node(*(Oracle *)h); }
int orc_prune(void *h) {
    Oracle &o = *(Oracle *)h;
    return prune(o.nodes, o.gamma);
}
void orc_predict_in_training(void *h, int k) { predict_in_training(*(Oracle *)h, k); }
void orc_build_tree(void *h, int k) { build_tree(*(Oracle *)h, k); }
float orc_metric(void *h) {
    Oracle &o = *(Oracle *)h;
    if (is_rank(o.objective)) return rank_metric(o.objective == "rank:ndcg", o.n, o.y.data(), o.y_pred.data(), o.group);
    return metric(o.objective, o.n, o.num_class, o.y.data(), o.y_pred.data());
}

// getters / setters
int orc_n_features(void *h) { return ((Oracle *)h)->F; }
int orc_n_bins(void *h) { return ((Oracle *)h)->n_bins; }
int orc_num_class(void *h) { return ((Oracle *)h)->num_class; }
int orc_tree_per_rounds(void *h) { return ((Oracle *)h)->tree_per_rounds; }
int orc_n_labels(void *h) { return (int)((Oracle *)h)->label.size(); }
float orc_base_score(void *h) { return ((Oracle *)h)->base_score; }
int orc_n_nodes(void *h) { return (1 << (((Oracle *)h)->depth + 1)) - 1; }
long orc_rows_built(void *h) { return ((Oracle *)h)->rows_built_total; }
void orc_get_labels(void *h, float *out) {
    Oracle &o = *(Oracle *)h;
    std::copy(o.label.begin(), o.label.end(), out);
}
void orc_get_y(void *h, float *out) {
    Oracle &o = *(Oracle *)h;
    std::copy(o.y.begin(), o.y.end(), out);
}
void orc_get_cuts(void *h, float *cut_val, int *cut_row_ptr, int *cut_fid) {
    Oracle &o = *(Oracle *)h;
    std::copy(o.cut_val.begin(), o.cut_val.end(), cut_val);
    std::copy(o.cut_row_ptr.begin(), o.cut_row_ptr.end(), cut_row_ptr);
    std::copy(o.cut_fid.begin(), o.cut_fid.end(), cut_fid);
}
void orc_get_bin_ids(void *h, int *out) {
    Oracle &o = *(Oracle *)h;
    std::copy(o.bin_id.begin(), o.bin_id.end(), out);
}
long orc_y_pred_size(void *h) { return (long)((Oracle *)h)->y_pred.size(); }
void orc_get_y_pred(void *h, float *out) {
    Oracle &o = *(Oracle *)h;
    std::copy(o.y_pred.begin(), o.y_pred.end(), out);
}
void orc_set_y_pred(void *h, const float *in) {
    Oracle &o = *(Oracle *)h;
    std::copy(in, in + o.y_pred.size(), o.y_pred.begin());
}
void orc_get_gh(void *h, float *out) {
    Oracle &o = *(Oracle *)h;
    std::memcpy(out, o.gh.data(), o.gh.size() * sizeof(GH));
}
void orc_set_gh(void *h, const float *in) {
    Oracle &o = *(Oracle *)h;
    std::memcpy(o.gh.data(), in, o.gh.size() * sizeof(GH));
}
void orc_get_nid(void *h, int *out) {
    Oracle &o = *(Oracle *)h;
    std::copy(o.nid.begin(), o.nid.end(), out);
}
void orc_set_nid(void *h, const int *in) {
    Oracle &o = *(Oracle *)h;
    std::copy(in, in + o.n, o.nid.begin());
}
void orc_get_nodes(void *h, void *out) {
    Oracle &o = *(Oracle *)h;
    std::memcpy(out, o.nodes.data(), o.nodes.size() * sizeof(Node));
}
void orc_set_nodes(void *h, const void *in) {
    Oracle &o = *(Oracle *)h;
    std::memcpy(o.nodes.data(), in, o.nodes.size() * sizeof(Node));
}
int orc_get_splits(void *h, void *out) {
    Oracle &o = *(Oracle *)h;
    std::memcpy(out, o.sp.data(), o.sp.size() * sizeof(Split));
    return (int)o.sp.size();
}
// raw histogram of node `node_in_level` of the level last passed to orc_find_split
void orc_get_level_hist(void *h, int node_in_level, float *out, double *out64) {
    Oracle &o = *(Oracle *)h;
    std::memcpy(out, o.hist_cur.data() + (size_t)node_in_level * o.n_bins, o.n_bins * sizeof(GH));
    if (out64 && o.shadow64)
        std::memcpy(out64, o.hist64_cur.data() + (size_t)node_in_level * o.n_bins * 2, o.n_bins * 2 * sizeof(double));
}
// debug views of the current tree (need orc_set_debug(keep_debug=1) before orc_tree_init)
void orc_get_tree_scores(void *h, float *out) {
    Oracle &o = *(Oracle *)h;
    std::copy(o.dbg_score.begin(), o.dbg_score.end(), out);
}
// probe: n_nodes global candidate indices (-1 = none), or nullptr to switch probing off; results are collected
// while the next tree is built
void orc_set_probes(void *h, const int *probe) {
    Oracle &o = *(Oracle *)h;
    const int n_nodes = (1 << (o.depth + 1)) - 1;
    if (probe == nullptr) {
        o.probe.clear();
        o.probe_out.clear();
        return;
    }
    o.probe.assign(probe, probe + n_nodes);
    o.probe_out.assign(n_nodes, ProbeResult{0.f, 0.f, 0.f, 0.f});
}
void orc_get_probes(void *h, ProbeResult *out) {
    Oracle &o = *(Oracle *)h;
    std::copy(o.probe_out.begin(), o.probe_out.end(), out);
}
void orc_get_tree_dir_gaps(void *h, float *out) {
    Oracle &o = *(Oracle *)h;
    std::copy(o.dbg_dir_gap.begin(), o.dbg_dir_gap.end(), out);
}
void orc_get_tree_hists(void *h, float *out, double *out64, int *built) {
    Oracle &o = *(Oracle *)h;
    std::memcpy(out, o.dbg_hist.data(), o.dbg_hist.size() * sizeof(GH));
    if (out64 && o.shadow64) std::copy(o.dbg_hist64.begin(), o.dbg_hist64.end(), out64);
    if (built) std::copy(o.dbg_built.begin(), o.dbg_built.end(), built);
}
int orc_model_size(void *h) { return (int)((Oracle *)h)->model.size(); }
void orc_get_model(void *h, void *out) {
    Oracle &o = *(Oracle *)h;
    char *p = (char *)out;
    for (auto &r : o.model) {
        std::memcpy(p, r.data(), r.size() * sizeof(Node));
        p += r.size() * sizeof(Node);
    }
}
int orc_get_metric_log(void *h, float *out) {
    Oracle &o = *(Oracle *)h;
    std::copy(o.metric_log.begin(), o.metric_log.end(), out);
    return (int)o.metric_log.size();
}
int orc_get_rows_built_level(void *h, long *out, int cap) {
    Oracle &o = *(Oracle *)h;
    int m = std::min<int>(cap, (int)o.rows_built_level.size());
    std::copy(o.rows_built_level.begin(), o.rows_built_level.begin() + m, out);
    return m;
}

// ---- stateless entry points ------------------------------------------------------------------
int orc_cut_points(int F, long nnz, const float *val, const int *col, int max_bin, float *cut_val, int *cut_row_ptr,
                   int *cut_fid) {
    std::vector<float> cv;
    std::vector<int> crp, cf;
    int nb = cut_points(F, nnz, val, col, max_bin, cv, crp, cf);
    std::copy(cv.begin(), cv.end(), cut_val);
    std::copy(crp.begin(), crp.end(), cut_row_ptr);
    std::copy(cf.begin(), cf.end(), cut_fid);
    return nb;
}
void orc_bin_ids(long nnz, const float *val, const int *col, const float *cut_val, const int *cut_row_ptr, int *out) {
#pragma omp parallel for
    for (long i = 0; i < nnz; ++i) out[i] = bin_of(cut_val, cut_row_ptr, col[i], val[i]);
}
void orc_gradient(const char *objective, int n, int num_class, const float *y, const float *yp, float *gh) {
    gradient(objective, n, num_class, y, yp, (GH *)gh);
}
float orc_metric_score(const char *objective, int n, int num_class, const float *y, const float *yp) {
    return metric(objective, n, num_class, y, yp);
}
int orc_prune_nodes(void *nodes, int n_nodes, float gamma) {
    std::vector<Node> v((Node *)nodes, (Node *)nodes + n_nodes);
    int np = prune(v, gamma);
    std::memcpy(nodes, v.data(), n_nodes * sizeof(Node));
    return np;
}
void orc_group_label(int n, float *y, float *label_out, int *n_label) {
    std::vector<float> yy(y, y + n), lab;
    group_label(yy, lab);
    std::copy(yy.begin(), yy.end(), y);
    std::copy(lab.begin(), lab.end(), label_out);
    *n_label = (int)lab.size();
}
void orc_predict_raw(int n, int F, const float *val, const int *row_ptr, const int *col, const void *model,
                     int n_iter, int n_class_trees, int n_nodes, float lr, float base_score, float *out) {
    predict_raw(n, F, val, row_ptr, col, (const Node *)model, n_iter, n_class_trees, n_nodes, lr, base_score, out);
}
long orc_predict_transform(const char *objective, int n, int num_class, const float *label, float *y) {
    return predict_transform(objective, n, num_class, label, y);
}
int orc_num_threads() {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
}
