// Host orchestration of a training session on one MI355X: Booster::init / Booster::boost /
// TreeBuilder::build_approximate of the reference (include/thundergbm/booster.h:36-93,
// src/thundergbm/builder/tree_builder.cu:147-194), restructured so that a whole tree is a
// stream-ordered chain of level-wide launches without host synchronisation.
#include "trainer.h"

#include <algorithm>
#include <thread>
#include <chrono>
#include <cmath>
#include <cstdlib>
#include <cstring>

namespace tgbm {

template <typename T>
T *Trainer::dalloc(size_t count) {
    void *p = nullptr;
    if (count == 0) count = 1;
    HIP_CHECK(hipMalloc(&p, count * sizeof(T)));
    allocs_.push_back(p);
    return static_cast<T *>(p);
}

template <typename T>
static T *upload(hipStream_t s, T *dst, const T *src, size_t count) {
    if (count) HIP_CHECK(hipMemcpyAsync(dst, src, count * sizeof(T), hipMemcpyHostToDevice, s));
    return dst;
}

// Host -> device copy of a large pageable array: chunks are copied by a few host threads into two pinned
// staging buffers and sent with asynchronous DMA, so the host copy of one chunk overlaps the transfer of
// the previous one (a plain hipMemcpy of pageable memory stages through one thread).
void upload_large(hipStream_t s, void *dst, const void *src, size_t bytes) {
    constexpr size_t kChunk = (size_t)32 << 20;
    if (bytes < 4 * kChunk) {
        if (bytes) HIP_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, s));
        return;
    }
    void *pin[2] = {nullptr, nullptr};
    hipEvent_t done[2];
    for (int b = 0; b < 2; ++b) {
        HIP_CHECK(hipHostMalloc(&pin[b], kChunk, hipHostMallocDefault));
        HIP_CHECK(hipEventCreateWithFlags(&done[b], hipEventDisableTiming));
    }
    const int n_thr = (int)std::min(8u, std::max(1u, std::thread::hardware_concurrency()));
    size_t off = 0;
    for (int i = 0; off < bytes; ++i, off += kChunk) {
        const int b = i & 1;
        const size_t len = std::min(kChunk, bytes - off);
        if (i >= 2) HIP_CHECK(hipEventSynchronize(done[b]));  // the DMA that last read this buffer
        std::vector<std::thread> pool;
        auto part = [&](int t) {
            const size_t pb = len * t / n_thr, pe = len * (t + 1) / n_thr;
            std::memcpy(static_cast<char *>(pin[b]) + pb, static_cast<const char *>(src) + off + pb, pe - pb);
        };
        for (int t = 1; t < n_thr; ++t) pool.emplace_back(part, t);
        part(0);
        for (auto &th : pool) th.join();
        HIP_CHECK(hipMemcpyAsync(static_cast<char *>(dst) + off, pin[b], len, hipMemcpyHostToDevice, s));
        HIP_CHECK(hipEventRecord(done[b], s));
    }
    HIP_CHECK(hipStreamSynchronize(s));
    for (int b = 0; b < 2; ++b) {
        HIP_CHECK(hipEventDestroy(done[b]));
        HIP_CHECK(hipHostFree(pin[b]));
    }
}

Trainer::Trainer(const DataSet &ds, GBMParam &param) {
    int n_dev = 0;
    hipError_t e = hipGetDeviceCount(&n_dev);
    TGBM_CHECK(e == hipSuccess && n_dev >= 1, "no HIP device available: this library has no CPU path");
    HIP_CHECK(hipStreamCreate(&stream_));
    n_ = (int)ds.n_instances();
    F_ = (int)ds.n_features();
    nnz_ = ds.nnz;
    TGBM_CHECK(n_ > 0, "empty dataset");
    TGBM_CHECK(param.depth >= 1 && param.depth <= 14, "depth %d out of the supported range 1..14", param.depth);
    TGBM_CHECK(param.max_num_bin >= 2 && param.max_num_bin <= 65535,
               "max_num_bin %d out of the supported range 2..65535", param.max_num_bin);
    TGBM_CHECK(objective_supported(param.objective), "undefined objective %s", param.objective.c_str());
    TGBM_CHECK(param.column_sampling_rate > 0.f, "column_sampling_rate must be positive");
    // class bookkeeping of TreeTrainer::train (src/thundergbm/trainer.cu:24-37)
    if (param.objective.find("multi:") != std::string::npos || param.objective.find("binary:") != std::string::npos) {
        int nc = (int)ds.label.size();
        if (param.num_class != nc) {
            log_info("updating number of classes from %d to %d", param.num_class, nc);
            param.num_class = nc;
        }
        if (param.num_class > 2) param.tree_per_rounds = param.num_class;
    } else if (param.objective.find("reg:") != std::string::npos) {
        param.num_class = 1;
    }
    if (objective_needs_groups(param.objective)) {
        // LambdaRank / LambdaRankNDCG with their default metrics (ranking_obj.cpp:98,115); one score per row
        objective_ = OBJ_RANK;
        metric_kind_ = param.objective == "rank:ndcg" ? RANK_METRIC_NDCG : RANK_METRIC_MAP;
        if (param.num_class != 1) {
            log_info("ranking objectives train one score per instance: num_class %d -> 1", param.num_class);
            param.num_class = 1;
        }
    } else if (param.objective == "reg:linear") {
        objective_ = OBJ_SQUARE;
        metric_kind_ = 0;
    } else if (param.objective == "reg:logistic") {
        objective_ = OBJ_LOGISTIC;
        metric_kind_ = 0;
    } else if (param.objective == "binary:logistic") {
        objective_ = OBJ_LOGISTIC;
        metric_kind_ = 1;
        TGBM_CHECK(ds.label.size() == 2, "binary:logistic needs exactly two distinct labels, got %zu",
                   ds.label.size());
    } else {
        objective_ = OBJ_SOFTMAX;
        metric_kind_ = 2;
        // the reference aborts here as well (tree_builder.cu:87-90 vs multiclass_obj.cu:8)
        TGBM_CHECK(param.num_class != 2, "multi:softmax/softprob with two classes is not supported; use binary:logistic");
    }
    param_ = param;

    // ---- upload CSR, cut points, bin matrix --------------------------------------------------
    float *d_val = nullptr;
    int *d_col = nullptr, *d_row_ptr = nullptr;
    HIP_CHECK(hipMalloc(&d_val, sizeof(float) * (size_t)std::max(nnz_, 1l)));
    HIP_CHECK(hipMalloc(&d_col, sizeof(int) * (size_t)std::max(nnz_, 1l)));
    HIP_CHECK(hipMalloc(&d_row_ptr, sizeof(int) * (size_t)(n_ + 1)));
    auto t_up = std::chrono::steady_clock::now();
    upload_large(stream_, d_val, ds.val, sizeof(float) * (size_t)nnz_);
    upload_large(stream_, d_col, ds.col_idx, sizeof(int) * (size_t)nnz_);
    upload(stream_, d_row_ptr, ds.row_ptr, (size_t)n_ + 1);
    HIP_CHECK(hipStreamSynchronize(stream_));
    log_debug("upload of %.2f GB: %.3f s", (double)nnz_ * 8e-9,
              std::chrono::duration<double>(std::chrono::steady_clock::now() - t_up).count());
    if (!ds.features_counted) {  // the number of features = largest column index + 1 (dataset.cpp:40-46)
        F_ = device_max_int(stream_, d_col, nnz_) + 1;
        log_info("#instances = %d, #features = %d", n_, F_);
    }
    log_info("Fast getting cut points...");
    auto t_cut = std::chrono::steady_clock::now();
    cuts_ = build_cut_points(stream_, F_, nnz_, d_val, d_col, param_.max_num_bin);
    log_debug("cut points: %.3f s", std::chrono::duration<double>(std::chrono::steady_clock::now() - t_cut).count());
    auto t_bin = std::chrono::steady_clock::now();
    n_bins_ = cuts_.n_bins;
    allocs_.push_back(cuts_.cut_row_ptr);
    if (cuts_.cut_val) allocs_.push_back(cuts_.cut_val);
    if (cuts_.cut_fid) allocs_.push_back(cuts_.cut_fid);
    log_info("TOTAL CP:%d", n_bins_);
    log_info("NNZ: %ld", nnz_);
    TGBM_CHECK(n_bins_ > 0, "the dataset has no stored feature value");
    h_cut_row_ptr_.resize(F_ + 1);
    HIP_CHECK(hipMemcpyAsync(h_cut_row_ptr_.data(), cuts_.cut_row_ptr, sizeof(int) * (size_t)(F_ + 1),
                             hipMemcpyDeviceToHost, stream_));
    HIP_CHECK(hipStreamSynchronize(stream_));

    // Layout choice. Dense: column-blocked uint8 matrix (needs max_num_bin <= 255 and room for
    // n x F bytes twice). Sparse: CSR rows of global bin ids, for wide data whose rows store few values.
    const double density = (double)nnz_ / ((double)n_ * (double)F_);
    size_t free_b = 0, total_b = 0;
    HIP_CHECK(hipMemGetInfo(&free_b, &total_b));
    const char *force = std::getenv("TGBM_LAYOUT");  // "dense" / "sparse" override the heuristic (tests)
    sparse_ = (F_ > 4096 && density < 0.05) || (size_t)n_ * F_ * 2 > free_b / 2 || n_ >= (1 << 29);
    if (force != nullptr && std::string(force) == "sparse") sparse_ = true;
    if (force != nullptr && std::string(force) == "dense") sparse_ = false;
    if (F_ >= 65536) {  // the dense kernels keep feature ids in 16 bits
        if (!sparse_) log_info("%d features: sparse layout whatever the density (%.4f)", F_, density);
        sparse_ = true;
    }
    // More than 255 cut points in a feature (max_num_bin above 255): the dense layout then keeps 16-bit bins in narrower
    // feature blocks (their LDS histograms hold as many bins as the byte layout's), as long as one feature's bins fit
    // the LDS; the CSR layout's global bin ids have no limit at all. Either way the split search runs one workgroup
    // per (feature, node) and the split bin travels in a side array (TreeNode::split_bid is a byte).
    int max_feature_bins = 0;
    for (int f = 0; f < F_; ++f) max_feature_bins = std::max(max_feature_bins, h_cut_row_ptr_[f + 1] - h_cut_row_ptr_[f]);
    const char *wide_env = std::getenv("TGBM_WIDE_EVAL");  // "1": that split search for any data (tests)
    const char *bytes_env = std::getenv("TGBM_DENSE_BIN_BYTES");  // "2": 16-bit bins whatever the bin counts (tests)
    wide_bins_ = max_feature_bins > 255;
    int bin_bytes = (wide_bins_ || (bytes_env != nullptr && std::string(bytes_env) == "2")) ? 2 : 1;
    if (bin_bytes == 2 && (2 * max_feature_bins > kDense16MaxBlockBins || (size_t)n_ * F_ * 4 > free_b / 2))
        sparse_ = true;  // two features' bins of a block must fit the LDS, matrix and column copy the memory
    if (sparse_) bin_bytes = 1;
    log_info("layout: %s (density %.4f)",
             sparse_ ? "sparse CSR bin ids" : (bin_bytes == 2 ? "dense column-blocked uint16" : "dense column-blocked uint8"),
             density);
    wide_eval_ = wide_bins_ || (wide_env != nullptr && std::string(wide_env) == "1");
    if (sparse_) {
        // TGBM_SPARSE_PASS=0 keeps the row-list kernels with per-node histograms in HBM (tests compare the two)
        const char *pe = std::getenv("TGBM_SPARSE_PASS");
        sparse_pass_ = param_.depth <= 11 && nnz_ > 0 && nnz_ < (1l << 31) && !(pe != nullptr && std::string(pe) == "0") &&
                       !wide_bins_;
        wide_eval_ = wide_bins_ || (!sparse_pass_ && wide_env != nullptr && std::string(wide_env) == "1");
        if (!sparse_pass_) {
            // the per-node path keeps a histogram of all cut points per node in HBM (the reference's structure,
            // hist_tree_builder_single.cu:811-832) and costs about three times the level pass per tree
            const char *why = param_.depth > 11 ? "depth above 11 (the level pass keeps 12-bit node ids)"
                              : wide_bins_      ? "features with more than 255 bins"
                              : nnz_ >= (1l << 31) ? "2^31 stored values or more"
                                                  : "switched off";
            log_info("sparse layout: per-node histograms instead of the level pass: %s", why);
        }
        if (wide_bins_)
            log_info("features with up to %d bins: CSR layout, split search per (feature, node)", max_feature_bins);
        int *d_bin = dalloc<int>((size_t)std::max(nnz_, 1l));
        // Head of the histogram: the most frequent features whose bins fit the LDS slots. Worth it when
        // they carry a real share of the stored values (skewed, e.g. Zipf-distributed, feature usage).
        std::vector<int> feat_slot(F_, -1), head_bin;
        {
            std::vector<int> order(F_);
            for (int f = 0; f < F_; ++f) order[f] = f;
            std::stable_sort(order.begin(), order.end(),
                             [&](int a, int b) { return cuts_.feature_nnz[a] > cuts_.feature_nnz[b]; });
            long head_nnz = 0;
            for (int f : order) {
                const int k = h_cut_row_ptr_[f + 1] - h_cut_row_ptr_[f];
                if (k == 0 || cuts_.feature_nnz[f] == 0) break;
                if ((int)head_bin.size() + k > kCsrHeadBins) continue;
                feat_slot[f] = (int)head_bin.size();
                for (int j = 0; j < k; ++j) head_bin.push_back(h_cut_row_ptr_[f] + j);
                head_nnz += cuts_.feature_nnz[f];
            }
            const char *he = std::getenv("TGBM_CSR_HEAD");  // "0" disables the head (tests of both kernels)
            if (head_nnz * 10 < nnz_ || (he != nullptr && std::string(he) == "0") || sparse_pass_) head_bin.clear();
            log_info("sparse histogram head: %zu bins in LDS carry %.1f%% of the stored values", head_bin.size(),
                     nnz_ > 0 ? 100.0 * (double)head_nnz / (double)nnz_ : 0.0);
        }
        if (!head_bin.empty()) {
            int *d_slot = nullptr;
            HIP_CHECK(hipMalloc(&d_slot, sizeof(int) * (size_t)F_));
            upload(stream_, d_slot, feat_slot.data(), (size_t)F_);
            int *d_word = dalloc<int>((size_t)std::max(nnz_, 1l));
            int *d_head = dalloc<int>(head_bin.size());
            upload(stream_, d_head, head_bin.data(), head_bin.size());
            launch_bin_csr(stream_, nnz_, d_col, d_val, cuts_.cut_val, cuts_.cut_row_ptr, d_bin, d_slot, d_word);
            HIP_CHECK(hipStreamSynchronize(stream_));
            HIP_CHECK(hipFree(d_slot));
            csr_.hist_word = d_word;
            csr_.head_bin = d_head;
            csr_.head_bins = (int)head_bin.size();
        } else {
            launch_bin_csr(stream_, nnz_, d_col, d_val, cuts_.cut_val, cuts_.cut_row_ptr, d_bin);
        }
        allocs_.push_back(d_row_ptr);  // kept for the whole session
        csr_.row_ptr = d_row_ptr;
        csr_.bin = d_bin;
        // bin-major copy for the root histogram (TGBM_CSC_ROOT=0: without, the root goes through the row-major
        // kernels like every other level; tests of both)
        const char *ce = std::getenv("TGBM_CSC_ROOT");
        if (nnz_ > 0 && (sparse_pass_ || !(ce != nullptr && std::string(ce) == "0"))) {
            PairSorter ps;
            ps.alloc(nnz_);
            // Sort key of every bin. The features that the level pass serves through (bin, node) tables need no bin
            // order: all their bins share one key, so the stable sort leaves their values in row order - the row ->
            // node map and the gradient pairs are then fetched at ascending, for frequent features nearly consecutive
            // addresses, and neighbouring lanes add to different table cells.
            int *d_sort_key = nullptr;
            if (sparse_pass_) {
                std::vector<int> sort_key((size_t)n_bins_);
                for (int f = 0; f < F_; ++f)
                    for (int b = h_cut_row_ptr_[f]; b < h_cut_row_ptr_[f + 1]; ++b)
                        sort_key[(size_t)b] = sparse_feature_in_tables(f) ? h_cut_row_ptr_[f] : b;
                HIP_CHECK(hipMalloc(&d_sort_key, sizeof(int) * (size_t)n_bins_));
                upload(stream_, d_sort_key, sort_key.data(), sort_key.size());
                HIP_CHECK(hipStreamSynchronize(stream_));
            }
            launch_csc_keys(stream_, n_, d_row_ptr, d_bin, d_sort_key, ps.keys[0], ps.vals[0]);
            int bits = 1;
            while (bits < 31 && (1l << bits) < (long)n_bins_) ++bits;
            const int cur = sort_pairs(stream_, ps, nnz_, bits);
            int *d_cbin = dalloc<int>((size_t)nnz_), *d_crow = dalloc<int>((size_t)nnz_);
            launch_csc_unpack(stream_, nnz_, ps.keys[cur], ps.vals[cur], d_cbin, d_crow);
            HIP_CHECK(hipStreamSynchronize(stream_));
            ps.release();
            if (d_sort_key != nullptr) HIP_CHECK(hipFree(d_sort_key));
            csr_.csc_bin = d_cbin;
            csr_.csc_row = d_crow;
            csr_.nnz = nnz_;
        }
        if (sparse_pass_) {
            // One byte per row (local bin id, 255 = no stored value) for the frequent features - the ones that win
            // most splits: the row -> node update then takes a row's side from one byte instead of searching the
            // row's bin ids. As many of the table features, most frequent first, as fit an eighth of the free memory.
            std::vector<int> order;
            for (int f = 0; f < F_; ++f)
                if (cuts_.feature_nnz[f] > 0 && cuts_.feature_nnz[f] > kSortedTile) order.push_back(f);
            std::stable_sort(order.begin(), order.end(),
                             [&](int a, int b) { return cuts_.feature_nnz[a] > cuts_.feature_nnz[b]; });
            HIP_CHECK(hipMemGetInfo(&free_b, &total_b));
            const size_t col_stride = ((size_t)n_ + 3) / 4 * 4;
            const char *ce2 = std::getenv("TGBM_SPARSE_COLS");  // "0": none (tests of the search path)
            size_t n_cols = std::min(order.size(), free_b / 8 / col_stride);
            if (ce2 != nullptr && std::string(ce2) == "0") n_cols = 0;
            if (n_cols > 0) {
                std::vector<int> col_of(F_, -1);
                for (size_t c = 0; c < n_cols; ++c) col_of[order[c]] = (int)c;
                int *d_col_of = dalloc<int>((size_t)F_);
                upload(stream_, d_col_of, col_of.data(), col_of.size());
                uint8_t *d_cols = dalloc<uint8_t>(n_cols * col_stride);
                launch_fill_u8(stream_, d_cols, (uint8_t)kMissingBin, n_cols * col_stride);
                launch_sparse_cols(stream_, nnz_, csr_.csc_bin, csr_.csc_row, cuts_.cut_fid, cuts_.cut_row_ptr, d_col_of,
                                   d_cols, col_stride);
                HIP_CHECK(hipStreamSynchronize(stream_));
                csr_.col_of_feature = d_col_of;
                csr_.colbin = d_cols;
                csr_.col_stride = col_stride;
                log_info("sparse level pass: %zu frequent features have a byte column (%.1f MB)", n_cols,
                         (double)(n_cols * col_stride) * 1e-6);
            }
        }
        bins_.W = 4;
        bins_.n_blocks = 1;
        HIP_CHECK(hipStreamSynchronize(stream_));
        HIP_CHECK(hipFree(d_val));
        HIP_CHECK(hipFree(d_col));
    } else {
        // dense column-blocked layout: blocks of W columns, each block n rows x W bins
        // Bundles: a run of consecutive features of which no row stores more than one (the columns of a one-hot
        // group) shares one column, as long as the run's bins fit a byte. No two features of [a, b) meet in a row
        // if and only if no row has a column of [a, b) directly followed by another one of it (columns ascend inside
        // a row), so the smallest successor of every column decides: one pass over the column indices.
        h_col_bin_begin_ = h_cut_row_ptr_;
        int P = F_;  // columns of the matrix
        bool rows_ascend = true;
        bool ascend_known = false;
        std::vector<int> h_feat_col;
        std::vector<uint8_t> h_feat_lo;
        const char *be = std::getenv("TGBM_BUNDLE");  // "0": one column per feature (tests, measurements)
        // (rows that store every feature leave nothing to bundle)
        if (bin_bytes == 1 && F_ > 1 && nnz_ < (long)n_ * F_ && !(be != nullptr && std::string(be) == "0")) {
            int *d_next = nullptr;
            HIP_CHECK(hipMalloc(&d_next, sizeof(int) * ((size_t)F_ + 1)));
            HIP_CHECK(hipMemsetAsync(d_next, 0x7f, sizeof(int) * (size_t)F_, stream_));  // 0x7f7f7f7f: above every column
            HIP_CHECK(hipMemsetAsync(d_next + F_, 0, sizeof(int), stream_));
            launch_min_next_col(stream_, n_, d_row_ptr, d_col, d_next, d_next + F_);
            std::vector<int> next((size_t)F_ + 1);
            HIP_CHECK(hipMemcpyAsync(next.data(), d_next, sizeof(int) * next.size(), hipMemcpyDeviceToHost, stream_));
            HIP_CHECK(hipStreamSynchronize(stream_));
            HIP_CHECK(hipFree(d_next));
            rows_ascend = next[F_] == 0;
            ascend_known = true;
            if (next[F_] == 0) {  // (rows whose columns do not ascend: the argument above does not hold)
                std::vector<int> col_of(F_), begin;
                std::vector<uint8_t> lo(F_);
                int p = 0;
                for (int a = 0; a < F_; ++p) {
                    auto nb = [&](int f) { return h_cut_row_ptr_[f + 1] - h_cut_row_ptr_[f]; };
                    int limit = next[a], total = nb(a), b = a + 1;
                    while (b < F_ && b < limit && total + nb(b) <= 255) {
                        total += nb(b);
                        limit = std::min(limit, next[b]);
                        ++b;
                    }
                    begin.push_back(h_cut_row_ptr_[a]);
                    for (int f = a; f < b; ++f) {
                        col_of[f] = p;
                        lo[f] = (uint8_t)(h_cut_row_ptr_[f] - h_cut_row_ptr_[a]);
                    }
                    a = b;
                }
                if (p < F_) {
                    begin.push_back(n_bins_);
                    h_col_bin_begin_ = begin;
                    h_feat_col = col_of;
                    h_feat_lo = lo;
                    P = p;
                    log_info("dense layout: %d features in %d columns (runs of features that never meet in a row share one)",
                             F_, P);
                }
            }
        }
        int W;
        auto block_bins = [&](int w) {  // bins of the largest block of w columns
            int most = 0;
            for (int c0 = 0; c0 < P; c0 += w)
                most = std::max(most, h_col_bin_begin_[std::min(P, c0 + w)] - h_col_bin_begin_[c0]);
            return most;
        };
        if (bin_bytes == 2) {
            // 16-bit bins: the widest block (a power of two, at most 32 features = 64-byte rows) whose histogram
            // leaves room for two workgroups per CU, else two features per block
            W = 32;
            while (W > 2 && (W / 2 >= P || block_bins(W) > kDense16BlockBins)) W /= 2;
            if (wide_bins_) log_info("features with up to %d bins: 16-bit bins, %d features per block", max_feature_bins, W);
        } else if (P <= 32) {
            W = 4;
            while (W < P) W *= 2;
        } else if (P <= 64 && n_bins_ <= 8192) {
            W = 64;
        } else {
            // Wide data. A 64-byte block row is one whole memory request of a gathered row (a 32-byte row shares it
            // with a neighbour that the node mostly does not hold), but 64 features of 255 bins fill the LDS of a CU
            // with one workgroup's histogram. Measured per tree, 32 against 64 features per block: 500 k x 2000
            // 2.26 / 2.01 ms, 1 M x 200 1.15 / 1.09, 500 k x 300 with 63 bins (two workgroups fit either way)
            // 0.53 / 0.48; but 2 M x 100 0.91 / 0.97, 200 k x 500 0.57 / 0.64, 100 k x 1000 0.57 / 0.77.
            W = 32;
            const int bins64 = block_bins(64);
            if (bins64 <= 8192 || (bins64 <= 16 * 1024 && P >= 128 && n_ >= 400000)) W = 64;
            if (const char *we = std::getenv("TGBM_DENSE_W")) {  // 32 / 64: override (measurements)
                const int w = atoi(we);
                if ((w == 32 || w == 64) && block_bins(w) <= kDense16MaxBlockBins) W = w;
            }
        }
        // (the histogram kernel addresses a block's rows, the gradient pairs and the row lists with unsigned 32-bit
        // byte offsets: a block stays below 4 GiB, the rows below 2^29)
        while (W * bin_bytes > 4 && (size_t)n_ * W * bin_bytes >= ((size_t)1 << 32)) W /= 2;
        TGBM_CHECK((size_t)n_ * W * bin_bytes < ((size_t)1 << 32) && n_ < (1 << 29),
                   "%d rows are more than the dense layout addresses; use TGBM_LAYOUT=sparse", n_);
        const int n_blocks = (P + W - 1) / W;
        bins_.W = W;
        bins_.n_blocks = n_blocks;
        bins_.bin_bytes = bin_bytes;
        bins_.n_cols = P;
        if (!h_feat_col.empty()) {
            int *d_fc = dalloc<int>((size_t)F_);
            uint8_t *d_fl = dalloc<uint8_t>(((size_t)F_ + 3) / 4 * 4);
            upload(stream_, d_fc, h_feat_col.data(), (size_t)F_);
            upload(stream_, d_fl, h_feat_lo.data(), (size_t)F_);
            HIP_CHECK(hipStreamSynchronize(stream_));  // (the host vectors go out of scope)
            bins_.feat_col = d_fc;
            bins_.feat_lo = d_fl;
            h_feat_col_ = h_feat_col;
        }
        const size_t mat_bytes = (size_t)n_ * W * n_blocks * bin_bytes;
        bins_.block_stride = (size_t)n_ * W * bin_bytes;
        TGBM_CHECK(mat_bytes + (size_t)n_ * P * bin_bytes < free_b / 2, "dense bin matrix of %zu bytes does not fit (free %zu)",
                   mat_bytes, free_b);
        d_binmat_ = dalloc<uint8_t>(mat_bytes);
        launch_fill_u8(stream_, d_binmat_, (uint8_t)kMissingBin, mat_bytes);  // (all-ones: the sentinel of both widths)
        const size_t col_stride = ((size_t)n_ + 3) / 4 * 4;
        uint8_t *d_colmat = dalloc<uint8_t>(col_stride * P * bin_bytes);
        launch_fill_u8(stream_, d_colmat, (uint8_t)kMissingBin, col_stride * P * bin_bytes);
        // (rows that store every feature cannot hold a column twice)
        if (!ascend_known && nnz_ != (long)n_ * F_) rows_ascend = device_rows_ascend(stream_, n_, d_row_ptr, d_col);
        if (!rows_ascend) log_info("rows with descending column indices: the dense bins are filled row by row");
        launch_bin_dense(stream_, n_, d_row_ptr, d_col, d_val, cuts_.cut_val, cuts_.cut_row_ptr, d_binmat_, W,
                         bins_.block_stride, d_colmat, col_stride, bin_bytes, P, bins_.feat_col, bins_.feat_lo, rows_ascend);
        bins_.col = d_colmat;
        bins_.col_stride = col_stride;
        bins_.data = d_binmat_;
        {
            // (TGBM_GH_WORD=0: the histogram kernels always gather the pairs from the gradient array; tests)
            const char *ge = std::getenv("TGBM_GH_WORD");
            const bool off = ge != nullptr && std::string(ge) == "0";
            const bool loss_ok = param.objective == "reg:linear" || param.objective == "binary:logistic";  // (labels 0 / 1)
            if (!off && loss_ok && param.tree_per_rounds == 1 && bin_bytes == 1 && n_blocks == 1 && W >= 16 && P <= W - 4) {
                gh_word_lane_ = W / 4 - 1;
                bins_.gh_lane = gh_word_lane_;
                d_gh_words_ = dalloc<unsigned>((size_t)n_);
                bins_.gh_words = d_gh_words_;
                log_info("gradient pairs ride in the spare bytes of the bin-matrix rows");
            }
        }
        HIP_CHECK(hipStreamSynchronize(stream_));
        HIP_CHECK(hipFree(d_val));
        HIP_CHECK(hipFree(d_col));
        HIP_CHECK(hipFree(d_row_ptr));
    }

    // ---- labels, predictions, gradients (Booster::init) --------------------------------------
    d_y_ = dalloc<float>(n_);
    upload(stream_, d_y_, ds.y.data(), (size_t)n_);
    log_debug("bin matrix: %.3f s", std::chrono::duration<double>(std::chrono::steady_clock::now() - t_bin).count());
    auto t_rest = std::chrono::steady_clock::now();
    n_yp_ = (long)param_.num_class * n_;
    if (param_.num_class == 2) n_yp_ = n_;
    d_yp_ = dalloc<float>((size_t)n_yp_);
    launch_fill_f32(stream_, d_yp_, 0.f, (size_t)n_yp_);
    d_gh_ = dalloc<GHPair>((size_t)param_.num_class * n_);
    launch_fill_f32(stream_, reinterpret_cast<float *>(d_gh_), 0.f, (size_t)param_.num_class * n_ * 2);
    alloc_tree_buffers();

    if (objective_ == OBJ_RANK) rank_.reset(new RankContext(stream_, ds.y, ds.group, param_.objective == "rank:ndcg"));

    // base score (regression_obj.h:35-53, :95-114; only for squared / logistic objectives)
    if (objective_ != OBJ_SOFTMAX && objective_ != OBJ_RANK) {
        launch_gradient(stream_, objective_, n_, param_.num_class, d_y_, d_yp_, d_gh_, nullptr, 0);
        launch_tree_init(stream_, tb_, d_gh_, param_.lambda);  // reuses the root-sum reduction
        TreeNode root;
        HIP_CHECK(hipMemcpyAsync(&root, tb_.nodes, sizeof(TreeNode), hipMemcpyDeviceToHost, stream_));
        HIP_CHECK(hipStreamSynchronize(stream_));
        float weight = (float)(-root.sum_gh_pair.g / std::fmax((double)root.sum_gh_pair.h, 1e-6));
        float base = weight;
        if (param_.objective == "binary:logistic") {
            weight = 1 / (1 + expf(-weight));
            base = -logf(1.0f / weight - 1.0f);
        }
        log_info("base_score %g", base);
        param_.base_score = base;
        launch_fill_f32(stream_, d_yp_, base, (size_t)n_yp_);
    } else {
        param_.base_score = 0;
    }
    param.base_score = param_.base_score;
    HIP_CHECK(hipStreamSynchronize(stream_));
    log_debug("training buffers and base score: %.3f s",
              std::chrono::duration<double>(std::chrono::steady_clock::now() - t_rest).count());
}

void Trainer::alloc_tree_buffers() {
    TreeBuffers &tb = tb_;
    const int depth = param_.depth;
    tb.n = n_;
    tb.n_bins = n_bins_;
    tb.sparse = sparse_ ? 1 : 0;
    tb.F = F_;
    tb.depth = depth;
    tb.n_nodes = (1 << (depth + 1)) - 1;
    const int max_level_nodes = 1 << (depth - 1 > 0 ? depth - 1 : 0);
    const int max_pairs = std::max(1, max_level_nodes / 2);
    tb.max_level_nodes = max_level_nodes;
    tb.target_hitems = std::min(512, std::max(4, 512 / bins_.n_blocks));  // ~2 resident workgroups per CU
    tb.max_hitems = tb.target_hitems + max_pairs + 1;
    tb.max_pitems = n_ / kPartChunk + max_level_nodes + 1;
    tb.n_partial = sparse_ ? 1 : (size_t)tb.max_hitems * n_bins_;
    tb.n_end_bound = ((size_t)row_blocks(n_) + 1) * (((size_t)1 << depth) - 1);
    tb.n_grad_blocks = row_blocks(n_);
    // One set of buffers per class tree of a round when that fits comfortably: the trees of a round are
    // independent and are then built together (class = blockIdx.z of every launch).
    const int K = param_.tree_per_rounds;
    if (sparse_pass_) build_sparse_tasks();
    // The per-node paths keep the node histograms of two levels. The reference sizes its `last_hist` buffer against
    // the free memory and builds both siblings from rows beyond the depth that fits
    // (hist_tree_builder_single.cu:811-832, :544-570); same here: the arena holds `hist_nodes` node histograms per
    // buffer - all of the deepest level when that fits, else the largest power of two that does - and deeper levels
    // are served in batches of that many nodes (find_split_sets). TGBM_HIST_ARENA_NODES caps it (tests).
    size_t free_b = 0, total_b = 0;
    HIP_CHECK(hipMemGetInfo(&free_b, &total_b));
    int hist_nodes = max_level_nodes;
    const size_t fixed_bytes = sparse_pass_ ? 0 : (size_t)n_ * 13 + tb.n_end_bound * sizeof(int);
    auto arena_bytes = [&](int nodes) {  // two buffers + the work items' partial histograms (dense layout)
        const size_t items = sparse_ ? 0 : (size_t)tb.target_hitems + (nodes < max_level_nodes ? nodes : max_pairs) + 2;
        return ((size_t)2 * nodes + items) * (size_t)n_bins_ * sizeof(longlong2);
    };
    if (!sparse_pass_) {
        if (const char *ae = std::getenv("TGBM_HIST_ARENA_NODES")) hist_nodes = std::max(2, std::min(hist_nodes, atoi(ae)));
        const size_t budget = free_b - free_b / 8;
        while (hist_nodes > 2 && fixed_bytes + arena_bytes(hist_nodes) > budget) hist_nodes /= 2;
        int p2 = 1;
        while (p2 * 2 <= hist_nodes) p2 *= 2;
        hist_nodes = std::max(max_level_nodes >= 2 ? 2 : 1, p2);
        TGBM_CHECK(fixed_bytes + arena_bytes(hist_nodes) <= free_b - free_b / 16,
                   "the histograms of %d bins need %.1f GB for a %d-node arena, %.1f GB are free", n_bins_,
                   (double)arena_bytes(hist_nodes) * 1e-9, hist_nodes, (double)free_b * 1e-9);
        if (hist_nodes < max_level_nodes) {
            // first level that does not fit: still has its parents (batches of sibling pairs); below it single nodes
            int lc = 0;
            while ((1 << lc) <= hist_nodes) ++lc;
            hist_cap_level_ = lc;
            tb.singles_from = lc + 1;
            tb.max_hitems = tb.target_hitems + max_level_nodes + 1;  // every node of a level may add a partly filled item
            tb.n_partial = sparse_ ? 1 : ((size_t)tb.target_hitems + hist_nodes + 2) * n_bins_;
            log_info("histogram arena: %d node histograms per buffer (%.2f GB); levels from %d on are built in batches, "
                     "both siblings from rows below level %d", hist_nodes, (double)arena_bytes(hist_nodes) * 1e-9, lc, lc);
        }
    }
    tb.hist_nodes = hist_nodes;
    const size_t set_bytes =
        sparse_pass_ ? (size_t)n_ * 15 + (size_t)sp_.n_partial_slots * sp_.partial_stride * sizeof(longlong2) +
                           (size_t)max_level_nodes * sp_.n_cand_slots * sizeof(SplitCand) +
                           (size_t)sp_.n_sorted * 32 + (size_t)nnz_ * sizeof(GHPair)
                     : fixed_bytes + arena_bytes(hist_nodes);
    const char *be = std::getenv("TGBM_BATCH_CLASSES");  // "0": build the trees of a round one after the other
    n_sets_ = (K > 1 && set_bytes * K < free_b / 2 && !(be != nullptr && std::string(be) == "0")) ? K : 1;
    tb.n_sets = n_sets_;
    const size_t S = (size_t)n_sets_;
    tb.nodes = dalloc<TreeNode>(S * tb.n_nodes);
    tb.seg = dalloc<int2>(S * tb.n_nodes);
    tb.nid = dalloc<int>(S * n_);
    tb.ridx[0] = dalloc<int>(S * n_);
    tb.ridx[1] = dalloc<int>(S * n_);
    tb.goes_right = dalloc<uint8_t>(S * (size_t)tb.max_pitems * 256);
    if (!sparse_pass_) {
        tb.hist_q[0] = dalloc<longlong2>(S * (size_t)hist_nodes * n_bins_);
        tb.hist_q[1] = dalloc<longlong2>(S * (size_t)hist_nodes * n_bins_);
    } else {
        tb.nid16 = dalloc<unsigned short>(S * (((size_t)n_ + 2) / 2 * 2));
        tb.node_rows = dalloc<int>(S * tb.n_nodes);
        tb.row_move = dalloc<uint8_t>(S * (((size_t)n_ + 63) / 64 * 64));
    }
    tb.partial = dalloc<longlong2>(S * tb.n_partial);
    tb.quant = dalloc<QuantCtl>(S);
    tb.hitem_shift = dalloc<int2>(S * (size_t)tb.max_hitems);
    tb.root_total = dalloc<long long>(S * 512);
    // a feature that is stored in every row (checked on the bin matrix itself: a row with a repeated column index
    // would make the stored-value count lie): its bins add up to the root's sums
    tb.complete_feature = -1;
    if (!sparse_) {
        for (int f = 0; f < F_ && tb.complete_feature < 0; ++f) {
            int c = f;
            if (!h_feat_col_.empty()) {
                // (a feature that shares its column: the others must be empty, so that every byte of the column that
                // is not the missing sentinel is this feature's - the same choice as without bundles)
                c = h_feat_col_[f];
                bool alone = true;
                for (int g = f - 1; g >= 0 && h_feat_col_[g] == c; --g) alone = alone && cuts_.feature_nnz[g] == 0;
                for (int g = f + 1; g < F_ && h_feat_col_[g] == c; ++g) alone = alone && cuts_.feature_nnz[g] == 0;
                if (!alone) continue;
            }
            if (cuts_.feature_nnz[f] != (long)n_) continue;
            const long absent =
                bins_.bin_bytes == 1
                    ? device_count_bytes(stream_, bins_.col + (size_t)c * bins_.col_stride, (size_t)n_, (uint8_t)kMissingBin)
                    : device_count_u16(stream_, reinterpret_cast<const uint16_t *>(bins_.col) + (size_t)c * bins_.col_stride,
                                       (size_t)n_, (uint16_t)kMissingBin16);
            if (absent == 0) tb.complete_feature = f;
        }
    }
    tb.hpair_begin = dalloc<int>(S * ((size_t)max_level_nodes + 1));
    tb.leaf_value = dalloc<float>(S * tb.n_nodes);
    tb.end_bound = dalloc<int>(S * tb.n_end_bound);
    tb.hpair_built = dalloc<int>(S * max_level_nodes);
    tb.pitem_begin = dalloc<int>(S * 2 * ((size_t)max_level_nodes + 1));
    tb.pitem_nleft = dalloc<int>(S * ((size_t)tb.max_pitems + 1));
    tb.pitem_loff = dalloc<int>(S * ((size_t)tb.max_pitems + 1));
    tb.node_nleft = dalloc<int>(S * max_level_nodes);
    tb.ctl = dalloc<LevelCtl>(S * ((size_t)depth + 2));
    tb.sp = dalloc<SplitPoint>(S * max_level_nodes);
    tb.root_partial = dalloc<GradStats>(S * tb.n_grad_blocks);
    tb.cut_row_ptr = cuts_.cut_row_ptr;
    tb.cut_fid = cuts_.cut_fid;
    tb.cut_val = cuts_.cut_val;

    // split-finder packs: whole features, at most kEvalPackBins bins per wavefront
    std::vector<int> pack_begin;
    pack_begin.push_back(0);
    int cur = 0;
    for (int f = 0; f < F_; ++f) {
        int k = h_cut_row_ptr_[f + 1] - h_cut_row_ptr_[f];
        if (k == 0) continue;
        TGBM_CHECK(k <= kEvalPackBins || wide_eval_, "feature %d has %d cut points, more than %d", f, k, kEvalPackBins);
        if (cur + k > kEvalPackBins) {
            pack_begin.push_back(h_cut_row_ptr_[f]);
            cur = 0;
        }
        cur += k;
    }
    pack_begin.push_back(n_bins_);
    tb.n_packs = sparse_pass_ ? sp_.n_cand_slots : (int)pack_begin.size() - 1;  // candidates per node
    if (wide_eval_) {
        tb.n_packs = F_;  // one candidate per feature
        tb.split_bin = dalloc<int>(S * tb.n_nodes);
    }
    if (sparse_pass_) {
        tb.best_key = dalloc<unsigned long long>(S * (size_t)max_level_nodes);
        HIP_CHECK(hipMemsetAsync(tb.best_key, 0, sizeof(unsigned long long) * S * (size_t)max_level_nodes, stream_));
        if (sp_.n_sorted_tasks > 0) {
            // static order of the sorted pass, then per set the two level orders and the live counts
            int *row0 = dalloc<int>((size_t)sp_.n_sorted);
            unsigned *key0 = dalloc<unsigned>((size_t)sp_.n_sorted);
            unsigned short *start0 = dalloc<unsigned short>((size_t)sp_.n_sorted);
            launch_sorted_setup(stream_, tb, csr_, sp_, row0, key0, start0);
            sp_.sorted_row0 = row0;
            sp_.sorted_key0 = key0;
            sp_.sorted_start0 = start0;
            for (int b = 0; b < 2; ++b) {
                sp_.sorted_row[b] = dalloc<int>(S * (size_t)sp_.n_sorted);
                sp_.sorted_key[b] = dalloc<unsigned>(S * (size_t)sp_.n_sorted);
                sp_.sorted_gh[b] = dalloc<GHPair>(S * (size_t)sp_.n_sorted);
            }
            sp_.sorted_live = dalloc<int>(S * (size_t)kSortedLevels * sp_.n_sorted_tasks);
            HIP_CHECK(hipMemsetAsync(sp_.sorted_live, 0, sizeof(int) * S * (size_t)kSortedLevels * sp_.n_sorted_tasks,
                                     stream_));
        }
        sp_.partial = dalloc<longlong2>(S * (size_t)sp_.n_partial_slots * sp_.partial_stride);
        // per-value gradient pairs in the order of the bin-major copy, when they fit comfortably
        sp_.nnz = nnz_;
        HIP_CHECK(hipMemGetInfo(&free_b, &total_b));
        const char *ge = std::getenv("TGBM_SPARSE_GH_COPY");  // "0": gather the pairs per value instead (tests)
        if (S * (size_t)nnz_ * sizeof(GHPair) < free_b / 4 && !(ge != nullptr && std::string(ge) == "0"))
            sp_.csc_gh = dalloc<GHPair>(S * (size_t)nnz_);
    }
    int *d_pack = dalloc<int>(pack_begin.size());
    upload(stream_, d_pack, pack_begin.data(), pack_begin.size());
    tb.pack_begin = d_pack;
    std::vector<unsigned short> bin_meta((size_t)n_bins_);
    for (int f = 0; f < F_; ++f)
        for (int b = h_cut_row_ptr_[f]; b < h_cut_row_ptr_[f + 1]; ++b)
            bin_meta[(size_t)b] = (unsigned short)((h_cut_row_ptr_[f + 1] - 1 - b) | (b == h_cut_row_ptr_[f] ? 0x100 : 0));
    unsigned short *d_meta = dalloc<unsigned short>(bin_meta.size());
    upload(stream_, d_meta, bin_meta.data(), bin_meta.size());
    tb.bin_meta = d_meta;
    tb.cand = dalloc<SplitCand>(S * max_level_nodes * tb.n_packs);

    // dense block tables
    const int W = bins_.W, nb = bins_.n_blocks;
    std::vector<int> blk_begin(nb + 1), feat_off((size_t)nb * W, 0);
    int max_block_bins = 0;
    // (columns of the matrix: features, or bundles of features whose bins follow each other)
    const std::vector<int> &cbb = sparse_ ? h_cut_row_ptr_ : h_col_bin_begin_;
    const int n_cols = (int)cbb.size() - 1;
    for (int b = 0; b <= nb; ++b) blk_begin[b] = cbb[std::min(b * W, n_cols)];
    for (int b = 0; b < nb; ++b) {
        max_block_bins = std::max(max_block_bins, blk_begin[b + 1] - blk_begin[b]);
        for (int j = 0; j < W; ++j) {
            int c = b * W + j;
            feat_off[(size_t)b * W + j] = c < n_cols ? cbb[c] - blk_begin[b] : 0;
        }
    }
    TGBM_CHECK(sparse_ || (size_t)max_block_bins * 8 <= 160 * 1024, "feature block histogram exceeds the LDS");
    tb.max_block_bins = max_block_bins;
    int *d_blk = dalloc<int>(blk_begin.size());
    int *d_off = dalloc<int>(feat_off.size());
    upload(stream_, d_blk, blk_begin.data(), blk_begin.size());
    upload(stream_, d_off, feat_off.data(), feat_off.size());
    tb.blk_bin_begin = d_blk;
    tb.feat_lds_off = d_off;
    HIP_CHECK(hipStreamSynchronize(stream_));  // the host vectors above go out of scope

    model_cap_trees_ = std::max(1, param_.n_trees) * param_.tree_per_rounds;
    d_model_ = dalloc<TreeNode>((size_t)model_cap_trees_ * tb.n_nodes);
    d_metric_ = dalloc<float>((size_t)std::max(1, param_.n_trees));
    d_metric_scratch_ = dalloc<double>((size_t)row_blocks(n_));
    HIP_CHECK_LAUNCHES("set-up (cut points, bin matrix)");
}

Trainer::~Trainer() {
    if (stream_) (void)hipStreamSynchronize(stream_);
    for (auto &m : marks_) (void)hipEventDestroy(m.ev);
    reorder_sorter_.release();
    for (void *p : allocs_) (void)hipFree(p);
    if (stream_) (void)hipStreamDestroy(stream_);
}

void Trainer::sync() { HIP_CHECK(hipStreamSynchronize(stream_)); }

void Trainer::mark(int phase, int level) {
    if (!profiling_) return;
    PhaseMark m;
    HIP_CHECK(hipEventCreate(&m.ev));
    m.phase = phase;
    m.level = level;
    HIP_CHECK(hipEventRecord(m.ev, stream_));
    marks_.push_back(m);
}

// The first two steps of Booster::boost (include/thundergbm/booster.h:80-84): the objective's gradients, then
// bagging when it is switched on.
void Trainer::compute_gradient() {
    next_round_ready_ = false;
    gh_array_stale_ = false;  // (recomputed below)
    if (objective_ == OBJ_RANK) {
        // the round's partner draws hang off the process-wide rand(), which is what the reference seeds its
        // per-group generators from (ranking_obj.cpp:53): srand() makes a run repeatable
        rank_->gradient(d_yp_, d_gh_, (unsigned)std::rand(), rank_order_fresh_);
        rank_order_fresh_ = false;
    } else {
        launch_gradient(stream_, objective_, n_, param_.num_class, d_y_, d_yp_, d_gh_, nullptr, 0);
    }
    gh_words_fresh_ = gh_records_fresh_ = false;
    if (gh_word_lane_ >= 0 && !param_.bagging) {  // (bagging multiplies the pairs by draw counts)
        launch_gh_words(stream_, objective_, n_, d_y_, d_yp_, d_gh_words_);
        gh_words_fresh_ = true;
    }
    if (param_.bagging) {
        const size_t N = (size_t)param_.num_class * n_;  // the whole gradient array, as in the reference
        TGBM_CHECK(N < ((size_t)1 << 31), "bagging: %zu gradient pairs exceed the int index range", N);
        if (d_bag_count_ == nullptr) {
            d_bag_count_ = dalloc<int>(N);
            HIP_CHECK(hipMemsetAsync(d_bag_count_, 0, sizeof(int) * N, stream_));
        }
        // row_sampler.cu:15. The gradient array may be longer than the rows (binary:logistic: 2n entries, the
        // rows use the first n); only the row entries are subject to the permutation.
        launch_bagging(stream_, (int)N, (unsigned)std::rand(), d_bag_count_, d_gh_, d_perm_, n_);
    }
}

// Shard::column_sampling (src/thundergbm/builder/shard.cu:8-22), once per boosting round
// (builder/tree_builder.cu:150-152): the columns 0..F-1 are shuffled the way libstdc++'s
// std::random_shuffle does it (i = 1..F-1: swap with position rand() % (i + 1), process-wide rand() as
// in the reference) and the first max(1, int(F * rate)) of them are ignored by this round's split search.
void Trainer::sample_columns() {
    if (!(param_.column_sampling_rate < 1.f)) return;
    std::vector<int> idx(F_);
    for (int i = 0; i < F_; ++i) idx[i] = i;
    for (int i = 1; i < F_; ++i) {
        const int j = std::rand() % (i + 1);
        if (i != j) std::swap(idx[i], idx[j]);
    }
    const int sample_count = std::max(1, (int)(F_ * param_.column_sampling_rate));
    h_ignored_.assign(F_, 0);
    for (int i = 0; i < sample_count; ++i) h_ignored_[idx[i]] = 1;
    if (d_ignored_ == nullptr) d_ignored_ = dalloc<uint8_t>((size_t)F_);
    HIP_CHECK(hipMemcpyAsync(d_ignored_, h_ignored_.data(), (size_t)F_, hipMemcpyHostToDevice, stream_));
    HIP_CHECK(hipStreamSynchronize(stream_));  // h_ignored_ is reused by the next round
    tb_.ignored = d_ignored_;
}

void Trainer::set_option(const std::string &key, double value) {
    if (key == "column_sampling_rate") {
        TGBM_CHECK(value > 0, "column_sampling_rate must be positive");
        param_.column_sampling_rate = (float)value;
        if (!(value < 1)) tb_.ignored = nullptr;
    } else if (key == "reorder_first") {
        reorder_first_ = (int)value;
    } else if (key == "reorder_burst") {
        reorder_burst_ = std::max(1, (int)value);
    } else if (key == "reorder_every") {
        reorder_every_ = (int)value;
    } else if (key == "reorder_min_rows") {
        reorder_min_rows_ = (long)value;
    } else if (key == "bagging") {
        ensure_gh_array();
        param_.bagging = value != 0;
        next_round_ready_ = false;
        gh_words_fresh_ = gh_records_fresh_ = false;
    } else {
        fatal("unknown trainer option %s", key.c_str());
    }
}

// Buffer set of class tree k, and the first set with the item target of a whole round built at once.
TreeBuffers Trainer::set_of(int k) const { return tb_.for_class(n_sets_ > 1 ? k : 0); }

void Trainer::tree_init(int k) {
    if (!in_boost_) ensure_gh_array();
    cur_class_ = k;
    HIP_CHECK_LAUNCHES("the stages before tree_init");  // gradients, bagging, column sampling, metric, re-ordering
    launch_tree_init(stream_, set_of(k), d_gh_ + (size_t)k * n_, param_.lambda, next_round_ready_);
    next_round_ready_ = false;
    lookup_level_ = -1;
    nid_materialized_ = false;
}

void Trainer::ensure_gh_array() {
    if (!gh_array_stale_) return;
    launch_gradient(stream_, objective_, n_, param_.num_class, d_y_, d_yp_, d_gh_, nullptr, 0);
    gh_array_stale_ = false;
}

void Trainer::find_split(int level) {
    if (!in_boost_) ensure_gh_array();
    if (sparse_pass_ && !in_boost_) ensure_hist_arena();
    find_split_sets(set_of(cur_class_), d_gh_ + (size_t)cur_class_ * n_, level, 1);
}

// The sparse level pass keeps no per-node histogram; callers that drive the stages one by one can look at them,
// so the first such call allocates the two level arenas the other layouts always have.
void Trainer::ensure_hist_arena() {
    if (tb_.hist_q[0] != nullptr) return;
    const size_t cells = (size_t)n_sets_ * tb_.max_level_nodes * n_bins_;
    size_t free_b = 0, total_b = 0;
    HIP_CHECK(hipMemGetInfo(&free_b, &total_b));
    TGBM_CHECK(cells * 2 * sizeof(longlong2) < free_b / 2,
               "per-node histograms for stage-wise inspection need %zu bytes (free %zu); use tgbm_trainer_boost",
               cells * 2 * sizeof(longlong2), free_b);
    tb_.hist_q[0] = dalloc<longlong2>(cells);
    tb_.hist_q[1] = dalloc<longlong2>(cells);
    tb_.hist_nodes = tb_.max_level_nodes;
}

// Which features the sparse level pass serves through (bin, node) tables: those with more values than a sorted-pass
// tile holds, and the feature that owns global bin 0 (its table is searched for every node even without values: the
// arg-max of a node without any positive gain ends there).
bool Trainer::sparse_feature_in_tables(int f) {
    if (sparse_bin0_owner_ == -2) {
        sparse_bin0_owner_ = -1;
        for (int q = 0; q < F_ && sparse_bin0_owner_ < 0; ++q)
            if (h_cut_row_ptr_[q + 1] > h_cut_row_ptr_[q]) sparse_bin0_owner_ = q;
        const char *se = std::getenv("TGBM_SPARSE_SORTED");  // "0": every feature through the tables (tests)
        sparse_sorted_on_ = !(se != nullptr && std::string(se) == "0");
        // the sorted pass keeps 40 bytes per stored value of its features for every class tree built together;
        // it is left out when that would take more than a quarter of the free memory
        size_t free_b = 0, total_b = 0;
        HIP_CHECK(hipMemGetInfo(&free_b, &total_b));
        if ((size_t)nnz_ * 40 * (size_t)std::max(1, param_.tree_per_rounds) > free_b / 4) sparse_sorted_on_ = false;
    }
    return !sparse_sorted_on_ || cuts_.feature_nnz[f] > kSortedTile || f == sparse_bin0_owner_;
}

// Work lists of the sparse level pass. Features with at most kSortedTile stored values go to the sorted pass (tasks:
// runs of such features whose values fit one tile); the others to table tasks: runs of consecutive such features
// with about kSparseTaskValues values, a feature with more values than that cut into chunks (tasks of their own)
// whose tables k_sparse_big adds up. The feature that owns global bin 0 is always a table feature (its table is
// searched for every node even without values: the arg-max of a node without any positive gain ends there).
void Trainer::build_sparse_tasks() {
    std::vector<int> fvb(F_ + 1, 0);
    for (int f = 0; f < F_; ++f) fvb[f + 1] = fvb[f] + (int)cuts_.feature_nnz[f];
    auto is_table = [&](int f) { return sparse_feature_in_tables(f); };
    std::vector<SparseTask> tasks;
    std::vector<SparseBig> big;
    std::vector<SortedTask> sorted_tasks;
    std::vector<int> sorted_fid;
    std::vector<int2> sorted_meta;
    std::vector<int> feat_slot(F_, -1);
    int n_small = 0, n_partial = 0, max_big_bins = 0;
    int f = 0;
    while (f < F_) {
        const long m = cuts_.feature_nnz[f];
        if (!is_table(f)) {
            if (m > 0) {
                sorted_fid.push_back(f);
                sorted_meta.push_back(make_int2(h_cut_row_ptr_[f], h_cut_row_ptr_[f + 1] - h_cut_row_ptr_[f]));
            }
            ++f;
            continue;
        }
        if (m > kSparseTaskValues) {
            SparseBig b;
            b.feature = f;
            b.slot_begin = n_partial;
            for (long v = 0; v < m; v += kSparseTaskValues) {
                SparseTask t{f, f + 1, fvb[f] + (int)v, fvb[f] + (int)std::min(m, v + kSparseTaskValues), -1, n_partial++};
                tasks.push_back(t);
            }
            b.slot_end = n_partial;
            b.cand_slot = -1;  // numbered below
            big.push_back(b);
            max_big_bins = std::max(max_big_bins, h_cut_row_ptr_[f + 1] - h_cut_row_ptr_[f]);
            ++f;
            continue;
        }
        int fe = f;
        long vals = 0;
        while (fe < F_ && is_table(fe) && cuts_.feature_nnz[fe] <= kSparseTaskValues &&
               vals + cuts_.feature_nnz[fe] <= kSparseTaskValues) {
            vals += cuts_.feature_nnz[fe];
            ++fe;
        }
        for (int q = f; q < fe; ++q) feat_slot[q] = n_small;
        SparseTask t{f, fe, fvb[f], fvb[fe], n_small++, -1};
        tasks.push_back(t);
        f = fe;
    }
    for (size_t i = 0; i < big.size(); ++i) {
        big[i].cand_slot = n_small + (int)i;
        feat_slot[big[i].feature] = big[i].cand_slot;
    }
    int next_slot = n_small + (int)big.size();
    long n_sorted = 0;
    for (size_t i = 0; i < sorted_fid.size();) {
        size_t e = i;
        long vals = 0;
        while (e < sorted_fid.size() && e - i < ((size_t)1 << (32 - kSortedFeatShift)) &&
               vals + cuts_.feature_nnz[sorted_fid[e]] <= kSortedTile)
            vals += cuts_.feature_nnz[sorted_fid[e++]];
        for (size_t q = i; q < e; ++q) feat_slot[sorted_fid[q]] = next_slot;
        sorted_tasks.push_back(SortedTask{(int)n_sorted, (int)vals, (int)i, (int)(e - i), next_slot++});
        n_sorted += vals;
        i = e;
    }
    // the biggest tasks first: they decide when the level is done
    std::stable_sort(tasks.begin(), tasks.end(),
                     [](const SparseTask &a, const SparseTask &b) { return a.v_end - a.v_begin > b.v_end - b.v_begin; });
    sp_.n_tasks = (int)tasks.size();
    sp_.n_big = (int)big.size();
    sp_.n_sorted_tasks = (int)sorted_tasks.size();
    sp_.n_sorted = n_sorted;
    sp_.n_cand_slots = std::max(1, next_slot);
    sp_.n_partial_slots = n_partial;
    sp_.partial_stride = (size_t)max_big_bins * (size_t)tb_.max_level_nodes;
    SparseTask *d_tasks = dalloc<SparseTask>(tasks.size());
    SparseBig *d_big = dalloc<SparseBig>(big.size());
    SortedTask *d_sorted = dalloc<SortedTask>(sorted_tasks.size());
    int *d_sorted_fid = dalloc<int>(sorted_fid.size());
    int2 *d_sorted_meta = dalloc<int2>(sorted_meta.size());
    int *d_feat_slot = dalloc<int>(feat_slot.size());
    int *d_fvb = dalloc<int>(fvb.size());
    upload(stream_, d_tasks, tasks.data(), tasks.size());
    upload(stream_, d_big, big.data(), big.size());
    upload(stream_, d_sorted, sorted_tasks.data(), sorted_tasks.size());
    upload(stream_, d_sorted_fid, sorted_fid.data(), sorted_fid.size());
    upload(stream_, d_sorted_meta, sorted_meta.data(), sorted_meta.size());
    upload(stream_, d_feat_slot, feat_slot.data(), feat_slot.size());
    upload(stream_, d_fvb, fvb.data(), fvb.size());
    HIP_CHECK(hipStreamSynchronize(stream_));  // the host vectors go out of scope
    sp_.tasks = d_tasks;
    sp_.big = d_big;
    sp_.sorted_tasks = d_sorted;
    sp_.sorted_fid = d_sorted_fid;
    sp_.sorted_meta = d_sorted_meta;
    sp_.feat_val_begin = d_fvb;
    tb_.feat_slot = d_feat_slot;
    log_info("sparse level pass: %d table tasks, %d features in chunks (%d chunks), %zu features (%ld values) in %d "
             "sorted tasks, %d candidate slots per node", sp_.n_tasks, sp_.n_big, n_partial, sorted_fid.size(), n_sorted,
             sp_.n_sorted_tasks, sp_.n_cand_slots);
}

void Trainer::find_split_sets(const TreeBuffers &tb, const GHPair *gh, int level, int n_class) {
    if (sparse_pass_ && level == 0) {
        launch_root_sum(stream_, tb, gh, param_.lambda, n_class);
        launch_sparse_gh_refresh(stream_, tb, csr_, sp_, gh, n_class);
    }
    if (hist_cap_level_ >= 0 && level >= hist_cap_level_) {
        // the level has more nodes than the histogram arena: batches of hist_nodes nodes, each through the whole
        // chain histogram -> merge -> split search -> update before the next one overwrites the arena
        const int nl = 1 << level;
        mark(level == 0 ? PH_GRADIENT : PH_PARTITION, level);
        for (int x0 = 0; x0 < nl; x0 += tb.hist_nodes) {
            TreeBuffers tbb = tb;
            tbb.lvl_x0 = x0;
            tbb.lvl_x1 = std::min(nl, x0 + tb.hist_nodes);
            // node x of the batch sits at (x - x0) * n_bins of the level's buffer (for every class set alike)
            longlong2 *&cur = (level & 1) ? tbb.hist_q[1] : tbb.hist_q[0];
            cur -= (size_t)x0 * n_bins_;
            build_level_hist(tbb, level, gh, n_class);
            mark(PH_HIST, level);
            if (!sparse_) launch_hist_merge(stream_, tbb, level, n_class);
            mark(PH_MERGE, level);
            if (wide_eval_) launch_eval_split_wide(stream_, tbb, level, param_.min_child_weight, param_.lambda, n_class, false);
            else launch_eval_split(stream_, tbb, level, param_.min_child_weight, param_.lambda, n_class, false);
            launch_best_update(stream_, tbb, level, param_.rt_eps, param_.lambda, n_class);
            mark(PH_SPLIT, level);
        }
        lookup_level_ = level;
        HIP_CHECK_LAUNCHES("find_split");
        return;
    }
    mark(level == 0 ? PH_GRADIENT : PH_PARTITION, level);  // closes what ran before this level's histogram
    build_level_hist(tb, level, gh, n_class);
    mark(PH_HIST, level);
    if (!sparse_pass_) {
        if (!sparse_) launch_hist_merge(stream_, tb, level, n_class);
        if (level == 0) launch_root_sum(stream_, tb, gh, param_.lambda, n_class);
        mark(PH_MERGE, level);
        // inside boost() nobody looks at the last level's derived histograms (the stage-wise API keeps them); the
        // last level that fits a capped arena keeps them for the batches of the next one
        if (wide_eval_)
            launch_eval_split_wide(stream_, tb, level, param_.min_child_weight, param_.lambda, n_class,
                                   !(in_boost_ && level == param_.depth - 1));
        else
            launch_eval_split(stream_, tb, level, param_.min_child_weight, param_.lambda, n_class,
                              !(in_boost_ && level == param_.depth - 1));
    }
    launch_best_update(stream_, tb, level, param_.rt_eps, param_.lambda, n_class);
    mark(PH_SPLIT, level);
    lookup_level_ = level;  // until partition(level) moves the rows into the children's lists
    HIP_CHECK_LAUNCHES("find_split");
}

void Trainer::build_level_hist(const TreeBuffers &tb, int level, const GHPair *gh, int n_class) {
    if (sparse_pass_) {
        // histogram and split search of the level in one pass; stage-wise driving also gets the per-node histograms
        launch_sparse_level(stream_, tb, csr_, sp_, gh, level, param_.min_child_weight, param_.lambda,
                            !in_boost_ && tb_.hist_q[0] != nullptr, n_class, level == param_.depth - 1);
    } else if (sparse_)
        launch_hist_csr(stream_, tb, csr_, gh, level, n_class);
    else {
        DenseBins b = bins_;
        // (the root level's launch of a tree moves the words into the records; the levels below use them there)
        if (level == 0) gh_records_fresh_ = gh_words_fresh_ && n_class == 1 && gh == d_gh_ && tb.lvl_x0 == 0;
        b.gh_fresh = gh_records_fresh_ && n_class == 1 && gh == d_gh_;
        b.gh_objective = objective_;
        launch_hist_dense(stream_, tb, b, gh, level, n_class);
    }
}

void Trainer::partition(int level) { partition_sets(set_of(cur_class_), level, 1); }

void Trainer::partition_sets(const TreeBuffers &tb, int level, int n_class) {
    // the last level is not partitioned: its split nodes keep their rows until the tree's final pass
    if (level < param_.depth - 1) lookup_level_ = -1;
    if (sparse_pass_) {
        launch_sparse_partition(stream_, tb, csr_, level, n_class);  // every level: the map is the only row state
        lookup_level_ = -1;
    } else if (sparse_)
        launch_partition_csr(stream_, tb, csr_, level, n_class);
    else
        launch_partition_dense(stream_, tb, bins_, level, n_class);
    mark(PH_PARTITION, level);
    HIP_CHECK_LAUNCHES("partition");
}

void Trainer::log_plan(const TreeBuffers &tb) {
    size_t off = ctl_log_.size();
    ctl_log_.resize(off + param_.depth + 1);
    if (sparse_pass_) {
        // rows of the nodes the reference would build from rows: the root, then the smaller child of every pair
        std::vector<int> rows((size_t)tb.n_nodes);
        HIP_CHECK(hipMemcpyAsync(rows.data(), tb.node_rows, sizeof(int) * rows.size(), hipMemcpyDeviceToHost, stream_));
        HIP_CHECK(hipStreamSynchronize(stream_));
        for (int level = 0; level <= param_.depth; ++level) {
            long built = level == 0 ? n_ : 0;
            if (level > 0 && level < param_.depth)
                for (int x = (1 << level) - 1; x < (2 << level) - 1; x += 2) built += std::min(rows[x], rows[x + 1]);
            ctl_log_[off + level] = LevelCtl{0, 0, 0, (int)built};
        }
        return;
    }
    HIP_CHECK(hipMemcpyAsync(ctl_log_.data() + off, tb.ctl, sizeof(LevelCtl) * (size_t)(param_.depth + 1),
                             hipMemcpyDeviceToHost, stream_));
    HIP_CHECK(hipStreamSynchronize(stream_));
}

void Trainer::finish_tree(int k, bool fuse_round_end) {
    const TreeBuffers tb = set_of(k);
    rank_order_fresh_ = false;  // the scores change below
    // (the tree is pruned by a workgroup of the same launches)
    if (fuse_round_end) {
        // one tree per round: prediction update + metric + next gradients + their statistics in one pass
        // (see gh_array_stale_: inside boost() the next tree may need the words only)
        const bool words_only = in_boost_ && d_gh_words_ != nullptr && tb.complete_feature >= 0;
        launch_round_end(stream_, tb, &bins_, &csr_, lookup_level_, objective_, metric_kind_, d_y_, d_yp_,
                         param_.learning_rate, words_only ? nullptr : d_gh_, d_metric_scratch_, d_metric_ + rounds_done_,
                         &param_.gamma, d_gh_words_);
        gh_array_stale_ = words_only;
        gh_words_fresh_ = d_gh_words_ != nullptr;
        gh_records_fresh_ = false;  // (the records still hold the finished tree's words)
        next_round_ready_ = true;
    } else {
        launch_predict_in_training(stream_, tb, &bins_, &csr_, lookup_level_, d_yp_ + (size_t)k * n_,
                                   param_.learning_rate, 1, &param_.gamma);
    }
    TGBM_CHECK(trees_built_ < model_cap_trees_, "more trees built than n_trees * tree_per_rounds");
    HIP_CHECK(hipMemcpyAsync(d_model_ + (size_t)trees_built_ * tb.n_nodes, tb.nodes,
                             sizeof(TreeNode) * (size_t)tb.n_nodes, hipMemcpyDeviceToDevice, stream_));
    mark(PH_TREE_END);
    if (profiling_) log_plan(tb);
    ++trees_built_;
    HIP_CHECK_LAUNCHES("finish_tree");
}

// All class trees of a round through the same launches (class = blockIdx.z): the trees are independent
// given the round's gradients, and one launch over K small trees costs about what one tree costs.
void Trainer::build_round_together() {
    const int K = param_.tree_per_rounds;
    TreeBuffers tb = tb_;
    // the K classes share the chip: size every class's histogram items for its share of the workgroup slots
    tb.target_hitems = std::max(4, tb_.target_hitems / K);
    launch_tree_init(stream_, tb, d_gh_, param_.lambda, false, K);
    lookup_level_ = -1;
    nid_materialized_ = false;
    for (int level = 0; level < param_.depth; ++level) {
        find_split_sets(tb, d_gh_, level, K);
        partition_sets(tb, level, K);
    }
    launch_predict_in_training(stream_, tb, &bins_, &csr_, lookup_level_, d_yp_, param_.learning_rate, K, &param_.gamma);
    TGBM_CHECK(trees_built_ + K <= model_cap_trees_, "more trees built than n_trees * tree_per_rounds");
    HIP_CHECK(hipMemcpyAsync(d_model_ + (size_t)trees_built_ * tb.n_nodes, tb.nodes,
                             sizeof(TreeNode) * (size_t)tb.n_nodes * K, hipMemcpyDeviceToDevice, stream_));
    mark(PH_TREE_END);
    if (profiling_)
        for (int k = 0; k < K; ++k) log_plan(tb.for_class(k));
    trees_built_ += K;
    cur_class_ = K - 1;
    HIP_CHECK_LAUNCHES("build_round_together");
}

void Trainer::run_metric(float *slot) {
    if (objective_ == OBJ_RANK) {
        rank_->metric(metric_kind_, d_yp_, slot);
        rank_order_fresh_ = true;
    } else
        launch_metric(stream_, metric_kind_, n_, param_.num_class, d_y_, d_yp_, d_metric_scratch_, slot);
}

float Trainer::metric() {
    float *slot = d_metric_ + std::min(rounds_done_, std::max(1, param_.n_trees) - 1);
    run_metric(slot);
    float v = 0;
    HIP_CHECK(hipMemcpyAsync(&v, slot, sizeof(float), hipMemcpyDeviceToHost, stream_));
    HIP_CHECK(hipStreamSynchronize(stream_));
    return v;
}

void Trainer::boost(int rounds) {
    static const char *names[] = {"RMSE", "test error", "multi-class accuracy", "MAP", "NDCG"};
    in_boost_ = true;
    for (int r = 0; r < rounds; ++r) {
        TGBM_CHECK(rounds_done_ < std::max(1, param_.n_trees), "boost called more often than n_trees");
        // (with bagging the next round's gradients are not the plain ones the fused pass would compute)
        const bool fuse = (objective_ == OBJ_SQUARE || objective_ == OBJ_LOGISTIC) && param_.tree_per_rounds == 1 &&
                          !param_.bagging;
        mark(-1);  // a round's first interval starts here (log_plan of the previous round waited for the device)
        if (profiling_) ++prof_rounds_;
        // the reference's order of the draws from rand(): gradients (ranking partner seed), bagging seed
        // (booster.h:80-84), then the column shuffle at the start of build_approximate (tree_builder.cu:150-152)
        if (!next_round_ready_) compute_gradient();
        sample_columns();
        if (n_sets_ > 1) {
            build_round_together();
        } else {
            for (int k = 0; k < param_.tree_per_rounds; ++k) {
                tree_init(k);
                // The reference leaves the level loop when no row sits in a node that was split
                // (tree_builder.cu:174-181). Running the remaining levels is a no-op on every output
                // (no valid node, no work item), so the loop is not cut short and needs no readback.
                for (int level = 0; level < param_.depth; ++level) {
                    find_split(level);
                    partition(level);
                }
                finish_tree(k, fuse);
            }
        }
        float *slot = d_metric_ + rounds_done_;
        if (!fuse) {
            mark(-1);
            run_metric(slot);
            mark(PH_METRIC);
        }
        if (g_verbose >= 1) {
            float v = 0;
            HIP_CHECK(hipMemcpyAsync(&v, slot, sizeof(float), hipMemcpyDeviceToHost, stream_));
            HIP_CHECK(hipStreamSynchronize(stream_));
            log_info("[%d/%d] %s = %g", rounds_done_ + 1, param_.n_trees, names[metric_kind_], v);
        }
        ++rounds_done_;
        // after each of the trees reorder_first_ .. reorder_first_ + reorder_burst_ - 1 (consecutive stable sorts
        // cluster the rows by the leaves of the last tree, inside those by the leaves of the one before), then
        // every reorder_every_ trees
        const char *always = std::getenv("TGBM_REORDER");
        if (reorder_allowed() &&
            ((always != nullptr && std::string(always) == "always") ||
             (rounds_done_ >= reorder_first_ && rounds_done_ < reorder_first_ + reorder_burst_) ||
             (reorder_every_ > 0 && rounds_done_ > reorder_first_ && (rounds_done_ - reorder_first_) % reorder_every_ == 0))) {
            mark(-1);
            reorder_rows();
            mark(PH_REORDER);
        }
        HIP_CHECK_LAUNCHES("boost");
    }
    in_boost_ = false;
}

// Rows that end in the same leaf of one tree tend to travel together through the next trees. Below the root
// a histogram work item gathers its rows through a row list, one 128-byte line per row for the bin bytes and
// one for the gradient pair; when the rows of a node sit next to each other those lines are shared. So every
// few trees the rows are physically re-ordered by the leaf they just ended in (stable: inside a leaf the
// previous order stays): the row-major and column-major bin matrices, labels and predictions move, the
// permutation is remembered, and everything the API hands out per row is translated back to the caller's row
// order. Histograms are exact integer sums, so the trees do not depend on the row order; only the float
// reductions over all rows (root sums, metric) see another order of additions.
// With several class trees per round the leaves of the round's last tree give the order (measured on 5 M rows,
// 4 classes: 2.9 -> 2.35 ms per round). Not done for: the sparse layout, ranking (groups are runs of rows),
// small data. (Bagging's draw counts belong to original row indices: they are applied through the permutation.)
bool Trainer::reorder_allowed() const {
    const char *e = std::getenv("TGBM_REORDER");  // "0": never; "always": after every tree, any size (tests)
    const bool env_off = e != nullptr && std::string(e) == "0";
    if (e != nullptr && std::string(e) == "always") return !sparse_ && objective_ != OBJ_RANK;
    return !env_off && reorder_first_ > 0 && !sparse_ && objective_ != OBJ_RANK && (long)n_ >= reorder_min_rows_;
}

void Trainer::reorder_rows() {
    const TreeBuffers tb = set_of(cur_class_);  // the tree built last (the one whose map the API hands out)
    const int n_planes = (int)(n_yp_ / n_);     // prediction planes: one per class
    if (reorder_sorter_.cap < n_) {
        reorder_sorter_.alloc(n_);
        d_perm_alt_ = dalloc<int>((size_t)n_);
        int *second = dalloc<int>((size_t)n_);
        d_binmat_alt_ = dalloc<uint8_t>((size_t)n_ * bins_.W * bins_.n_blocks * bins_.bin_bytes);
        d_y_alt_ = dalloc<float>((size_t)n_);
        d_yp_alt_ = dalloc<float>((size_t)n_yp_);
        perm_spare_ = second;
    }
    // the finished tree's row -> node map (its row lists are intact until the next tree starts)
    launch_nid_rebuild(stream_, tb, &bins_, &csr_, lookup_level_);
    launch_reorder_keys(stream_, n_, param_.depth, tb.nid, reorder_sorter_.keys[0], reorder_sorter_.vals[0]);
    const int cur = sort_pairs(stream_, reorder_sorter_, n_, param_.depth);
    const int *from = reorder_sorter_.vals[cur];
    const size_t blk = bins_.block_stride;
    for (int b = 0; b < bins_.n_blocks; ++b)
        launch_gather_rows(stream_, n_, bins_.W * bins_.bin_bytes, from, d_binmat_ + b * blk, d_binmat_alt_ + b * blk);
    launch_gather_rows(stream_, n_, 4, from, d_y_, d_y_alt_);
    for (int k = 0; k < n_planes; ++k)
        launch_gather_rows(stream_, n_, 4, from, d_yp_ + (size_t)k * n_, d_yp_alt_ + (size_t)k * n_);
    int *perm_new = d_perm_ == d_perm_alt_ ? perm_spare_ : d_perm_alt_;
    launch_gather_perm(stream_, n_, from, d_perm_, perm_new);
    // the row -> node map moves along, so that it can still be handed out for this tree
    launch_gather_rows(stream_, n_, 4, from, tb.nid, reorder_sorter_.vals[cur ^ 1]);
    HIP_CHECK(hipMemcpyAsync(tb.nid, reorder_sorter_.vals[cur ^ 1], sizeof(int) * (size_t)n_, hipMemcpyDeviceToDevice,
                             stream_));
    std::swap(d_binmat_, d_binmat_alt_);
    std::swap(d_y_, d_y_alt_);
    std::swap(d_yp_, d_yp_alt_);
    d_perm_ = perm_new;
    bins_.data = d_binmat_;
    launch_cols_from_rows(stream_, n_, bins_.W, bins_.n_cols, bins_.n_blocks, d_binmat_, bins_.block_stride,
                          const_cast<uint8_t *>(bins_.col), bins_.col_stride, bins_.bin_bytes);
    h_perm_valid_ = false;
    nid_materialized_ = true;
    lookup_level_ = -1;
    // gradients (of this or already of the next round) and their block statistics are in the old order
    next_round_ready_ = false;
    gh_words_fresh_ = gh_records_fresh_ = false;
    gh_array_stale_ = false;  // (recomputed here)
    launch_gradient(stream_, objective_, n_, param_.num_class, d_y_, d_yp_, d_gh_, nullptr, 0);
    ++reorders_done_;
}

const std::vector<int> &Trainer::host_perm() {
    if (d_perm_ == nullptr) {
        h_perm_.clear();
    } else if (!h_perm_valid_) {
        h_perm_.resize((size_t)n_);
        HIP_CHECK(hipMemcpy(h_perm_.data(), d_perm_, sizeof(int) * (size_t)n_, hipMemcpyDeviceToHost));
    }
    h_perm_valid_ = true;
    return h_perm_;
}

std::vector<std::vector<Tree>> Trainer::model_to_host() {
    sync();
    std::vector<TreeNode> flat((size_t)trees_built_ * tb_.n_nodes);
    if (!flat.empty())
        HIP_CHECK(hipMemcpy(flat.data(), d_model_, flat.size() * sizeof(TreeNode), hipMemcpyDeviceToHost));
    std::vector<std::vector<Tree>> out;
    const int tpr = param_.tree_per_rounds;
    for (int t = 0; t < trees_built_; ++t) {
        if (t % tpr == 0) out.emplace_back();
        Tree tr;
        tr.nodes.assign(flat.begin() + (size_t)t * tb_.n_nodes, flat.begin() + (size_t)(t + 1) * tb_.n_nodes);
        out.back().push_back(std::move(tr));
    }
    return out;
}

std::vector<float> Trainer::metric_log() {
    sync();
    std::vector<float> v((size_t)rounds_done_);
    if (!v.empty()) HIP_CHECK(hipMemcpy(v.data(), d_metric_, v.size() * sizeof(float), hipMemcpyDeviceToHost));
    return v;
}

void Trainer::set_profiling(bool on) {
    sync();
    profiling_ = on;
}

HistProfile Trainer::profile() {
    sync();
    HistProfile p;
    p.rounds = prof_rounds_;
    for (size_t i = 1; i < marks_.size(); ++i) {
        if (marks_[i].phase < 0) continue;
        float ms = 0;
        HIP_CHECK(hipEventElapsedTime(&ms, marks_[i - 1].ev, marks_[i].ev));
        p.phase_ms[marks_[i].phase] += ms;
        if (marks_[i].phase == PH_HIST) {
            p.hist_ms += ms;
            p.hist_launches++;
            if (marks_[i].level == 0) {
                p.root_ms += ms;
                p.root_launches++;
            } else {
                p.below_ms += ms;
                p.below_launches++;
            }
        }
    }
    // algorithmic bytes: every visited row reads its bin bytes (one per feature), its gradient pair
    // and, below the root, its row index; every launch writes the level's built histograms once.
    const int per_tree = param_.depth + 1;
    for (size_t t = 0; t * per_tree < ctl_log_.size(); ++t) {
        for (int level = 0; level < param_.depth; ++level) {
            const LevelCtl &c = ctl_log_[t * per_tree + level];
            p.rows_built += c.rows_built;
            long long b;
            if (sparse_)  // CSR: 4-byte bin id per stored value + row pointer, gradient pair and row index per row
                b = (long long)((double)c.rows_built * ((double)nnz_ / n_ * 4 + 8 + 8 + (level > 0 ? 4 : 0)));
            else
                b = (long long)c.rows_built * (F_ * bins_.bin_bytes + 8 + (level > 0 ? 4 : 0));
            p.hist_bytes += b;
            (level == 0 ? p.root_bytes : p.below_bytes) += b;
        }
    }
    return p;
}

int Trainer::info(const std::string &key) const {
    if (key == "n") return n_;
    if (key == "n_features") return F_;
    if (key == "n_bins") return n_bins_;
    if (key == "num_class") return param_.num_class;
    if (key == "tree_per_rounds") return param_.tree_per_rounds;
    if (key == "n_nodes") return tb_.n_nodes;
    if (key == "n_sets") return n_sets_;
    if (key == "sparse") return sparse_ ? 1 : 0;
    if (key == "sparse_pass") return sparse_pass_ ? 1 : 0;
    if (key == "wide_bins") return wide_bins_ ? 1 : 0;
    if (key == "wide_eval") return wide_eval_ ? 1 : 0;
    if (key == "row_lists") return sparse_pass_ ? 0 : 1;  // the sparse level pass keeps a row -> node map only
    if (key == "dense_W") return bins_.W;
    if (key == "gh_word_lane") return gh_word_lane_;  // dword of a row's record that carries its gradient word, -1: none
    if (key == "dense_cols") return sparse_ ? 0 : bins_.n_cols;  // columns of the bin matrix (fewer than features: bundles)
    if (key == "dense_bin_bytes") return sparse_ ? 0 : bins_.bin_bytes;
    if (key == "reorders_done") return reorders_done_;
    if (key == "device_free_mb") {
        size_t free_b = 0, total_b = 0;
        HIP_CHECK(hipMemGetInfo(&free_b, &total_b));
        return (int)(free_b >> 20);
    }
    if (key == "dense_blocks") return bins_.n_blocks;
    if (key == "trees_built") return trees_built_;
    if (key == "rounds_done") return rounds_done_;
    if (key == "n_packs") return tb_.n_packs;
    if (key == "depth") return param_.depth;
    if (key == "y_pred_size") return (int)n_yp_;
    if (key == "max_hitems") return tb_.max_hitems;
    fatal("unknown info key %s", key.c_str());
}

size_t Trainer::get(const std::string &name, void *out, size_t cap) {
    sync();
    const void *src = nullptr;
    size_t bytes = 0;
    const int max_level_nodes = 1 << (param_.depth - 1 > 0 ? param_.depth - 1 : 0);
    const TreeBuffers cur = set_of(cur_class_);  // per-tree buffers: those of the class tree built last
    if (name == "cut_val") src = cuts_.cut_val, bytes = sizeof(float) * (size_t)n_bins_;
    else if (name == "cut_row_ptr") src = cuts_.cut_row_ptr, bytes = sizeof(int) * (size_t)(F_ + 1);
    else if (name == "cut_fid") src = cuts_.cut_fid, bytes = sizeof(int) * (size_t)n_bins_;
    else if (name == "binmat") src = d_binmat_, bytes = sparse_ ? 0 : (size_t)n_ * bins_.W * bins_.n_blocks * bins_.bin_bytes;
    else if (name == "csr_bin") src = csr_.bin, bytes = sparse_ ? sizeof(int) * (size_t)nnz_ : 0;
    else if (name == "feat_col") src = bins_.feat_col, bytes = bins_.feat_col != nullptr ? sizeof(int) * (size_t)F_ : 0;
    else if (name == "feat_lo") src = bins_.feat_lo, bytes = bins_.feat_lo != nullptr ? (size_t)F_ : 0;
    else if (name == "nid") {
        // the map is kept as row lists; materialise it on demand (a re-ordering of the rows has done so already)
        if (!nid_materialized_) launch_nid_rebuild(stream_, cur, &bins_, &csr_, lookup_level_);
        sync();
        src = cur.nid, bytes = sizeof(int) * (size_t)n_;
    }
    else if (name == "gh") {
        ensure_gh_array();
        sync();
        src = d_gh_, bytes = sizeof(GHPair) * (size_t)param_.num_class * n_;
    }
    else if (name == "y_pred") src = d_yp_, bytes = sizeof(float) * (size_t)n_yp_;
    else if (name == "y") src = d_y_, bytes = sizeof(float) * (size_t)n_;
    else if (name == "nodes") src = cur.nodes, bytes = sizeof(TreeNode) * (size_t)tb_.n_nodes;
    else if (name == "sp") src = cur.sp, bytes = sizeof(SplitPoint) * (size_t)max_level_nodes;
    else if (name == "hist_q0") src = cur.hist_q[0], bytes = tb_.hist_q[0] ? sizeof(longlong2) * (size_t)max_level_nodes * n_bins_ : 0;
    else if (name == "hist_q1") src = cur.hist_q[1], bytes = tb_.hist_q[1] ? sizeof(longlong2) * (size_t)max_level_nodes * n_bins_ : 0;
    else if (name == "quant") src = cur.quant, bytes = sizeof(QuantCtl);
    else if (name == "ctl") src = cur.ctl, bytes = sizeof(LevelCtl) * (size_t)(param_.depth + 1);
    else if (name == "seg") src = cur.seg, bytes = sizeof(int2) * (size_t)tb_.n_nodes;
    else if (name == "ridx0") src = cur.ridx[0], bytes = sizeof(int) * (size_t)n_;
    else if (name == "ridx1") src = cur.ridx[1], bytes = sizeof(int) * (size_t)n_;
    else if (name == "model") src = d_model_, bytes = sizeof(TreeNode) * (size_t)trees_built_ * tb_.n_nodes;
    else if (name == "metric_log") src = d_metric_, bytes = sizeof(float) * (size_t)rounds_done_;
    else if (name == "rank_order") {
        // rows in the order the last ranking gradient / metric pass sorted them
        TGBM_CHECK(rank_ != nullptr, "rank_order belongs to the ranking objectives");
        src = rank_->last_sorted_rows(), bytes = sizeof(int) * (size_t)n_;
    }
    else fatal("unknown buffer %s", name.c_str());
    if (out != nullptr && cap >= bytes && bytes > 0) {
        HIP_CHECK(hipMemcpy(out, src, bytes, hipMemcpyDeviceToHost));
        if (name == "binmat" && gh_word_lane_ >= 0) {
            // (the records' spare dword carries the rows' gradient words: the matrix is handed out as bins only)
            const size_t rb = (size_t)bins_.W;
            unsigned char *m = static_cast<unsigned char *>(out);
            for (int r = 0; r < n_; ++r) std::memset(m + (size_t)r * rb + rb - 4, kMissingBin, 4);
        }
        // per-row buffers are handed out in the caller's row order, whatever the physical order is by now
        size_t row_bytes = 0, n_planes = 1;
        if (name == "nid" || name == "y") row_bytes = 4;
        else if (name == "y_pred") row_bytes = 4, n_planes = (size_t)(n_yp_ / n_);
        else if (name == "gh") row_bytes = sizeof(GHPair), n_planes = (size_t)param_.num_class;
        else if (name == "binmat") row_bytes = (size_t)bins_.W * bins_.bin_bytes, n_planes = (size_t)bins_.n_blocks;
        const bool row_list = name == "ridx0" || name == "ridx1";
        static const std::vector<int> identity;
        const std::vector<int> &perm = (row_bytes || row_list) ? host_perm() : identity;
        if (!perm.empty()) {
            if (row_bytes) {
                std::vector<char> phys(static_cast<char *>(out), static_cast<char *>(out) + bytes);
                for (size_t pl = 0; pl < n_planes; ++pl) {
                    const char *ps = phys.data() + pl * (size_t)n_ * row_bytes;
                    char *pd = static_cast<char *>(out) + pl * (size_t)n_ * row_bytes;
                    for (int p = 0; p < n_; ++p) std::memcpy(pd + (size_t)perm[p] * row_bytes, ps + (size_t)p * row_bytes, row_bytes);
                }
            } else if (row_list) {  // row lists: the entries are row positions
                int *v = static_cast<int *>(out);
                for (int i = 0; i < n_; ++i)
                    if (v[i] >= 0 && v[i] < n_) v[i] = perm[v[i]];
            }
        }
    }
    return bytes;
}

void Trainer::set(const std::string &name, const void *in, size_t bytes) {
    if (name == "gh") gh_array_stale_ = false;  // (overwritten below)
    else ensure_gh_array();                      // (the pairs of the predictions as they are now)
    sync();
    next_round_ready_ = false;
    rank_order_fresh_ = false;
    void *dst = nullptr;
    size_t want = 0;
    if (name == "gh") dst = d_gh_, want = sizeof(GHPair) * (size_t)param_.num_class * n_, gh_words_fresh_ = gh_records_fresh_ = false;
    else if (name == "y_pred") dst = d_yp_, want = sizeof(float) * (size_t)n_yp_;
    else fatal("buffer %s cannot be set", name.c_str());
    TGBM_CHECK(bytes == want, "set %s: got %zu bytes, expected %zu", name.c_str(), bytes, want);
    const std::vector<int> &perm = host_perm();
    if (!perm.empty()) {  // caller's row order -> physical order (re-ordering only happens with one value per row)
        const size_t row_bytes = name == "gh" ? sizeof(GHPair) : sizeof(float);
        const size_t n_planes = bytes / ((size_t)n_ * row_bytes);  // one per class
        std::vector<char> phys(bytes);
        for (size_t pl = 0; pl < n_planes; ++pl) {
            const char *src_pl = static_cast<const char *>(in) + pl * (size_t)n_ * row_bytes;
            char *dst_pl = phys.data() + pl * (size_t)n_ * row_bytes;
            for (int p = 0; p < n_; ++p)
                std::memcpy(dst_pl + (size_t)p * row_bytes, src_pl + (size_t)perm[p] * row_bytes, row_bytes);
        }
        HIP_CHECK(hipMemcpy(dst, phys.data(), bytes, hipMemcpyHostToDevice));
        return;
    }
    HIP_CHECK(hipMemcpy(dst, in, bytes, hipMemcpyHostToDevice));
}

// ---------------------------------------------------------------------------------------------
// TreeTrainer::train (src/thundergbm/trainer.cu:18-57)
std::vector<std::vector<Tree>> train(GBMParam &param, const DataSet &dataset) {
    if (param.tree_method == "auto") param.tree_method = "hist";  // this build has the histogram method only
    TGBM_CHECK(param.tree_method == "hist", "tree_method %s is not part of this build (hist only)",
               param.tree_method.c_str());
    if (param.n_device != 1) log_info("n_gpus=%d requested; this build trains on one GPU", param.n_device);
    Trainer trainer(dataset, param);
    // `profiling` (thundergbm_train.cpp:28-30 switches the reference's performance tracking on with it): per-stage
    // timers around every launch group of the boosting loop, reported after the run
    if (param.profiling) trainer.set_profiling(true);
    auto start = std::chrono::high_resolution_clock::now();
    trainer.boost(param.n_trees);
    trainer.sync();
    auto stop = std::chrono::high_resolution_clock::now();
    log_info("training time = %g", std::chrono::duration<float>(stop - start).count());
    if (param.profiling) {
        const HistProfile p = trainer.profile();
        static const char *names[PH_COUNT] = {"gradients and tree init", "build hist", "merge and subtract",
                                              "evaluate and update tree", "data partitioning", "end of tree",
                                              "metric", "row re-ordering"};
        for (int i = 0; i < PH_COUNT; ++i) log_info("profiling: %-26s %10.3f ms", names[i], p.phase_ms[i]);
        log_info("profiling: histogram launches: root %lld x %.1f us, below the root %lld x %.1f us", p.root_launches,
                 p.root_launches ? p.root_ms * 1e3 / p.root_launches : 0.0, p.below_launches,
                 p.below_launches ? p.below_ms * 1e3 / p.below_launches : 0.0);
    }
    std::vector<std::vector<Tree>> model = trainer.model_to_host();
    log_debug("model to host: %.3f s",
              std::chrono::duration<double>(std::chrono::high_resolution_clock::now() - stop).count());
    return model;
}

}  // namespace tgbm
