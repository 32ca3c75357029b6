// Host side of prediction: the reference's Predictor (src/thundergbm/predictor.cu:11-86).
#include <algorithm>
#include <chrono>
#include <cstring>

#include "device_api.h"
#include "host.h"
#include "rank.h"

namespace tgbm {

static int transform_kind(const std::string &objective) {
    if (objective == "binary:logistic") return 1;
    if (objective == "multi:softmax") return 2;
    if (objective == "multi:softprob") return 3;
    if (objective == "reg:logistic") return 4;
    return 0;
}

int compact_records_apply(const TreeNode *model, size_t n_total, int n_nodes, int F) {
    if (n_nodes < 1 || n_nodes > 0x1fff || F < 1 || (size_t)F * 128 * sizeof(float) > 48 * 1024) return 0;
    const size_t dense_bytes = (size_t)(F + 2) * compact_rows_per_group(F) * sizeof(float);
    if (dense_bytes + (size_t)n_nodes * sizeof(uint2) > 64 * 1024) return 0;
    int deepest = 0;
    std::vector<int> level((size_t)n_nodes);
    for (size_t t0 = 0; t0 + (size_t)n_nodes <= n_total; t0 += (size_t)n_nodes) {
        std::fill(level.begin(), level.end(), -1);
        level[0] = 0;
        for (int self = 0; self < n_nodes; ++self) {
            const TreeNode &nd = model[t0 + self];
            const bool children_ok = nd.lch_index >= 0 && nd.lch_index < n_nodes && nd.rch_index >= 0 && nd.rch_index < n_nodes;
            if (nd.is_leaf || !children_ok) continue;  // (a walk ends here)
            if (nd.rch_index != nd.lch_index + 1 || nd.lch_index <= self) return 0;
            if (nd.split_value != nd.split_value) return 0;  // (a NaN threshold: the two comparisons would disagree)
            if (level[self] < 0) continue;  // (not reachable from the root)
            level[nd.lch_index] = level[nd.rch_index] = level[self] + 1;
            deepest = std::max(deepest, level[self] + 1);
        }
    }
    return std::max(deepest, 1);
}

// Runs the traversal kernel and, if asked, the objective's transform and the training metric.
static std::vector<float> run_predict(const GBMParam &param, const std::vector<std::vector<Tree>> &model,
                                      const DataSet &ds, bool transform, bool log_metric) {
    int n_dev = 0;
    hipError_t e = hipGetDeviceCount(&n_dev);
    TGBM_CHECK(e == hipSuccess && n_dev >= 1, "no HIP device available: this library has no CPU path");
    const int n = (int)ds.n_instances();
    int F = (int)ds.n_features();
    const long nnz = ds.nnz;
    TGBM_CHECK(!model.empty() && !model.front().empty(), "empty model");
    const int n_iter = (int)model.size();
    const int nct = (int)model.front().size();
    const int n_nodes = (int)model[0][0].nodes.size();
    std::vector<TreeNode> flat((size_t)n_iter * nct * n_nodes);
    size_t t = 0;
    for (const auto &iter : model) {
        TGBM_CHECK((int)iter.size() == nct, "ragged model");
        for (const Tree &tr : iter) {
            TGBM_CHECK((int)tr.nodes.size() == n_nodes, "trees of different size in one model");
            std::memcpy(flat.data() + t * n_nodes, tr.nodes.data(), sizeof(TreeNode) * (size_t)n_nodes);
            ++t;
        }
    }
    auto t_begin = std::chrono::steady_clock::now();
    auto lap = [&](const char *what) {
        auto now = std::chrono::steady_clock::now();
        log_debug("predict: %s %.3f s", what, std::chrono::duration<double>(now - t_begin).count());
        t_begin = now;
    };
    hipStream_t s;
    HIP_CHECK(hipStreamCreate(&s));
    float *d_val = nullptr, *d_out = nullptr, *d_label = nullptr;
    int *d_col = nullptr, *d_row_ptr = nullptr;
    TreeNode *d_model = nullptr;
    PackedNode *d_packed = nullptr;
    uint2 *d_compact = nullptr;
    int compact_depth = 0;
    const size_t n_out = (size_t)n * nct;
    HIP_CHECK(hipMalloc(&d_val, sizeof(float) * (size_t)std::max(nnz, 1l)));
    HIP_CHECK(hipMalloc(&d_col, sizeof(int) * (size_t)std::max(nnz, 1l)));
    HIP_CHECK(hipMalloc(&d_row_ptr, sizeof(int) * (size_t)(n + 1)));
    HIP_CHECK(hipMalloc(&d_model, sizeof(TreeNode) * flat.size()));
    HIP_CHECK(hipMalloc(&d_packed, sizeof(PackedNode) * flat.size()));
    HIP_CHECK(hipMalloc(&d_out, sizeof(float) * std::max(n_out, (size_t)1)));
    HIP_CHECK(hipMemcpyAsync(d_row_ptr, ds.row_ptr, sizeof(int) * (size_t)(n + 1), hipMemcpyHostToDevice, s));
    HIP_CHECK(hipMemcpyAsync(d_model, flat.data(), sizeof(TreeNode) * flat.size(), hipMemcpyHostToDevice, s));
    launch_pack_model(s, d_model, (long)flat.size(), n_nodes, d_packed);
    launch_fill_f32(s, d_out, 0.f, n_out);
    // The column indices go up first (the feature count, which selects the traversal kernel, may have to be
    // taken from them), then the values in slices of whole rows on a second stream: the traversal of a
    // slice runs while the next slice crosses PCIe.
    if (nnz) upload_large(s, d_col, ds.col_idx, sizeof(int) * (size_t)nnz);
    if (!ds.features_counted) F = device_max_int(s, d_col, nnz) + 1;
    compact_depth = compact_records_apply(flat.data(), flat.size(), n_nodes, F);  // (F is known only now)
    if (compact_depth > 0) {
        HIP_CHECK(hipMalloc(&d_compact, sizeof(uint2) * flat.size()));
        launch_pack_compact(s, d_model, n_iter, nct, n_nodes, F, d_compact);
    }
    HIP_CHECK(hipStreamSynchronize(s));
    lap("allocation, model and column indices");
    {
        hipStream_t s_up;
        HIP_CHECK(hipStreamCreate(&s_up));
        const long slice_entries = 64l << 20;  // ~256 MB of values per slice
        int r0 = 0;
        while (r0 < n) {
            const long e0 = ds.row_ptr[r0];
            // last row whose entries still fit the slice (at least one row)
            const int *first = ds.row_ptr + r0 + 1, *last = ds.row_ptr + n + 1;
            int r1 = (int)(std::upper_bound(first, last, (int)std::min<long>(e0 + slice_entries, nnz)) - ds.row_ptr) - 1;
            r1 = std::max(r1, r0 + 1);
            const long e1 = ds.row_ptr[r1];
            if (e1 > e0) upload_large(s_up, d_val + e0, ds.val + e0, sizeof(float) * (size_t)(e1 - e0));
            HIP_CHECK(hipStreamSynchronize(s_up));  // small copies return before they are done
            launch_predict(s, r1 - r0, F, d_row_ptr + r0, d_col, d_val, d_model, n_iter, nct, n_nodes,
                           param.learning_rate, param.base_score, d_out + r0, (size_t)n, d_packed, d_compact, compact_depth);
            HIP_CHECK_LAUNCHES("predict");
            r0 = r1;
        }
        HIP_CHECK(hipStreamSynchronize(s));
        HIP_CHECK(hipStreamDestroy(s_up));
    }
    lap("values and traversal");
    size_t n_ret = n_out;
    if (log_metric && objective_needs_groups(param.objective)) {
        // MAP / NDCG need the query groups of the rows that are scored (Predictor::predict configures the
        // objective with the dataset's groups, predictor.cu:16-24); without them the metric line is left out
        long covered = 0;
        for (int g : ds.group) covered += g;
        if (!ds.group.empty() && covered == (long)n && (int)ds.y.size() == n) {
            const bool ndcg = param.objective == "rank:ndcg";
            RankContext rc(s, ds.y, ds.group, ndcg);
            float *d_m = nullptr;
            HIP_CHECK(hipMalloc(&d_m, sizeof(float)));
            rc.metric(ndcg ? RANK_METRIC_NDCG : RANK_METRIC_MAP, d_out, d_m);
            float v = 0;
            HIP_CHECK(hipMemcpyAsync(&v, d_m, sizeof(float), hipMemcpyDeviceToHost, s));
            HIP_CHECK(hipStreamSynchronize(s));
            log_info("%s = %g", ndcg ? "NDCG" : "MAP", v);
            HIP_CHECK(hipFree(d_m));
        }
    } else if (log_metric && (int)ds.y.size() == n && n > 0) {
        int kind = 0;
        if (param.objective == "binary:logistic") kind = 1;
        if (param.objective.find("multi:") == 0) kind = 2;
        static const char *names[] = {"RMSE", "test error", "multi-class accuracy"};
        float *d_y = nullptr, *d_m = nullptr;
        double *d_scratch = nullptr;
        HIP_CHECK(hipMalloc(&d_y, sizeof(float) * (size_t)n));
        HIP_CHECK(hipMalloc(&d_m, sizeof(float)));
        HIP_CHECK(hipMalloc(&d_scratch, sizeof(double) * (size_t)row_blocks(n)));
        HIP_CHECK(hipMemcpyAsync(d_y, ds.y.data(), sizeof(float) * (size_t)n, hipMemcpyHostToDevice, s));
        launch_metric(s, kind, n, nct, d_y, d_out, d_scratch, d_m);
        float v = 0;
        HIP_CHECK(hipMemcpyAsync(&v, d_m, sizeof(float), hipMemcpyDeviceToHost, s));
        HIP_CHECK(hipStreamSynchronize(s));
        log_info("%s = %g", names[kind], v);
        HIP_CHECK(hipFree(d_y));
        HIP_CHECK(hipFree(d_m));
        HIP_CHECK(hipFree(d_scratch));
    }
    if (transform) {
        const int kind = transform_kind(param.objective);
        if (kind == 1 || kind == 2) {
            const size_t need = kind == 1 ? 2 : (size_t)std::max(param.num_class, 1);
            TGBM_CHECK(ds.label.size() >= need, "predict: %zu class labels given, %zu needed", ds.label.size(), need);
            HIP_CHECK(hipMalloc(&d_label, sizeof(float) * ds.label.size()));
            HIP_CHECK(hipMemcpyAsync(d_label, ds.label.data(), sizeof(float) * ds.label.size(), hipMemcpyHostToDevice, s));
        }
        launch_predict_transform(s, kind, n, kind == 2 || kind == 3 ? nct : param.num_class, d_label, d_out);
        if (kind == 1 || kind == 2) n_ret = (size_t)n;
    }
    HIP_CHECK_LAUNCHES("predict (metric, transform)");
    std::vector<float> out(n_ret);
    if (n_ret) HIP_CHECK(hipMemcpyAsync(out.data(), d_out, sizeof(float) * n_ret, hipMemcpyDeviceToHost, s));
    HIP_CHECK(hipStreamSynchronize(s));
    lap("transform and download");
    HIP_CHECK(hipFree(d_val));
    HIP_CHECK(hipFree(d_col));
    HIP_CHECK(hipFree(d_row_ptr));
    HIP_CHECK(hipFree(d_model));
    HIP_CHECK(hipFree(d_packed));
    if (d_compact) HIP_CHECK(hipFree(d_compact));
    HIP_CHECK(hipFree(d_out));
    if (d_label) HIP_CHECK(hipFree(d_label));
    HIP_CHECK(hipStreamDestroy(s));
    lap("release");
    return out;
}

std::vector<float> predict_raw(const GBMParam &param, const std::vector<std::vector<Tree>> &model,
                               const DataSet &dataset) {
    return run_predict(param, model, dataset, false, false);
}

std::vector<float> predict(const GBMParam &param, const std::vector<std::vector<Tree>> &model, const DataSet &dataset,
                           bool log_metric) {
    return run_predict(param, model, dataset, true, log_metric);
}

}  // namespace tgbm
