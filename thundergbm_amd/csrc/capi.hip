// extern "C" layer declared in include/thundergbm.h.
#include <chrono>
#include <cstring>
#include <memory>
#include <mutex>

#include "../../include/thundergbm.h"
#include "model_handle.h"
#include "trainer.h"

using namespace tgbm;

struct tgbm_trainer {
    std::unique_ptr<Trainer> impl;
    DataSet dataset;  // labels only after creation (CSR arrays are released)
    GBMParam param;
};

namespace {

// Training and prediction calls of the reference's interface are serialised process-wide, as the reference's
// global mutex does for Booster::boost (include/thundergbm/booster.h:17,78): two threads that call fit() at
// once run one after the other instead of competing for the device.
std::mutex g_call_mutex;

std::vector<std::vector<Tree>> to_nested(const tgbm_model *m, int n_trees, int per_iter) {
    TGBM_CHECK(m != nullptr, "model is null!");
    TGBM_CHECK((size_t)n_trees * per_iter <= m->trees.size(), "model holds %zu trees, %d x %d requested",
               m->trees.size(), n_trees, per_iter);
    std::vector<std::vector<Tree>> out((size_t)n_trees);
    for (int i = 0; i < n_trees; ++i)
        for (int j = 0; j < per_iter; ++j) out[i].push_back(m->trees[(size_t)i * per_iter + j]);
    return out;
}

tgbm_model *from_nested(const std::vector<std::vector<Tree>> &nested) {
    tgbm_model *m = new tgbm_model;
    for (const auto &iter : nested)
        for (const Tree &t : iter) m->trees.push_back(t);
    return m;
}

}  // namespace

extern "C" {

void set_logger(int verbose) { g_verbose = verbose; }

void sparse_train_scikit(int row_size, float *val, int *row_ptr, int *col_ptr, float *label, int depth, int n_trees,
                         int n_device, float min_child_weight, float lambda, float gamma, int max_num_bin,
                         int verbose, float column_sampling_rate, int bagging, int n_parallel_trees,
                         float learning_rate, char *obj_type, int *num_class, char *tree_method, tgbm_model **model,
                         int *tree_per_iter, float *group_label, int *group, int num_group) {
    std::lock_guard<std::mutex> lock(g_call_mutex);
    GBMParam p;
    p.depth = depth;
    p.n_trees = n_trees;
    p.n_device = n_device;
    p.min_child_weight = min_child_weight;
    p.lambda = lambda;
    p.gamma = gamma;
    p.max_num_bin = max_num_bin;
    p.verbose = verbose;
    p.column_sampling_rate = column_sampling_rate;
    p.bagging = bagging != 0;
    p.n_parallel_trees = n_parallel_trees;
    p.learning_rate = learning_rate;
    p.objective = obj_type;
    p.num_class = *num_class;
    p.tree_method = tree_method;
    p.rt_eps = 1e-6f;
    p.tree_per_rounds = 1;
    set_logger(verbose);
    DataSet ds;
    auto t0 = std::chrono::steady_clock::now();
    ds.load_from_sparse(row_size, val, row_ptr, col_ptr, label, group, num_group, p, false);
    log_debug("host-side dataset checks and label grouping: %.3f s",
              std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count());
    *num_class = p.num_class;
    std::vector<std::vector<Tree>> boosted = train(p, ds);
    TGBM_CHECK((int)boosted.size() == n_trees, "%d v.s. %zu", n_trees, boosted.size());
    *tree_per_iter = (int)boosted[0].size();
    *model = from_nested(boosted);
    for (size_t i = 0; i < ds.label.size(); ++i) group_label[i] = ds.label[i];
}

void sparse_predict_scikit(int row_size, float *val, int *row_ptr, int *col_ptr, float *y_pred, tgbm_model **model,
                           int n_trees, int trees_per_iter, char *objective, int num_class, float learning_rate,
                           float *group_label, int *group, int num_group, int verbose) {
    std::lock_guard<std::mutex> lock(g_call_mutex);
    GBMParam p;  // base_score stays 0 on this path, as in the reference (scikit_tgbm.cpp:87-90)
    p.objective = objective;
    p.learning_rate = learning_rate;
    p.num_class = num_class;
    DataSet ds;
    GBMParam load_param = p;
    set_logger(verbose);
    auto t0 = std::chrono::steady_clock::now();
    ds.load_from_sparse(row_size, val, row_ptr, col_ptr, nullptr, group, num_group, load_param, false);
    log_debug("predict: host-side dataset %.3f s",
              std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count());
    ds.label.clear();
    if (group_label != nullptr && objective_needs_group_label(p.objective))
        for (int i = 0; i < num_class; ++i) ds.label.push_back(group_label[i]);
    TGBM_CHECK(model != nullptr && *model != nullptr, "model is null!");
    std::vector<float> out = predict(p, to_nested(*model, n_trees, trees_per_iter), ds, false);
    std::memcpy(y_pred, out.data(), out.size() * sizeof(float));
}

void save(char *model_path, char *objective, float learning_rate, int num_class, int n_trees, int trees_per_iter,
          tgbm_model **model, float *group_label) {
    GBMParam p;
    p.objective = objective;
    p.learning_rate = learning_rate;
    p.num_class = num_class;
    p.n_trees = n_trees;
    TGBM_CHECK(model != nullptr && *model != nullptr, "model is null!");
    DataSet ds;
    if (num_class != 1 && group_label != nullptr)
        for (int i = 0; i < num_class; ++i) ds.label.push_back(group_label[i]);
    Parser::save_model(model_path, p, to_nested(*model, n_trees, trees_per_iter), ds);
}

void load_model(char *model_path, float *learning_rate, int *num_class, int *n_trees, int *trees_per_iter,
                tgbm_model **model) {
    GBMParam p;
    std::vector<std::vector<Tree>> boosted;
    DataSet ds;
    Parser::load_model(model_path, p, boosted, ds);
    *learning_rate = p.learning_rate;
    *num_class = p.num_class;
    *n_trees = p.n_trees;
    TGBM_CHECK(!boosted.empty(), "model file %s holds no tree", model_path);
    *trees_per_iter = (int)boosted[0].size();
    TGBM_CHECK(*n_trees == (int)boosted.size(), "%d v.s. %zu", *n_trees, boosted.size());
    *model = from_nested(boosted);
}

void load_config(char *model_path, float *group_label) {
    GBMParam p;
    std::vector<std::vector<Tree>> boosted;
    DataSet ds;
    Parser::load_model(model_path, p, boosted, ds);
    for (size_t i = 0; i < ds.label.size(); ++i) group_label[i] = ds.label[i];
}

void get_n_nodes(tgbm_model **model, int *n_nodes, int n_trees, int tree_per_iter) {
    TGBM_CHECK(model != nullptr && *model != nullptr, "model is null!");
    const tgbm_model *m = *model;
    TGBM_CHECK((size_t)n_trees * tree_per_iter <= m->trees.size(), "model holds %zu trees", m->trees.size());
    for (int i = 0; i < n_trees * tree_per_iter; ++i) n_nodes[i] = (int)m->trees[(size_t)i].nodes.size();
}

void get_a_tree(tgbm_model **model, int tree_id, int n_nodes, int *children_left, int *children_right,
                int *children_default, int *features, float *thresholds, float *values,
                float *node_sample_weights) {
    TGBM_CHECK(model != nullptr && *model != nullptr, "model is null!");
    const tgbm_model *m = *model;
    TGBM_CHECK(tree_id >= 0 && (size_t)tree_id < m->trees.size(), "tree id %d out of range", tree_id);
    const Tree &tree = m->trees[(size_t)tree_id];
    TGBM_CHECK(n_nodes == (int)tree.nodes.size(), "n_nodes %d != %zu", n_nodes, tree.nodes.size());
    for (int i = 0; i < n_nodes; ++i) {
        const TreeNode &nd = tree.nodes[(size_t)i];
        children_left[i] = nd.lch_index;
        children_right[i] = nd.rch_index;
        children_default[i] = nd.default_right ? nd.rch_index : nd.lch_index;
        if (nd.is_leaf) {
            children_left[i] = children_right[i] = children_default[i] = -1;
            values[i] = nd.base_weight;
        } else {
            values[i] = 0;
        }
        features[i] = nd.split_feature_id;
        thresholds[i] = nd.split_value;
        node_sample_weights[i] = nd.sum_gh_pair.h;
    }
}

void model_free(tgbm_model **model) {
    if (model != nullptr && *model != nullptr) {
        delete *model;
        *model = nullptr;
    }
}

// ----------------------------------------------------------------------------- R entry points
// R's .C() convention: every argument is a pointer, strings arrive as char**. File in, file out.
void train_R(int *depth, int *n_trees, int *n_gpus, int *verbose, int *profiling, char **data, int *max_num_bin,
             double *column_sampling_rate, int *bagging, int *n_parallel_trees, double *learning_rate,
             char **objective, int *num_class, int *min_child_weight, double *lambda_tgbm, double *gamma,
             char **tree_method, char **model_out) {
    std::lock_guard<std::mutex> lock(g_call_mutex);
    set_logger(*verbose);
    GBMParam p;
    p.depth = *depth;
    p.n_trees = *n_trees;
    p.n_device = *n_gpus;
    p.verbose = *verbose;
    p.profiling = *profiling != 0;
    p.path = data[0];
    p.max_num_bin = *max_num_bin;
    p.column_sampling_rate = (float)*column_sampling_rate;
    p.bagging = *bagging != 0;
    p.n_parallel_trees = *n_parallel_trees;
    p.learning_rate = (float)*learning_rate;
    p.objective = objective[0];
    p.num_class = *num_class;
    p.min_child_weight = (float)*min_child_weight;
    p.lambda = (float)*lambda_tgbm;
    p.gamma = (float)*gamma;
    p.tree_method = tree_method[0];
    p.rt_eps = 1e-6f;
    p.tree_per_rounds = 1;
    DataSet dataset;
    dataset.load_from_file(p.path, p);
    std::vector<std::vector<Tree>> model = train(p, dataset);
    Parser::save_model(model_out[0], p, model, dataset);
}

void predict_R(char **data, char **model_in, int *verbose) {
    std::lock_guard<std::mutex> lock(g_call_mutex);
    set_logger(*verbose);
    GBMParam p;
    DataSet dataset;
    std::vector<std::vector<Tree>> model;
    Parser::load_model(model_in[0], p, model, dataset);
    std::vector<float> model_labels = dataset.label;
    dataset.load_from_file(data[0], p);
    if (!objective_needs_group_label(p.objective)) dataset.label = model_labels;
    (void)predict(p, model, dataset, true);
}

// ------------------------------------------------------------------------------- session API
tgbm_trainer *tgbm_trainer_create(int row_size, const float *val, const int *row_ptr, const int *col_ptr,
                                  const float *label, int depth, int n_trees, float min_child_weight, float lambda,
                                  float gamma, int max_num_bin, float learning_rate, const char *objective,
                                  int num_class, int verbose) {
    return tgbm_trainer_create_grouped(row_size, val, row_ptr, col_ptr, label, depth, n_trees, min_child_weight,
                                       lambda, gamma, max_num_bin, learning_rate, objective, num_class, verbose,
                                       nullptr, 0);
}

tgbm_trainer *tgbm_trainer_create_grouped(int row_size, const float *val, const int *row_ptr, const int *col_ptr,
                                          const float *label, int depth, int n_trees, float min_child_weight,
                                          float lambda, float gamma, int max_num_bin, float learning_rate,
                                          const char *objective, int num_class, int verbose, const int *group,
                                          int num_group) {
    set_logger(verbose);
    tgbm_trainer *t = new tgbm_trainer;
    GBMParam &p = t->param;
    p.depth = depth;
    p.n_trees = n_trees;
    p.min_child_weight = min_child_weight;
    p.lambda = lambda;
    p.gamma = gamma;
    p.max_num_bin = max_num_bin;
    p.learning_rate = learning_rate;
    p.objective = objective;
    p.num_class = num_class;
    p.verbose = verbose;
    p.tree_method = "hist";
    t->dataset.load_from_sparse(row_size, val, row_ptr, col_ptr, label, group, num_group, p, false);
    t->impl.reset(new Trainer(t->dataset, p));
    t->dataset.val = nullptr;  // the caller's buffers are not referenced after this call
    t->dataset.col_idx = nullptr;
    t->dataset.row_ptr = nullptr;
    return t;
}

void tgbm_trainer_destroy(tgbm_trainer *t) { delete t; }

void tgbm_trainer_set_option(tgbm_trainer *t, const char *key, double value) { t->impl->set_option(key, value); }
void tgbm_trainer_sample_columns(tgbm_trainer *t) { t->impl->sample_columns(); }

void tgbm_trainer_boost(tgbm_trainer *t, int rounds) {
    t->impl->boost(rounds);
    t->impl->sync();
}
void tgbm_trainer_gradient(tgbm_trainer *t) { t->impl->compute_gradient(); }
void tgbm_trainer_tree_init(tgbm_trainer *t, int class_id) { t->impl->tree_init(class_id); }
void tgbm_trainer_find_split(tgbm_trainer *t, int level) { t->impl->find_split(level); }
void tgbm_trainer_partition(tgbm_trainer *t, int level) { t->impl->partition(level); }
void tgbm_trainer_finish_tree(tgbm_trainer *t, int class_id) { t->impl->finish_tree(class_id); }
float tgbm_trainer_metric(tgbm_trainer *t) { return t->impl->metric(); }
int tgbm_trainer_info(tgbm_trainer *t, const char *key) {
    if (std::strcmp(key, "n_labels") == 0) return (int)t->dataset.label.size();
    return t->impl->info(key);
}
float tgbm_trainer_base_score(tgbm_trainer *t) { return t->impl->param().base_score; }
size_t tgbm_trainer_get(tgbm_trainer *t, const char *name, void *out, size_t cap) {
    if (std::strcmp(name, "labels") == 0) {
        size_t bytes = t->dataset.label.size() * sizeof(float);
        if (out != nullptr && cap >= bytes) std::memcpy(out, t->dataset.label.data(), bytes);
        return bytes;
    }
    return t->impl->get(name, out, cap);
}
void tgbm_trainer_set(tgbm_trainer *t, const char *name, const void *in, size_t bytes) {
    t->impl->set(name, in, bytes);
}
void tgbm_trainer_set_profiling(tgbm_trainer *t, int on) { t->impl->set_profiling(on != 0); }
void tgbm_trainer_get_profile(tgbm_trainer *t, double *out4) {
    HistProfile p = t->impl->profile();
    out4[0] = p.hist_ms;
    out4[1] = (double)p.hist_launches;
    out4[2] = (double)p.rows_built;
    out4[3] = (double)p.hist_bytes;
}
int tgbm_trainer_get_phase_profile(tgbm_trainer *t, double *out, int cap) {
    HistProfile p = t->impl->profile();
    const double v[] = {(double)p.rounds,
                        p.phase_ms[PH_GRADIENT], p.phase_ms[PH_HIST], p.phase_ms[PH_MERGE], p.phase_ms[PH_SPLIT],
                        p.phase_ms[PH_PARTITION], p.phase_ms[PH_TREE_END], p.phase_ms[PH_METRIC], p.phase_ms[PH_REORDER],
                        p.root_ms, (double)p.root_launches, (double)p.root_bytes,
                        p.below_ms, (double)p.below_launches, (double)p.below_bytes};
    const int n = (int)(sizeof(v) / sizeof(v[0]));
    for (int i = 0; i < n && i < cap; ++i) out[i] = v[i];
    return n;
}
tgbm_model *tgbm_trainer_export_model(tgbm_trainer *t) { return from_nested(t->impl->model_to_host()); }

void tgbm_predict_raw(int row_size, const float *val, const int *row_ptr, const int *col_ptr, tgbm_model *model,
                      int n_trees, int trees_per_iter, float learning_rate, float base_score, float *out) {
    GBMParam p;
    p.learning_rate = learning_rate;
    p.base_score = base_score;
    DataSet ds;
    GBMParam load_param = p;
    int saved = g_verbose;
    g_verbose = 0;
    ds.load_from_sparse(row_size, val, row_ptr, col_ptr, nullptr, nullptr, 0, load_param, false);
    g_verbose = saved;
    std::vector<float> r = predict_raw(p, to_nested(model, n_trees, trees_per_iter), ds);
    std::memcpy(out, r.data(), r.size() * sizeof(float));
}

int tgbm_cut_points(int row_size, int n_features, const float *val, const int *row_ptr, const int *col_ptr,
                    int max_num_bin, float *cut_val, int *cut_row_ptr, int *cut_fid, int *bin_id) {
    const long nnz = row_ptr[row_size];
    hipStream_t s;
    HIP_CHECK(hipStreamCreate(&s));
    float *d_val = nullptr;
    int *d_col = nullptr, *d_bin = nullptr;
    HIP_CHECK(hipMalloc(&d_val, sizeof(float) * (size_t)std::max(nnz, 1l)));
    HIP_CHECK(hipMalloc(&d_col, sizeof(int) * (size_t)std::max(nnz, 1l)));
    if (nnz) {
        HIP_CHECK(hipMemcpyAsync(d_val, val, sizeof(float) * (size_t)nnz, hipMemcpyHostToDevice, s));
        HIP_CHECK(hipMemcpyAsync(d_col, col_ptr, sizeof(int) * (size_t)nnz, hipMemcpyHostToDevice, s));
    }
    DeviceCuts c = build_cut_points(s, n_features, nnz, d_val, d_col, max_num_bin);
    HIP_CHECK(hipMemcpyAsync(cut_row_ptr, c.cut_row_ptr, sizeof(int) * (size_t)(n_features + 1),
                             hipMemcpyDeviceToHost, s));
    if (c.n_bins) {
        HIP_CHECK(hipMemcpyAsync(cut_val, c.cut_val, sizeof(float) * (size_t)c.n_bins, hipMemcpyDeviceToHost, s));
        HIP_CHECK(hipMemcpyAsync(cut_fid, c.cut_fid, sizeof(int) * (size_t)c.n_bins, hipMemcpyDeviceToHost, s));
    }
    if (bin_id != nullptr && nnz) {
        HIP_CHECK(hipMalloc(&d_bin, sizeof(int) * (size_t)nnz));
        launch_bin_csr(s, nnz, d_col, d_val, c.cut_val, c.cut_row_ptr, d_bin);
        HIP_CHECK(hipMemcpyAsync(bin_id, d_bin, sizeof(int) * (size_t)nnz, hipMemcpyDeviceToHost, s));
    }
    HIP_CHECK(hipStreamSynchronize(s));
    HIP_CHECK(hipFree(d_val));
    HIP_CHECK(hipFree(d_col));
    if (d_bin) HIP_CHECK(hipFree(d_bin));
    HIP_CHECK(hipFree(c.cut_row_ptr));
    if (c.cut_val) HIP_CHECK(hipFree(c.cut_val));
    if (c.cut_fid) HIP_CHECK(hipFree(c.cut_fid));
    HIP_CHECK(hipStreamDestroy(s));
    return c.n_bins;
}

}  // extern "C"
