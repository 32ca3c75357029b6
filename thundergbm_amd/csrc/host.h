// Host-side pieces that mirror the reference's DataSet, Parser, TreeTrainer and Predictor.
#pragma once
#include <memory>
#include <string>
#include <vector>

#include "common.h"

namespace tgbm {

// Host CSR dataset (the reference's DataSet, include/thundergbm/dataset.h).
struct DataSet {
    // Owned CSR arrays (filled by load_from_file only).
    std::vector<float> csr_val;
    std::vector<int> csr_row_ptr;
    std::vector<int> csr_col_idx;
    // The CSR arrays the device code uploads: the caller's buffers after load_from_sparse (not copied; they
    // must stay valid while the trainer / predictor is being constructed), the owned vectors after
    // load_from_file.
    const float *val = nullptr;
    const int *row_ptr = nullptr;
    const int *col_idx = nullptr;
    long nnz = 0;
    std::vector<float> y;
    std::vector<float> label;  // distinct class labels, ascending
    std::vector<int> group;
    size_t n_features_ = 0;
    bool features_counted = true;  // false: load_from_sparse left the column scan to the device code

    size_t n_features() const { return n_features_; }
    size_t n_instances() const { return y.size(); }

    // src/thundergbm/dataset.cpp:20-63
    // count_features = false skips the scan of all column indices for the largest one (n_features() stays 0
    // and features_counted false): the trainer / predictor take the maximum on the device after the upload,
    // where the scan of a few hundred million indices costs a fraction of a millisecond instead of tens
    void load_from_sparse(int n_instances, const float *csr_val, const int *csr_row_ptr, const int *csr_col_idx,
                          const float *y, const int *group, int num_group, GBMParam &param,
                          bool count_features = true);
    // src/thundergbm/dataset.cpp:170-320 (LIBSVM text, 1-based feature ids)
    void load_from_file(const std::string &file_name, GBMParam &param);
    // src/thundergbm/dataset.cpp:83-101
    void group_label();
    // src/thundergbm/dataset.cpp:71-81 (sizes of the query groups, one number per token)
    void load_group_file(const std::string &file_name);
};

bool objective_needs_group_label(const std::string &objective);
bool objective_needs_groups(const std::string &objective);  // rank:pairwise, rank:ndcg
bool objective_supported(const std::string &objective);

// Parameter parsing and the raw binary model format (src/thundergbm/parser.cpp).
struct Parser {
    static void parse_param(GBMParam &param, int argc, char **argv);
    static void load_model(const std::string &path, GBMParam &param, std::vector<std::vector<Tree>> &model,
                           DataSet &dataset);
    static void save_model(const std::string &path, const GBMParam &param,
                           const std::vector<std::vector<Tree>> &model, const DataSet &dataset);
};

class Trainer;  // device trainer, trainer.hip

// src/thundergbm/trainer.cu:18-57
std::vector<std::vector<Tree>> train(GBMParam &param, const DataSet &dataset);

// src/thundergbm/predictor.cu:11-30 / :32-189. Returns class-major raw scores (predict_raw) or the
// transformed predictions (predict).
std::vector<float> predict_raw(const GBMParam &param, const std::vector<std::vector<Tree>> &model,
                               const DataSet &dataset);
std::vector<float> predict(const GBMParam &param, const std::vector<std::vector<Tree>> &model,
                           const DataSet &dataset, bool log_metric);

}  // namespace tgbm
