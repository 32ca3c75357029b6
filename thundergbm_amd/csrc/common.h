// Shared POD types, error handling and logging of the MI355X histogram GBDT library.
#pragma once
#include <cstdarg>
#include <cstddef>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <string>
#include <vector>

namespace tgbm {

// Gradient / hessian pair, same bytes as the reference's GHPair (include/thundergbm/common.h:43-80).
struct GHPair {
    float g, h;
};

// Model node. Byte-for-byte the reference's Tree::TreeNode (include/thundergbm/tree.h:14-30): it is
// written raw into model files and exposed through get_a_tree, so the layout is part of the ABI.
struct TreeNode {
    int final_id;
    int lch_index;
    int rch_index;
    int parent_index;
    float gain;
    float base_weight;
    int split_feature_id;
    float split_value;
    unsigned char split_bid;
    bool default_right;
    bool is_leaf;
    bool is_valid;
    bool is_pruned;
    GHPair sum_gh_pair;
};
static_assert(sizeof(TreeNode) == 48, "TreeNode layout is part of the model file format");
static_assert(offsetof(TreeNode, split_bid) == 32 && offsetof(TreeNode, sum_gh_pair) == 40, "TreeNode layout");

// Best split of one node (the content of the reference's SplitPoint, include/thundergbm/builder/shard.h:23-47).
struct SplitPoint {
    float gain;
    GHPair fea_missing_gh;
    GHPair lch_sum_gh;
    int default_right;
    int nid;
    int split_fea_id;
    float fval;
    int split_bid;
    int best_index;  // global bin index of the winning candidate
    int pad;
};
static_assert(sizeof(SplitPoint) == 48, "SplitPoint is read back by tests as 48-byte records");

// Training parameters (include/thundergbm/common.h:86-111).
struct GBMParam {
    int depth = 6;
    int n_trees = 40;
    float min_child_weight = 1;
    float lambda = 1;
    float gamma = 1;
    float rt_eps = 1e-6f;
    float column_sampling_rate = 1;
    std::string path = "../dataset/test_dataset.txt";
    int verbose = 1;
    bool profiling = false;
    bool bagging = false;
    int n_parallel_trees = 1;
    float learning_rate = 1;
    std::string objective = "reg:linear";
    int num_class = 1;
    int tree_per_rounds = 1;
    int max_num_bin = 255;
    float base_score = 0;
    int n_device = 1;
    std::string tree_method = "auto";
};

// A trained tree as the host sees it.
struct Tree {
    std::vector<TreeNode> nodes;
};

// ---- logging: verbose 0 = silent, 1 = info, 2 = debug (scikit_tgbm.cpp:13-23) -------------------
extern int g_verbose;
void log_info(const char *fmt, ...);
void log_debug(const char *fmt, ...);
[[noreturn]] void fatal(const char *fmt, ...);  // the reference aborts on any failed CHECK

}  // namespace tgbm

#define TGBM_CHECK(cond, ...)                    \
    do {                                         \
        if (!(cond)) ::tgbm::fatal(__VA_ARGS__); \
    } while (0)
