// Device trainer: owns every HBM buffer of a training session and drives the kernels.
#pragma once
#include <hip/hip_runtime.h>

#include <map>
#include <memory>
#include <string>
#include <vector>

#include "device_api.h"
#include "host.h"
#include "rank.h"

namespace tgbm {

// Stages of a boosting round that the profiling switch times with HIP events on the trainer's stream (the
// reference accumulates host timers for histogram, evaluation and data partitioning under its `profiling` switch,
// hist_tree_builder_single.cu:19-27, :196-219, :392, :400-418).
enum Phase {
    PH_GRADIENT = 0,  // gradients, column sampling, tree initialisation
    PH_HIST,          // histogram build of a level
    PH_MERGE,         // sum of the work items' histograms, sibling = parent - built, exact root sums
    PH_SPLIT,         // split search and tree update of a level
    PH_PARTITION,     // row -> child decision and the next level's row lists
    PH_TREE_END,      // pruning, prediction update (with metric and next gradients where fused), model copy
    PH_METRIC,        // training metric when it is a pass of its own
    PH_REORDER,       // physical re-ordering of the rows
    PH_COUNT
};

struct HistProfile {
    double hist_ms = 0;          // summed duration of the histogram-build launches
    long long hist_launches = 0;
    long long rows_built = 0;    // rows visited by those launches
    long long hist_bytes = 0;    // algorithmic bytes of those launches
    double phase_ms[PH_COUNT] = {0};
    // the histogram launches of the root level and of the levels below it
    double root_ms = 0, below_ms = 0;
    long long root_launches = 0, below_launches = 0, root_bytes = 0, below_bytes = 0;
    long long rounds = 0;
};

class Trainer {
   public:
    // Uploads the dataset, builds cut points and bin ids on the device and initialises the base
    // score (HistTreeBuilder_single::init + Booster::init of the reference).
    Trainer(const DataSet &dataset, GBMParam &param);
    ~Trainer();
    Trainer(const Trainer &) = delete;
    Trainer &operator=(const Trainer &) = delete;

    // One call = `rounds` iterations of Booster::boost: gradients, tree_per_rounds trees, metric.
    void boost(int rounds);
    // step-wise driving (used by parity tests)
    void sample_columns();  // column sampling of one boosting round (no-op for rate >= 1); boost() calls it
    // "column_sampling_rate", "bagging", "reorder_first", "reorder_burst", "reorder_every", "reorder_min_rows"
    void set_option(const std::string &key, double value);
    void compute_gradient();
    void tree_init(int k);
    void find_split(int level);  // histogram, merge/subtract, split search, update_tree
    void partition(int level);   // update_ins2node_id + next level's row lists
    // prune, prediction update, append the tree to the model; fuse_round_end also computes the metric and
    // the next round's gradients in the same pass (single-tree objectives inside boost())
    void finish_tree(int k, bool fuse_round_end = false);
    float metric();
    void sync();

    // results
    std::vector<std::vector<Tree>> model_to_host();
    std::vector<float> metric_log();
    const GBMParam &param() const { return param_; }
    int info(const std::string &key) const;
    size_t get(const std::string &name, void *out, size_t cap);  // returns bytes, copies if cap suffices
    void set(const std::string &name, const void *in, size_t bytes);
    void set_profiling(bool on);
    HistProfile profile();

   private:
    TreeBuffers set_of(int k) const;
    void find_split_sets(const TreeBuffers &tb, const GHPair *gh, int level, int n_class);
    void partition_sets(const TreeBuffers &tb, int level, int n_class);
    void build_level_hist(const TreeBuffers &tb, int level, const GHPair *gh, int n_class);
    void build_round_together();
    void log_plan(const TreeBuffers &tb);
    bool reorder_allowed() const;
    void reorder_rows();                 // physical re-ordering of the rows by the leaves of the tree just built
    const std::vector<int> &host_perm();  // original row of every physical position (empty: identity)
    void run_metric(float *slot);
    void alloc_tree_buffers();
    template <typename T>
    T *dalloc(size_t count);

    GBMParam param_;
    hipStream_t stream_ = nullptr;
    int n_ = 0, F_ = 0, n_bins_ = 0;
    long nnz_ = 0;
    int objective_ = OBJ_SQUARE, metric_kind_ = 0;
    // Dense layout with a spare dword at the end of every row's record, one tree per round, squared or binary logistic
    // loss: the rows' gradient pairs also travel as one word in that dword (DenseBins::gh_lane), written by whatever
    // computes the round's gradients (into an array of their own; the root level's histogram launch moves them).
    int gh_word_lane_ = -1;
    bool gh_words_fresh_ = false;   // d_gh_words_ matches d_gh_
    bool gh_records_fresh_ = false;  // and the root level's histogram launch of this tree has copied it into the records
    unsigned *d_gh_words_ = nullptr;  // [n]
    // Inside boost() the fused end of a round leaves the next gradients as words only when nothing of the next tree
    // reads the pair array (the histogram kernels take the words, the root's sums come from a complete feature's
    // bins, the tree's scales from the pass's own statistics); whoever wants the array then - the stage-wise API, a
    // getter - has it recomputed from the predictions first (the same kernel, the same values).
    bool gh_array_stale_ = false;
    void ensure_gh_array();
    std::vector<void *> allocs_;
    // dataset
    float *d_y_ = nullptr;
    float *d_yp_ = nullptr;
    long n_yp_ = 0;
    GHPair *d_gh_ = nullptr;
    DeviceCuts cuts_;
    std::vector<int> h_cut_row_ptr_;
    std::vector<int> h_col_bin_begin_;  // dense layout: first global bin of every column of the matrix (+ the bin count)
    std::vector<int> h_feat_col_;       // dense layout with bundles: column of every feature (else empty)
    uint8_t *d_binmat_ = nullptr;
    DenseBins bins_;
    bool sparse_ = false;
    CsrBins csr_;
    // sparse layout: one pass per level over the bin-major copy instead of per-node histograms (depth <= 11)
    bool sparse_pass_ = false;
    bool wide_bins_ = false;        // a feature has more than 255 cut points (max_num_bin above 255)
    bool wide_eval_ = false;        // split search with one workgroup per (feature, node)
    int hist_cap_level_ = -1;       // first level with more nodes than the histogram arena holds (-1: none)
    int sparse_bin0_owner_ = -2;    // -2: not looked up yet
    bool sparse_sorted_on_ = true;
    bool sparse_feature_in_tables(int f);
    SparsePass sp_;
    void build_sparse_tasks();
    void ensure_hist_arena();  // per-node histograms for stage-wise inspection (the level pass itself keeps none)
    TreeBuffers tb_;      // buffer set 0; set k = tb_.for_class(k)
    int n_sets_ = 1;      // tree_per_rounds when the class trees of a round are built together, else 1
    // model
    TreeNode *d_model_ = nullptr;
    int trees_built_ = 0, rounds_done_ = 0, model_cap_trees_ = 0;
    float *d_metric_ = nullptr;
    double *d_metric_scratch_ = nullptr;
    std::vector<uint8_t> h_ignored_;
    uint8_t *d_ignored_ = nullptr;
    int cur_class_ = 0;
    std::unique_ptr<RankContext> rank_;  // ranking objectives only
    // physical row order: position p holds original row d_perm_[p] (nullptr: the original order)
    int *d_perm_ = nullptr, *d_perm_alt_ = nullptr, *perm_spare_ = nullptr;
    uint8_t *d_binmat_alt_ = nullptr;
    float *d_y_alt_ = nullptr, *d_yp_alt_ = nullptr;
    PairSorter reorder_sorter_;
    std::vector<int> h_perm_;
    bool h_perm_valid_ = false;
    bool nid_materialized_ = false;  // tb_.nid already holds the finished tree's row -> node map (in physical order)
    // after trees 1, 2 and 3, then every 32 trees (first 0: never); see reorder_allowed()
    int reorder_first_ = 1, reorder_burst_ = 3, reorder_every_ = 32;
    long reorder_min_rows_ = 1l << 20;
    int reorders_done_ = 0;
    int *d_bag_count_ = nullptr;         // bagging: draws per gradient entry (zero between rounds)
    bool rank_order_fresh_ = false;      // d_yp_ unchanged since the last ranking metric pass
    bool in_boost_ = false;
    int lookup_level_ = -1;          // level whose split nodes have not been partitioned into row lists yet
    bool next_round_ready_ = false;  // d_gh_ and the root statistics already belong to the next round
    // profiling
    bool profiling_ = false;
    // a mark closes the stage that ran since the previous mark
    struct PhaseMark {
        hipEvent_t ev;
        int phase;  // -1: start of a timed span (nothing is attributed to the interval before it)
        int level;
    };
    std::vector<PhaseMark> marks_;
    long long prof_rounds_ = 0;
    void mark(int phase, int level = -1);
    std::vector<LevelCtl> ctl_log_;  // per tree, depth + 1 entries (copied at tree end when profiling)
    HistProfile prof_;
};

}  // namespace tgbm
