// Ranking objectives and metrics on the device: LambdaRank gradients (rank:pairwise, rank:ndcg) and
// the list metrics MAP and NDCG over query groups of consecutive rows.
#pragma once
#include <hip/hip_runtime.h>

#include <vector>

#include "device_api.h"

namespace tgbm {

enum RankMetric { RANK_METRIC_MAP = 3, RANK_METRIC_NDCG = 4 };

// Groups of at most this many rows are ordered by counting (every row counts the rows of its segment that go before
// it: one launch, quadratic in the segment length); data with a longer group takes the radix sort.
constexpr int kRankCountSortMax = 2048;
constexpr int kRankCountSortMean = 384;  // ... and only while sum(len^2) / rows stays below this

// One run of equal labels inside a query group, in the group's label-descending order. The run owns the
// positions [begin, end) of that order; [first_l, end) are the positions that draw a partner (the reference's
// loop over a group skips the first position of a run that follows a processed run,
// src/thundergbm/objective/ranking_obj.cpp:55-92), first_l == end for a run that draws nothing.
struct RankRun {
    int group_begin, group_end;  // positions of the whole group
    int first_l, end;
    int group;
    int begin;
};

class RankContext {
   public:
    // y: labels of all rows; group: sizes of the query groups (consecutive rows), their sum must be y.size()
    RankContext(hipStream_t s, const std::vector<float> &y, const std::vector<int> &group, bool ndcg);
    ~RankContext();
    RankContext(const RankContext &) = delete;
    RankContext &operator=(const RankContext &) = delete;

    // LambdaRank::get_gradient (ranking_obj.cpp:20-96): gh[row] = sum of the lambdas of the sampled pairs the
    // row takes part in. `seed` selects the round's partner draws.
    // order_is_fresh: d_score has not changed since the last metric() call, whose (group, score) order then
    // only needs a stable re-sort by run id
    void gradient(const float *d_score, GHPair *d_gh, unsigned seed, bool order_is_fresh = false);
    // RankListMetric::get_score with MAP or NDCG (metric/rank_metric.cpp:9-104); writes one float to d_out
    void metric(int kind, const float *d_score, float *d_out);
    // the row order and partner draws of the last gradient() call (tests): sorted rows [n]
    const int *last_sorted_rows() const { return sorter_.vals[last_cur_]; }
    int n() const { return n_; }

   private:
    template <typename T>
    T *dalloc(size_t count);
    hipStream_t stream_;
    int n_ = 0, n_groups_ = 0, n_runs_ = 0;
    bool ndcg_ = false;
    int run_bits_ = 0, group_bits_ = 0;
    int zero_hit_groups_ = 0;   // groups without a non-zero label: MAP = 1 by definition
    int ndcg_one_groups_ = 0;   // groups with IDCG == 0: NDCG = 1 by definition
    bool idcg_valid_ = false;   // all labels in 0..30
    std::vector<void *> allocs_;
    float *d_y_ = nullptr;
    int *d_static_row_ = nullptr;  // rows of every group by label descending (ties: row ascending)
    int *d_run_of_ = nullptr;      // run of a position of that order
    int *d_run_of_row_ = nullptr;  // run of a row
    RankRun *d_runs_ = nullptr;
    int *d_group_of_ = nullptr;    // group of a row
    int *d_gptr_ = nullptr;
    float *d_idcg_ = nullptr;
    int *d_group_hits_ = nullptr;  // rows with a non-zero label per group
    long long *d_acc_ = nullptr;   // [2n] fixed-point gradient / hessian sums
    unsigned *d_flags_ = nullptr, *d_hits_before_ = nullptr;
    double *d_partial_ = nullptr;
    int n_partial_ = 0;
    PairSorter sorter_;
    int last_cur_ = 0;
    bool have_metric_order_ = false;  // sorter_.vals[last_cur_] is the (group, score) order of a metric() call
    bool short_groups_ = false;       // groups short enough to be ordered by counting (kRankCountSortMax / Mean)
};

}  // namespace tgbm
