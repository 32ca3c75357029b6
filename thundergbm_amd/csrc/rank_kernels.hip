// LambdaRank gradients and the list metrics MAP / NDCG on the device.
//
// The reference computes these on the host, one query group per OpenMP iteration
// (src/thundergbm/objective/ranking_obj.cpp:20-96, src/thundergbm/metric/rank_metric.cpp:9-104). Here a
// round is a handful of data-parallel passes over all rows:
//   * labels never change, so the label-descending order of every group, its runs of equal labels and the
//     part of each run that draws partners are tables built once on the host;
//   * per round one stable radix sort of (run, descending score) keys orders the rows inside their runs,
//     which reproduces "sort by score, then stably by label";
//   * one thread per position draws its partner, evaluates the pair and adds the lambdas to both rows with
//     64-bit fixed-point atomics (exact integer sums: the result does not depend on the order of the adds).
// Two things differ from the reference by necessity, because there they are not reproducible: ties between
// equal scores keep the row order (std::sort leaves it unspecified), and the partner of a position is a
// pure function of (round seed, position) instead of a std::mt19937 stream seeded with std::rand() from
// whichever thread reaches the group first.
#include <algorithm>
#include <cmath>
#include <cstdlib>
#include <string>

#include "rank.h"

namespace tgbm {
namespace {

constexpr int kBlock = 256;

// Order-preserving map float -> uint32 (-0.0 folded into +0.0: they compare equal).
__device__ __forceinline__ unsigned float_key(float v) {
    if (v == 0.f) v = 0.f;
    unsigned u = __float_as_uint(v);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

// Partner draw of position `pos` in round `seed`: a 64-bit finaliser of the pair, scaled to [0, range).
__device__ __forceinline__ unsigned rank_draw(unsigned seed, unsigned pos, unsigned range) {
    unsigned long long x = ((unsigned long long)seed << 32) | pos;
    x += 0x9E3779B97F4A7C15ull;
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
    x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
    x ^= x >> 31;
    return (unsigned)(((x >> 32) * (unsigned long long)range) >> 32);
}

// NDCG::discounted_gain (include/thundergbm/metric/ranking_metric.h:43-45)
__device__ __forceinline__ float discounted_gain(int label, int rank) {
    return (float)((1 << label) - 1) / log2f((float)(rank + 2));
}

// bits of the fixed-point fraction for a group of `len` rows: a row collects at most len + 1 lambdas of
// magnitude <= 2, so sums stay below 2^62
__device__ __forceinline__ int acc_bits(int len) { return 59 - (32 - __clz(max(len, 1))); }

int grid_for(size_t n) {
    size_t b = (n + kBlock - 1) / kBlock;
    return (int)std::max<size_t>(1, b);
}

__global__ __launch_bounds__(kBlock) void k_rank_train_keys(int n, const int *__restrict__ static_row,
                                                           const int *__restrict__ run_of,
                                                           const float *__restrict__ score,
                                                           unsigned long long *__restrict__ keys, int *__restrict__ vals) {
    const int p = blockIdx.x * kBlock + threadIdx.x;
    if (p >= n) return;
    const int row = static_row[p];
    keys[p] = ((unsigned long long)(unsigned)run_of[p] << 32) | (unsigned)~float_key(score[row]);
    vals[p] = row;
}

// Keys for the short re-sort of rows that are already in (group, score) order: the run id alone.
__global__ __launch_bounds__(kBlock) void k_rank_run_keys(int n, const int *__restrict__ run_of_row,
                                                         const int *sorted_row, unsigned long long *__restrict__ keys,
                                                         int *vals) {
    const int p = blockIdx.x * kBlock + threadIdx.x;
    if (p >= n) return;
    const int row = sorted_row[p];  // may alias vals: every thread reads and writes its own element
    keys[p] = (unsigned long long)(unsigned)run_of_row[row];
    vals[p] = row;
}

__global__ __launch_bounds__(kBlock) void k_rank_metric_keys(int n, const int *__restrict__ group_of,
                                                            const float *__restrict__ score,
                                                            unsigned long long *__restrict__ keys, int *__restrict__ vals) {
    const int row = blockIdx.x * kBlock + threadIdx.x;
    if (row >= n) return;
    keys[row] = ((unsigned long long)(unsigned)group_of[row] << 32) | (unsigned)~float_key(score[row]);
    vals[row] = row;
}

// Stable order by descending score inside every segment through counting: the place of an element is the number of
// elements of its segment with a smaller key (the radix sort's key: ~float_key(score)) or with the same key and an
// earlier position - the order the stable radix sort of (segment, key) pairs gives, in one launch. Segments are short
// (kRankCountSortMax at most) and the threads of a wavefront mostly walk the same one, so the loads of the walk are
// shared. RUNS: segments are the runs of equal labels in the label-descending order (positions -> rows through
// static_row); otherwise the query groups in row order.
// (the keys of all elements in segment order first, so that the walk loads them from consecutive addresses)
__global__ __launch_bounds__(kBlock) void k_rank_sort_keys(int n, const float *__restrict__ score,
                                                          const int *__restrict__ static_row, unsigned *__restrict__ key) {
    const int p = blockIdx.x * kBlock + threadIdx.x;
    if (p < n) key[p] = ~float_key(score[static_row != nullptr ? static_row[p] : p]);
}

template <bool RUNS>
__global__ __launch_bounds__(kBlock) void k_rank_count_sort(int n, const unsigned *__restrict__ keys,
                                                           const int *__restrict__ static_row,
                                                           const int *__restrict__ run_of,
                                                           const RankRun *__restrict__ runs,
                                                           const int *__restrict__ group_of,
                                                           const int *__restrict__ gptr, int *__restrict__ sorted) {
    const int p = blockIdx.x * kBlock + threadIdx.x;
    if (p >= n) return;
    int sb, se;
    if (RUNS) {
        const RankRun r = runs[run_of[p]];
        sb = r.begin;
        se = r.end;
    } else {
        const int g = group_of[p];
        sb = gptr[g];
        se = gptr[g + 1];
    }
    const unsigned key = keys[p];
    int before = 0;
    constexpr int kAhead = 8;
    for (int j0 = sb; j0 < se; j0 += kAhead) {
        unsigned kj[kAhead];
#pragma unroll
        for (int u = 0; u < kAhead; ++u) kj[u] = keys[min(j0 + u, se - 1)];
#pragma unroll
        for (int u = 0; u < kAhead; ++u) {
            const int j = j0 + u;
            before += (j < se && (kj[u] < key || (kj[u] == key && j < p))) ? 1 : 0;
        }
    }
    sorted[sb + before] = RUNS ? static_row[p] : p;
}

// One thread per position of the (label descending, score descending) order of its group; the body is the
// inner loop of LambdaRank::get_gradient (ranking_obj.cpp:63-90) for l = that position.
__global__ __launch_bounds__(kBlock) void k_rank_pairs(int n, const RankRun *__restrict__ runs,
                                                      const int *__restrict__ run_of, const int *__restrict__ sorted_row,
                                                      const float *__restrict__ score, const float *__restrict__ y,
                                                      const float *__restrict__ idcg, unsigned seed,
                                                      unsigned long long *__restrict__ acc) {
    const int p = blockIdx.x * kBlock + threadIdx.x;
    if (p >= n) return;
    const RankRun r = runs[run_of[p]];
    if (p < r.first_l) return;
    const int nleft = r.first_l - r.group_begin;
    const int nright = r.group_end - r.end;
    if (nleft + nright == 0) return;
    const int m = (int)rank_draw(seed, (unsigned)p, (unsigned)(nleft + nright));
    const int l = p - r.group_begin;
    int high, low;  // positions inside the group; `high` is the one nearer the top of the label order
    if (m < nleft) {
        high = m;
        low = l;
    } else {
        high = l;
        low = m - nleft + (r.end - r.group_begin);
    }
    const int high_row = sorted_row[r.group_begin + high];
    const int low_row = sorted_row[r.group_begin + low];
    float dz = 1.f;  // LambdaRank::get_delta_z
    if (idcg != nullptr) {  // LambdaRankNDCG::get_delta_z (ranking_obj.cpp:105-113)
        const float z = idcg[r.group];
        if (z == 0.f) {
            dz = 0.f;
        } else {
            const int li = (int)y[high_row], lj = (int)y[low_row];
            dz = (discounted_gain(li, high) + discounted_gain(lj, low) - discounted_gain(li, low) -
                  discounted_gain(lj, high)) / z;
        }
    }
    const float adz = fabsf(dz);
    const float rho = 1.f / (1.f + expf(score[high_row] - score[low_row]));
    const float lambda = -adz * rho;
    const float hess = 2.f * fmaxf(adz * rho * (1.f - rho), 1e-16f);
    const int sb = acc_bits(r.group_end - r.group_begin);
    const long long ql = __double2ll_rn(ldexp((double)lambda, sb));
    const unsigned long long qh = (unsigned long long)__double2ll_rn(ldexp((double)hess, sb));
    atomicAdd(acc + 2 * (size_t)high_row, (unsigned long long)ql);
    atomicAdd(acc + 2 * (size_t)high_row + 1, qh);
    atomicAdd(acc + 2 * (size_t)low_row, (unsigned long long)(-ql));
    atomicAdd(acc + 2 * (size_t)low_row + 1, qh);
}

// fixed point -> GHPair, and the accumulators are cleared for the next round
__global__ __launch_bounds__(kBlock) void k_rank_finish(int n, const int *__restrict__ group_of,
                                                       const int *__restrict__ gptr, long long *__restrict__ acc,
                                                       GHPair *__restrict__ gh) {
    const int row = blockIdx.x * kBlock + threadIdx.x;
    if (row >= n) return;
    const int g = group_of[row];
    const int sb = acc_bits(gptr[g + 1] - gptr[g]);
    const long long ag = acc[2 * (size_t)row], ah = acc[2 * (size_t)row + 1];
    acc[2 * (size_t)row] = 0;
    acc[2 * (size_t)row + 1] = 0;
    gh[row] = GHPair{(float)ldexp((double)ag, -sb), (float)ldexp((double)ah, -sb)};
}

// Sum of a block's per-thread doubles in thread order (the same bits on every run).
__device__ __forceinline__ void store_block_sum(double v, double *__restrict__ out) {
    __shared__ double s[kBlock];
    s[threadIdx.x] = v;
    __syncthreads();
    for (int w = kBlock / 2; w > 0; w >>= 1) {
        if ((int)threadIdx.x < w) s[threadIdx.x] += s[threadIdx.x + w];
        __syncthreads();
    }
    if (threadIdx.x == 0) out[blockIdx.x] = s[0];
}

// NDCG::eval_query_group (rank_metric.cpp:81-104): position p of the score order adds gain / IDCG of its group.
__global__ __launch_bounds__(kBlock) void k_rank_ndcg_partial(int n, const int *__restrict__ sorted_row,
                                                             const int *__restrict__ group_of,
                                                             const int *__restrict__ gptr, const float *__restrict__ y,
                                                             const float *__restrict__ idcg,
                                                             double *__restrict__ partial) {
    const int p = blockIdx.x * kBlock + threadIdx.x;
    double c = 0;
    if (p < n) {
        const int g = group_of[p];  // groups are runs of consecutive rows, so position p lies in row p's group
        const float z = idcg[g];
        if (z != 0.f) c = (double)discounted_gain((int)y[sorted_row[p]], p - gptr[g]) / (double)z;
    }
    store_block_sum(c, partial);
}

__global__ __launch_bounds__(kBlock) void k_rank_hit_flags(int n, const int *__restrict__ sorted_row,
                                                          const float *__restrict__ y, unsigned *__restrict__ flags) {
    const int p = blockIdx.x * kBlock + threadIdx.x;
    if (p < n) flags[p] = y[sorted_row[p]] != 0.f ? 1u : 0u;
}

// MAP::eval_query_group (rank_metric.cpp:47-72): a hit at rank i adds (hits so far) / (i + 1) / (hits of the group).
__global__ __launch_bounds__(kBlock) void k_rank_map_partial(int n, const unsigned *__restrict__ flags,
                                                            const unsigned *__restrict__ hits_before,
                                                            const int *__restrict__ group_of,
                                                            const int *__restrict__ gptr,
                                                            const int *__restrict__ group_hits,
                                                            double *__restrict__ partial) {
    const int p = blockIdx.x * kBlock + threadIdx.x;
    double c = 0;
    if (p < n && flags[p] != 0u) {
        const int g = group_of[p];
        const int b = gptr[g];
        const unsigned nh = hits_before[p] - hits_before[b] + 1u;
        c = (double)nh / (double)(p - b + 1) / (double)group_hits[g];
    }
    store_block_sum(c, partial);
}

// (sum of the partials + groups that score 1 by definition) / number of groups; one workgroup, fixed order
__global__ __launch_bounds__(kBlock) void k_rank_metric_final(const double *__restrict__ partial, int n_partial,
                                                             double constant, int n_groups, float *__restrict__ out) {
    __shared__ double s[kBlock];
    double v = 0;
    for (int i = threadIdx.x; i < n_partial; i += kBlock) v += partial[i];
    s[threadIdx.x] = v;
    __syncthreads();
    for (int w = kBlock / 2; w > 0; w >>= 1) {
        if ((int)threadIdx.x < w) s[threadIdx.x] += s[threadIdx.x + w];
        __syncthreads();
    }
    if (threadIdx.x == 0) *out = (float)((s[0] + constant) / (double)n_groups);
}

int bits_for(long count) {
    int b = 0;
    while ((1l << b) < count) ++b;
    return b;
}

}  // namespace

template <typename T>
T *RankContext::dalloc(size_t count) {
    void *p = nullptr;
    HIP_CHECK(hipMalloc(&p, sizeof(T) * std::max<size_t>(count, 1)));
    allocs_.push_back(p);
    return static_cast<T *>(p);
}

RankContext::RankContext(hipStream_t s, const std::vector<float> &y, const std::vector<int> &group, bool ndcg)
    : stream_(s), ndcg_(ndcg) {
    n_ = (int)y.size();
    n_groups_ = (int)group.size();
    TGBM_CHECK(n_groups_ > 0, "ranking needs query groups (a .group file or the group argument)");
    std::vector<int> gptr(n_groups_ + 1, 0);  // RankListMetric::configure_gptr (rank_metric.cpp:39-44)
    for (int g = 0; g < n_groups_; ++g) {
        TGBM_CHECK(group[g] >= 0, "negative size of query group %d", g);
        TGBM_CHECK((long)gptr[g] + group[g] <= (long)n_, "query groups cover more than the %d instances", n_);
        gptr[g + 1] = gptr[g] + group[g];
    }
    TGBM_CHECK(gptr.back() == n_, "query groups cover %d instances, the dataset has %d", gptr.back(), n_);

    bool labels_ok = true;  // NDCG takes labels as small non-negative integers (1 << label)
    for (float v : y) labels_ok = labels_ok && v >= 0.f && v < 31.f;
    TGBM_CHECK(!ndcg || labels_ok, "rank:ndcg needs labels in 0..30");

    std::vector<int> static_row(n_), run_of(n_), run_of_row(n_), group_of(n_), hits(n_groups_, 0);
    std::vector<RankRun> runs;
    std::vector<float> idcg(n_groups_, 0.f);
    int ndcg_one = 0;  // groups whose NDCG is 1 by definition (IDCG == 0)
    for (int g = 0; g < n_groups_; ++g) {
        const int b = gptr[g], e = gptr[g + 1];
        for (int i = b; i < e; ++i) {
            static_row[i] = i;
            group_of[i] = g;
            if (y[i] != 0.f) ++hits[g];
        }
        std::stable_sort(static_row.begin() + b, static_row.begin() + e,
                         [&](int a, int c) { return y[a] > y[c]; });
        if (labels_ok) {  // NDCG::get_IDCG (rank_metric.cpp:106-123): float sum in descending label order
            float z = 0.f;
            for (int i = b; i < e; ++i)
                z += (float)((1 << (int)y[static_row[i]]) - 1) / log2f((float)(i - b + 2));
            idcg[g] = z;
        }
        if (idcg[g] == 0.f) ++ndcg_one;
        if (hits[g] == 0) ++zero_hit_groups_;
        bool skip_first = false;
        for (int i = b; i < e;) {
            int j = i + 1;
            while (j < e && y[static_row[j]] == y[static_row[i]]) ++j;
            RankRun r;
            r.group_begin = b;
            r.group_end = e;
            r.end = j;
            r.first_l = std::min(j, i + (skip_first ? 1 : 0));
            r.group = g;
            r.begin = i;
            skip_first = r.first_l < j;  // a processed run makes the loop step over the next run's first position
            for (int k = i; k < j; ++k) {
                run_of[k] = (int)runs.size();
                run_of_row[static_row[k]] = (int)runs.size();
            }
            runs.push_back(r);
            i = j;
        }
    }
    ndcg_one_groups_ = ndcg_one;
    idcg_valid_ = labels_ok;
    n_runs_ = (int)runs.size();
    // ordering by counting costs sum(len^2) steps (measured: 50 us for a million rows in groups of 120, where the radix
    // sort takes 220 us): taken while the average row sits in a group of at most kRankCountSortMean rows
    int longest = 0;
    double steps = 0;
    for (int g : group) {
        longest = std::max(longest, g);
        steps += (double)g * (double)g;
    }
    const char *sort_env = std::getenv("TGBM_RANK_SORT");  // "radix": the radix sort whatever the group sizes (tests)
    short_groups_ = longest <= kRankCountSortMax && steps <= (double)kRankCountSortMean * (double)std::max(n_, 1) &&
                    !(sort_env != nullptr && std::string(sort_env) == "radix");
    run_bits_ = bits_for(n_runs_);
    group_bits_ = bits_for(n_groups_);

    d_y_ = dalloc<float>(n_);
    d_static_row_ = dalloc<int>(n_);
    d_run_of_ = dalloc<int>(n_);
    d_run_of_row_ = dalloc<int>(n_);
    d_group_of_ = dalloc<int>(n_);
    d_runs_ = dalloc<RankRun>(runs.size());
    d_gptr_ = dalloc<int>(gptr.size());
    d_idcg_ = dalloc<float>(n_groups_);
    d_group_hits_ = dalloc<int>(n_groups_);
    d_acc_ = dalloc<long long>(2 * (size_t)n_);
    d_flags_ = dalloc<unsigned>(n_);
    d_hits_before_ = dalloc<unsigned>((size_t)n_ + 1);
    n_partial_ = grid_for(n_);
    d_partial_ = dalloc<double>(n_partial_);
    auto up = [&](void *dst, const void *src, size_t bytes) {
        if (bytes) HIP_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, stream_));
    };
    up(d_y_, y.data(), sizeof(float) * (size_t)n_);
    up(d_static_row_, static_row.data(), sizeof(int) * (size_t)n_);
    up(d_run_of_, run_of.data(), sizeof(int) * (size_t)n_);
    up(d_run_of_row_, run_of_row.data(), sizeof(int) * (size_t)n_);
    up(d_group_of_, group_of.data(), sizeof(int) * (size_t)n_);
    up(d_runs_, runs.data(), sizeof(RankRun) * runs.size());
    up(d_gptr_, gptr.data(), sizeof(int) * gptr.size());
    up(d_idcg_, idcg.data(), sizeof(float) * (size_t)n_groups_);
    up(d_group_hits_, hits.data(), sizeof(int) * (size_t)n_groups_);
    HIP_CHECK(hipMemsetAsync(d_acc_, 0, sizeof(long long) * 2 * (size_t)std::max(n_, 1), stream_));
    sorter_.alloc(n_);
    HIP_CHECK(hipStreamSynchronize(stream_));  // the host vectors go out of scope
}

RankContext::~RankContext() {
    sorter_.release();
    for (void *p : allocs_) (void)hipFree(p);
}

void RankContext::gradient(const float *d_score, GHPair *d_gh, unsigned seed, bool order_is_fresh) {
    if (n_ == 0) return;
    const int grid = grid_for(n_);
    if (short_groups_) {
        last_cur_ = 0;
        unsigned *keys = reinterpret_cast<unsigned *>(sorter_.keys[0]);
        k_rank_sort_keys<<<grid, kBlock, 0, stream_>>>(n_, d_score, d_static_row_, keys);
        k_rank_count_sort<true><<<grid, kBlock, 0, stream_>>>(n_, keys, d_static_row_, d_run_of_, d_runs_, nullptr, nullptr,
                                                             sorter_.vals[0]);
    } else if (order_is_fresh && have_metric_order_) {
        // rows already ordered by (group, score descending, row): a stable sort by run id yields
        // (run, score descending, row), the same order as the full sort below
        k_rank_run_keys<<<grid, kBlock, 0, stream_>>>(n_, d_run_of_row_, sorter_.vals[last_cur_], sorter_.keys[0],
                                                     sorter_.vals[0]);
        last_cur_ = sort_pairs(stream_, sorter_, n_, run_bits_);
    } else {
        k_rank_train_keys<<<grid, kBlock, 0, stream_>>>(n_, d_static_row_, d_run_of_, d_score, sorter_.keys[0],
                                                       sorter_.vals[0]);
        last_cur_ = sort_pairs(stream_, sorter_, n_, 32 + run_bits_);
    }
    have_metric_order_ = false;
    k_rank_pairs<<<grid, kBlock, 0, stream_>>>(n_, d_runs_, d_run_of_, sorter_.vals[last_cur_], d_score, d_y_,
                                              ndcg_ ? d_idcg_ : nullptr, seed,
                                              reinterpret_cast<unsigned long long *>(d_acc_));
    k_rank_finish<<<grid, kBlock, 0, stream_>>>(n_, d_group_of_, d_gptr_, d_acc_, d_gh);
}

void RankContext::metric(int kind, const float *d_score, float *d_out) {
    TGBM_CHECK(kind == RANK_METRIC_MAP || kind == RANK_METRIC_NDCG, "unknown ranking metric %d", kind);
    const int grid = grid_for(n_);
    int cur = 0;
    if (short_groups_) {
        unsigned *keys = reinterpret_cast<unsigned *>(sorter_.keys[0]);
        k_rank_sort_keys<<<grid, kBlock, 0, stream_>>>(n_, d_score, nullptr, keys);
        k_rank_count_sort<false><<<grid, kBlock, 0, stream_>>>(n_, keys, nullptr, nullptr, nullptr, d_group_of_, d_gptr_,
                                                              sorter_.vals[0]);
    } else {
        k_rank_metric_keys<<<grid, kBlock, 0, stream_>>>(n_, d_group_of_, d_score, sorter_.keys[0], sorter_.vals[0]);
        cur = sort_pairs(stream_, sorter_, n_, 32 + group_bits_);
    }
    const int *sorted = sorter_.vals[cur];
    double constant;
    if (kind == RANK_METRIC_NDCG) {
        TGBM_CHECK(idcg_valid_, "NDCG needs labels in 0..30");
        k_rank_ndcg_partial<<<grid, kBlock, 0, stream_>>>(n_, sorted, d_group_of_, d_gptr_, d_y_, d_idcg_, d_partial_);
        constant = ndcg_one_groups_;
    } else {
        k_rank_hit_flags<<<grid, kBlock, 0, stream_>>>(n_, sorted, d_y_, d_flags_);
        device_exclusive_scan(stream_, d_flags_, d_hits_before_, n_, sorter_.d_total, sorter_.scan);
        k_rank_map_partial<<<grid, kBlock, 0, stream_>>>(n_, d_flags_, d_hits_before_, d_group_of_, d_gptr_,
                                                        d_group_hits_, d_partial_);
        constant = zero_hit_groups_;
    }
    k_rank_metric_final<<<1, kBlock, 0, stream_>>>(d_partial_, n_partial_, constant, n_groups_, d_out);
    last_cur_ = cur;
    have_metric_order_ = true;
}

}  // namespace tgbm
