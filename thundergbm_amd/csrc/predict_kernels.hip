// Tree-traversal prediction (the reference's Predictor::predict_raw, src/thundergbm/predictor.cu:32-189)
// and the objectives' predict_transform.
#include "device_api.h"

namespace tgbm {
namespace {

constexpr int kBlock = 256;

// Value of feature `f` in a CSR row with ascending column indices; `missing` when not stored.
__device__ __forceinline__ float row_value(const int *__restrict__ ci, const float *__restrict__ cv, int len, int f,
                                           bool *missing) {
    int lo = 0, hi = len;
    while (lo < hi) {
        int mid = lo + (hi - lo) / 2;
        int c = ci[mid];
        if (c == f) {
            *missing = false;
            return cv[mid];
        }
        if (c > f)
            hi = mid;
        else
            lo = mid + 1;
    }
    *missing = true;
    return 0.f;
}

// One thread per row; the model (all trees, 48-byte nodes) is read through the caches. ACC is
// double where the reference takes its shared-memory path (n_features * 128 * 4 <= 48 KB, :85) and
// float otherwise (:166); in the double path a stored +inf counts as missing (:96-118).
template <typename ACC, bool INF_IS_MISSING>
__global__ __launch_bounds__(kBlock) void k_predict(int n, const int *__restrict__ row_ptr, const int *__restrict__ col,
                                                   const float *__restrict__ val, const TreeNode *__restrict__ model,
                                                   int n_iter, int n_class_trees, int n_nodes, float lr,
                                                   float base_score, float *__restrict__ out, size_t out_stride) {
    const int i = blockIdx.x * kBlock + threadIdx.x;
    if (i >= n) return;
    const int rb = row_ptr[i];
    const int len = row_ptr[i + 1] - rb;
    const int *ci = col + rb;
    const float *cv = val + rb;
    for (int t = 0; t < n_class_trees; ++t) {
        ACC sum = base_score;
        for (int it = 0; it < n_iter; ++it) {
            const TreeNode *nd = model + ((size_t)it * n_class_trees + t) * n_nodes;
            int cur = 0;
            while (!nd[cur].is_leaf) {
                const TreeNode &c = nd[cur];
                bool missing;
                float v = row_value(ci, cv, len, c.split_feature_id, &missing);
                if (INF_IS_MISSING && !(v < INFINITY)) missing = true;
                if (!missing)
                    cur = v < c.split_value ? c.lch_index : c.rch_index;
                else
                    cur = c.default_right ? c.rch_index : c.lch_index;
            }
            sum += lr * nd[cur].base_weight;
        }
        out[(size_t)t * out_stride + i] += (float)sum;
    }
}

// The reference's shared-memory path (predictor.cu:85-160): every thread first spreads its row into a dense
// vector of F floats (+inf = not stored, which is why a stored +inf counts as missing there), then walks
// all trees with one LDS read per node instead of a binary search of the CSR row. Feature-major LDS layout
// (f * kStageBlock + thread) keeps the reads of a wavefront on distinct banks. Sums are double as in the
// reference's path.
constexpr int kStageBlock = 128;

__global__ __launch_bounds__(kStageBlock) void k_predict_staged(int n, int F, const int *__restrict__ row_ptr,
                                                               const int *__restrict__ col,
                                                               const float *__restrict__ val,
                                                               const TreeNode *__restrict__ model, int n_iter,
                                                               int n_class_trees, int n_nodes, float lr,
                                                               float base_score, float *__restrict__ out,
                                                               size_t out_stride) {
    extern __shared__ float dense[];  // [F][kStageBlock]
    const int i = blockIdx.x * kStageBlock + threadIdx.x;
    for (int f = 0; f < F; ++f) dense[f * kStageBlock + threadIdx.x] = INFINITY;
    if (i >= n) return;  // no barrier below: a thread only reads what it wrote
    const int rb = row_ptr[i], re = row_ptr[i + 1];
    for (int e = rb; e < re; ++e) {
        const int c = col[e];
        if (c < F) dense[c * kStageBlock + threadIdx.x] = val[e];
    }
    for (int t = 0; t < n_class_trees; ++t) {
        double sum = base_score;
        for (int it = 0; it < n_iter; ++it) {
            const TreeNode *nd = model + ((size_t)it * n_class_trees + t) * n_nodes;
            int cur = 0;
            while (!nd[cur].is_leaf) {
                const TreeNode &c = nd[cur];
                const int f = c.split_feature_id;
                const float v = f < F ? dense[f * kStageBlock + threadIdx.x] : INFINITY;
                if (v < INFINITY)
                    cur = v < c.split_value ? c.lch_index : c.rch_index;
                else
                    cur = c.default_right ? c.rch_index : c.lch_index;
            }
            sum += lr * nd[cur].base_weight;
        }
        out[(size_t)t * out_stride + i] += (float)sum;
    }
}

// The same walk with the trees in LDS: the workgroup's rows are spread into the dense vector as above, then the trees
// of a class are staged a few at a time as 16-byte records (one LDS read per node visit instead of several cached
// global reads of the 48-byte node) and every thread walks the staged trees. Same operations in the same order as
// k_predict_staged, hence the same bits. A walk is cut off after n_nodes steps (a malformed model file).
__global__ void k_pack_model(const TreeNode *__restrict__ model, long n_total, int n_nodes, PackedNode *__restrict__ packed) {
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n_total; i += (long)gridDim.x * blockDim.x) {
        const TreeNode nd = model[i];
        PackedNode p;
        p.split_value = nd.split_value;
        p.base_weight = nd.base_weight;
        const bool children_ok = nd.lch_index >= 0 && nd.lch_index < n_nodes && nd.rch_index >= 0 && nd.rch_index < n_nodes;
        const bool leaf = nd.is_leaf || !children_ok;  // (an index outside the tree ends the walk instead of leaving it)
        p.children = leaf ? 0u : ((unsigned)nd.lch_index | (unsigned)nd.rch_index << 16);
        const unsigned f = (nd.split_feature_id >= 0 && nd.split_feature_id < 0xffffff) ? (unsigned)nd.split_feature_id : 0xffffffu;
        p.meta = f | (nd.default_right ? 1u << 30 : 0u) | (leaf ? 1u << 31 : 0u);
        packed[i] = p;
    }
}

template <int B>
__global__ __launch_bounds__(B) void k_predict_lds(int n, int F, const int *__restrict__ row_ptr,
                                                   const int *__restrict__ col, const float *__restrict__ val,
                                                   const PackedNode *__restrict__ packed, int n_iter, int n_class_trees,
                                                   int n_nodes, float lr, float base_score, float *__restrict__ out,
                                                   size_t out_stride, int trees_per_stage) {
    extern __shared__ float smem[];
    float *dense = smem;                                       // [F][B]
    uint4 *nodes = reinterpret_cast<uint4 *>(smem + F * B);    // [trees_per_stage][n_nodes]
    const int i = blockIdx.x * B + threadIdx.x;
    const bool live = i < n;
    for (int f = 0; f < F; ++f) dense[f * B + threadIdx.x] = INFINITY;
    if (live) {
        const int rb = row_ptr[i], re = row_ptr[i + 1];
        for (int e = rb; e < re; ++e) {
            const int c = col[e];
            if (c < F) dense[c * B + threadIdx.x] = val[e];
        }
    }
    const uint4 *__restrict__ src = reinterpret_cast<const uint4 *>(packed);
    for (int t = 0; t < n_class_trees; ++t) {
        double sum = base_score;
        for (int it0 = 0; it0 < n_iter; it0 += trees_per_stage) {
            const int staged = min(trees_per_stage, n_iter - it0);
            __syncthreads();  // the walks of the previous stage are done
            for (int idx = threadIdx.x; idx < staged * n_nodes; idx += B) {
                const int k = idx / n_nodes, j = idx - k * n_nodes;
                nodes[idx] = src[((size_t)(it0 + k) * n_class_trees + t) * n_nodes + j];
            }
            __syncthreads();
            if (!live) continue;
            for (int k = 0; k < staged; ++k) {
                const uint4 *tree = nodes + k * n_nodes;
                int cur = 0;
                uint4 nd = tree[0];
                for (int step = 0; step < n_nodes && !(nd.w >> 31); ++step) {
                    const unsigned f = nd.w & 0xffffffu;
                    const float v = f < (unsigned)F ? dense[f * B + threadIdx.x] : INFINITY;
                    const unsigned l = nd.z & 0xffffu, r = nd.z >> 16;
                    if (v < INFINITY)
                        cur = v < __uint_as_float(nd.x) ? l : r;
                    else
                        cur = ((nd.w >> 30) & 1u) ? r : l;
                    nd = tree[cur];
                }
                sum += lr * __uint_as_float(nd.y);
            }
        }
        if (live) out[(size_t)t * out_stride + i] += (float)sum;
    }
}

// ---- the walk on order-preserving integer keys
// A float that is not a NaN maps to an unsigned key with the floats' order (-0 counts as +0): `v < t` is
// `key(v) < key(t)`. In a row's dense vector a value that is missing - not stored, or stored as +inf or NaN, which the
// reference's shared-memory path takes for missing (predictor.cu:96-118) - is the largest key, 0xffffffff; nothing else
// maps there. A split node whose default direction is left adds one to the value's key before it compares (the missing
// key wraps to 0 and goes left; every other key keeps its order, as does the node's threshold key, which has the one
// added when the record is packed), so the default direction costs no comparison of its own.
__device__ __forceinline__ unsigned order_key(float v) {
    if (v == 0.f) v = 0.f;  // -0 -> +0
    const unsigned b = __float_as_uint(v);
    return b ^ ((unsigned)((int)b >> 31) | 0x80000000u);
}
constexpr unsigned kMissingKey = 0xffffffffu;
__device__ __forceinline__ unsigned value_key(float v) { return v < INFINITY ? order_key(v) : kMissingKey; }

// Eight-byte records for models whose trees keep the two children of a node side by side and below it (every tree the
// trainer builds, and the reference's: heap order), walked by k_predict_compact:
//   x: a split: key(threshold) + (default left ? 1 : 0) - 1, so that "goes right" is `value key + that one > x`;
//      a leaf: the bits of its weight
//   y: dword offset of the split feature's keys in the workgroup's dense vectors (15 bits; a feature the data does not
//      have: that of the all-missing feature F; a leaf: that of the all-zero feature F + 1, whose key never exceeds x)
//      | byte offset of the left child in the tree << 15 (16 bits; a leaf: of the leaf itself)
//      | default left << 31 (a leaf: 0)
// A leaf therefore walks to itself, and a walk of `depth` steps needs no test for the end.
// Half the LDS bytes per node visit of the 16-byte record. B: rows per workgroup of the kernel that reads the records.
__global__ void k_pack_compact(const TreeNode *__restrict__ model, int n_iter, int n_class_trees, int n_nodes, int F,
                               int B, uint2 *__restrict__ packed) {
    const long n_total = (long)n_iter * n_class_trees * n_nodes;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n_total; i += (long)gridDim.x * blockDim.x) {
        const TreeNode nd = model[i];
        const bool children_ok = nd.lch_index >= 0 && nd.lch_index < n_nodes && nd.rch_index >= 0 && nd.rch_index < n_nodes;
        const bool leaf = nd.is_leaf || !children_ok;
        const unsigned f = (nd.split_feature_id >= 0 && nd.split_feature_id < F) ? (unsigned)nd.split_feature_id : (unsigned)F;
        const long tree = i / n_nodes;
        const int self = (int)(i - tree * n_nodes);
        uint2 p;
        if (leaf) {
            p.x = __float_as_uint(nd.base_weight);
            p.y = (unsigned)(F + 1) * (unsigned)B | (unsigned)self * 8u << 15;
        } else {
            const unsigned left = nd.default_right ? 0u : 1u;
            p.x = order_key(nd.split_value) + left - 1u;
            p.y = f * (unsigned)B | (unsigned)nd.lch_index * 8u << 15 | left << 31;
        }
        // the model is stored round by round; the records class by class, so that the trees a workgroup stages
        // together (consecutive rounds of one class) are one contiguous run
        const long it = tree / n_class_trees, t = tree - it * n_class_trees;
        packed[(t * n_iter + it) * n_nodes + self] = p;
    }
}

// k_predict_lds with the eight-byte records, ILP trees walked at a time by every thread and `depth` steps for every tree:
// the walks of different trees do not depend on each other, so their LDS round trips (node, feature key, node, ...)
// overlap; a walk that has reached its leaf stays there until the deepest possible walk is done (straight-line
// code: eight vector instructions and two LDS reads per step). The leaf weights are added in the order of the
// trees, as in the other kernels: same bits.
// Rows of equal length with ascending columns (dense data handed over as CSR) are spread into the LDS vectors by
// consecutive lanes reading consecutive entries - whole cache lines per load instruction instead of one 4-byte word from
// each of 64 lines; anything else takes the row-per-thread loop (whose result for a repeated column, the later entry,
// does not depend on the order in which lanes write).
template <int B, int ILP, int kFetch>
__global__ __launch_bounds__(B) void k_predict_compact(int n, int F, const int *__restrict__ row_ptr,
                                                       const int *__restrict__ col, const float *__restrict__ val,
                                                       const uint2 *__restrict__ packed, int n_iter, int n_class_trees,
                                                       int n_nodes, int depth, float lr, float base_score,
                                                       float *__restrict__ out, size_t out_stride, int trees_per_stage,
                                                       int coalesced_fill) {
    extern __shared__ unsigned smem_u[];
    unsigned *dense = smem_u;                                        // [F + 2][B] keys; feature F: missing, F + 1: zero
    uint2 *nodes = reinterpret_cast<uint2 *>(smem_u + (F + 2) * B);  // [trees_per_stage][n_nodes]
    const int row0 = blockIdx.x * B;
    const int i = row0 + threadIdx.x;
    const bool live = i < n;
    for (int f = 0; f <= F; ++f) dense[f * B + threadIdx.x] = kMissingKey;
    dense[(F + 1) * B + threadIdx.x] = 0u;
    const int rb = live ? row_ptr[i] : 0, re = live ? row_ptr[i + 1] : 0;
    const int len0 = row_ptr[row0 + 1] - row_ptr[row0];  // (row0 < n: the grid covers no workgroup without rows)
    bool per_row = true;
    if (coalesced_fill && __syncthreads_and(!live || re - rb == len0) && len0 > 0) {
        // (the barrier above also orders the clearing before the writes of other lanes below)
        const int rows = min(B, n - row0);
        const int e0 = row_ptr[row0];
        const int total = rows * len0;
        int r = threadIdx.x / len0, slot = threadIdx.x - r * len0;
        const int dr = B / len0, ds = B - dr * len0;
        bool bad = false;
        // (four entries per lane in flight: the loop is a chain of memory round trips otherwise)
        for (int idx0 = threadIdx.x; idx0 < total; idx0 += 4 * B) {
            int c[4], before[4];
            float v[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int idx = min(idx0 + u * B, total - 1);
                c[u] = col[e0 + idx];
                v[u] = val[e0 + idx];
                // ascending inside the row: the entry before this one sits in the lane below (or, for lane 0, in memory)
                before[u] = (threadIdx.x & 63) == 0 && idx > 0 ? col[e0 + idx - 1] : 0;
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int below = __shfl_up(c[u], 1);
                if ((threadIdx.x & 63) != 0) before[u] = below;
                if (idx0 + u * B < total) {
                    if (slot > 0 && before[u] >= c[u]) bad = true;
                    if ((unsigned)c[u] < (unsigned)F) dense[c[u] * B + r] = value_key(v[u]);
                }
                r += dr;
                slot += ds;
                if (slot >= len0) {
                    slot -= len0;
                    ++r;
                }
            }
        }
        per_row = __syncthreads_or(bad);
        if (per_row)
            for (int f = 0; f < F; ++f) dense[f * B + threadIdx.x] = kMissingKey;
    }
    if (per_row) {
        for (int e = rb; e < re; e += 4) {  // (four entries in flight, written in their order)
            int c[4];
            float v[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                c[u] = col[min(e + u, re - 1)];
                v[u] = val[min(e + u, re - 1)];
            }
#pragma unroll
            for (int u = 0; u < 4; ++u)
                if (e + u < re && (unsigned)c[u] < (unsigned)F) dense[c[u] * B + threadIdx.x] = value_key(v[u]);
        }
    }
    // (byte offsets into the workgroup's LDS, so that a step adds record fields to them without further scaling)
    const char *lds = reinterpret_cast<const char *>(smem_u);
    const unsigned mine = threadIdx.x * 4u;  // this row's key of feature 0
    const unsigned trees0 = (unsigned)(F + 2) * B * 4u;
    // The trees of a stage are fetched into registers while the stage before is walked and go to the LDS between two
    // barriers after it, so that no walk waits for global memory (kFetch records per thread, as many as the stage needs:
    // the loads are unconditional - clamped -, or the compiler waits for them at once; stages of more than 8 records
    // per thread are copied after the barrier instead).
    const bool prefetch = trees_per_stage * n_nodes <= kFetch * B;
    uint2 fetched[kFetch];
    auto fetch = [&](int t, int it0) {
        const int count = min(trees_per_stage, n_iter - it0) * n_nodes;
        const uint2 *src = packed + ((size_t)t * n_iter + it0) * n_nodes;
#pragma unroll
        for (int q = 0; q < kFetch; ++q) fetched[q] = src[min((int)threadIdx.x + q * B, count - 1)];
    };
    if (prefetch) fetch(0, 0);
    for (int t = 0; t < n_class_trees; ++t) {
        double sum = base_score;
        for (int it0 = 0; it0 < n_iter; it0 += trees_per_stage) {
            const int staged = min(trees_per_stage, n_iter - it0);
            __syncthreads();  // the walks of the previous stage are done (and, the first time, the vectors are filled)
            if (prefetch) {
#pragma unroll
                for (int q = 0; q < kFetch; ++q) {
                    const int idx = threadIdx.x + q * B;
                    if (idx < staged * n_nodes) nodes[idx] = fetched[q];
                }
                // the next stage: of this class, or the first of the next class
                if (it0 + trees_per_stage < n_iter) fetch(t, it0 + trees_per_stage);
                else if (t + 1 < n_class_trees) fetch(t + 1, 0);
            } else {
                const uint2 *src = packed + ((size_t)t * n_iter + it0) * n_nodes;
                for (int idx = threadIdx.x; idx < staged * n_nodes; idx += B) nodes[idx] = src[idx];
            }
            __syncthreads();
            if (!live) continue;
            for (int k = 0; k < staged; k += ILP) {
                unsigned tree[ILP];
                uint2 nd[ILP];
#pragma unroll
                for (int j = 0; j < ILP; ++j) {
                    // (past the last staged tree: the last one is walked again and not added)
                    tree[j] = trees0 + (unsigned)(min(k + j, staged - 1) * n_nodes) * 8u;
                    nd[j] = *reinterpret_cast<const uint2 *>(lds + tree[j]);
                }
                for (int step = 0; step < depth; ++step) {
                    unsigned key[ILP];
#pragma unroll
                    for (int j = 0; j < ILP; ++j)
                        key[j] = *reinterpret_cast<const unsigned *>(lds + (mine + ((nd[j].y & 0x7fffu) << 2)));
#pragma unroll
                    for (int j = 0; j < ILP; ++j) {
                        const bool right = key[j] + (nd[j].y >> 31) > nd[j].x;
                        nd[j] = *reinterpret_cast<const uint2 *>(lds + (tree[j] + ((nd[j].y >> 15) & 0xffffu) + (right ? 8u : 0u)));
                    }
                }
#pragma unroll
                for (int j = 0; j < ILP; ++j)
                    if (k + j < staged) sum += lr * __uint_as_float(nd[j].x);
            }
        }
        if (live) out[(size_t)t * out_stride + i] += (float)sum;
    }
}

// kind 1: binary label lookup, 2: arg-max label lookup, 3: softmax probabilities in place,
// 4: sigmoid (reg:logistic). regression_obj.h:27-32,76-92 and multiclass_obj.cu:44-88 of the reference.
__global__ void k_predict_transform(int kind, int n, int K, const float *__restrict__ label, float *__restrict__ y) {
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x) {
        if (kind == 1) {
            y[i] = label[y[i] > 0 ? 1 : 0];
        } else if (kind == 2) {
            int nc = K == 2 ? 1 : K;
            int mk = 0;
            float mp = y[i];
            for (int k = 1; k < nc; ++k) {
                float v = y[(size_t)k * n + i];
                if (mp < v) {
                    mp = v;
                    mk = k;
                }
            }
            y[i] = label[mk];
        } else if (kind == 3) {
            float mx = y[i];
            for (int k = 1; k < K; ++k) mx = fmaxf(mx, y[(size_t)k * n + i]);
            float sum = 0;
            for (int k = 0; k < K; ++k) {
                float e = expf(y[(size_t)k * n + i] - mx);
                y[(size_t)k * n + i] = e;
                sum += e;
            }
            for (int k = 0; k < K; ++k) y[(size_t)k * n + i] /= sum;
        } else if (kind == 4) {
            y[i] = 1.f / (1.f + expf(-y[i]));
        }
    }
}

}  // namespace

void launch_predict(hipStream_t s, int n, int F, const int *row_ptr, const int *col, const float *val,
                    const TreeNode *model, int n_iter, int n_class_trees, int n_nodes, float lr, float base_score,
                    float *out, size_t out_stride, const PackedNode *packed, const uint2 *compact, int compact_depth) {
    if (n == 0) return;
    if (out_stride == 0) out_stride = (size_t)n;
    if (n_class_trees > 1) base_score = 0;  // predictor.cu:81-83
    const bool dense_path = (size_t)F * 128 * sizeof(float) <= 48 * 1024;
    int grid = (n + kBlock - 1) / kBlock;
    // (TGBM_PREDICT_TPS: trees staged at a time, 0 = walk the 48-byte nodes in global memory; measurements)
    // (both switches are read at every call, so a test can compare the kernels within one process)
    const int tps_given = std::getenv("TGBM_PREDICT_TPS") ? atoi(std::getenv("TGBM_PREDICT_TPS")) : -1;
    int tps_env = tps_given < 0 ? 2 : tps_given;
    // (TGBM_PREDICT_COMPACT=0: the 16-byte records also where the 8-byte ones apply; =2: those without the coalesced
    // spreading of equal-length rows; measurements and tests)
    const int compact_env = std::getenv("TGBM_PREDICT_COMPACT") ? atoi(std::getenv("TGBM_PREDICT_COMPACT")) : 1;
    if (compact != nullptr && compact_env > 0 && tps_env > 0) {
        const int B = compact_rows_per_group(F);
        const size_t dense_bytes = (size_t)(F + 2) * B * sizeof(float), tree_bytes = (size_t)n_nodes * sizeof(uint2);
        const size_t fit = (64 * 1024 - dense_bytes) / tree_bytes;  // (>= 1: compact_records_apply)
        // two trees per stage and thread (more were not faster: 10 M rows x 40 trees of depth 8 take 2.0 ms with two,
        // 2.1 ms with four, 2.7 ms with one)
        const int tps = (int)std::max<size_t>(1, std::min<size_t>(std::min(tps_env, 2), fit));
        const size_t lds = dense_bytes + (size_t)tps * tree_bytes;
        const int fill = compact_env == 2 ? 0 : 1;
        const int g = (n + B - 1) / B;
        const int per_thread = (tps * n_nodes + B - 1) / B;  // records of a stage
#define TGBM_PREDICT_COMPACT_LAUNCH(BLK, ILP, FETCH)                                                                  \
    k_predict_compact<BLK, ILP, FETCH><<<g, BLK, lds, s>>>(n, F, row_ptr, col, val, compact, n_iter, n_class_trees,  \
                                                           n_nodes, compact_depth, lr, base_score, out, out_stride, \
                                                           tps, fill)
#define TGBM_PREDICT_COMPACT_FETCH(BLK, ILP)                               \
    if (per_thread <= 2) TGBM_PREDICT_COMPACT_LAUNCH(BLK, ILP, 2);         \
    else if (per_thread <= 4) TGBM_PREDICT_COMPACT_LAUNCH(BLK, ILP, 4);    \
    else TGBM_PREDICT_COMPACT_LAUNCH(BLK, ILP, 8)
        if (B == 256) {
            if (tps >= 2) { TGBM_PREDICT_COMPACT_FETCH(256, 2); }
            else { TGBM_PREDICT_COMPACT_FETCH(256, 1); }
        } else {
            if (tps >= 2) { TGBM_PREDICT_COMPACT_FETCH(128, 2); }
            else { TGBM_PREDICT_COMPACT_FETCH(128, 1); }
        }
#undef TGBM_PREDICT_COMPACT_FETCH
#undef TGBM_PREDICT_COMPACT_LAUNCH
        return;
    }
    tps_env = tps_given < 0 ? 4 : tps_given;
    if (dense_path && packed != nullptr && tps_env > 0 && n_nodes <= 0xffff) {  // (16-bit child indices)
        // trees in LDS: 256 rows per workgroup while their dense vectors take at most 48 KB, else 128; trees are staged
        // one at a time unless several fit next to the vectors in 40 KB (four workgroups per CU: measured on 10 M rows
        // x 40 trees of depth 8, 6.0 ms with one tree per stage, 8.0 ms with four, 14.3 ms from global memory)
        const int B = (size_t)F * 256 * sizeof(float) <= 48 * 1024 ? 256 : 128;
        const size_t dense_bytes = (size_t)F * B * sizeof(float), tree_bytes = (size_t)n_nodes * sizeof(PackedNode);
        if (dense_bytes + tree_bytes <= 64 * 1024) {
            size_t fit = dense_bytes + tree_bytes <= 40 * 1024 ? (40 * 1024 - dense_bytes) / tree_bytes : 1;
            const int tps = (int)std::max<size_t>(1, std::min<size_t>((size_t)tps_env, fit));
            const size_t lds = dense_bytes + (size_t)tps * tree_bytes;
            if (B == 256)
                k_predict_lds<256><<<(n + 255) / 256, 256, lds, s>>>(n, F, row_ptr, col, val, packed, n_iter, n_class_trees,
                                                                  n_nodes, lr, base_score, out, out_stride, tps);
            else
                k_predict_lds<128><<<(n + 127) / 128, 128, lds, s>>>(n, F, row_ptr, col, val, packed, n_iter, n_class_trees,
                                                                  n_nodes, lr, base_score, out, out_stride, tps);
            return;
        }
    }
    if (dense_path)
        k_predict_staged<<<(n + kStageBlock - 1) / kStageBlock, kStageBlock, (size_t)F * kStageBlock * sizeof(float), s>>>(
            n, F, row_ptr, col, val, model, n_iter, n_class_trees, n_nodes, lr, base_score, out, out_stride);
    else
        k_predict<float, false><<<grid, kBlock, 0, s>>>(n, row_ptr, col, val, model, n_iter, n_class_trees, n_nodes, lr,
                                                       base_score, out, out_stride);
}

void launch_pack_model(hipStream_t s, const TreeNode *model, long n_total, int n_nodes, PackedNode *packed) {
    if (n_total <= 0) return;
    k_pack_model<<<(int)std::min<long>((n_total + 255) / 256, 4096), 256, 0, s>>>(model, n_total, n_nodes, packed);
}

int compact_rows_per_group(int F) { return (size_t)(F + 2) * 256 * sizeof(float) <= 50 * 1024 ? 256 : 128; }

void launch_pack_compact(hipStream_t s, const TreeNode *model, int n_iter, int n_class_trees, int n_nodes, int F,
                         uint2 *packed) {
    const long n_total = (long)n_iter * n_class_trees * n_nodes;
    if (n_total <= 0) return;
    k_pack_compact<<<(int)std::min<long>((n_total + 255) / 256, 4096), 256, 0, s>>>(model, n_iter, n_class_trees, n_nodes,
                                                                                    F, compact_rows_per_group(F), packed);
}

void launch_predict_transform(hipStream_t s, int kind, int n, int num_class, const float *label, float *y) {
    if (n == 0 || kind == 0) return;
    int grid = (n + kBlock - 1) / kBlock;
    if (grid > 4096) grid = 4096;
    k_predict_transform<<<grid, kBlock, 0, s>>>(kind, n, num_class, label, y);
}

}  // namespace tgbm
