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
                    float *out, size_t out_stride, const PackedNode *packed) {
    if (n == 0) return;
    if (out_stride == 0) out_stride = (size_t)n;
    if (n_class_trees > 1) base_score = 0;  // predictor.cu:81-83
    const bool dense_path = (size_t)F * 128 * sizeof(float) <= 48 * 1024;
    int grid = (n + kBlock - 1) / kBlock;
    // (TGBM_PREDICT_TPS: trees staged at a time, 0 = walk the 48-byte nodes in global memory; measurements)
    static const int tps_env = std::getenv("TGBM_PREDICT_TPS") ? atoi(std::getenv("TGBM_PREDICT_TPS")) : 4;
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

void launch_predict_transform(hipStream_t s, int kind, int n, int num_class, const float *label, float *y) {
    if (n == 0 || kind == 0) return;
    int grid = (n + kBlock - 1) / kBlock;
    if (grid > 4096) grid = 4096;
    k_predict_transform<<<grid, kBlock, 0, s>>>(kind, n, num_class, label, y);
}

}  // namespace tgbm
