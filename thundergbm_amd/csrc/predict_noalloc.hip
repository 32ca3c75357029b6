// tgbm_predict_raw for callers that must not allocate: the device copies of the rows, of the model and of the
// scores live in one file-scope device array instead of per-call hipMalloc'ed buffers.
#include <cstdio>
#include <mutex>

#include "../../include/thundergbm.h"
#include "device_api.h"
#include "model_handle.h"

using namespace tgbm;

namespace {

// Limits of one call (the array below is sized for exactly these).
constexpr long kMaxRows = 1l << 16;    // rows
constexpr long kMaxValues = 1l << 20;  // stored values (row_ptr[row_size])
constexpr long kMaxScores = 1l << 19;  // row_size * trees_per_iter
constexpr long kMaxNodes = 1l << 19;   // nodes of all trees used (n_trees * trees_per_iter * nodes per tree)

constexpr size_t align256(size_t b) { return (b + 255) / 256 * 256; }
constexpr size_t kOffVal = 0;
constexpr size_t kOffCol = kOffVal + align256(sizeof(float) * kMaxValues);
constexpr size_t kOffRowPtr = kOffCol + align256(sizeof(int) * kMaxValues);
constexpr size_t kOffScores = kOffRowPtr + align256(sizeof(int) * (kMaxRows + 1));
constexpr size_t kOffModel = kOffScores + align256(sizeof(float) * kMaxScores);
constexpr size_t kScratchBytes = kOffModel + align256(sizeof(TreeNode) * kMaxNodes);  // ~34.3 MiB

// Every GPU the library runs on holds its own copy of this array until the process ends. In host code the name is
// only a handle for hipGetSymbolAddress; kernels and copies get the address that call returns.
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

constexpr int kMaxDevices = 64;
unsigned char *g_scratch_ptr[kMaxDevices] = {};  // per device: address of that device's `scratch`
std::mutex g_mutex;                              // calls share the device's array: one at a time

// Address of the current device's array; resolved on the first call on that device.
unsigned char *scratch_of_current_device() {
    int dev = -1;
    HIP_CHECK(hipGetDevice(&dev));
    TGBM_CHECK(dev >= 0 && dev < kMaxDevices, "device index %d out of range", dev);
    if (g_scratch_ptr[dev] == nullptr) {
        void *p = nullptr;
        HIP_CHECK(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        TGBM_CHECK(p != nullptr, "hipGetSymbolAddress returned a null address");
        g_scratch_ptr[dev] = static_cast<unsigned char *>(p);
    }
    return g_scratch_ptr[dev];
}

int reject(const char *what, long got, long limit) {
    std::fprintf(stderr, "tgbm_predict_raw_noalloc: %s = %ld exceeds the limit of %ld; use tgbm_predict_raw\n", what, got,
                 limit);
    std::fflush(stderr);
    return 1;
}

}  // namespace

extern "C" int tgbm_predict_raw_noalloc(int row_size, const float *val, const int *row_ptr, const int *col_ptr,
                                        tgbm_model *model, int n_trees, int trees_per_iter, float learning_rate,
                                        float base_score, float *out) {
    TGBM_CHECK(model != nullptr, "model is null!");
    TGBM_CHECK(row_size >= 0 && n_trees >= 1 && trees_per_iter >= 1, "bad sizes: %d rows, %d x %d trees", row_size,
               n_trees, trees_per_iter);
    const size_t n_used = (size_t)n_trees * trees_per_iter;
    TGBM_CHECK(n_used <= model->trees.size(), "model holds %zu trees, %d x %d requested", model->trees.size(), n_trees,
               trees_per_iter);
    const long n_nodes = (long)model->trees[0].nodes.size();
    for (size_t t = 0; t < n_used; ++t)
        TGBM_CHECK((long)model->trees[t].nodes.size() == n_nodes, "trees of different size in one model");
    if (row_size == 0) return 0;
    TGBM_CHECK(row_ptr[0] == 0, "CSR input: row_ptr[0] is %d, expected 0", row_ptr[0]);
    for (int i = 0; i < row_size; ++i)
        TGBM_CHECK(row_ptr[i + 1] >= row_ptr[i], "CSR input: row_ptr decreases at row %d", i);
    const long nnz = row_ptr[row_size];
    if (row_size > kMaxRows) return reject("row_size", row_size, kMaxRows);
    if (nnz > kMaxValues) return reject("stored values", nnz, kMaxValues);
    if ((long)row_size * trees_per_iter > kMaxScores) return reject("row_size * trees_per_iter", (long)row_size * trees_per_iter, kMaxScores);
    if ((long)n_used * n_nodes > kMaxNodes) return reject("model nodes", (long)n_used * n_nodes, kMaxNodes);
    // number of features = largest column index + 1 (dataset.cpp:40-46); the indices address per-row staging in
    // the kernel, so they are checked here
    int max_col = -1;
    for (long e = 0; e < nnz; ++e) {
        TGBM_CHECK(col_ptr[e] >= 0, "CSR input: negative column index %d", col_ptr[e]);
        max_col = col_ptr[e] > max_col ? col_ptr[e] : max_col;
    }
    const int F = max_col + 1;

    std::lock_guard<std::mutex> lock(g_mutex);
    unsigned char *base = scratch_of_current_device();
    float *d_val = reinterpret_cast<float *>(base + kOffVal);
    int *d_col = reinterpret_cast<int *>(base + kOffCol);
    int *d_row_ptr = reinterpret_cast<int *>(base + kOffRowPtr);
    float *d_scores = reinterpret_cast<float *>(base + kOffScores);
    TreeNode *d_model = reinterpret_cast<TreeNode *>(base + kOffModel);
    hipStream_t s = nullptr;  // the default stream: nothing is created per call
    const size_t n_scores = (size_t)row_size * trees_per_iter;
    if (nnz) {
        HIP_CHECK(hipMemcpyAsync(d_val, val, sizeof(float) * (size_t)nnz, hipMemcpyHostToDevice, s));
        HIP_CHECK(hipMemcpyAsync(d_col, col_ptr, sizeof(int) * (size_t)nnz, hipMemcpyHostToDevice, s));
    }
    HIP_CHECK(hipMemcpyAsync(d_row_ptr, row_ptr, sizeof(int) * (size_t)(row_size + 1), hipMemcpyHostToDevice, s));
    for (size_t t = 0; t < n_used; ++t)
        HIP_CHECK(hipMemcpyAsync(d_model + t * (size_t)n_nodes, model->trees[t].nodes.data(),
                                 sizeof(TreeNode) * (size_t)n_nodes, hipMemcpyHostToDevice, s));
    // the array keeps the previous call's scores and the traversal adds to them: clear this call's part (with a
    // kernel, not a memset node, so that the sequence can be recorded into a HIP graph)
    launch_fill_f32(s, d_scores, 0.f, n_scores);
    launch_predict(s, row_size, F, d_row_ptr, d_col, d_val, d_model, n_trees, trees_per_iter, (int)n_nodes,
                   learning_rate, base_score, d_scores, (size_t)row_size);
    HIP_CHECK_LAUNCHES("tgbm_predict_raw_noalloc");
    HIP_CHECK(hipMemcpyAsync(out, d_scores, sizeof(float) * n_scores, hipMemcpyDeviceToHost, s));
    HIP_CHECK(hipStreamSynchronize(s));
    return 0;
}
