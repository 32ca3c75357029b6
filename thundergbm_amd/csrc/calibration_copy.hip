// Profiler calibration helper, built as a library of its own (libtgbm_calibration.so) and not part of the training
// library's ABI: a plain streaming copy of known size, against which the HBM byte counters of rocprofv3 (FETCH_SIZE,
// WRITE_SIZE) are scaled. The reference has no counterpart.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>

namespace {

__global__ void k_calibration_copy(const uint4 *__restrict__ src, uint4 *__restrict__ dst, size_t n) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x)
        dst[i] = src[i];
}

void check(hipError_t e, const char *what) {
    if (e == hipSuccess) return;
    std::fprintf(stderr, "tgbm_calibration_copy: %s: %s\n", what, hipGetErrorString(e));
    std::abort();
}

}  // namespace

// Runs `repeats` launches of the copy kernel over `bytes` bytes (two fresh device buffers).
extern "C" void tgbm_calibration_copy(size_t bytes, int repeats) {
    void *src = nullptr, *dst = nullptr;
    check(hipMalloc(&src, bytes), "hipMalloc");
    check(hipMalloc(&dst, bytes), "hipMalloc");
    check(hipMemset(src, 1, bytes), "hipMemset");
    check(hipMemset(dst, 0, bytes), "hipMemset");
    const size_t n = bytes / 16;
    const int block = 256;
    size_t grid = (n + block - 1) / block;
    if (grid > 16384) grid = 16384;
    if (grid < 1) grid = 1;
    for (int i = 0; i < repeats && n > 0; ++i)
        k_calibration_copy<<<(int)grid, block, 0, nullptr>>>(static_cast<const uint4 *>(src), static_cast<uint4 *>(dst), n);
    check(hipGetLastError(), "launch");
    check(hipDeviceSynchronize(), "hipDeviceSynchronize");
    check(hipFree(src), "hipFree");
    check(hipFree(dst), "hipFree");
}
