// Small device helpers shared by the kernel sources (wave64 indexing, 64-bit shuffles, the reference's gain
// formula and left/right rule). Everything here is inlined into its callers.
#pragma once
#include <hip/hip_runtime.h>

#include "device_api.h"

namespace tgbm {
namespace {

__device__ __forceinline__ int lane_id() { return threadIdx.x & 63; }
__device__ __forceinline__ int wave_id() { return threadIdx.x >> 6; }
__device__ __forceinline__ int lanes_below(unsigned long long mask) {
    return __builtin_amdgcn_mbcnt_hi((unsigned)(mask >> 32), __builtin_amdgcn_mbcnt_lo((unsigned)mask, 0));
}


// Round-to-nearest-even of a float (|x| < 2^51) as a 64-bit integer: the integer sits in the low mantissa bits of
// x + 1.5 * 2^52 (bit pattern 0x4338000000000000, whose low word is zero: only the high word is corrected).
__device__ __forceinline__ long long round_to_ll(float x) {
    const long long b = __double_as_longlong((double)x + 6755399441055744.0);
    const unsigned hi = (unsigned)((unsigned long long)b >> 32) - 0x43380000u;
    return (long long)(((unsigned long long)hi << 32) | (unsigned)b);
}

__device__ __forceinline__ bool node_splits(const TreeNode &nd) {
    return nd.is_valid && !nd.is_leaf && nd.split_feature_id >= 0;
}


__device__ __forceinline__ long long shfl_up_ll(long long v, int d) {
    int lo = __shfl_up((int)(unsigned)(unsigned long long)v, d);
    int hi = __shfl_up((int)((unsigned long long)v >> 32), d);
    return (long long)(((unsigned long long)(unsigned)hi << 32) | (unsigned)lo);
}


__device__ __forceinline__ long long wave_sum_ll(long long v) {
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) {
        const int lo = __shfl_xor((int)(unsigned)(unsigned long long)v, d);
        const int hi = __shfl_xor((int)((unsigned long long)v >> 32), d);
        v += (long long)(((unsigned long long)(unsigned)hi << 32) | (unsigned)lo);
    }
    return v;
}


// Left/right decision of the sparse layout: binary search of the row's bin ids for the one inside
// the split feature's bin range (absent = missing), hist_tree_builder_single.cu:941-1011.
// Does the row go right at a split of the feature whose global bins are [cb, ce)? Binary search of the
// row's ascending bin ids for one inside the feature's range; none = missing -> default direction.
__device__ __forceinline__ bool csr_goes_right(const CsrBins &bins, int row, int cb, int ce, int sbid, bool dr) {
    int lo = bins.row_ptr[row], hi = bins.row_ptr[row + 1];
    int found = -1;
    while (lo < hi) {
        int mid = lo + (hi - lo) / 2;
        int b = bins.bin[mid];
        if (b >= cb && b < ce) {
            found = b;
            break;
        }
        if (b < cb)
            lo = mid + 1;
        else
            hi = mid;
    }
    return found < 0 ? dr : (found >= sbid);
}


// Power of two by which the dense work items of a node that add at most `rows` rows between two drains coarsen one
// of the tree's scales: the smallest s >= 0 with rows * (qmax / 2^s + 0.5) < 2^bits (qmax: the most one row adds at the tree's
// scale, bits: magnitude bits of the packed field).
__device__ __forceinline__ int item_shift(float qmax, int rows, int bits) {
    const double lim = ldexp(1.0, bits) / (double)rows * (1.0 - 1e-6) - 0.5;
    const double q = (double)qmax;
    if (!(q >= lim)) return 0;
    return ilogb(q / lim) + 1;  // 2^s > q / lim
}

// ------------------------------------------------------------------------ split finding
__device__ __forceinline__ float split_gain(GHPair f, GHPair l, float mcw, float lambda) {
#pragma clang fp contract(off)
    GHPair r{f.g - l.g, f.h - l.h};
    float gain = 0.f;
    if (l.h >= mcw && r.h >= mcw)
        gain = (l.g * l.g) / (l.h + lambda) + (r.g * r.g) / (r.h + lambda) - (f.g * f.g) / (f.h + lambda);
    return fmaxf(0.f, gain);
}



}  // namespace
}  // namespace tgbm
