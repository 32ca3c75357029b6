// One-off data preparation on the device: quantile cut points (a stable LSD radix sort of
// (feature, value) keys, run-length flags, exclusive scan, strided selection) and the dense
// column-blocked bin matrix. Runs once per training call, outside the boosting loop.
#include <algorithm>
#include <vector>

#include "device_api.h"

namespace tgbm {
namespace {

constexpr int kBlock = 256;
constexpr int kWaves = kBlock / 64;
constexpr int kSortRounds = 64;               // keys per lane and tile
constexpr int kSortTile = 64 * kSortRounds;   // keys per wavefront tile
constexpr int kScanItems = 8;
constexpr int kScanTile = kBlock * kScanItems;

__device__ __forceinline__ int lane_id() { return threadIdx.x & 63; }
__device__ __forceinline__ int wave_id() { return threadIdx.x >> 6; }
__device__ __forceinline__ int lanes_below(unsigned long long mask) {
    return __builtin_amdgcn_mbcnt_hi((unsigned)(mask >> 32), __builtin_amdgcn_mbcnt_lo((unsigned)mask, 0));
}

// Order-preserving map float -> uint32 (-0.0 is folded into +0.0 so that == duplicates share a key).
__device__ __forceinline__ unsigned float_key(float v) {
    if (v == 0.f) v = 0.f;
    unsigned u = __float_as_uint(v);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float key_float(unsigned k) {
    unsigned u = (k & 0x80000000u) ? (k & 0x7fffffffu) : ~k;
    return __uint_as_float(u);
}

__global__ void k_make_keys(long n, const float *__restrict__ val, const int *__restrict__ col,
                            unsigned long long *__restrict__ keys) {
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x)
        keys[i] = ((unsigned long long)(unsigned)col[i] << 32) | float_key(val[i]);
}

// ---- radix sort, 8 bits per pass; every wavefront owns one tile of kSortTile consecutive keys ----
__global__ __launch_bounds__(kBlock) void k_radix_count(const unsigned long long *__restrict__ keys, long n, int shift,
                                                       long n_tiles, unsigned *__restrict__ counts) {
    __shared__ unsigned cnt[kWaves][256];
    const int w = wave_id(), lane = lane_id();
    const long tile = (long)blockIdx.x * kWaves + w;
    if (tile >= n_tiles) return;  // a wavefront only touches its own row of counters: no workgroup barrier
    for (int d = lane; d < 256; d += 64) cnt[w][d] = 0;
    __builtin_amdgcn_wave_barrier();
    const long base = tile * kSortTile;
    constexpr int kBatch = 16;
    for (int r0 = 0; r0 < kSortRounds; r0 += kBatch) {
        unsigned long long k[kBatch];
#pragma unroll
        for (int b = 0; b < kBatch; ++b) {
            const long i = base + (long)(r0 + b) * 64 + lane;
            k[b] = i < n ? keys[i] : 0ull;
        }
#pragma unroll
        for (int b = 0; b < kBatch; ++b) {
            const long i = base + (long)(r0 + b) * 64 + lane;
            if (i < n) atomicAdd(&cnt[w][(unsigned)(k[b] >> shift) & 255u], 1u);
        }
    }
    __builtin_amdgcn_wave_barrier();
    for (int d = lane; d < 256; d += 64) counts[(size_t)d * n_tiles + tile] = cnt[w][d];
}

// A workgroup owns one tile. Its keys are first ordered by digit inside LDS (every wavefront ranks its quarter of the
// tile round by round, in order, so equal digits keep their order: per-wavefront digit counts, a scan over the digits
// and the wavefronts, then a running position per wavefront and digit), then written out in that order: the keys of
// one digit go to consecutive addresses (runs of 16 keys on average instead of single 8-byte stores).
template <bool PAYLOAD>
__global__ __launch_bounds__(kBlock) void k_radix_scatter(const unsigned long long *__restrict__ in,
                                                         unsigned long long *__restrict__ out, long n, int shift,
                                                         long n_tiles, const unsigned *__restrict__ offsets,
                                                         const int *__restrict__ in_val, int *__restrict__ out_val) {
    static_assert(kBlock == 256, "one thread per digit");
    __shared__ unsigned long long s_key[kSortTile];
    __shared__ int s_val[PAYLOAD ? kSortTile : 1];
    __shared__ unsigned s_run[kWaves][256];  // per wavefront and digit: count, then the next local position
    __shared__ unsigned s_delta[256];        // per digit: global position of its first key - local position of it
    __shared__ unsigned s_wsum[kWaves];
    const int w = wave_id(), lane = lane_id();
    const long tile = blockIdx.x;
    const long base = tile * kSortTile;
    const int count = (int)((n - base) < (long)kSortTile ? (n - base) : (long)kSortTile);
    constexpr int kRounds = kSortTile / kBlock;  // rounds of 64 keys per wavefront
    for (int d = lane; d < 256; d += 64) s_run[w][d] = 0;
    unsigned long long keys[kRounds];
    int payload[kRounds];
#pragma unroll
    for (int b = 0; b < kRounds; ++b) {
        const int li = w * (kSortTile / kWaves) + b * 64 + lane;
        const int lc = li < count ? li : count - 1;  // (clamped: unconditional loads; count >= 1)
        keys[b] = in[base + lc];
        payload[b] = PAYLOAD ? in_val[base + lc] : 0;
    }
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int b = 0; b < kRounds; ++b) {
        const int li = w * (kSortTile / kWaves) + b * 64 + lane;
        if (li < count) atomicAdd(&s_run[w][(unsigned)(keys[b] >> shift) & 255u], 1u);
    }
    __syncthreads();
    {
        const int d = threadIdx.x;
        unsigned c[kWaves], tot = 0;
#pragma unroll
        for (int i = 0; i < kWaves; ++i) {
            c[i] = s_run[i][d];
            tot += c[i];
        }
        unsigned inc = tot;
#pragma unroll
        for (int k = 1; k < 64; k <<= 1) {
            const unsigned t = __shfl_up(inc, k);
            if (lane >= k) inc += t;
        }
        if (lane == 63) s_wsum[w] = inc;
        __syncthreads();
        unsigned run = inc - tot;
        for (int i = 0; i < w; ++i) run += s_wsum[i];
        s_delta[d] = offsets[(size_t)d * n_tiles + tile] - run;  // (modulo 2^32; the sum below is a position < n)
#pragma unroll
        for (int i = 0; i < kWaves; ++i) {
            s_run[i][d] = run;
            run += c[i];
        }
    }
    __syncthreads();
#pragma unroll
    for (int b = 0; b < kRounds; ++b) {
        const int li = w * (kSortTile / kWaves) + b * 64 + lane;
        const bool valid = li < count;
        const unsigned long long key = keys[b];
        const unsigned d = (unsigned)(key >> shift) & 255u;
        // lanes holding the same digit (match-any built from eight ballots)
        unsigned long long mask = __ballot(valid);
#pragma unroll
        for (int bit_i = 0; bit_i < 8; ++bit_i) {
            const bool bit = (d >> bit_i) & 1u;
            const unsigned long long m = __ballot(bit);
            mask &= bit ? m : ~m;
        }
        const unsigned first = valid ? s_run[w][d] : 0u;
        const int rank = lanes_below(mask);
        __builtin_amdgcn_wave_barrier();
        if (valid) {
            s_key[first + rank] = key;
            if (PAYLOAD) s_val[first + rank] = payload[b];
            if (rank == 0) s_run[w][d] = first + (unsigned)__popcll(mask);
        }
        __builtin_amdgcn_wave_barrier();
    }
    __syncthreads();
    for (int i = threadIdx.x; i < count; i += kBlock) {
        const unsigned long long key = s_key[i];
        const unsigned pos = s_delta[(unsigned)(key >> shift) & 255u] + (unsigned)i;
        out[pos] = key;
        if (PAYLOAD) out_val[pos] = s_val[i];
    }
}

// ---- exclusive scan of 32-bit counters (tile scan + recursive scan of tile sums + add) ----------
template <bool FROM_KEYS>
__device__ __forceinline__ unsigned scan_load(const void *in, long i) {
    if (FROM_KEYS) {
        const unsigned long long *k = static_cast<const unsigned long long *>(in);
        return (i == 0 || k[i] != k[i - 1]) ? 1u : 0u;  // 1 at the first entry of every (feature, value) run
    }
    return static_cast<const unsigned *>(in)[i];
}

template <bool FROM_KEYS>
__global__ __launch_bounds__(kBlock) void k_scan_tiles(const void *__restrict__ in, unsigned *__restrict__ out, long n,
                                                      unsigned *__restrict__ tile_sums) {
    __shared__ unsigned ws[kWaves];
    const long base = (long)blockIdx.x * kScanTile + (long)threadIdx.x * kScanItems;
    unsigned v[kScanItems];
    unsigned local = 0;
#pragma unroll
    for (int j = 0; j < kScanItems; ++j) {
        long i = base + j;
        v[j] = i < n ? scan_load<FROM_KEYS>(in, i) : 0u;
        local += v[j];
    }
    unsigned inc = local;
    const int lane = lane_id(), w = wave_id();
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        unsigned t = __shfl_up(inc, d);
        if (lane >= d) inc += t;
    }
    if (lane == 63) ws[w] = inc;
    __syncthreads();
    unsigned wbase = 0, tot = 0;
#pragma unroll
    for (int i = 0; i < kWaves; ++i) {
        if (i < w) wbase += ws[i];
        tot += ws[i];
    }
    unsigned run = wbase + inc - local;
#pragma unroll
    for (int j = 0; j < kScanItems; ++j) {
        long i = base + j;
        if (i < n) out[i] = run;
        run += v[j];
    }
    if (threadIdx.x == 0) tile_sums[blockIdx.x] = tot;
}

__global__ __launch_bounds__(kBlock) void k_scan_add(unsigned *__restrict__ out, long n,
                                                    const unsigned *__restrict__ tile_offsets) {
    const unsigned add = tile_offsets[blockIdx.x];
    const long base = (long)blockIdx.x * kScanTile;
#pragma unroll
    for (int j = 0; j < kScanItems; ++j) {
        long i = base + (long)j * kBlock + threadIdx.x;
        if (i < n) out[i] += add;
    }
}

// out[i] = sum of in[0..i); returns nothing, the total is written to *d_total (device). The tile sums of
// every recursion level live in `sc`, which grows on demand and is reused by later calls.
template <bool FROM_KEYS>
void exclusive_scan(hipStream_t s, const void *in, unsigned *out, long n, unsigned *d_total, ScanScratch &sc,
                    size_t level = 0) {
    long tiles = (n + kScanTile - 1) / kScanTile;
    if (sc.levels.size() <= level) sc.levels.resize(level + 1);
    ScanScratch::Level &lv = sc.levels[level];
    if (lv.cap < (size_t)tiles + 1) {
        if (lv.sums) HIP_CHECK(hipFree(lv.sums));
        if (lv.scanned) HIP_CHECK(hipFree(lv.scanned));
        lv.cap = (size_t)tiles + 1;
        HIP_CHECK(hipMalloc(&lv.sums, sizeof(unsigned) * lv.cap));
        HIP_CHECK(hipMalloc(&lv.scanned, sizeof(unsigned) * lv.cap));
    }
    unsigned *sums = lv.sums, *sums_scanned = lv.scanned;  // the recursion may move sc.levels
    k_scan_tiles<FROM_KEYS><<<(unsigned)tiles, kBlock, 0, s>>>(in, out, n, sums);
    if (tiles > 1) {
        exclusive_scan<false>(s, sums, sums_scanned, tiles, d_total, sc, level + 1);
        k_scan_add<<<(unsigned)tiles, kBlock, 0, s>>>(out, n, sums_scanned);
    } else {
        HIP_CHECK(hipMemcpyAsync(d_total, sums, sizeof(unsigned), hipMemcpyDeviceToDevice, s));
    }
}

// First sorted entry of every feature (binary search of f << 32), estart[F] = nnz.
__global__ void k_feature_starts(const unsigned long long *__restrict__ keys, long n, int F, long *__restrict__ estart) {
    for (int f = blockIdx.x * blockDim.x + threadIdx.x; f <= F; f += gridDim.x * blockDim.x) {
        unsigned long long target = (unsigned long long)(unsigned)f << 32;
        long lo = 0, hi = n;
        while (lo < hi) {
            long mid = lo + (hi - lo) / 2;
            if (keys[mid] < target)
                lo = mid + 1;
            else
                hi = mid;
        }
        estart[f] = lo;
    }
}

// ustart[f] = number of distinct (feature, value) pairs of features < f.
__global__ void k_unique_starts(const long *__restrict__ estart, const unsigned *__restrict__ uidx, long n, int F,
                                const unsigned *__restrict__ d_total, unsigned *__restrict__ ustart) {
    for (int f = blockIdx.x * blockDim.x + threadIdx.x; f <= F; f += gridDim.x * blockDim.x) {
        long e = estart[f];
        ustart[f] = e < n ? uidx[e] : *d_total;
    }
}

// Strided selection of the reference (hist_cut.cu:259-265): with m distinct values and
// step = m / max_bin, keep all of them if step == 0, else the values at ranks 0, step, 2 step, ...
// (max_bin of them).
__global__ void k_emit_cuts(const unsigned long long *__restrict__ keys, const unsigned *__restrict__ uidx, long n,
                            const unsigned *__restrict__ ustart, const int *__restrict__ cut_row_ptr, int max_bin,
                            float *__restrict__ cut_val, int *__restrict__ cut_fid) {
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) {
        unsigned long long k = keys[i];
        if (i != 0 && k == keys[i - 1]) continue;
        int f = (int)(k >> 32);
        unsigned j = uidx[i] - ustart[f];
        unsigned m = ustart[f + 1] - ustart[f];
        unsigned step = m / (unsigned)max_bin;
        int out = -1;
        if (step == 0)
            out = cut_row_ptr[f] + (int)j;
        else if (j % step == 0 && j / step < (unsigned)max_bin)
            out = cut_row_ptr[f] + (int)(j / step);
        if (out >= 0) {
            cut_val[out] = key_float((unsigned)k);
            cut_fid[out] = f;
        }
    }
}

// Bin of a stored value (the reference's clamped upper bound, hist_tree_builder_single.cu:81-119):
// min(#cuts <= v, k - 1), as a local (per-feature) bin id.
__device__ __forceinline__ int local_bin(const float *__restrict__ cuts, int k, float v) {
    int left = 0, right = k - 1;
    while (left < right) {
        int mid = left + (right - left) / 2;
        if (cuts[mid] <= v)
            left = mid + 1;
        else
            right = mid;
    }
    return left;
}

// Row-major blocks of the dense bin matrix (BinT = uint8_t or uint16_t; block_stride counts bins). Sixteen lanes
// share a row: its column indices and values are read in 64-byte pieces and the bins of neighbouring columns land
// in neighbouring bytes (one thread per row, the first version, read addresses a whole row apart: 45 ms for the
// 10^9 values of the 500k x 2000 configuration). Of two entries with the same column in a row the later one counts
// (adjacent ones, as in rows with ascending columns, are told apart here; the column-major copy is derived from
// this matrix afterwards, k_cols_from_rows).
template <typename BinT>
__global__ __launch_bounds__(kBlock) void k_bin_dense(int n, const int *__restrict__ row_ptr, const int *__restrict__ col,
                                                     const float *__restrict__ val, const float *__restrict__ cut_val,
                                                     const int *__restrict__ cut_row_ptr, BinT *__restrict__ binmat,
                                                     int W, size_t block_stride, const int *__restrict__ feat_col,
                                                     const uint8_t *__restrict__ feat_lo) {
    constexpr int kLanes = 16;
    const int sub = threadIdx.x % kLanes;
    for (int i = blockIdx.x * (kBlock / kLanes) + threadIdx.x / kLanes; i < n; i += gridDim.x * (kBlock / kLanes)) {
        const int e1 = row_ptr[i + 1];
        for (int e = row_ptr[i] + sub; e < e1; e += kLanes) {
            const int f = col[e];
            if (e + 1 < e1 && col[e + 1] == f) continue;
            const int cb = cut_row_ptr[f];
            const int k = cut_row_ptr[f + 1] - cb;
            int c = f, b = local_bin(cut_val + cb, k, val[e]);
            if (feat_col != nullptr) {  // (a bundled feature: its bins follow those of the bundle's earlier features)
                c = feat_col[f];
                b += feat_lo[f];
            }
            binmat[(size_t)(c / W) * block_stride + (size_t)i * W + (c % W)] = (BinT)b;
        }
    }
}

// The same for data with rows whose columns do not ascend (nothing the reference's wrappers produce: they sort the
// indices of every row, thundergbm.py:103): a row may then store a column twice with other entries in between, and
// sixteen lanes writing one cell would leave whichever bin arrived last. One thread walks its row front to back, so
// the later entry counts, as for adjacent ones. (The reference adds both entries to the histogram and searches the
// row's bin ids by bisection, which needs ascending columns: its own result for such rows is not defined.)
template <typename BinT>
__global__ __launch_bounds__(kBlock) void k_bin_dense_serial(int n, const int *__restrict__ row_ptr, const int *__restrict__ col,
                                                            const float *__restrict__ val, const float *__restrict__ cut_val,
                                                            const int *__restrict__ cut_row_ptr, BinT *__restrict__ binmat,
                                                            int W, size_t block_stride) {
    for (int i = blockIdx.x * kBlock + threadIdx.x; i < n; i += gridDim.x * kBlock) {
        for (int e = row_ptr[i]; e < row_ptr[i + 1]; ++e) {
            const int f = col[e];
            const int cb = cut_row_ptr[f];
            const int b = local_bin(cut_val + cb, cut_row_ptr[f + 1] - cb, val[e]);
            binmat[(size_t)(f / W) * block_stride + (size_t)i * W + (f % W)] = (BinT)b;
        }
    }
}

// Sets *descending when a row holds a column index below its predecessor's.
__global__ __launch_bounds__(kBlock) void k_rows_ascend(int n, const int *__restrict__ row_ptr, const int *__restrict__ col,
                                                       int *__restrict__ descending) {
    constexpr int kLanes = 16;
    const int sub = threadIdx.x % kLanes;
    bool bad = false;
    for (int i = blockIdx.x * (kBlock / kLanes) + threadIdx.x / kLanes; i < n; i += gridDim.x * (kBlock / kLanes)) {
        const int e1 = row_ptr[i + 1];
        for (int e = row_ptr[i] + sub; e + 1 < e1; e += kLanes) bad |= col[e + 1] < col[e];
    }
    if (bad) *descending = 1;
}

// Which columns follow which inside the rows (sixteen lanes per row, as above).
__global__ __launch_bounds__(kBlock) void k_min_next_col(int n, const int *__restrict__ row_ptr, const int *__restrict__ col,
                                                        int *__restrict__ min_next, int *__restrict__ descending) {
    constexpr int kLanes = 16;
    const int sub = threadIdx.x % kLanes;
    for (int i = blockIdx.x * (kBlock / kLanes) + threadIdx.x / kLanes; i < n; i += gridDim.x * (kBlock / kLanes)) {
        const int e1 = row_ptr[i + 1];
        for (int e = row_ptr[i] + sub; e + 1 < e1; e += kLanes) {
            const int c = col[e], next = col[e + 1];
            if (next < c) *descending = 1;
            // (the plain read keeps the atomics to the few that lower the entry)
            if (next > c && next < min_next[c]) atomicMin(&min_next[c], next);
        }
    }
}

// One wavefront per row: (global bin, row) of every stored value, for the bin-major copy.
__global__ __launch_bounds__(kBlock) void k_csc_keys(int n_rows, const int *__restrict__ row_ptr,
                                                    const int *__restrict__ bin, const int *__restrict__ sort_key,
                                                    unsigned long long *__restrict__ keys, int *__restrict__ vals) {
    const int r = blockIdx.x * (kBlock / 64) + (threadIdx.x >> 6);
    if (r >= n_rows) return;
    const int e1 = row_ptr[r + 1];
    for (int e = row_ptr[r] + (threadIdx.x & 63); e < e1; e += 64) {
        const unsigned b = (unsigned)bin[e];
        keys[e] = ((unsigned long long)b << 32) | (sort_key != nullptr ? (unsigned)sort_key[b] : b);
        vals[e] = r;
    }
}

__global__ __launch_bounds__(kBlock) void k_csc_unpack(long nnz, const unsigned long long *__restrict__ keys,
                                                      const int *__restrict__ vals, int *__restrict__ csc_bin,
                                                      int *__restrict__ csc_row) {
    for (long e = (long)blockIdx.x * kBlock + threadIdx.x; e < nnz; e += (long)gridDim.x * kBlock) {
        csc_bin[e] = (int)(keys[e] >> 32);
        csc_row[e] = vals[e];
    }
}

__global__ void k_bin_csr(long nnz, const int *__restrict__ col, const float *__restrict__ val,
                          const float *__restrict__ cut_val, const int *__restrict__ cut_row_ptr,
                          int *__restrict__ bin_id, const int *__restrict__ feat_slot, int *__restrict__ hist_word) {
    for (long e = (long)blockIdx.x * blockDim.x + threadIdx.x; e < nnz; e += (long)gridDim.x * blockDim.x) {
        int f = col[e];
        int cb = cut_row_ptr[f];
        int k = cut_row_ptr[f + 1] - cb;
        int local = local_bin(cut_val + cb, k, val[e]);
        bin_id[e] = cb + local;
        if (hist_word != nullptr) {
            int slot = feat_slot[f];
            hist_word[e] = slot >= 0 ? ~(slot + local) : cb + local;
        }
    }
}

int grid_for(size_t n, int cap = 8192) {
    size_t b = (n + kBlock - 1) / kBlock;
    if (b < 1) b = 1;
    if (b > (size_t)cap) b = cap;
    return (int)b;
}

}  // namespace

// Cut points of the reference's HistCut::get_cut_points_single (src/thundergbm/hist_cut.cu:232-286).
DeviceCuts build_cut_points(hipStream_t s, int F, long nnz, const float *d_val, const int *d_col, int max_num_bin) {
    DeviceCuts out;
    HIP_CHECK(hipMalloc(&out.cut_row_ptr, sizeof(int) * (size_t)(F + 1)));
    if (nnz == 0) {
        HIP_CHECK(hipMemsetAsync(out.cut_row_ptr, 0, sizeof(int) * (size_t)(F + 1), s));
        HIP_CHECK(hipStreamSynchronize(s));
        out.feature_nnz.assign(F, 0);
        return out;
    }
    ScanScratch scratch;
    unsigned long long *keys[2];
    HIP_CHECK(hipMalloc(&keys[0], sizeof(unsigned long long) * (size_t)nnz));
    HIP_CHECK(hipMalloc(&keys[1], sizeof(unsigned long long) * (size_t)nnz));
    k_make_keys<<<grid_for(nnz), kBlock, 0, s>>>(nnz, d_val, d_col, keys[0]);

    int fid_bits = 0;
    while ((1ll << fid_bits) < (long long)F) ++fid_bits;
    const int passes = (32 + fid_bits + 7) / 8;
    const long n_tiles = (nnz + kSortTile - 1) / kSortTile;
    const size_t n_counts = (size_t)256 * n_tiles;
    unsigned *counts = nullptr, *offsets = nullptr, *d_total = nullptr;
    HIP_CHECK(hipMalloc(&counts, sizeof(unsigned) * n_counts));
    HIP_CHECK(hipMalloc(&offsets, sizeof(unsigned) * (n_counts + 1)));
    HIP_CHECK(hipMalloc(&d_total, sizeof(unsigned)));
    const unsigned sort_grid = (unsigned)((n_tiles + kWaves - 1) / kWaves);
    int cur = 0;
    for (int p = 0; p < passes; ++p) {
        const int shift = 8 * p;
        k_radix_count<<<sort_grid, kBlock, 0, s>>>(keys[cur], nnz, shift, n_tiles, counts);
        exclusive_scan<false>(s, counts, offsets, (long)n_counts, d_total, scratch);
        k_radix_scatter<false><<<(unsigned)n_tiles, kBlock, 0, s>>>(keys[cur], keys[cur ^ 1], nnz, shift, n_tiles, offsets,
                                                            nullptr, nullptr);
        cur ^= 1;
    }
    const unsigned long long *sorted = keys[cur];
    unsigned *uidx = nullptr;
    HIP_CHECK(hipMalloc(&uidx, sizeof(unsigned) * (size_t)nnz));
    exclusive_scan<true>(s, sorted, uidx, nnz, d_total, scratch);
    long *estart = nullptr;
    unsigned *ustart = nullptr;
    HIP_CHECK(hipMalloc(&estart, sizeof(long) * (size_t)(F + 1)));
    HIP_CHECK(hipMalloc(&ustart, sizeof(unsigned) * (size_t)(F + 1)));
    k_feature_starts<<<grid_for(F + 1), kBlock, 0, s>>>(sorted, nnz, F, estart);
    k_unique_starts<<<grid_for(F + 1), kBlock, 0, s>>>(estart, uidx, nnz, F, d_total, ustart);
    std::vector<unsigned> h_ustart(F + 1);
    std::vector<long> h_estart(F + 1);
    HIP_CHECK(hipMemcpyAsync(h_ustart.data(), ustart, sizeof(unsigned) * (size_t)(F + 1), hipMemcpyDeviceToHost, s));
    HIP_CHECK(hipMemcpyAsync(h_estart.data(), estart, sizeof(long) * (size_t)(F + 1), hipMemcpyDeviceToHost, s));
    HIP_CHECK(hipStreamSynchronize(s));
    out.feature_nnz.resize(F);
    for (int f = 0; f < F; ++f) out.feature_nnz[f] = h_estart[f + 1] - h_estart[f];
    std::vector<int> h_crp(F + 1, 0);
    for (int f = 0; f < F; ++f) {
        unsigned m = h_ustart[f + 1] - h_ustart[f];
        unsigned k = (m / (unsigned)max_num_bin == 0) ? m : (unsigned)max_num_bin;
        h_crp[f + 1] = h_crp[f] + (int)k;
    }
    out.n_bins = h_crp[F];
    HIP_CHECK(hipMemcpyAsync(out.cut_row_ptr, h_crp.data(), sizeof(int) * (size_t)(F + 1), hipMemcpyHostToDevice, s));
    HIP_CHECK(hipMalloc(&out.cut_val, sizeof(float) * (size_t)std::max(out.n_bins, 1)));
    HIP_CHECK(hipMalloc(&out.cut_fid, sizeof(int) * (size_t)std::max(out.n_bins, 1)));
    k_emit_cuts<<<grid_for(nnz), kBlock, 0, s>>>(sorted, uidx, nnz, ustart, out.cut_row_ptr, max_num_bin, out.cut_val,
                                               out.cut_fid);
    HIP_CHECK(hipStreamSynchronize(s));
    scratch.release();
    HIP_CHECK(hipFree(keys[0]));
    HIP_CHECK(hipFree(keys[1]));
    HIP_CHECK(hipFree(counts));
    HIP_CHECK(hipFree(offsets));
    HIP_CHECK(hipFree(d_total));
    HIP_CHECK(hipFree(uidx));
    HIP_CHECK(hipFree(estart));
    HIP_CHECK(hipFree(ustart));
    return out;
}

// Largest element of n ints, with a check that none is negative (the values are column indices that the
// callers are about to use as array indices): returns 0 for n == 0 and aborts on a negative entry.
__global__ __launch_bounds__(256) void k_min_max_int(const int *__restrict__ v, long n, int *__restrict__ out) {
    int m = 0, lo = 0;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) {
        const int x = v[i];
        m = max(m, x);
        lo = min(lo, x);
    }
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) {
        m = max(m, __shfl_xor(m, d));
        lo = min(lo, __shfl_xor(lo, d));
    }
    if ((threadIdx.x & 63) == 0) {
        atomicMax(out, m);
        atomicMin(out + 1, lo);
    }
}

int device_max_int(hipStream_t s, const int *d_v, long n) {
    if (n <= 0) return 0;
    int *d_out = nullptr;
    HIP_CHECK(hipMalloc(&d_out, 2 * sizeof(int)));
    HIP_CHECK(hipMemsetAsync(d_out, 0, 2 * sizeof(int), s));
    k_min_max_int<<<grid_for((size_t)n, 4096), 256, 0, s>>>(d_v, n, d_out);
    int h[2] = {0, 0};
    HIP_CHECK(hipMemcpyAsync(h, d_out, 2 * sizeof(int), hipMemcpyDeviceToHost, s));
    HIP_CHECK(hipStreamSynchronize(s));
    HIP_CHECK(hipFree(d_out));
    TGBM_CHECK(h[1] >= 0, "CSR input: negative column index %d", h[1]);
    TGBM_CHECK(h[0] < 2147483647, "CSR input: column index %d leaves no room for the feature count", h[0]);
    return h[0];
}

// ---- physical re-ordering of the rows (see Trainer::reorder_rows) ---------------------------------
// Sort keys: the node a row ended in, numbered by its path from the root (left = 0, right = 1, padded to
// `depth` bits), so that the rows of every subtree - not only of every leaf - end up next to each other;
// payload: the row's current position.
__global__ __launch_bounds__(256) void k_reorder_keys(int n, int depth, const int *__restrict__ nid,
                                                     unsigned long long *__restrict__ keys, int *__restrict__ vals) {
    const int p = blockIdx.x * 256 + threadIdx.x;
    if (p >= n) return;
    const int x = max(nid[p], 0);                       // heap order: children of x are 2x + 1 and 2x + 2
    const int level = 31 - __clz(x + 1);
    const unsigned path = (unsigned)(x + 1 - (1 << level));
    keys[p] = (unsigned long long)(path << max(depth - level, 0));
    vals[p] = p;
}

// dst[p] = src[from[p]] for n rows of `words` dwords; consecutive lanes take consecutive dwords of a row.
__global__ __launch_bounds__(256) void k_gather_rows(int n, int words, const int *__restrict__ from,
                                                    const unsigned *__restrict__ src, unsigned *__restrict__ dst) {
    const size_t total = (size_t)n * words;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (size_t)gridDim.x * 256) {
        const size_t p = i / words, w = i % words;
        dst[i] = src[(size_t)from[p] * words + w];
    }
}

// perm_new[p] = perm_old[from[p]], or from[p] itself while the rows are still in their original order
__global__ __launch_bounds__(256) void k_gather_perm(int n, const int *__restrict__ from,
                                                    const int *__restrict__ perm_old, int *__restrict__ perm_new) {
    const int p = blockIdx.x * 256 + threadIdx.x;
    if (p >= n) return;
    const int f = from[p];
    perm_new[p] = perm_old != nullptr ? perm_old[f] : f;
}

// Column-major copy of one feature block from its row-major form: a tile of 256 rows x W bins goes through
// LDS so that both the reads (whole rows) and the writes (256 consecutive bins of one feature) are coalesced.
template <typename BinT>
__global__ __launch_bounds__(256) void k_cols_from_rows(int n, int W, int F, int block, const uint8_t *__restrict__ rows,
                                                       BinT *__restrict__ colmat, size_t col_stride) {
    extern __shared__ uint8_t tile[];  // [256][row bytes + 4]: the padding spreads a column's bins over the banks
    const int r0 = blockIdx.x * 256;
    const int row_bytes = W * (int)sizeof(BinT);
    const int pitch = row_bytes + 4;
    const int words = row_bytes / 4;
    for (int i = threadIdx.x; i < 256 * words; i += 256) {
        const int r = i / words, w = i % words;
        unsigned v = 0xffffffffu;
        if (r0 + r < n) v = reinterpret_cast<const unsigned *>(rows + (size_t)(r0 + r) * row_bytes)[w];
        *reinterpret_cast<unsigned *>(tile + r * pitch + w * 4) = v;
    }
    __syncthreads();
    const int r = threadIdx.x;
    if (r0 + r >= n) return;
    for (int j = 0; j < W; ++j) {
        const int f = block * W + j;
        if (f < F) colmat[(size_t)f * col_stride + r0 + r] = reinterpret_cast<const BinT *>(tile + r * pitch)[j];
    }
}

void launch_reorder_keys(hipStream_t s, int n, int depth, const int *nid, unsigned long long *keys, int *vals) {
    if (n > 0) k_reorder_keys<<<(n + 255) / 256, 256, 0, s>>>(n, depth, nid, keys, vals);
}

void launch_gather_rows(hipStream_t s, int n, int bytes_per_row, const int *from, const void *src, void *dst) {
    if (n <= 0) return;
    TGBM_CHECK(bytes_per_row % 4 == 0, "rows of %d bytes cannot be gathered by dwords", bytes_per_row);
    const int words = bytes_per_row / 4;
    k_gather_rows<<<grid_for((size_t)n * words, 65536), 256, 0, s>>>(n, words, from, static_cast<const unsigned *>(src),
                                                                      static_cast<unsigned *>(dst));
}

void launch_gather_perm(hipStream_t s, int n, const int *from, const int *perm_old, int *perm_new) {
    if (n > 0) k_gather_perm<<<(n + 255) / 256, 256, 0, s>>>(n, from, perm_old, perm_new);
}

void launch_cols_from_rows(hipStream_t s, int n, int W, int F, int n_blocks, const uint8_t *binmat, size_t block_stride,
                           uint8_t *colmat, size_t col_stride, int bin_bytes) {
    if (n <= 0) return;
    const size_t lds = (size_t)256 * (W * bin_bytes + 4);
    for (int b = 0; b < n_blocks; ++b) {
        const uint8_t *rows = binmat + (size_t)b * block_stride;
        if (bin_bytes == 2)
            k_cols_from_rows<uint16_t><<<(n + 255) / 256, 256, lds, s>>>(n, W, F, b, rows,
                                                                      reinterpret_cast<uint16_t *>(colmat), col_stride);
        else
            k_cols_from_rows<uint8_t><<<(n + 255) / 256, 256, lds, s>>>(n, W, F, b, rows, colmat, col_stride);
    }
}

void ScanScratch::release() {
    for (Level &lv : levels) {
        if (lv.sums) (void)hipFree(lv.sums);
        if (lv.scanned) (void)hipFree(lv.scanned);
    }
    levels.clear();
}

void device_exclusive_scan(hipStream_t s, const unsigned *in, unsigned *out, long n, unsigned *d_total,
                           ScanScratch &sc) {
    exclusive_scan<false>(s, in, out, n, d_total, sc);
}

void PairSorter::alloc(long n) {
    cap = n;
    const size_t m = (size_t)std::max(n, 1l);
    n_tiles = (n + kSortTile - 1) / kSortTile;
    const size_t n_counts = (size_t)256 * (size_t)std::max(n_tiles, 1l);
    for (int b = 0; b < 2; ++b) {
        HIP_CHECK(hipMalloc(&keys[b], sizeof(unsigned long long) * m));
        HIP_CHECK(hipMalloc(&vals[b], sizeof(int) * m));
    }
    HIP_CHECK(hipMalloc(&counts, sizeof(unsigned) * n_counts));
    HIP_CHECK(hipMalloc(&offsets, sizeof(unsigned) * (n_counts + 1)));
    HIP_CHECK(hipMalloc(&d_total, sizeof(unsigned)));
}

void PairSorter::release() {
    for (int b = 0; b < 2; ++b) {
        if (keys[b]) (void)hipFree(keys[b]);
        if (vals[b]) (void)hipFree(vals[b]);
        keys[b] = nullptr;
        vals[b] = nullptr;
    }
    if (counts) (void)hipFree(counts);
    if (offsets) (void)hipFree(offsets);
    if (d_total) (void)hipFree(d_total);
    counts = offsets = d_total = nullptr;
    scan.release();
    cap = 0;
}

int sort_pairs(hipStream_t s, PairSorter &ps, long n, int key_bits) {
    TGBM_CHECK(n <= ps.cap, "sort_pairs: %ld pairs exceed the sorter's capacity %ld", n, ps.cap);
    if (n <= 1) return 0;
    const long n_tiles = (n + kSortTile - 1) / kSortTile;
    const size_t n_counts = (size_t)256 * n_tiles;
    const unsigned sort_grid = (unsigned)((n_tiles + kWaves - 1) / kWaves);
    const int passes = (key_bits + 7) / 8;
    int cur = 0;
    for (int p = 0; p < passes; ++p) {
        const int shift = 8 * p;
        k_radix_count<<<sort_grid, kBlock, 0, s>>>(ps.keys[cur], n, shift, n_tiles, ps.counts);
        exclusive_scan<false>(s, ps.counts, ps.offsets, (long)n_counts, ps.d_total, ps.scan);
        k_radix_scatter<true><<<(unsigned)n_tiles, kBlock, 0, s>>>(ps.keys[cur], ps.keys[cur ^ 1], n, shift, n_tiles, ps.offsets,
                                                           ps.vals[cur], ps.vals[cur ^ 1]);
        cur ^= 1;
    }
    return cur;
}

void launch_bin_dense(hipStream_t s, int n, const int *row_ptr, const int *col, const float *val, const float *cut_val,
                      const int *cut_row_ptr, uint8_t *binmat, int W, size_t block_stride, uint8_t *colmat,
                      size_t col_stride, int bin_bytes, int F, const int *feat_col, const uint8_t *feat_lo,
                      bool rows_ascend) {
    const int grid = grid_for((size_t)n * 16, 1 << 20);
    if (!rows_ascend) {  // (no bundles then: the layout is chosen with one column per feature)
        if (bin_bytes == 2)
            k_bin_dense_serial<uint16_t><<<grid_for((size_t)n, 1 << 20), kBlock, 0, s>>>(
                n, row_ptr, col, val, cut_val, cut_row_ptr, reinterpret_cast<uint16_t *>(binmat), W, block_stride / 2);
        else
            k_bin_dense_serial<uint8_t><<<grid_for((size_t)n, 1 << 20), kBlock, 0, s>>>(n, row_ptr, col, val, cut_val,
                                                                                      cut_row_ptr, binmat, W, block_stride);
    } else if (bin_bytes == 2)
        k_bin_dense<uint16_t><<<grid, kBlock, 0, s>>>(n, row_ptr, col, val, cut_val, cut_row_ptr,
                                                     reinterpret_cast<uint16_t *>(binmat), W, block_stride / 2, nullptr,
                                                     nullptr);
    else
        k_bin_dense<uint8_t><<<grid, kBlock, 0, s>>>(n, row_ptr, col, val, cut_val, cut_row_ptr, binmat, W, block_stride,
                                                    feat_col, feat_lo);
    launch_cols_from_rows(s, n, W, F, (F + W - 1) / W, binmat, block_stride, colmat, col_stride, bin_bytes);
}

bool device_rows_ascend(hipStream_t s, int n, const int *row_ptr, const int *col) {
    if (n == 0) return true;
    int *d_flag = nullptr, h = 0;
    HIP_CHECK(hipMalloc(&d_flag, sizeof(int)));
    HIP_CHECK(hipMemsetAsync(d_flag, 0, sizeof(int), s));
    k_rows_ascend<<<grid_for((size_t)n * 16, 1 << 20), kBlock, 0, s>>>(n, row_ptr, col, d_flag);
    HIP_CHECK(hipMemcpyAsync(&h, d_flag, sizeof(int), hipMemcpyDeviceToHost, s));
    HIP_CHECK(hipStreamSynchronize(s));
    HIP_CHECK(hipFree(d_flag));
    return h == 0;
}

void launch_min_next_col(hipStream_t s, int n, const int *row_ptr, const int *col, int *min_next, int *descending) {
    if (n == 0) return;
    k_min_next_col<<<grid_for((size_t)n * 16, 1 << 20), kBlock, 0, s>>>(n, row_ptr, col, min_next, descending);
}

void launch_csc_keys(hipStream_t s, int n_rows, const int *row_ptr, const int *bin, const int *sort_key,
                     unsigned long long *keys, int *vals) {
    if (n_rows == 0) return;
    const int rows_per_block = kBlock / 64;
    k_csc_keys<<<(n_rows + rows_per_block - 1) / rows_per_block, kBlock, 0, s>>>(n_rows, row_ptr, bin, sort_key, keys,
                                                                                vals);
}

void launch_csc_unpack(hipStream_t s, long nnz, const unsigned long long *keys, const int *vals, int *csc_bin,
                       int *csc_row) {
    if (nnz == 0) return;
    k_csc_unpack<<<grid_for(nnz), kBlock, 0, s>>>(nnz, keys, vals, csc_bin, csc_row);
}

void launch_bin_csr(hipStream_t s, long nnz, const int *col, const float *val, const float *cut_val,
                    const int *cut_row_ptr, int *bin_id, const int *feat_slot, int *hist_word) {
    if (nnz == 0) return;
    k_bin_csr<<<grid_for(nnz), kBlock, 0, s>>>(nnz, col, val, cut_val, cut_row_ptr, bin_id, feat_slot, hist_word);
}

}  // namespace tgbm
