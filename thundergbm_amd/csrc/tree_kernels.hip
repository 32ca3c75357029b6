// Tree-building kernels for gfx950 (wave64): gradients, LDS-privatised histograms, merge + sibling
// subtraction, wavefront segmented-scan split finding, ballot/popcount row partition, pruning and the
// in-training prediction update. Every stage of a level is one launch over all nodes of the level;
// work lists are planned on the device so the host never waits inside a tree.
#include <algorithm>

#include "device_api.h"

namespace tgbm {
namespace {

constexpr int kBlock = 256;
constexpr int kWaves = kBlock / 64;
constexpr int kHistMinChunk = 1024;
#ifndef TGBM_HIST_BLOCK
#define TGBM_HIST_BLOCK 1024
#endif
constexpr int kHistBlock = TGBM_HIST_BLOCK;  // threads per histogram workgroup (they share one LDS histogram)
#ifndef TGBM_FLUSH_EVERY
#define TGBM_FLUSH_EVERY 8192
#endif
constexpr int kHistFlushEvery = TGBM_FLUSH_EVERY;  // timing experiments only; must equal kHistFlushRows
constexpr int kHistFlushRows = 8192;         // rows a packed 32+32-bit LDS bin may absorb before it is drained

__device__ __forceinline__ int lane_id() { return threadIdx.x & 63; }
__device__ __forceinline__ int wave_id() { return threadIdx.x >> 6; }
__device__ __forceinline__ int lanes_below(unsigned long long mask) {
    return __builtin_amdgcn_mbcnt_hi((unsigned)(mask >> 32), __builtin_amdgcn_mbcnt_lo((unsigned)mask, 0));
}

// Exclusive scan of one int per thread over a 256-thread block; lds needs kWaves ints.
__device__ int block_excl_scan(int v, int *lds, int *total) {
    int lane = lane_id(), w = wave_id();
    int inc = v;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        int t = __shfl_up(inc, d);
        if (lane >= d) inc += t;
    }
    if (lane == 63) lds[w] = inc;
    __syncthreads();
    int base = 0, tot = 0;
#pragma unroll
    for (int i = 0; i < kWaves; ++i) {
        int c = lds[i];
        if (i < w) base += c;
        tot += c;
    }
    *total = tot;
    __syncthreads();
    return base + inc - v;
}

__device__ int block_sum(int v, int *lds) {
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) v += __shfl_xor(v, d);
    if (lane_id() == 0) lds[wave_id()] = v;
    __syncthreads();
    int tot = 0;
#pragma unroll
    for (int i = 0; i < kWaves; ++i) tot += lds[i];
    __syncthreads();
    return tot;
}

__device__ __forceinline__ float wave_sum_f(float v) {
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) v += __shfl_xor(v, d);
    return v;
}

// Largest p in [0, n) with begin[p] <= item (begin is non-decreasing, begin[0] <= item < begin[n]).
__device__ int find_owner(const int *begin, int n, int item) {
    int lo = 0, hi = n;
    while (hi - lo > 1) {
        int mid = (lo + hi) >> 1;
        if (begin[mid] <= item)
            lo = mid;
        else
            hi = mid;
    }
    return lo;
}

// Plain streaming copy of 16-byte words; used to calibrate the profiler's HBM byte counters.
__global__ void k_calibration_copy(const uint4 *__restrict__ src, uint4 *__restrict__ dst, size_t n) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x)
        dst[i] = src[i];
}

// ------------------------------------------------------------------------------------ fills
__global__ void k_fill_f32(float *p, float v, size_t n) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) p[i] = v;
}
__global__ void k_fill_u32(unsigned *p, unsigned v, size_t n) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) p[i] = v;
}

// -------------------------------------------------------------------------------- gradients
// Squared / logistic: include/thundergbm/objective/regression_obj.h:130-154 of the reference.
__global__ void k_gradient_pointwise(int objective, int n, const float *__restrict__ y, const float *__restrict__ yp,
                                     GHPair *__restrict__ gh) {
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x) {
        float p = yp[i];
        GHPair o;
        if (objective == OBJ_SQUARE) {
            o.g = p - y[i];
            o.h = 1.f;
        } else {
            float s = 1.f / (1.f + expf(-p));
            o.g = s - y[i];
            o.h = fmaxf(s * (1.f - s), 1e-16f);
        }
        gh[i] = o;
    }
}

// Softmax: src/thundergbm/objective/multiclass_obj.cu:6-35 (class-major predictions and gradients,
// hessian 2p(1-p)).
__global__ void k_gradient_softmax(int n, int K, const float *__restrict__ y, const float *__restrict__ yp,
                                   GHPair *__restrict__ gh) {
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x) {
        float mx = yp[i];
        for (int k = 1; k < K; ++k) mx = fmaxf(mx, yp[(size_t)k * n + i]);
        float sum = 0;
        for (int k = 0; k < K; ++k) sum += expf(yp[(size_t)k * n + i] - mx);
        float yi = y[i];
        for (int k = 0; k < K; ++k) {
            float p = expf(yp[(size_t)k * n + i] - mx) / sum;
            GHPair o;
            o.g = (k == yi) ? (p - 1.f) : p;
            o.h = fmaxf(2.f * p * (1.f - p), 1e-16f);
            gh[(size_t)k * n + i] = o;
        }
    }
}

// Block sums of (g,h) and block maxima of |g|, h for one tree; fixed grid and fixed reduction order.
__global__ __launch_bounds__(kBlock) void k_sum_gh(int n, const GHPair *__restrict__ gh, GradStats *__restrict__ out) {
    __shared__ float sg[kWaves], sh[kWaves], mg[kWaves], mh[kWaves];
    float g = 0, h = 0, gm = 0, hm = 0;
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x) {
        GHPair v = gh[i];
        g += v.g;
        h += v.h;
        gm = fmaxf(gm, fabsf(v.g));
        hm = fmaxf(hm, v.h);
    }
    g = wave_sum_f(g);
    h = wave_sum_f(h);
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) {
        gm = fmaxf(gm, __shfl_xor(gm, d));
        hm = fmaxf(hm, __shfl_xor(hm, d));
    }
    if (lane_id() == 0) {
        sg[wave_id()] = g;
        sh[wave_id()] = h;
        mg[wave_id()] = gm;
        mh[wave_id()] = hm;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        GradStats o{0, 0, 0, 0};
        for (int i = 0; i < kWaves; ++i) {
            o.g += sg[i];
            o.h += sh[i];
            o.gmax = fmaxf(o.gmax, mg[i]);
            o.hmax = fmaxf(o.hmax, mh[i]);
        }
        out[blockIdx.x] = o;
    }
}

// Largest power of two s with rows * (vmax * s + 0.5) < limit; 1 when vmax is 0 or not finite.
__device__ float pow2_scale(float vmax, int rows, float limit) {
    if (!(vmax > 0.f) || !(vmax < INFINITY)) return 1.f;
    float bound = (limit / (float)rows - 0.5f) / vmax;
    if (!(bound < 1e18f)) bound = 1e18f;  // tiny gradients: keep the scale and its inverse well inside float range
    int e;
    frexpf(bound, &e);             // bound = m * 2^e, m in [0.5, 1)
    return ldexpf(1.f, e - 1);     // 2^(e-1) <= bound
}

// ------------------------------------------------------------------------------- tree init
// Node array initialisation of the reference's Tree::init2 (src/thundergbm/tree.cu:8-39), root sum
// from the block partials, root segment and the histogram plan of level 0. One workgroup.
__global__ __launch_bounds__(kBlock) void k_tree_init(TreeBuffers tb, const GradStats *__restrict__ block_sums,
                                                     float lambda) {
    __shared__ float sg[kWaves], sh[kWaves], mg[kWaves], mh[kWaves];
    const int nn = tb.n_nodes;
    for (int i = threadIdx.x; i < nn; i += kBlock) {
        TreeNode nd;
        nd.final_id = i;
        nd.parent_index = i == 0 ? -1 : (i - 1) / 2;
        nd.gain = 0;
        nd.base_weight = 0;
        nd.split_feature_id = -1;
        nd.split_value = 0;
        nd.split_bid = 0;
        nd.default_right = false;
        nd.is_valid = false;
        nd.is_pruned = false;
        nd.sum_gh_pair = GHPair{0, 0};
        if (i < nn / 2) {
            nd.is_leaf = false;
            nd.lch_index = 2 * i + 1;
            nd.rch_index = 2 * i + 2;
        } else {
            nd.is_leaf = true;
            nd.lch_index = -1;
            nd.rch_index = -1;
        }
        // zero the padding bytes too: nodes are written raw into model files
        unsigned *raw = reinterpret_cast<unsigned *>(&nd);
        raw[9] &= 0x000000ffu;  // bytes 37..39 are padding (byte 36 = is_pruned)
        tb.nodes[i] = nd;
        tb.seg[i] = make_int2(0, 0);
    }
    float g = 0, h = 0, gm = 0, hm = 0;
    for (int i = threadIdx.x; i < tb.n_grad_blocks; i += kBlock) {
        g += block_sums[i].g;
        h += block_sums[i].h;
        gm = fmaxf(gm, block_sums[i].gmax);
        hm = fmaxf(hm, block_sums[i].hmax);
    }
    g = wave_sum_f(g);
    h = wave_sum_f(h);
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) {
        gm = fmaxf(gm, __shfl_xor(gm, d));
        hm = fmaxf(hm, __shfl_xor(hm, d));
    }
    if (lane_id() == 0) {
        sg[wave_id()] = g;
        sh[wave_id()] = h;
        mg[wave_id()] = gm;
        mh[wave_id()] = hm;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        GHPair s{0, 0};
        gm = 0;
        hm = 0;
        for (int i = 0; i < kWaves; ++i) {
            s.g += sg[i];
            s.h += sh[i];
            gm = fmaxf(gm, mg[i]);
            hm = fmaxf(hm, mh[i]);
        }
        TreeNode &root = tb.nodes[0];
        root.sum_gh_pair = s;
        root.is_valid = true;
        root.base_weight = -s.g / (s.h + lambda);
        tb.seg[0] = make_int2(0, tb.n);
        int chunk = (tb.n + tb.target_hitems - 1) / tb.target_hitems;
        chunk = max(kHistMinChunk, (chunk + 255) / 256 * 256);
        int items = (tb.n + chunk - 1) / chunk;
        tb.hpair_begin[0] = 0;
        tb.hpair_begin[1] = items;
        tb.hpair_built[0] = 0;
        LevelCtl c;
        c.hchunk = chunk;
        c.n_hitems = items;
        c.n_pitems = 0;
        c.rows_built = tb.n;
        tb.ctl[0] = c;
        // One pair of scales serves the whole tree: between two drains of the LDS histogram at most
        // kHistFlushRows rows are added, which keeps a bin's gradient sum inside a signed and its
        // hessian sum inside an unsigned 32-bit field.
        QuantCtl q;
        if (tb.sparse) {
            // sums go straight into 64-bit integers: the whole dataset must fit below 2^62
            q.scale_g = pow2_scale(gm, tb.n, 4.6e18f);
            q.scale_h = pow2_scale(hm, tb.n, 4.6e18f);
        } else {
            q.scale_g = pow2_scale(gm, kHistFlushRows, 2147483520.f);  // largest float below 2^31
            q.scale_h = pow2_scale(hm, kHistFlushRows, 4294967040.f);  // largest float below 2^32
        }
        q.inv_g = 1.f / q.scale_g;
        q.inv_h = 1.f / q.scale_h;
        *tb.quant = q;
    }
}

// ------------------------------------------------------------------------- dense histogram
// One workgroup = one work item (a run of rows of one node) x one feature block. The block's
// histogram lives in LDS as one 64-bit integer per bin holding the fixed-point gradient sum in the
// high and the hessian sum in the low half; a row contributes with a single ds_add_u64 per feature
// (float LDS atomics run at ~0.3 lanes/clk/CU on gfx950, 64-bit integer ones at ~5). The 32-bit
// fields are safe for kHistFlushRows rows (that bound sets the fixed-point scales), so after at most
// that many rows every thread drains the bins it owns into 64-bit register accumulators and clears
// them; at the end the registers go to the item's slot of `partial`.
// LPR consecutive lanes cover one row (one dword = four bin bytes per lane), so a wavefront load
// instruction reads 256 contiguous bytes and the 64 atomics of one step spread over many features.
// (Packing each row's gradient pair next to its bins so that a gathered row costs one 128-byte line
// instead of two was measured: it halves the fetched bytes below the root, but the per-tree refresh of
// the pairs costs what the gathers save.)
template <int LPR, bool DIRECT, int BLK, int SLOTS>
__global__ __launch_bounds__(BLK) __attribute__((amdgpu_waves_per_eu(SLOTS <= 8 ? 8 : 4)))  // two 1024-thread groups per CU
void k_hist_dense(DenseBins bins, const GHPair *__restrict__ gh,
                                                    const int *__restrict__ ridx, const int2 *__restrict__ seg,
                                                    const int *__restrict__ hpair_begin,
                                                    const int *__restrict__ hpair_built, int n_pairs,
                                                    const LevelCtl *__restrict__ ctl,
                                                    const QuantCtl *__restrict__ quant,
                                                    const int *__restrict__ blk_bin_begin,
                                                    const int *__restrict__ feat_lds_off,
                                                    longlong2 *__restrict__ partial, int n_bins) {
    extern __shared__ unsigned long long lds[];
    __shared__ int s_range[2];
    const LevelCtl c = *ctl;
    const int item = blockIdx.x;
    if (item >= c.n_hitems) return;
    const int fb = blockIdx.y;
    const int bin0 = blk_bin_begin[fb];
    const int nb = blk_bin_begin[fb + 1] - bin0;
    if (nb == 0) return;
    if (threadIdx.x == 0) {
        int p = find_owner(hpair_begin, n_pairs, item);
        int node = hpair_built[p];
        int2 sg = seg[node];
        int b = sg.x + (item - hpair_begin[p]) * c.hchunk;
        s_range[0] = b;
        s_range[1] = min(sg.y, b + c.hchunk);
    }
    for (int i = threadIdx.x; i < nb; i += BLK) lds[i] = 0ull;
    __syncthreads();
    const int begin = s_range[0], end = s_range[1];
    const float scale_g = quant->scale_g, scale_h = quant->scale_h;
    constexpr int RPS = BLK / LPR;  // rows per step of the whole block
    constexpr int U = 4;
    static_assert(RPS * U <= kHistFlushRows, "one iteration must not exceed the flush interval");
    const int q = threadIdx.x % LPR;
    const int rsub = threadIdx.x / LPR;
    const int W = LPR * 4;
    const int *fo = feat_lds_off + fb * W + q * 4;
    const int o0 = fo[0], o1 = fo[1], o2 = fo[2], o3 = fo[3];
    const uint8_t *blk = bins.data + (size_t)fb * bins.block_stride + q * 4;
    long long accg[SLOTS], acch[SLOTS];
#pragma unroll
    for (int k = 0; k < SLOTS; ++k) accg[k] = acch[k] = 0;
    int pending = 0;  // rows accumulated in LDS since the last drain (uniform across the block)
    unsigned pk[U], pk_next[U];
    GHPair s[U], s_next[U];
    auto load_rows = [&](int base, unsigned(&opk)[U], GHPair(&os)[U]) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            int pos = base + rsub + u * RPS;
            bool ok = pos < end;
            int r = 0;
            if (ok) r = DIRECT ? pos : ridx[pos];
            opk[u] = ok ? *reinterpret_cast<const unsigned *>(blk + (size_t)r * W) : 0xffffffffu;
            os[u] = ok ? gh[r] : GHPair{0, 0};
        }
    };
    if (begin < end) load_rows(begin, pk, s);
    for (int base = begin; base < end; base += RPS * U) {
        // the next step's rows are requested before this step's atomics (and before a drain's
        // barriers), so the memory pipeline stays busy
        if (base + RPS * U < end) load_rows(base + RPS * U, pk_next, s_next);
        if (pending + RPS * U > kHistFlushEvery) {
            __syncthreads();
#pragma unroll
            for (int k = 0; k < SLOTS; ++k) {
                const int i = threadIdx.x + k * BLK;
                if (i < nb) {
                    const unsigned long long t = lds[i];
                    lds[i] = 0ull;
                    const unsigned lo = (unsigned)t;
                    accg[k] += (int)((long long)(t - lo) >> 32);
                    acch[k] += lo;
                }
            }
            __syncthreads();
            pending = 0;
        }
        pending += RPS * U;
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const unsigned v = pk[u];
            const int gq = __float2int_rn(s[u].g * scale_g);
            const unsigned hq = __float2uint_rn(s[u].h * scale_h);
            const unsigned long long add = ((unsigned long long)(long long)gq << 32) + hq;
            const unsigned b0 = v & 0xff, b1 = (v >> 8) & 0xff, b2 = (v >> 16) & 0xff, b3 = v >> 24;
            if (b0 != kMissingBin) atomicAdd(lds + o0 + b0, add);
            if (b1 != kMissingBin) atomicAdd(lds + o1 + b1, add);
            if (b2 != kMissingBin) atomicAdd(lds + o2 + b2, add);
            if (b3 != kMissingBin) atomicAdd(lds + o3 + b3, add);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            pk[u] = pk_next[u];
            s[u] = s_next[u];
        }
    }
    __syncthreads();
    longlong2 *out = partial + (size_t)item * n_bins + bin0;
#pragma unroll
    for (int k = 0; k < SLOTS; ++k) {
        const int i = threadIdx.x + k * BLK;
        if (i < nb) {
            const unsigned long long t = lds[i];
            const unsigned lo = (unsigned)t;
            out[i] = make_longlong2(accg[k] + (int)((long long)(t - lo) >> 32), acch[k] + lo);
        }
    }
}

// (Adding the work items' histograms straight into the node's histogram with global 64-bit atomics
// instead of storing and merging them was measured: 0.5 ms per tree slower on the 10M x 28 benchmark.)
// Sum the private histograms of the node that was built from rows (64-bit integers, exact, any
// order gives the same bits) and derive its sibling as parent - built (the reference's subtraction
// trick, hist_tree_builder_single.cu:526-540). A block covers 32 bins of one sibling pair; its eight
// thread groups stride over the pair's work items and are combined through LDS.
constexpr int kMergeBins = 32;
constexpr int kMergeGroups = kBlock / kMergeBins;

__global__ __launch_bounds__(kBlock) void k_hist_merge(const longlong2 *__restrict__ partial,
                                                      longlong2 *__restrict__ cur_q,
                                                      const longlong2 *__restrict__ prev_q,
                                                      const int *__restrict__ hpair_begin,
                                                      const int *__restrict__ hpair_built, int level, int n_bins) {
    __shared__ long long s_g[kMergeGroups][kMergeBins], s_h[kMergeGroups][kMergeBins];
    const int p = blockIdx.y;
    const int built = hpair_built[p];
    if (built < 0) return;
    const int jl = threadIdx.x % kMergeBins, ig = threadIdx.x / kMergeBins;
    const int j = blockIdx.x * kMergeBins + jl;
    const int ib = hpair_begin[p], ie = hpair_begin[p + 1];
    long long sg = 0, sh = 0;
    if (j < n_bins) {
        for (int it = ib + ig; it < ie; it += kMergeGroups) {
            longlong2 v = partial[(size_t)it * n_bins + j];
            sg += v.x;
            sh += v.y;
        }
    }
    s_g[ig][jl] = sg;
    s_h[ig][jl] = sh;
    __syncthreads();
    if (ig != 0 || j >= n_bins) return;
#pragma unroll
    for (int k = 1; k < kMergeGroups; ++k) {
        sg += s_g[k][jl];
        sh += s_h[k][jl];
    }
    const int off = (1 << level) - 1;
    cur_q[(size_t)(built - off) * n_bins + j] = make_longlong2(sg, sh);
    if (level > 0) {
        const int sib = (built & 1) ? built + 1 : built - 1;
        const longlong2 par = prev_q[(size_t)p * n_bins + j];
        cur_q[(size_t)(sib - off) * n_bins + j] = make_longlong2(par.x - sg, par.y - sh);
    }
}

// --------------------------------------------------------------------------- sparse histogram
// CSR rows of global bin ids: the histogram is too large for LDS (one slot per cut point of every
// feature), so every stored value adds its row's fixed-point gradient pair to the node's histogram
// in HBM with two 64-bit integer atomics (exact and order-independent, unlike the float atomics of
// hist_tree_builder_single.cu:203-216 / :485-505). One wavefront walks one row at a time.
__global__ __launch_bounds__(kBlock) void k_hist_zero_built(longlong2 *__restrict__ cur_q,
                                                           const int *__restrict__ hpair_built, int level,
                                                           int n_bins) {
    const int built = hpair_built[blockIdx.y];
    if (built < 0) return;
    const int off = (1 << level) - 1;
    longlong2 *h = cur_q + (size_t)(built - off) * n_bins;
    for (int j = blockIdx.x * kBlock + threadIdx.x; j < n_bins; j += gridDim.x * kBlock) h[j] = make_longlong2(0, 0);
}

template <bool DIRECT>
__global__ __launch_bounds__(kBlock) void k_hist_csr(TreeBuffers tb, CsrBins bins, const GHPair *__restrict__ gh,
                                                    const int *__restrict__ ridx, longlong2 *__restrict__ cur_q,
                                                    int n_pairs, int level) {
    __shared__ int s_info[3];
    const LevelCtl c = tb.ctl[level];
    const int item = blockIdx.x;
    if (item >= c.n_hitems) return;
    if (threadIdx.x == 0) {
        int p = find_owner(tb.hpair_begin, n_pairs, item);
        int node = tb.hpair_built[p];
        int2 sg = tb.seg[node];
        int b = sg.x + (item - tb.hpair_begin[p]) * c.hchunk;
        s_info[0] = b;
        s_info[1] = min(sg.y, b + c.hchunk);
        s_info[2] = node - ((1 << level) - 1);
    }
    __syncthreads();
    const int begin = s_info[0], end = s_info[1];
    unsigned long long *h = reinterpret_cast<unsigned long long *>(cur_q + (size_t)s_info[2] * tb.n_bins);
    const float scale_g = tb.quant->scale_g, scale_h = tb.quant->scale_h;
    const int lane = lane_id(), w = wave_id();
    for (int pos = begin + w; pos < end; pos += kWaves) {
        const int r = DIRECT ? pos : ridx[pos];
        const GHPair s = gh[r];
        const long long gq = __float2ll_rn(s.g * scale_g);
        const long long hq = __float2ll_rn(s.h * scale_h);
        const int e0 = bins.row_ptr[r], e1 = bins.row_ptr[r + 1];
        for (int e = e0 + lane; e < e1; e += 64) {
            const int b = bins.bin[e];
            atomicAdd(h + 2 * (size_t)b, (unsigned long long)gq);
            atomicAdd(h + 2 * (size_t)b + 1, (unsigned long long)hq);
        }
    }
}

__global__ __launch_bounds__(kBlock) void k_hist_sub_csr(longlong2 *__restrict__ cur_q,
                                                        const longlong2 *__restrict__ prev_q,
                                                        const int *__restrict__ hpair_built, int level, int n_bins) {
    const int p = blockIdx.y;
    const int built = hpair_built[p];
    if (built < 0) return;
    const int off = (1 << level) - 1;
    const int sib = (built & 1) ? built + 1 : built - 1;
    const longlong2 *b = cur_q + (size_t)(built - off) * n_bins;
    longlong2 *sq = cur_q + (size_t)(sib - off) * n_bins;
    const longlong2 *par = prev_q + (size_t)p * n_bins;
    for (int j = blockIdx.x * kBlock + threadIdx.x; j < n_bins; j += gridDim.x * kBlock) {
        longlong2 pv = par[j], bv = b[j];
        sq[j] = make_longlong2(pv.x - bv.x, pv.y - bv.y);
    }
}

// Left/right decision of the sparse layout: binary search of the row's bin ids for the one inside
// the split feature's bin range (absent = missing), hist_tree_builder_single.cu:941-1011.
template <bool DIRECT>
__global__ __launch_bounds__(kBlock) void k_part_count_csr(TreeBuffers tb, CsrBins bins, const int *__restrict__ ridx,
                                                          int level) {
    __shared__ int lds[kWaves];
    __shared__ int s_x;
    const int item = blockIdx.x;
    if (item >= tb.ctl[level].n_pitems) return;
    const int nl = 1 << level, off = nl - 1;
    if (threadIdx.x == 0) s_x = find_owner(tb.pitem_begin, nl, item);
    __syncthreads();
    const int x_in = s_x;
    const TreeNode &nd = tb.nodes[off + x_in];
    const int2 sg = tb.seg[off + x_in];
    const int pb = sg.x + (item - tb.pitem_begin[x_in]) * kPartChunk;
    const int pe = min(sg.y, pb + kPartChunk);
    const int f = nd.split_feature_id;
    const int cb = tb.cut_row_ptr[f], ce = tb.cut_row_ptr[f + 1];
    const int sbid = cb + nd.split_bid;
    const bool dr = nd.default_right;
    int nleft = 0;
#pragma unroll
    for (int k = 0; k < kPartChunk / kBlock; ++k) {
        int pos = pb + k * kBlock + threadIdx.x;
        if (pos < pe) {
            int row = DIRECT ? pos : ridx[pos];
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
            bool right = found < 0 ? dr : (found >= sbid);
            tb.goes_right[pos] = right ? 1 : 0;
            nleft += right ? 0 : 1;
        }
    }
    int tot = block_sum(nleft, lds);
    if (threadIdx.x == 0) tb.pitem_nleft[item] = tot;
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

__device__ __forceinline__ long long shfl_up_ll(long long v, int d) {
    int lo = __shfl_up((int)(unsigned)(unsigned long long)v, d);
    int hi = __shfl_up((int)((unsigned long long)v >> 32), d);
    return (long long)(((unsigned long long)(unsigned)hi << 32) | (unsigned)lo);
}

// Split search. One wavefront scans one pack of whole features (at most 256 bins, 4 consecutive bins
// per lane) of one node with a segmented inclusive prefix sum over the exact 64-bit fixed-point
// histogram: integer sums are associative, so the parallel scan returns bit-for-bit what a
// sequential one would, and candidates separated only by empty bins tie exactly. Per candidate:
// left = sum of the feature's bins below it, missing = node sum - feature total, gain with missing
// values sent right and left (hist_tree_builder_single.cu:257-325 / :614-681 of the reference);
// the wavefront keeps its best candidate: largest |gain|, ties to the smaller bin index (:330-335).
__global__ __launch_bounds__(kBlock) void k_eval_split(TreeBuffers tb, const longlong2 *__restrict__ hist_q, int level,
                                                      float mcw, float lambda) {
#pragma clang fp contract(off)
    __shared__ GHPair s_miss[kWaves][kEvalPackBins];
    const int lane = lane_id(), w = wave_id();
    const int pack = blockIdx.x * kWaves + w;
    const int x_in = blockIdx.y;
    const int x = (1 << level) - 1 + x_in;
    const TreeNode nd = tb.nodes[x];
    const bool active = pack < tb.n_packs && nd.is_valid;
    int b_begin = 0, b_end = 0;
    if (active) {
        b_begin = tb.pack_begin[pack];
        b_end = tb.pack_begin[pack + 1];
    }
    const GHPair S = nd.sum_gh_pair;
    const longlong2 *h = hist_q + (size_t)x_in * tb.n_bins;
    const double inv_g = tb.quant->inv_g, inv_h = tb.quant->inv_h;

    long long incg[4], inch[4];
    int lastb[4];  // pack-relative index of the last bin of the element's feature
    bool valid[4], head[4], last[4];
    long long rung = 0, runh = 0;
    bool any_head = false;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        int b = b_begin + lane * 4 + j;
        valid[j] = b < b_end;
        lastb[j] = 0;
        head[j] = false;
        last[j] = false;
        incg[j] = inch[j] = 0;
        if (valid[j]) {
            longlong2 v = h[b];
            const int f = tb.cut_fid[b];
            const int fend = tb.cut_row_ptr[f + 1];
            head[j] = tb.cut_row_ptr[f] == b;
            last[j] = fend == b + 1;
            lastb[j] = fend - 1 - b_begin;
            if (head[j]) {
                rung = v.x;
                runh = v.y;
                any_head = true;
            } else {
                rung += v.x;
                runh += v.y;
            }
            incg[j] = rung;
            inch[j] = runh;
        }
    }
    // wavefront segmented inclusive scan of the lane aggregates
    long long aggg = rung, aggh = runh;
    int flag = any_head ? 1 : 0;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        long long pg = shfl_up_ll(aggg, d);
        long long ph = shfl_up_ll(aggh, d);
        int pf = __shfl_up(flag, d);
        if (lane >= d) {
            if (!flag) {
                aggg += pg;
                aggh += ph;
            }
            flag |= pf;
        }
    }
    long long carryg = shfl_up_ll(aggg, 1), carryh = shfl_up_ll(aggh, 1);
    if (lane == 0) carryg = carryh = 0;
    bool seen = false;
    long long exg[4], exh[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        if (valid[j]) {
            if (head[j]) seen = true;
            if (!seen) {
                incg[j] += carryg;
                inch[j] += carryh;
            }
        }
        if (head[j]) {
            exg[j] = exh[j] = 0;
        } else {
            exg[j] = (j == 0) ? carryg : incg[j > 0 ? j - 1 : 0];
            exh[j] = (j == 0) ? carryh : inch[j > 0 ? j - 1 : 0];
        }
        if (valid[j] && last[j]) {
            const float tg = (float)((double)incg[j] * inv_g), th = (float)((double)inch[j] * inv_h);
            s_miss[w][lastb[j]] = GHPair{S.g - tg, S.h - th};
        }
    }
    __syncthreads();
    float best = -1.f;  // |score| of the lane's best candidate
    float best_score = 0.f;
    int best_idx = 0x7fffffff;
    GHPair best_miss{0, 0}, best_left{0, 0};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        if (valid[j]) {
            const GHPair m = s_miss[w][lastb[j]];
            const GHPair l{(float)((double)exg[j] * inv_g), (float)((double)exh[j] * inv_h)};
            float gr = split_gain(S, l, mcw, lambda);
            GHPair l2{l.g + m.g, l.h + m.h};
            float gl = split_gain(S, l2, mcw, lambda);
            float score = (gl > gr) ? gl : -gr;
            float a = fabsf(score);
            if (a > best) {
                best = a;
                best_score = score;
                best_idx = b_begin + lane * 4 + j;
                best_miss = m;
                best_left = l;
            }
        }
    }
    // wavefront arg-max: larger |score| wins, ties go to the smaller bin index
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) {
        float oa = __shfl_xor(best, d);
        float os = __shfl_xor(best_score, d);
        int oi = __shfl_xor(best_idx, d);
        float omg = __shfl_xor(best_miss.g, d), omh = __shfl_xor(best_miss.h, d);
        float olg = __shfl_xor(best_left.g, d), olh = __shfl_xor(best_left.h, d);
        if (oa > best || (oa == best && oi < best_idx)) {
            best = oa;
            best_score = os;
            best_idx = oi;
            best_miss = GHPair{omg, omh};
            best_left = GHPair{olg, olh};
        }
    }
    if (active && lane == 0) {
        SplitCand c;
        c.score = best_score;
        c.index = best_idx;
        c.miss = best_miss;
        c.left = best_left;
        c.pad[0] = c.pad[1] = 0;
        tb.cand[(size_t)x_in * tb.n_packs + pack] = c;
    }
}

// Per node: reduce the wavefront candidates, fill the split record (hist_tree_builder_single.cu
// :365-389) and apply it to the tree (update_tree, :860-899). One workgroup per node of the level.
__global__ __launch_bounds__(kBlock) void k_best_update(TreeBuffers tb, int level, float rt_eps, float lambda) {
    __shared__ float s_abs[kWaves];
    __shared__ int s_idx[kWaves];
    __shared__ int s_pack[kWaves];
    const int x_in = blockIdx.x;
    const int x = (1 << level) - 1 + x_in;
    TreeNode &node = tb.nodes[x];
    SplitPoint &sp = tb.sp[x_in];
    if (!node.is_valid) {
        if (threadIdx.x == 0) {
            SplitPoint z{};
            z.nid = -1;
            z.split_fea_id = -1;
            sp = z;
        }
        return;
    }
    float best = -1.f;
    int best_idx = 0x7fffffff, best_pack = -1;
    for (int p = threadIdx.x; p < tb.n_packs; p += kBlock) {
        const SplitCand &c = tb.cand[(size_t)x_in * tb.n_packs + p];
        if (c.index == 0x7fffffff) continue;  // a wavefront whose features have no bins
        float a = fabsf(c.score);
        if (a > best || (a == best && c.index < best_idx)) {
            best = a;
            best_idx = c.index;
            best_pack = p;
        }
    }
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) {
        float oa = __shfl_xor(best, d);
        int oi = __shfl_xor(best_idx, d);
        int op = __shfl_xor(best_pack, d);
        if (oa > best || (oa == best && oi < best_idx)) {
            best = oa;
            best_idx = oi;
            best_pack = op;
        }
    }
    if (lane_id() == 0) {
        s_abs[wave_id()] = best;
        s_idx[wave_id()] = best_idx;
        s_pack[wave_id()] = best_pack;
    }
    __syncthreads();
    if (threadIdx.x != 0) return;
    for (int i = 0; i < kWaves; ++i) {
        if (s_abs[i] > best || (s_abs[i] == best && s_idx[i] < best_idx)) {
            best = s_abs[i];
            best_idx = s_idx[i];
            best_pack = s_pack[i];
        }
    }
    const SplitCand c = tb.cand[(size_t)x_in * tb.n_packs + best_pack];
    const int f = tb.cut_fid[c.index];
    const int fbegin = tb.cut_row_ptr[f];
    SplitPoint s{};
    s.split_fea_id = f;
    s.nid = x;
    s.gain = fabsf(c.score);
    s.split_bid = (int)(unsigned char)(c.index - fbegin);
    s.fea_missing_gh = c.miss;
    s.default_right = c.score < 0;
    s.best_index = c.index;
    if (c.index != fbegin) {
        s.lch_sum_gh = c.left;
        s.fval = tb.cut_val[c.index - 1];
    } else {
        s.lch_sum_gh = GHPair{0, 0};
        float c0 = tb.cut_val[fbegin];
        s.fval = (float)((double)(c0 - fabsf(c0)) - 1e-5);
    }
    sp = s;
    if (s.gain > rt_eps) {
        node.gain = s.gain;
        TreeNode &l = tb.nodes[node.lch_index];
        TreeNode &r = tb.nodes[node.rch_index];
        l.is_valid = true;
        r.is_valid = true;
        node.split_feature_id = f;
        node.split_value = s.fval;
        node.split_bid = (unsigned char)s.split_bid;
        GHPair ls = s.lch_sum_gh;
        if (!s.default_right) {
            ls.g += s.fea_missing_gh.g;
            ls.h += s.fea_missing_gh.h;
            node.default_right = false;
        } else {
            node.default_right = true;
        }
        GHPair rs{node.sum_gh_pair.g - ls.g, node.sum_gh_pair.h - ls.h};
        l.sum_gh_pair = ls;
        r.sum_gh_pair = rs;
        l.base_weight = -ls.g / (ls.h + lambda);
        r.base_weight = -rs.g / (rs.h + lambda);
    } else {
        node.is_leaf = true;
        tb.nodes[node.lch_index].is_valid = false;
        tb.nodes[node.rch_index].is_valid = false;
    }
}

// ------------------------------------------------------------------------------ partition
__device__ __forceinline__ bool node_splits(const TreeNode &nd) {
    return nd.is_valid && !nd.is_leaf && nd.split_feature_id >= 0;
}

// Partition work items: every node of the level that was split gets ceil(rows / kPartChunk) items.
__global__ __launch_bounds__(kBlock) void k_part_plan(TreeBuffers tb, int level) {
    __shared__ int lds[kWaves];
    const int nl = 1 << level, off = nl - 1;
    int carry = 0;
    for (int base = 0; base < nl; base += kBlock) {
        int x_in = base + threadIdx.x;
        int cnt = 0;
        if (x_in < nl) {
            const TreeNode &nd = tb.nodes[off + x_in];
            int2 sg = tb.seg[off + x_in];
            if (node_splits(nd)) cnt = (sg.y - sg.x + kPartChunk - 1) / kPartChunk;
        }
        int tot;
        int ex = block_excl_scan(cnt, lds, &tot);
        if (x_in < nl) tb.pitem_begin[x_in] = carry + ex;
        carry += tot;
    }
    if (threadIdx.x == 0) {
        tb.pitem_begin[nl] = carry;
        tb.ctl[level].n_pitems = carry;
    }
}

// Decide left/right for every row of a work item from the split feature's column of the bin matrix
// (missing -> default direction, else right iff bin >= split bin; the reference's rule at
// hist_tree_builder_single.cu:986-1011) and count the rows that go left.
template <bool DIRECT>
__global__ __launch_bounds__(kBlock) void k_part_count_dense(TreeBuffers tb, DenseBins bins,
                                                            const int *__restrict__ ridx, int level) {
    __shared__ int lds[kWaves];
    __shared__ int s_x;
    const int item = blockIdx.x;
    if (item >= tb.ctl[level].n_pitems) return;
    const int nl = 1 << level, off = nl - 1;
    if (threadIdx.x == 0) s_x = find_owner(tb.pitem_begin, nl, item);
    __syncthreads();
    const int x_in = s_x;
    const TreeNode &nd = tb.nodes[off + x_in];
    const int2 sg = tb.seg[off + x_in];
    const int pb = sg.x + (item - tb.pitem_begin[x_in]) * kPartChunk;
    const int pe = min(sg.y, pb + kPartChunk);
    const int f = nd.split_feature_id;
    const int sbid = nd.split_bid;
    const bool dr = nd.default_right;
    const uint8_t *column = bins.col + (size_t)f * bins.col_stride;
    int nleft = 0;
#pragma unroll
    for (int k = 0; k < kPartChunk / kBlock; ++k) {
        int pos = pb + k * kBlock + threadIdx.x;
        if (pos < pe) {
            int row = DIRECT ? pos : ridx[pos];
            int b = column[row];
            bool right = (b == kMissingBin) ? dr : (b >= sbid);
            tb.goes_right[pos] = right ? 1 : 0;
            nleft += right ? 0 : 1;
        }
    }
    int tot = block_sum(nleft, lds);
    if (threadIdx.x == 0) tb.pitem_nleft[item] = tot;
}

// Scan the per-item left counts, publish the children's row segments and plan the histogram work
// of the next level: per sibling pair the child with fewer rows is built (ties: the left one, as
// hist_tree_builder_single.cu:466-467), the other one comes from subtraction. One workgroup.
__global__ __launch_bounds__(kBlock) void k_part_scan_plan(TreeBuffers tb, int level) {
    __shared__ int lds[kWaves];
    const int nl = 1 << level, off = nl - 1;
    const int n_p = tb.ctl[level].n_pitems;
    int carry = 0;
    constexpr int IPT = 8;  // items per thread and step
    for (int base = 0; base < n_p; base += kBlock * IPT) {
        const int i0 = base + threadIdx.x * IPT;
        int v[IPT];
        int local = 0;
#pragma unroll
        for (int j = 0; j < IPT; ++j) {
            v[j] = (i0 + j) < n_p ? tb.pitem_nleft[i0 + j] : 0;
            local += v[j];
        }
        int tot;
        int run = carry + block_excl_scan(local, lds, &tot);
#pragma unroll
        for (int j = 0; j < IPT; ++j) {
            if (i0 + j < n_p) tb.pitem_loff[i0 + j] = run;
            run += v[j];
        }
        carry += tot;
    }
    if (threadIdx.x == 0) tb.pitem_loff[n_p] = carry;
    __syncthreads();
    // children segments + rows of the built child of every pair
    int rows_sum = 0;
    for (int x_in = threadIdx.x; x_in < nl; x_in += kBlock) {
        const TreeNode &nd = tb.nodes[off + x_in];
        const int2 sg = tb.seg[off + x_in];
        int built = -1;
        if (node_splits(nd)) {
            int nleft = tb.pitem_loff[tb.pitem_begin[x_in + 1]] - tb.pitem_loff[tb.pitem_begin[x_in]];
            int nright = (sg.y - sg.x) - nleft;
            tb.node_nleft[x_in] = nleft;
            tb.seg[nd.lch_index] = make_int2(sg.x, sg.x + nleft);
            tb.seg[nd.rch_index] = make_int2(sg.x + nleft, sg.y);
            built = (nleft <= nright) ? nd.lch_index : nd.rch_index;
            rows_sum += min(nleft, nright);
        } else {
            tb.node_nleft[x_in] = 0;
            tb.seg[nd.lch_index] = make_int2(0, 0);
            tb.seg[nd.rch_index] = make_int2(0, 0);
        }
        tb.hpair_built[x_in] = built;
    }
    const int total_rows = block_sum(rows_sum, lds);
    int chunk = (total_rows + tb.target_hitems - 1) / tb.target_hitems;
    chunk = max(kHistMinChunk, (chunk + 255) / 256 * 256);
    carry = 0;
    for (int base = 0; base < nl; base += kBlock) {
        int x_in = base + threadIdx.x;
        int cnt = 0;
        if (x_in < nl) {
            int built = tb.hpair_built[x_in];
            if (built >= 0) {
                int2 sg = tb.seg[built];
                cnt = (sg.y - sg.x + chunk - 1) / chunk;
            }
        }
        int tot;
        int ex = block_excl_scan(cnt, lds, &tot);
        if (x_in < nl) tb.hpair_begin[x_in] = carry + ex;
        carry += tot;
    }
    if (threadIdx.x == 0) {
        tb.hpair_begin[nl] = carry;
        LevelCtl c;
        c.hchunk = chunk;
        c.n_hitems = carry;
        c.n_pitems = 0;
        c.rows_built = total_rows;
        tb.ctl[level + 1] = c;
    }
}

// Stable two-way compaction of a work item's rows into the children's segments with wavefront
// ballots and popcounts. (Moving the gradient pairs along with the row ids was measured: it makes
// the histogram's gradient reads sequential but costs more in this kernel than it saves there.) The row -> node map is not touched here; it is rebuilt from the segments
// when it is needed (k_nid_plan / k_nid_write).
template <bool DIRECT>
__global__ __launch_bounds__(kBlock) void k_part_scatter(TreeBuffers tb, const int *__restrict__ ridx_cur,
                                                        int *__restrict__ ridx_next, int level) {
    __shared__ int s_x;
    __shared__ int s_cnt[2][kWaves];
    const int item = blockIdx.x;
    if (item >= tb.ctl[level].n_pitems) return;
    const int nl = 1 << level, off = nl - 1;
    if (threadIdx.x == 0) s_x = find_owner(tb.pitem_begin, nl, item);
    __syncthreads();
    const int x_in = s_x;
    const int2 sg = tb.seg[off + x_in];
    const int first_item = tb.pitem_begin[x_in];
    const int pb = sg.x + (item - first_item) * kPartChunk;
    const int pe = min(sg.y, pb + kPartChunk);
    const int loff = tb.pitem_loff[item] - tb.pitem_loff[first_item];
    int left_base = sg.x + loff;
    int right_base = sg.x + tb.node_nleft[x_in] + ((pb - sg.x) - loff);
    const int lane = lane_id(), w = wave_id();
    for (int k = 0; k < kPartChunk / kBlock; ++k) {
        int pos = pb + k * kBlock + threadIdx.x;
        bool valid = pos < pe;
        int row = 0;
        bool right = false;
        if (valid) {
            row = DIRECT ? pos : ridx_cur[pos];
            right = tb.goes_right[pos] != 0;
        }
        unsigned long long mL = __ballot(valid && !right);
        unsigned long long mR = __ballot(valid && right);
        if (lane == 0) {
            s_cnt[0][w] = __popcll(mL);
            s_cnt[1][w] = __popcll(mR);
        }
        __syncthreads();
        int bL = 0, bR = 0, tL = 0, tR = 0;
#pragma unroll
        for (int i = 0; i < kWaves; ++i) {
            int cl = s_cnt[0][i], cr = s_cnt[1][i];
            if (i < w) {
                bL += cl;
                bR += cr;
            }
            tL += cl;
            tR += cr;
        }
        if (valid) {
            int dest = right ? right_base + bR + lanes_below(mR) : left_base + bL + lanes_below(mL);
            ridx_next[dest] = row;
        }
        left_base += tL;
        right_base += tR;
        __syncthreads();
    }
}

// Row -> node map (the reference's ins2node_id) from the row lists: a node holds rows iff it is valid
// and was not split; its rows are its segment of the row list of its level's parity. Planning is one
// workgroup over all nodes, writing is one workgroup per kPartChunk rows.
__global__ __launch_bounds__(kBlock) void k_nid_plan(TreeBuffers tb) {
    __shared__ int lds[kWaves];
    int carry = 0;
    for (int base = 0; base < tb.n_nodes; base += kBlock) {
        int x = base + threadIdx.x;
        int cnt = 0;
        if (x < tb.n_nodes) {
            const TreeNode &nd = tb.nodes[x];
            int2 sg = tb.seg[x];
            if (nd.is_valid && nd.split_feature_id < 0) cnt = (sg.y - sg.x + kPartChunk - 1) / kPartChunk;
        }
        int tot;
        int ex = block_excl_scan(cnt, lds, &tot);
        if (x < tb.n_nodes) tb.fitem_begin[x] = carry + ex;
        carry += tot;
    }
    if (threadIdx.x == 0) tb.fitem_begin[tb.n_nodes] = carry;
}

__global__ __launch_bounds__(kBlock) void k_nid_write(TreeBuffers tb) {
    __shared__ int s_x;
    const int item = blockIdx.x;
    if (item >= tb.fitem_begin[tb.n_nodes]) return;
    if (threadIdx.x == 0) s_x = find_owner(tb.fitem_begin, tb.n_nodes, item);
    __syncthreads();
    const int x = s_x;
    const int level = 31 - __clz(x + 1);
    const int2 sg = tb.seg[x];
    const int pb = sg.x + (item - tb.fitem_begin[x]) * kPartChunk;
    const int pe = min(sg.y, pb + kPartChunk);
    const int *ridx = tb.ridx[level & 1];
    for (int pos = pb + threadIdx.x; pos < pe; pos += kBlock) {
        int row = level == 0 ? pos : ridx[pos];
        tb.nid[row] = x;
    }
}

// ---------------------------------------------------------------------------------- prune
// Bottom-up, level-parallel form of the reference's Tree::prune_self (src/thundergbm/tree.cu:96-128):
// a node whose two children are valid leaves and whose gain is below gamma becomes a leaf and its
// children are marked pruned; then final ids are renumbered over valid, unpruned nodes.
__global__ __launch_bounds__(kBlock) void k_prune(TreeBuffers tb, float gamma) {
    __shared__ int lds[kWaves];
    for (int level = tb.depth - 1; level >= 0; --level) {
        const int nl = 1 << level, off = nl - 1;
        for (int x_in = threadIdx.x; x_in < nl; x_in += kBlock) {
            TreeNode &p = tb.nodes[off + x_in];
            if (p.is_valid && !p.is_leaf) {
                TreeNode &l = tb.nodes[p.lch_index];
                TreeNode &r = tb.nodes[p.rch_index];
                if (l.is_valid && l.is_leaf && r.is_valid && r.is_leaf && p.gain < gamma) {
                    l.is_pruned = true;
                    r.is_pruned = true;
                    p.is_leaf = true;
                }
            }
        }
        __syncthreads();
    }
    int carry = 0;
    for (int base = 0; base < tb.n_nodes; base += kBlock) {
        int i = base + threadIdx.x;
        int keep = 0;
        if (i < tb.n_nodes) keep = (tb.nodes[i].is_valid && !tb.nodes[i].is_pruned) ? 1 : 0;
        int tot;
        int ex = block_excl_scan(keep, lds, &tot);
        if (keep) tb.nodes[i].final_id = carry + ex;
        carry += tot;
    }
}

// y_pred += lr * weight of the (unpruned) leaf the row ended in (tree_builder.cu:62-74).
__global__ void k_predict_in_training(int n, const int *__restrict__ nid, const TreeNode *__restrict__ nodes,
                                      float *__restrict__ yp, float lr) {
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x) {
        int x = nid[i];
        while (x != -1 && nodes[x].is_pruned) x = nodes[x].parent_index;
        yp[i] += lr * nodes[x].base_weight;
    }
}

// ------------------------------------------------------------------- fused end of a round
// For objectives with one tree per round: the in-training prediction update (tree_builder.cu:62-74),
// the training metric partials (pointwise_metric.cu:13-20 / multiclass_metric.cu:39-44), the next
// round's gradients (regression_obj.h:130-154) and their block statistics for the next tree's root
// in one pass over the rows. Same grids, loops and arithmetic as k_predict_in_training,
// k_metric_partial, k_gradient_pointwise and k_sum_gh, so the results are bit-identical to running
// those four kernels.
__global__ __launch_bounds__(kBlock) void k_round_end_fused(int n, int objective, int metric_kind,
                                                           const int *__restrict__ nid,
                                                           const TreeNode *__restrict__ nodes,
                                                           const float *__restrict__ y, float *__restrict__ yp,
                                                           float lr, GHPair *__restrict__ gh,
                                                           GradStats *__restrict__ stats,
                                                           double *__restrict__ metric_out) {
    __shared__ float sg[kWaves], sh[kWaves], mg[kWaves], mh[kWaves];
    __shared__ double sd[kWaves];
    float g = 0, h = 0, gm = 0, hm = 0;
    double acc = 0;
    float accf = 0;
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x) {
        int x = nid[i];
        while (x != -1 && nodes[x].is_pruned) x = nodes[x].parent_index;
        float p = yp[i];
        p += lr * nodes[x].base_weight;
        yp[i] = p;
        const float yi = y[i];
        if (metric_kind == 0) {
            float e = p - yi;
            accf += e * e;
        } else {
            int k = (1.0 / (1.0 + exp(-(double)p)) > 0.5) ? 1 : 0;
            acc += (k == yi) ? 1 : 0;
        }
        GHPair o;
        if (objective == OBJ_SQUARE) {
            o.g = p - yi;
            o.h = 1.f;
        } else {
            float sgm = 1.f / (1.f + expf(-p));
            o.g = sgm - yi;
            o.h = fmaxf(sgm * (1.f - sgm), 1e-16f);
        }
        gh[i] = o;
        g += o.g;
        h += o.h;
        gm = fmaxf(gm, fabsf(o.g));
        hm = fmaxf(hm, o.h);
    }
    acc += (double)accf;
    g = wave_sum_f(g);
    h = wave_sum_f(h);
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) {
        gm = fmaxf(gm, __shfl_xor(gm, d));
        hm = fmaxf(hm, __shfl_xor(hm, d));
        acc += __shfl_xor(acc, d);
    }
    if (lane_id() == 0) {
        sg[wave_id()] = g;
        sh[wave_id()] = h;
        mg[wave_id()] = gm;
        mh[wave_id()] = hm;
        sd[wave_id()] = acc;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        GradStats o{0, 0, 0, 0};
        double s = 0;
        for (int i = 0; i < kWaves; ++i) {
            o.g += sg[i];
            o.h += sh[i];
            o.gmax = fmaxf(o.gmax, mg[i]);
            o.hmax = fmaxf(o.hmax, mh[i]);
            s += sd[i];
        }
        stats[blockIdx.x] = o;
        metric_out[blockIdx.x] = s;
    }
}

// ---------------------------------------------------------------------------------- metric
// kind 0: sum of squared errors; 1: correct binary decisions (sigmoid > 0.5 in double, like
// multiclass_metric.cu:40); 2: correct arg-max decisions (first maximum wins, :17-29).
__global__ __launch_bounds__(kBlock) void k_metric_partial(int kind, int n, int K, const float *__restrict__ y,
                                                          const float *__restrict__ yp, double *__restrict__ out) {
    __shared__ double sd[kWaves];
    double acc = 0;
    float accf = 0;
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x) {
        if (kind == 0) {
            float e = yp[i] - y[i];
            accf += e * e;
        } else if (kind == 1) {
            int k = (1.0 / (1.0 + exp(-(double)yp[i])) > 0.5) ? 1 : 0;
            acc += (k == y[i]) ? 1 : 0;
        } else {
            int mk = 0;
            float mp = yp[i];
            for (int k = 1; k < K; ++k) {
                float v = yp[(size_t)k * n + i];
                if (v > mp) {
                    mp = v;
                    mk = k;
                }
            }
            acc += (mk == y[i]) ? 1 : 0;
        }
    }
    acc += (double)accf;
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) acc += __shfl_xor(acc, d);
    if (lane_id() == 0) sd[wave_id()] = acc;
    __syncthreads();
    if (threadIdx.x == 0) {
        double s = 0;
        for (int i = 0; i < kWaves; ++i) s += sd[i];
        out[blockIdx.x] = s;
    }
}

__global__ __launch_bounds__(kBlock) void k_metric_final(int kind, int n, int n_blocks, const double *__restrict__ in,
                                                        float *__restrict__ out) {
    __shared__ double sd[kWaves];
    double acc = 0;
    for (int i = threadIdx.x; i < n_blocks; i += kBlock) acc += in[i];
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) acc += __shfl_xor(acc, d);
    if (lane_id() == 0) sd[wave_id()] = acc;
    __syncthreads();
    if (threadIdx.x == 0) {
        double s = 0;
        for (int i = 0; i < kWaves; ++i) s += sd[i];
        if (kind == 0) {
            out[0] = sqrtf((float)s / n);
        } else {
            float a = (float)s / (float)n;
            out[0] = kind == 1 ? 1.f - a : a;
        }
    }
}

constexpr int kMetricBlocks = 1024;

int grid_for(size_t n, int cap = 4096) {
    size_t b = (n + kBlock - 1) / kBlock;
    if (b < 1) b = 1;
    if (b > (size_t)cap) b = cap;
    return (int)b;
}

}  // namespace

// =================================================================================== launchers
void launch_calibration_copy(hipStream_t s, const void *src, void *dst, size_t bytes) {
    size_t n = bytes / 16;
    if (n == 0) return;
    k_calibration_copy<<<grid_for(n, 16384), kBlock, 0, s>>>(static_cast<const uint4 *>(src), static_cast<uint4 *>(dst), n);
}

void launch_fill_f32(hipStream_t s, float *p, float v, size_t n) {
    if (n == 0) return;
    k_fill_f32<<<grid_for(n), kBlock, 0, s>>>(p, v, n);
}

void launch_fill_u8(hipStream_t s, uint8_t *p, uint8_t v, size_t n) {
    // n must be a multiple of 4 (all users allocate padded buffers)
    if (n == 0) return;
    unsigned w = v * 0x01010101u;
    k_fill_u32<<<grid_for(n / 4), kBlock, 0, s>>>(reinterpret_cast<unsigned *>(p), w, n / 4);
}

void launch_gradient(hipStream_t s, int objective, int n, int num_class, const float *y, const float *yp, GHPair *gh,
                     GHPair *, int) {
    if (objective == OBJ_SOFTMAX)
        k_gradient_softmax<<<grid_for(n), kBlock, 0, s>>>(n, num_class, y, yp, gh);
    else
        k_gradient_pointwise<<<grid_for(n), kBlock, 0, s>>>(objective, n, y, yp, gh);
}

void launch_round_end_fused(hipStream_t s, const TreeBuffers &tb, int objective, int metric_kind, const float *y,
                            float *yp, float lr, GHPair *gh, double *metric_scratch, float *metric_out) {
    // grid == the grids of k_sum_gh and k_metric_partial (both min(1024, ceil(n / 256)))
    k_round_end_fused<<<tb.n_grad_blocks, kBlock, 0, s>>>(tb.n, objective, metric_kind, tb.nid, tb.nodes, y, yp, lr, gh,
                                                         tb.root_partial, metric_scratch);
    k_metric_final<<<1, kBlock, 0, s>>>(metric_kind, tb.n, tb.n_grad_blocks, metric_scratch, metric_out);
}

void launch_tree_init(hipStream_t s, const TreeBuffers &tb, const GHPair *gh_class, float lambda, bool stats_ready) {
    if (!stats_ready) k_sum_gh<<<tb.n_grad_blocks, kBlock, 0, s>>>(tb.n, gh_class, tb.root_partial);
    k_tree_init<<<1, kBlock, 0, s>>>(tb, tb.root_partial, lambda);
}

template <int LPR, int SLOTS>
static void hist_dense_launch(hipStream_t s, const TreeBuffers &tb, const DenseBins &bins, const GHPair *gh,
                              int level) {
    const int n_pairs = level == 0 ? 1 : (1 << (level - 1));
    dim3 grid(tb.max_hitems, bins.n_blocks);
    size_t lds = (size_t)tb.max_block_bins * sizeof(unsigned long long);
    if (lds > 64 * 1024) {
        // more than the default dynamic LDS window: opt in once per kernel instance and size
        static size_t opted = 0;
        if (lds > opted) {
            HIP_CHECK(hipFuncSetAttribute(
                reinterpret_cast<const void *>(&k_hist_dense<LPR, true, kHistBlock, SLOTS>),
                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
            HIP_CHECK(hipFuncSetAttribute(
                reinterpret_cast<const void *>(&k_hist_dense<LPR, false, kHistBlock, SLOTS>),
                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
            opted = lds;
        }
    }
    if (level == 0) {
        k_hist_dense<LPR, true, kHistBlock, SLOTS><<<grid, kHistBlock, lds, s>>>(
            bins, gh, nullptr, tb.seg, tb.hpair_begin, tb.hpair_built, n_pairs, tb.ctl + level, tb.quant,
            tb.blk_bin_begin, tb.feat_lds_off, tb.partial, tb.n_bins);
    } else {
        k_hist_dense<LPR, false, kHistBlock, SLOTS><<<grid, kHistBlock, lds, s>>>(
            bins, gh, tb.ridx[level & 1], tb.seg, tb.hpair_begin, tb.hpair_built, n_pairs, tb.ctl + level, tb.quant,
            tb.blk_bin_begin, tb.feat_lds_off, tb.partial, tb.n_bins);
    }
}

template <int LPR>
static void hist_dense_dispatch(hipStream_t s, const TreeBuffers &tb, const DenseBins &bins, const GHPair *gh,
                                int level) {
    const int slots = (tb.max_block_bins + kHistBlock - 1) / kHistBlock;  // bins drained per thread
    if (slots <= 1) hist_dense_launch<LPR, 1>(s, tb, bins, gh, level);
    else if (slots <= 2) hist_dense_launch<LPR, 2>(s, tb, bins, gh, level);
    else if (slots <= 4) hist_dense_launch<LPR, 4>(s, tb, bins, gh, level);
    else if (slots <= 8) hist_dense_launch<LPR, 8>(s, tb, bins, gh, level);
    else if (slots <= 20) hist_dense_launch<LPR, 20>(s, tb, bins, gh, level);
    else fatal("feature block with %d bins does not fit the histogram kernel", tb.max_block_bins);
}

void launch_hist_dense(hipStream_t s, const TreeBuffers &tb, const DenseBins &bins, const GHPair *gh, int level) {
    switch (bins.W / 4) {
        case 1: hist_dense_dispatch<1>(s, tb, bins, gh, level); break;
        case 2: hist_dense_dispatch<2>(s, tb, bins, gh, level); break;
        case 4: hist_dense_dispatch<4>(s, tb, bins, gh, level); break;
        case 8: hist_dense_dispatch<8>(s, tb, bins, gh, level); break;
        case 16: hist_dense_dispatch<16>(s, tb, bins, gh, level); break;
        default: fatal("unsupported dense block width %d", bins.W);
    }
}

void launch_hist_merge(hipStream_t s, const TreeBuffers &tb, int level) {
    const int n_pairs = level == 0 ? 1 : (1 << (level - 1));

    dim3 grid((tb.n_bins + kMergeBins - 1) / kMergeBins, n_pairs);
    k_hist_merge<<<grid, kBlock, 0, s>>>(tb.partial, tb.hist_q[level & 1], tb.hist_q[(level + 1) & 1], tb.hpair_begin,
                                        tb.hpair_built, level, tb.n_bins);
}

void launch_hist_csr(hipStream_t s, const TreeBuffers &tb, const CsrBins &bins, const GHPair *gh, int level) {
    const int n_pairs = level == 0 ? 1 : (1 << (level - 1));
    const int zgrid = std::min(1024, (tb.n_bins + kBlock - 1) / kBlock);
    longlong2 *cur = tb.hist_q[level & 1];
    k_hist_zero_built<<<dim3(zgrid, n_pairs), kBlock, 0, s>>>(cur, tb.hpair_built, level, tb.n_bins);
    if (level == 0) {
        k_hist_csr<true><<<tb.max_hitems, kBlock, 0, s>>>(tb, bins, gh, nullptr, cur, n_pairs, level);
    } else {
        k_hist_csr<false><<<tb.max_hitems, kBlock, 0, s>>>(tb, bins, gh, tb.ridx[level & 1], cur, n_pairs, level);
        k_hist_sub_csr<<<dim3(zgrid, n_pairs), kBlock, 0, s>>>(cur, tb.hist_q[(level + 1) & 1], tb.hpair_built, level,
                                                              tb.n_bins);
    }
}

void launch_eval_split(hipStream_t s, const TreeBuffers &tb, int level, float mcw, float lambda) {
    dim3 grid((tb.n_packs + kWaves - 1) / kWaves, 1 << level);
    k_eval_split<<<grid, kBlock, 0, s>>>(tb, tb.hist_q[level & 1], level, mcw, lambda);
}

void launch_best_update(hipStream_t s, const TreeBuffers &tb, int level, float rt_eps, float lambda) {
    k_best_update<<<1 << level, kBlock, 0, s>>>(tb, level, rt_eps, lambda);
}

void launch_partition_dense(hipStream_t s, const TreeBuffers &tb, const DenseBins &bins, int level) {
    k_part_plan<<<1, kBlock, 0, s>>>(tb, level);
    const int *cur = tb.ridx[level & 1];
    int *next = tb.ridx[(level + 1) & 1];
    if (level == 0) {
        k_part_count_dense<true><<<tb.max_pitems, kBlock, 0, s>>>(tb, bins, cur, level);
        k_part_scan_plan<<<1, kBlock, 0, s>>>(tb, level);
        k_part_scatter<true><<<tb.max_pitems, kBlock, 0, s>>>(tb, cur, next, level);
    } else {
        k_part_count_dense<false><<<tb.max_pitems, kBlock, 0, s>>>(tb, bins, cur, level);
        k_part_scan_plan<<<1, kBlock, 0, s>>>(tb, level);
        k_part_scatter<false><<<tb.max_pitems, kBlock, 0, s>>>(tb, cur, next, level);
    }
}

void launch_partition_csr(hipStream_t s, const TreeBuffers &tb, const CsrBins &bins, int level) {
    k_part_plan<<<1, kBlock, 0, s>>>(tb, level);
    const int *cur = tb.ridx[level & 1];
    int *next = tb.ridx[(level + 1) & 1];
    if (level == 0) {
        k_part_count_csr<true><<<tb.max_pitems, kBlock, 0, s>>>(tb, bins, cur, level);
        k_part_scan_plan<<<1, kBlock, 0, s>>>(tb, level);
        k_part_scatter<true><<<tb.max_pitems, kBlock, 0, s>>>(tb, cur, next, level);
    } else {
        k_part_count_csr<false><<<tb.max_pitems, kBlock, 0, s>>>(tb, bins, cur, level);
        k_part_scan_plan<<<1, kBlock, 0, s>>>(tb, level);
        k_part_scatter<false><<<tb.max_pitems, kBlock, 0, s>>>(tb, cur, next, level);
    }
}

void launch_nid_rebuild(hipStream_t s, const TreeBuffers &tb) {
    k_nid_plan<<<1, kBlock, 0, s>>>(tb);
    k_nid_write<<<tb.max_fitems, kBlock, 0, s>>>(tb);
}

void launch_prune(hipStream_t s, const TreeBuffers &tb, float gamma) { k_prune<<<1, kBlock, 0, s>>>(tb, gamma); }

void launch_predict_in_training(hipStream_t s, const TreeBuffers &tb, float *yp_class, float lr) {
    k_predict_in_training<<<grid_for(tb.n), kBlock, 0, s>>>(tb.n, tb.nid, tb.nodes, yp_class, lr);
}

void launch_metric(hipStream_t s, int kind, int n, int num_class, const float *y, const float *yp, double *scratch,
                   float *out) {
    int blocks = grid_for(n, kMetricBlocks);
    k_metric_partial<<<blocks, kBlock, 0, s>>>(kind, n, num_class, y, yp, scratch);
    k_metric_final<<<1, kBlock, 0, s>>>(kind, n, blocks, scratch, out);
}

}  // namespace tgbm
