// Tree-building kernels for gfx950 (wave64): gradients, LDS-privatised histograms, merge + sibling
// subtraction, wavefront segmented-scan split finding, ballot/popcount row partition, pruning and the
// in-training prediction update. Every stage of a level is one launch over all nodes of the level;
// work lists are planned on the device so the host never waits inside a tree.
#include <algorithm>

#include "device_api.h"
#include "kernel_common.h"

namespace tgbm {
namespace {

constexpr int kBlock = 256;
constexpr int kWaves = kBlock / 64;
constexpr int kHistMinChunk = 1024;
constexpr int kHistBlock = 1024;      // threads per histogram workgroup (they share one LDS histogram)

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

// ------------------------------------------------------------------------------------ fills
__global__ void k_fill_f32(float *p, float v, size_t n) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) p[i] = v;
}
__global__ void k_fill_u32(unsigned *p, unsigned v, size_t n) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) p[i] = v;
}

// -------------------------------------------------------------------------------- gradients
// Squared / logistic: include/thundergbm/objective/regression_obj.h:130-154 of the reference.
__device__ __forceinline__ GHPair pointwise_gradient(int objective, float yi, float p) {
    GHPair o;
    if (objective == OBJ_SQUARE) {
        o.g = p - yi;
        o.h = 1.f;
    } else {
        float s = 1.f / (1.f + expf(-p));
        o.g = s - yi;
        o.h = fmaxf(s * (1.f - s), 1e-16f);
    }
    return o;
}

__global__ void k_gradient_pointwise(int objective, int n, const float *__restrict__ y, const float *__restrict__ yp,
                                     GHPair *__restrict__ gh) {
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x)
        gh[i] = pointwise_gradient(objective, y[i], yp[i]);
}

// The gradient pair of a row as one 32-bit word that rides in the spare bytes of the row's bin-matrix record
// (DenseBins::gh_lane), so that a histogram work item that gathers a row gets its pair with the same memory request
// instead of a second one. Whatever computes a round's gradients also leaves the words in an array of their own
// (launch_gh_words, k_tree_end); the root level's histogram launch, which streams every record anyway, reads them
// there and writes the records back with the word in place - whole records, so that memory sees full-sector writes
// (4 bytes of every 32 written by themselves cost a read-modify-write per sector: 90 us per tree on 10 M rows). Squared loss: the gradient itself (the hessian is 1). Logistic loss with 0/1 labels: the
// sigmoid s (never negative) with the label in the sign bit; pair_from_word repeats pointwise_gradient's operations on
// s, so both give the same bits.
__device__ __forceinline__ unsigned word_from_row(int objective, float yi, float p) {
    if (objective == OBJ_SQUARE) return __float_as_uint(p - yi);
    const float s = 1.f / (1.f + expf(-p));
    return __float_as_uint(s) | (yi != 0.f ? 0x80000000u : 0u);
}
__device__ __forceinline__ GHPair pair_from_word(int objective, unsigned w) {
    GHPair o;
    if (objective == OBJ_SQUARE) {
        o.g = __uint_as_float(w);
        o.h = 1.f;
    } else {
        const float s = __uint_as_float(w & 0x7fffffffu);
        const float yi = (w >> 31) ? 1.f : 0.f;
        o.g = s - yi;
        o.h = fmaxf(s * (1.f - s), 1e-16f);
    }
    return o;
}

__global__ void k_gh_words(int objective, int n, const float *__restrict__ y, const float *__restrict__ yp,
                           unsigned *__restrict__ words) {
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x)
        words[i] = word_from_row(objective, y[i], yp[i]);
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

// Bagging, RowSampler::do_bagging (src/thundergbm/row_sampler.cu:9-38): entry i of the gradient array draws
// idx_i from thrust::default_random_engine(seed) after discard(i) through
// thrust::uniform_int_distribution<int>(0, N - 1); every gradient pair is multiplied by the number of draws
// that hit its index. thrust's default engine is minstd_rand (x <- 48271 x mod 2^31 - 1, a seed of 0 mod m
// becomes 1), its integer distribution maps the engine's output u in [1, m - 1] to
// int((u - 1) / (m - 1) * N) in double precision. The i + 1 steps of the engine are one modular power.
__global__ void k_bagging_draw(int N, unsigned seed, int *__restrict__ count) {
    constexpr unsigned long long M = 2147483647ull, A = 48271ull;
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < N; i += gridDim.x * blockDim.x) {
        unsigned long long x = seed % M;
        if (x == 0) x = 1;
        unsigned long long base = A, e = (unsigned long long)i + 1ull;  // discard(i), then one draw
        while (e) {
            if (e & 1ull) x = x * base % M;
            base = base * base % M;
            e >>= 1;
        }
        double r = (double)(unsigned)(x - 1ull);
        r /= 1.0 + (double)(unsigned)(M - 2ull);  // 1 + (max - min) with min = 1, max = m - 1
        const double lo = 0.0, hi = (double)(N - 1) + 1.0;
        const int idx = (int)(r * (hi - lo) + lo);
        atomicAdd(count + idx, 1);
    }
}

// perm (may be null): original row of every physical position; the draw counts belong to original rows
__global__ void k_bagging_apply(int N, int *__restrict__ count, GHPair *__restrict__ gh, const int *__restrict__ perm,
                                int n_rows) {
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < N; i += gridDim.x * blockDim.x) {
        // entry i = (plane, position): the plane (class) stays, the position maps to its original row
        const int src = perm != nullptr ? (i / n_rows) * n_rows + perm[i % n_rows] : i;
        const int c = count[src];
        count[src] = 0;  // ready for the next round (perm is a bijection: every counter is cleared once)
        GHPair v = gh[i];
        v.g = v.g * c;
        v.h = v.h * c;
        gh[i] = v;
    }
}

// Row-blocked reductions: workgroup b owns rows [b * kRowBlock, (b + 1) * kRowBlock), thread t adds its
// rows t, t + kBlock, ... in that order, then lanes, then wavefronts. Every kernel that produces
// gradient statistics or metric partials follows this order, so fused and separate passes give the
// same bits.
struct RowStats {
    float g = 0, h = 0, gm = 0, hm = 0, hf = 0;
    __device__ __forceinline__ void add(GHPair v) {
        g += v.g;
        h += v.h;
        gm = fmaxf(gm, fabsf(v.g));
        hm = fmaxf(hm, v.h);
        hf = fmaxf(hf, fabsf(v.h - rintf(v.h)));
    }
};

constexpr int kStatsLds = 5 * kWaves;  // floats of LDS that store_block_stats needs

// lds: kStatsLds floats; every thread of the block must call
__device__ void store_block_stats(RowStats r, float *lds, GradStats *out) {
    float *sg = lds, *sh = lds + kWaves, *mg = lds + 2 * kWaves, *mh = lds + 3 * kWaves, *fh = lds + 4 * kWaves;
    float g = wave_sum_f(r.g), h = wave_sum_f(r.h), gm = r.gm, hm = r.hm, hf = r.hf;
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) {
        gm = fmaxf(gm, __shfl_xor(gm, d));
        hm = fmaxf(hm, __shfl_xor(hm, d));
        hf = fmaxf(hf, __shfl_xor(hf, d));
    }
    if (lane_id() == 0) {
        sg[wave_id()] = g;
        sh[wave_id()] = h;
        mg[wave_id()] = gm;
        mh[wave_id()] = hm;
        fh[wave_id()] = hf;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        GradStats o{0, 0, 0, 0, 0};
        for (int i = 0; i < kWaves; ++i) {
            o.g += sg[i];
            o.h += sh[i];
            o.gmax = fmaxf(o.gmax, mg[i]);
            o.hmax = fmaxf(o.hmax, mh[i]);
            o.hfrac = fmaxf(o.hfrac, fh[i]);
        }
        *out = o;
    }
}

// lds: kWaves doubles
__device__ void store_block_sum_d(double acc, double *lds, double *out) {
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) acc += __shfl_xor(acc, d);
    if (lane_id() == 0) lds[wave_id()] = acc;
    __syncthreads();
    if (threadIdx.x == 0) {
        double t = 0;
        for (int i = 0; i < kWaves; ++i) t += lds[i];
        *out = t;
    }
}

// Block sums of (g,h) and block maxima of |g|, h for one tree.
// Class trees of a round: blockIdx.z selects the class (gradients and outputs are class-major).
__global__ __launch_bounds__(kBlock) void k_sum_gh(int n, const GHPair *__restrict__ gh, GradStats *__restrict__ out) {
    __shared__ float lds[kStatsLds];
    gh += (size_t)blockIdx.z * n;
    out += (size_t)blockIdx.z * gridDim.x;
    const int r0 = blockIdx.x * kRowBlock, r1 = min(n, r0 + kRowBlock);
    RowStats st;
    for (int i = r0 + threadIdx.x; i < r1; i += kBlock) st.add(gh[i]);
    store_block_stats(st, lds, out + blockIdx.x);
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
__global__ __launch_bounds__(kBlock) void k_tree_init(TreeBuffers tb_all, float lambda) {
    __shared__ float sg[kWaves], sh[kWaves], mg[kWaves], mh[kWaves], fh[kWaves];
    const TreeBuffers tb = tb_all.for_class(blockIdx.z);
    const GradStats *__restrict__ block_sums = tb.root_partial;
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
        if (tb.node_rows != nullptr) tb.node_rows[i] = i == 0 ? tb.n : 0;
    }
    float g = 0, h = 0, gm = 0, hm = 0, hf = 0;
    for (int i = threadIdx.x; i < tb.n_grad_blocks; i += kBlock) {
        g += block_sums[i].g;
        h += block_sums[i].h;
        gm = fmaxf(gm, block_sums[i].gmax);
        hm = fmaxf(hm, block_sums[i].hmax);
        hf = fmaxf(hf, block_sums[i].hfrac);
    }
    g = wave_sum_f(g);
    h = wave_sum_f(h);
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) {
        gm = fmaxf(gm, __shfl_xor(gm, d));
        hm = fmaxf(hm, __shfl_xor(hm, d));
        hf = fmaxf(hf, __shfl_xor(hf, d));
    }
    if (lane_id() == 0) {
        sg[wave_id()] = g;
        sh[wave_id()] = h;
        mg[wave_id()] = gm;
        mh[wave_id()] = hm;
        fh[wave_id()] = hf;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        GHPair s{0, 0};
        gm = 0;
        hm = 0;
        hf = 0;
        for (int i = 0; i < kWaves; ++i) {
            s.g += sg[i];
            s.h += sh[i];
            gm = fmaxf(gm, mg[i]);
            hm = fmaxf(hm, mh[i]);
            hf = fmaxf(hf, fh[i]);
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
        c.n_pitems = (tb.n + kPartChunk - 1) / kPartChunk;  // the root's partition items (used if it splits)
        c.rows_built = tb.n;
        tb.ctl[0] = c;
        tb.pbegin(0)[0] = 0;
        tb.pbegin(0)[1] = c.n_pitems;
        tb.ctl[tb.depth] = LevelCtl{0, 0, 0, 0};  // the last level plans no further one
        // The tree's scales keep the 64-bit sums over all n rows below 2^62; a dense work item coarsens them by its
        // own power of two so that its packed LDS fields hold the rows between two drains (item_shifts).
        QuantCtl q;
        // (the sparse layout's kernels round with round_to_ll, good below 2^51: its scales are those of at least
        // 4096 rows, which keeps every row's integers below 2^50)
        const int scale_rows = tb.sparse ? max(tb.n, 4096) : tb.n;
        q.scale_g = pow2_scale(gm, scale_rows, 4.6e18f);
        q.scale_h = pow2_scale(hm, scale_rows, 4.6e18f);
        q.h_bits = 32;
        q.h_integer = 0;
        // every hessian a non-negative integer (squared loss; bagging multiplies by draw counts): the hessian field
        // takes the bits that kHistFlushRowsInt such rows need, the gradient field the rest
        q.flush_rows = kHistFlushRows;
        const float hrows = hm * (float)kHistFlushRowsInt;
        if (!tb.sparse && hf == 0.f && hm >= 1.f && hrows < 4.0e9f) {
            q.h_integer = 1;
            q.h_bits = ilogbf(hrows) + 1;
            q.scale_h = 1.f;
            q.flush_rows = kHistFlushRowsInt;
        }
        q.inv_g = 1.f / q.scale_g;
        q.inv_h = 1.f / q.scale_h;
        q.gq_max = gm * q.scale_g;
        q.hq_max = hm * q.scale_h;
        *tb.quant = q;
    }
}

// ------------------------------------------------------------------------- dense histogram
// One workgroup = one work item (a run of rows of one node) x one feature block. The block's
// histogram lives in LDS as one 64-bit integer per bin holding the fixed-point gradient sum in the
// high and the hessian sum in the low field (QuantCtl::h_bits wide); a row contributes with a single
// ds_add_u64 per feature (float LDS atomics run at ~0.3 lanes/clk/CU on gfx950, 64-bit integer ones at ~5).
// The fields are safe for the rows added between two drains (at most kHistFlushRows; fewer in a node with fewer
// rows, whose items therefore count finer: item_shift), so after at most that many rows every thread drains the
// bins it owns into 64-bit register accumulators and clears them; at the end the registers go to the item's slot
// of `partial`, at the item's scale (k_hist_merge shifts them to the tree's).
// LPR consecutive lanes cover one row (one dword = four bin bytes per lane, or two 16-bit bins with BIN16), so a
// wavefront load instruction reads 256 contiguous bytes and the 64 atomics of one step spread over many features.
// (Packing each row's gradient pair next to its bins so that a gathered row costs one 128-byte line
// instead of two was measured: it halves the fetched bytes below the root, but the per-tree refresh of
// the pairs costs what the gathers save.)
// The value that the last of the LPR lanes of a row holds, in every lane of the row (LPR = 4, 8 or 16 consecutive
// lanes): a DPP broadcast inside the 16-lane row of the wavefront, no trip through the LDS crossbar.
template <int LPR>
__device__ __forceinline__ unsigned last_lane_of_row(unsigned v) {
    if (LPR == 4) return (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, 0xff, 0xf, 0xf, false);  // quad_perm:[3,3,3,3]
    const unsigned hi = (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, 0x15f, 0xf, 0xf, false);  // row_newbcast:15
    if (LPR == 16) return hi;
    const unsigned lo = (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, 0x157, 0xf, 0xf, false);  // row_newbcast:7
    return (threadIdx.x & 8u) ? hi : lo;
}

// GHW: the rows' gradient pairs come from 32-bit words (word_from_row). Below the root the word sits in the last
// dword of the row's record, which the row's last lane has loaded with the bins anyway: no second gather per row. The
// root launch (DIRECT) reads the words from their own array and puts them there, storing every record back.
template <int LPR, bool DIRECT, int BLK, int SLOTS, bool BIN16, bool GHW = false>
__global__ __launch_bounds__(BLK) __attribute__((amdgpu_waves_per_eu(SLOTS <= 8 ? 8 : 4)))  // two 1024-thread groups per CU
void k_hist_dense(TreeBuffers tb_all, DenseBins bins, const GHPair *__restrict__ gh, int level, int n_pairs) {
    extern __shared__ unsigned long long lds[];
    __shared__ int s_shift[2];  // the item's scale shifts (gradient, hessian)
    const TreeBuffers tb = tb_all.for_class(blockIdx.z);
    gh += (size_t)blockIdx.z * tb.n;
    const int *__restrict__ ridx = tb.list(level);
    const int2 *__restrict__ seg = tb.seg;
    const int *__restrict__ hpair_begin = tb.hpair_begin;
    const int *__restrict__ hpair_built = tb.hpair_built;
    const QuantCtl *__restrict__ quant = tb.quant;
    const int *__restrict__ blk_bin_begin = tb.blk_bin_begin;
    const int *__restrict__ feat_lds_off = tb.feat_lds_off;
    longlong2 *__restrict__ partial = tb.partial;
    const int n_bins = tb.n_bins;
    const LevelCtl c = tb.ctl[level];
    // (the feature blocks of an item are neighbours in the launch order: the item's row list and gradient pairs, which
    // every block reads again, are then fetched while they still sit in an L2 - with the items of a block as
    // neighbours, every block of 500 k x 2000 data fetched them from HBM again: 2.72 -> 2.29 ms per tree)
    const int item = blockIdx.y;
    if (item >= c.n_hitems) return;
    const int fb = blockIdx.x;
    const int bin0 = blk_bin_begin[fb];
    const int nb = blk_bin_begin[fb + 1] - bin0;
    if (nb == 0) return;
    const int h_bits = quant->h_bits;
    const int flush_rows = quant->flush_rows;
    const int gh_objective = bins.gh_objective;
    const bool word_lane = bins.gh_lane >= 0 && (int)(threadIdx.x % LPR) == bins.gh_lane;
    // The item's node and rows: the same few look-ups in every lane (uniform addresses: scalar loads), so that the
    // first row loads can be issued before the barrier that publishes the LDS histogram's clearing.
    const int p = find_owner(hpair_begin, n_pairs, item);
    const int node = hpair_built[p];
    const int2 sg = seg[node];
    const int begin = __builtin_amdgcn_readfirstlane(sg.x + (item - hpair_begin[p]) * c.hchunk);
    const int end = __builtin_amdgcn_readfirstlane(min(sg.y, begin + c.hchunk));
    const int x_in = node - ((1 << level) - 1);
    if (x_in < tb.lvl_x0 || x_in >= tb.lvl_x1) return;  // not in the batch of nodes this launch serves
    if (threadIdx.x == 0) {
        // (the node's rows, not the item's: what a row adds must not depend on the item it falls into, or the sums
        // would change with the order of the rows)
        const int rows = max(1, min(sg.y - sg.x, quant->flush_rows));
        const int2 shift = make_int2(item_shift(quant->gq_max, rows, 63 - h_bits),
                                     quant->h_integer ? 0 : item_shift(quant->hq_max, rows, h_bits));
        s_shift[0] = shift.x;
        s_shift[1] = shift.y;
        if (fb == 0) tb.hitem_shift[item] = shift;
    }
    // (slots of `partial` count from the first item of the served batch of nodes: item 0 unless the arena is capped)
    const int item0 = hpair_begin[tb.hpair_lo(level)];
    const unsigned long long h_mask = (1ull << h_bits) - 1ull;  // h_bits <= 32
    constexpr int RPS = BLK / LPR;  // rows per step of the whole block
    // rows per thread and stage: what the registers left over by the drain accumulators hold without spills (64
    // registers per thread with two workgroups per CU)
    constexpr int U = (SLOTS <= 4 || SLOTS == 16) ? 4 : 2;
    static_assert(RPS * U <= kHistFlushRows, "one iteration must not exceed the flush interval");
    const int q = threadIdx.x % LPR;
    const int rsub = threadIdx.x / LPR;
    constexpr int FPL = BIN16 ? 2 : 4;  // features per lane (one dword of the row)
    constexpr int ROWB = LPR * 4;       // bytes per row of the block
    const int *fo = feat_lds_off + fb * (LPR * FPL) + q * FPL;
    const int o0 = fo[0], o1 = fo[1], o2 = BIN16 ? 0 : fo[2], o3 = BIN16 ? 0 : fo[3];
    // (a block is smaller than 4 GiB and has fewer than 2^29 rows - checked when the layout is chosen -, so a lane
    // addresses its dword, its gradient pair and its row id with an unsigned 32-bit offset from a uniform base)
    const uint8_t *blk = bins.data + (size_t)fb * bins.block_stride;
    const unsigned qoff = q * 4;
    long long accg[SLOTS], acch[SLOTS];
#pragma unroll
    for (int k = 0; k < SLOTS; ++k) accg[k] = acch[k] = 0;
    int pending = 0;  // rows accumulated in LDS since the last drain (uniform across the block)
    unsigned pk[U], pk_next[U];
    GHPair s[U], s_next[U];
    // Three stages in flight per thread: the row ids of the step after next, the bins and gradient pairs of the next
    // step (gathered through row ids that arrived during the previous iteration), the atomics of this step. All
    // loads are unconditional - positions past the item's end are clamped to its last row and their bins replaced by
    // the sentinel - and each stage's loads are issued back to back, so that no load waits for an unrelated one.
    int r_next[U];
    auto load_ids = [&](int base, int(&r)[U]) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int pos = min(base + rsub + u * RPS, end - 1);
            r[u] = DIRECT ? pos : *reinterpret_cast<const int *>(reinterpret_cast<const char *>(ridx) + (unsigned)pos * 4u);
        }
    };
    auto load_rows = [&](const int(&r)[U], unsigned(&opk)[U], GHPair(&os)[U]) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            opk[u] = *reinterpret_cast<const unsigned *>(blk + ((unsigned)r[u] * (unsigned)ROWB + qoff));
            if (!GHW) os[u] = *reinterpret_cast<const GHPair *>(reinterpret_cast<const char *>(gh) + (unsigned)r[u] * 8u);
            if (GHW && DIRECT)  // (the word travels in the pair's first slot)
                os[u].g = __uint_as_float(*reinterpret_cast<const unsigned *>(reinterpret_cast<const char *>(bins.gh_words) + (unsigned)r[u] * 4u));
        }
    };
    constexpr int STEP = RPS * U;
    if (begin < end) {
        load_ids(begin, r_next);
        load_rows(r_next, pk, s);
        if (begin + STEP < end) load_ids(begin + STEP, r_next);
    }
    // the first rows are on their way: clear the histogram meanwhile
    for (int i = threadIdx.x; i < nb; i += BLK) lds[i] = 0ull;
    __syncthreads();
    // the item's scales: powers of two well inside the float range, so the products below are exact
    const float scale_g = ldexpf(quant->scale_g, -__builtin_amdgcn_readfirstlane(s_shift[0]));
    const float scale_h = ldexpf(quant->scale_h, -__builtin_amdgcn_readfirstlane(s_shift[1]));
    for (int base = begin; base < end; base += STEP) {
        // the next step's rows are requested before this step's atomics (and before a drain's
        // barriers), so the memory pipeline stays busy
        if (base + STEP < end) {
            load_rows(r_next, pk_next, s_next);
            if (base + 2 * STEP < end) load_ids(base + 2 * STEP, r_next);
        }
        const int step_rows = min(RPS * U, end - base);
        if (pending + step_rows > flush_rows) {
            __syncthreads();
#pragma unroll
            for (int k = 0; k < SLOTS; ++k) {
                const int i = threadIdx.x + k * BLK;
                if (i < nb) {
                    const unsigned long long t = lds[i];
                    lds[i] = 0ull;
                    const unsigned long long lo = t & h_mask;
                    accg[k] += (long long)(t - lo) >> h_bits;
                    acch[k] += (long long)lo;
                }
            }
            __syncthreads();
            pending = 0;
        }
        pending += step_rows;
#pragma unroll
        for (int u = 0; u < U; ++u) {
            unsigned v = (base + rsub + u * RPS < end) ? pk[u] : 0xffffffffu;  // (a clamped position adds nothing)
            GHPair sv = s[u];
            if constexpr (GHW && DIRECT) {
                const unsigned w = __float_as_uint(s[u].g);
                sv = pair_from_word(gh_objective, w);
                // the record goes back with the word in its last dword (whole records: full-sector writes)
                const int pos = base + rsub + u * RPS;
                if (pos < end)
                    *reinterpret_cast<unsigned *>(const_cast<uint8_t *>(blk) + ((unsigned)pos * (unsigned)ROWB + qoff)) = word_lane ? w : pk[u];
            } else if constexpr (GHW) {
                // the row's last lane holds the word: every lane of the row takes it from there
                sv = pair_from_word(gh_objective, last_lane_of_row<LPR>(pk[u]));
            }
            if (word_lane) v = 0xffffffffu;  // (that lane's dword holds no bins, whether the word is used or not)
            // exact products (the scales are powers of two), rounded once to the nearest integer
            const long long gq = round_to_ll(sv.g * scale_g);
            const long long hq = round_to_ll(fmaxf(sv.h, 0.f) * scale_h);
            const unsigned long long add = ((unsigned long long)gq << h_bits) + (unsigned long long)hq;
            if (BIN16) {
                const unsigned b0 = v & 0xffff, b1 = v >> 16;
                if (b0 != kMissingBin16) atomicAdd(lds + o0 + b0, add);
                if (b1 != kMissingBin16) atomicAdd(lds + o1 + b1, add);
            } else {
                const unsigned b0 = v & 0xff, b1 = (v >> 8) & 0xff, b2 = (v >> 16) & 0xff, b3 = v >> 24;
                if (b0 != kMissingBin) atomicAdd(lds + o0 + b0, add);
                if (b1 != kMissingBin) atomicAdd(lds + o1 + b1, add);
                if (b2 != kMissingBin) atomicAdd(lds + o2 + b2, add);
                if (b3 != kMissingBin) atomicAdd(lds + o3 + b3, add);
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            pk[u] = pk_next[u];
            if (!GHW || DIRECT) s[u] = s_next[u];
        }
    }
    __syncthreads();
    if (c.hchunk <= flush_rows) {
        // an item this short was never drained: its packed LDS words are the complete sums and go out as
        // they are (8 bytes per bin instead of 16; k_hist_merge unpacks them)
        unsigned long long *out = reinterpret_cast<unsigned long long *>(partial) + (size_t)(item - item0) * n_bins + bin0;
        for (int i = threadIdx.x; i < nb; i += BLK) out[i] = lds[i];
        return;
    }
    longlong2 *out = partial + (size_t)(item - item0) * n_bins + bin0;
#pragma unroll
    for (int k = 0; k < SLOTS; ++k) {
        const int i = threadIdx.x + k * BLK;
        if (i < nb) {
            const unsigned long long t = lds[i];
            const unsigned long long lo = t & h_mask;
            out[i] = make_longlong2(accg[k] + ((long long)(t - lo) >> h_bits), acch[k] + (long long)lo);
        }
    }
}

// (Adding the work items' histograms straight into the node's histogram with global 64-bit atomics
// instead of storing and merging them was measured: 0.5 ms per tree slower on the 10M x 28 benchmark.)
// Sum the private histograms of the node that was built from rows (64-bit integers, exact, any
// order gives the same bits) and derive its sibling as parent - built (the reference's subtraction
// trick, hist_tree_builder_single.cu:526-540). A block covers kMergeBins bins of one sibling pair; its
// thread groups stride over the pair's work items and are combined through LDS. Near the root a pair has
// hundreds of items and the level only a few pairs, so narrow blocks (8 bins, 32 groups) are used there:
// four times the workgroups and a quarter of the loads per thread.
template <int kMergeBins>
__global__ __launch_bounds__(kBlock) void k_hist_merge(TreeBuffers tb_all, int level) {
    constexpr int kMergeGroups = kBlock / kMergeBins;
    __shared__ long long s_g[kMergeGroups][kMergeBins], s_h[kMergeGroups][kMergeBins];
    const TreeBuffers tb = tb_all.for_class(blockIdx.z);
    const longlong2 *__restrict__ partial = tb.partial;
    longlong2 *__restrict__ cur_q = tb.hist(level);
    const longlong2 *__restrict__ prev_q = tb.hist(level + 1);
    const int *__restrict__ hpair_begin = tb.hpair_begin;
    const int *__restrict__ hpair_built = tb.hpair_built;
    const int n_bins = tb.n_bins;
    const int p = blockIdx.y + tb.hpair_lo(level);
    const int built = hpair_built[p];
    if (built < 0) return;
    const int jl = threadIdx.x % kMergeBins, ig = threadIdx.x / kMergeBins;
    const int j = blockIdx.x * kMergeBins + jl;
    const int ib = hpair_begin[p], ie = hpair_begin[p + 1];
    const int item0 = hpair_begin[tb.hpair_lo(level)];  // `partial` slots count from the served batch's first item
    long long sg = 0, sh = 0;
    if (j < n_bins) {
        // every item counted at its own scale (item_shift): shift its sums to the tree's
        const int2 *__restrict__ shift = tb.hitem_shift;
        if (tb.ctl[level].hchunk <= tb.quant->flush_rows) {  // packed 8-byte partials (see k_hist_dense)
            const unsigned long long *packed = reinterpret_cast<const unsigned long long *>(partial);
            const int h_bits = tb.quant->h_bits;
            const unsigned long long h_mask = (1ull << h_bits) - 1ull;
            for (int it = ib + ig; it < ie; it += kMergeGroups) {
                const unsigned long long t = packed[(size_t)(it - item0) * n_bins + j];
                const int2 s = shift[it];
                const unsigned long long lo = t & h_mask;
                sg += ((long long)(t - lo) >> h_bits) << s.x;
                sh += (long long)lo << s.y;
            }
        } else {
            for (int it = ib + ig; it < ie; it += kMergeGroups) {
                longlong2 v = partial[(size_t)(it - item0) * n_bins + j];
                const int2 s = shift[it];
                sg += v.x << s.x;
                sh += v.y << s.y;
            }
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
    if (level > 0 && !tb.singles(level)) {
        const int sib = (built & 1) ? built + 1 : built - 1;
        const longlong2 par = prev_q[(size_t)p * n_bins + j];
        cur_q[(size_t)(sib - off) * n_bins + j] = make_longlong2(par.x - sg, par.y - sh);
    }
}

// ------------------------------------------------------------------------------ exact root sums
// k_tree_init sets the root's sums from a float reduction over the rows, whose last bits depend on the physical
// order of the rows; every later quantity of a tree (child sums, weights, gains, predictions, the next gradients)
// derives from it. These kernels replace it by the exact fixed-point total - the same integers in any order - so
// that a tree does not depend on the row order at all.
__device__ void set_root_sums(const TreeBuffers &tb, long long G, long long H, float lambda) {
    GHPair s{(float)((double)G * (double)tb.quant->inv_g), (float)((double)H * (double)tb.quant->inv_h)};
    TreeNode &root = tb.nodes[0];
    root.sum_gh_pair = s;
    root.base_weight = -s.g / (s.h + lambda);
}

// From the root histogram: the bins of a feature that is stored in every row add up to the root. One workgroup.
__global__ __launch_bounds__(kBlock) void k_root_sum_bins(TreeBuffers tb_all, float lambda) {
    __shared__ long long s_g[kWaves], s_h[kWaves];
    const TreeBuffers tb = tb_all.for_class(blockIdx.z);
    const longlong2 *__restrict__ h = tb.hist(0);
    const int b0 = tb.cut_row_ptr[tb.complete_feature], b1 = tb.cut_row_ptr[tb.complete_feature + 1];
    long long g = 0, hh = 0;
    for (int b = b0 + threadIdx.x; b < b1; b += kBlock) {
        const longlong2 v = h[b];
        g += v.x;
        hh += v.y;
    }
    g = wave_sum_ll(g);
    hh = wave_sum_ll(hh);
    if (lane_id() == 0) {
        s_g[wave_id()] = g;
        s_h[wave_id()] = hh;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int i = 1; i < kWaves; ++i) {
            g += s_g[i];
            hh += s_h[i];
        }
        set_root_sums(tb, g, hh, lambda);
    }
}

// From the gradients (no feature is stored in every row): every row's pair rounded at the tree's scales, one pair of
// 64-bit block sums per workgroup into root_total[2 i], [2 i + 1]; k_root_sum_final (one workgroup) adds them up.
// (A ticket that lets the last workgroup finish the job needs a device-scope fence, which writes a whole L2 back on
// this chip: 288 us per round of 8 class trees against 2 x 5 us for two launches.)
constexpr int kRootSumBlocks = 256;
__global__ __launch_bounds__(kBlock) void k_root_sum_rows(TreeBuffers tb_all, const GHPair *__restrict__ gh) {
    __shared__ long long s_g[kWaves], s_h[kWaves];
    const TreeBuffers tb = tb_all.for_class(blockIdx.z);
    gh += (size_t)blockIdx.z * tb.n;
    const float scale_g = tb.quant->scale_g, scale_h = tb.quant->scale_h;
    long long g = 0, hh = 0;
    for (int i = blockIdx.x * kBlock + threadIdx.x; i < tb.n; i += gridDim.x * kBlock) {
        const GHPair v = gh[i];
        g += __float2ll_rn(v.g * scale_g);
        hh += __float2ll_rn(fmaxf(v.h, 0.f) * scale_h);
    }
    g = wave_sum_ll(g);
    hh = wave_sum_ll(hh);
    if (lane_id() == 0) {
        s_g[wave_id()] = g;
        s_h[wave_id()] = hh;
    }
    __syncthreads();
    if (threadIdx.x != 0) return;
    for (int i = 1; i < kWaves; ++i) {
        g += s_g[i];
        hh += s_h[i];
    }
    tb.root_total[2 * blockIdx.x] = g;
    tb.root_total[2 * blockIdx.x + 1] = hh;
}

__global__ __launch_bounds__(kBlock) void k_root_sum_final(TreeBuffers tb_all, int n_blocks, float lambda) {
    __shared__ long long s_g[kWaves], s_h[kWaves];
    const TreeBuffers tb = tb_all.for_class(blockIdx.z);
    long long g = 0, hh = 0;
    for (int i = threadIdx.x; i < n_blocks; i += kBlock) {
        g += tb.root_total[2 * i];
        hh += tb.root_total[2 * i + 1];
    }
    g = wave_sum_ll(g);
    hh = wave_sum_ll(hh);
    if (lane_id() == 0) {
        s_g[wave_id()] = g;
        s_h[wave_id()] = hh;
    }
    __syncthreads();
    if (threadIdx.x != 0) return;
    for (int i = 1; i < kWaves; ++i) {
        g += s_g[i];
        hh += s_h[i];
    }
    set_root_sums(tb, g, hh, lambda);
}

__global__ __launch_bounds__(kBlock) void k_count_bytes(const uint8_t *__restrict__ v, size_t n, uint8_t value,
                                                       unsigned long long *__restrict__ out) {
    unsigned long long c = 0;
    for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (size_t)gridDim.x * kBlock) c += v[i] == value;
    c = (unsigned long long)wave_sum_ll((long long)c);
    if (lane_id() == 0 && c) atomicAdd(out, c);
}

__global__ __launch_bounds__(kBlock) void k_count_u16(const uint16_t *__restrict__ v, size_t n, uint16_t value,
                                                     unsigned long long *__restrict__ out) {
    unsigned long long c = 0;
    for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (size_t)gridDim.x * kBlock) c += v[i] == value;
    c = (unsigned long long)wave_sum_ll((long long)c);
    if (lane_id() == 0 && c) atomicAdd(out, c);
}

// --------------------------------------------------------------------------- sparse histogram
// CSR rows of global bin ids: the histogram is too large for LDS (one slot per cut point of every
// feature), so every stored value adds its row's fixed-point gradient pair to the node's histogram
// in HBM with two 64-bit integer atomics (exact and order-independent, unlike the float atomics of
// hist_tree_builder_single.cu:203-216 / :485-505). One wavefront walks one row at a time.
__global__ __launch_bounds__(kBlock) void k_hist_zero_built(TreeBuffers tb_all, int level) {
    const TreeBuffers tb = tb_all.for_class(blockIdx.z);
    longlong2 *__restrict__ cur_q = tb.hist(level);
    const int n_bins = tb.n_bins;
    const int built = tb.hpair_built[blockIdx.y + tb.hpair_lo(level)];
    if (built < 0) return;
    const int off = (1 << level) - 1;
    longlong2 *h = cur_q + (size_t)(built - off) * n_bins;
    for (int j = blockIdx.x * kBlock + threadIdx.x; j < n_bins; j += gridDim.x * kBlock) h[j] = make_longlong2(0, 0);
}

template <bool DIRECT>
__global__ __launch_bounds__(kBlock) void k_hist_csr(TreeBuffers tb_all, CsrBins bins, const GHPair *__restrict__ gh,
                                                    int n_pairs, int level) {
    __shared__ int s_info[3];
    const TreeBuffers tb = tb_all.for_class(blockIdx.z);
    gh += (size_t)blockIdx.z * tb.n;
    const int *__restrict__ ridx = tb.list(level);
    longlong2 *__restrict__ cur_q = tb.hist(level);
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
        if (s_info[2] < tb.lvl_x0 || s_info[2] >= tb.lvl_x1) s_info[1] = b;  // not in the served batch: no rows
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

// The same with the bins of the most frequent features ("head") accumulated in LDS: with a skewed feature
// distribution most stored values hit a few thousand bins, and global atomics on those serialise (the
// root level of a 2M x 100k Zipf matrix spent 10 ms there). Every head slot is a pair of 64-bit sums, so
// no drain is needed; at the end the workgroup adds its non-zero slots to the node's histogram in HBM.
// 1024 threads (16 wavefronts, one row each, the next row's header prefetched), two workgroups per CU.
template <bool DIRECT>
__global__ __launch_bounds__(kHistBlock) __attribute__((amdgpu_waves_per_eu(8)))
void k_hist_csr_head(TreeBuffers tb_all, CsrBins bins, const GHPair *__restrict__ gh, int n_pairs, int level) {
    extern __shared__ unsigned long long lds[];  // [2 * head_bins]: gradient, hessian of every slot
    __shared__ int s_info[3];
    const TreeBuffers tb = tb_all.for_class(blockIdx.z);
    gh += (size_t)blockIdx.z * tb.n;
    const int *__restrict__ ridx = tb.list(level);
    longlong2 *__restrict__ cur_q = tb.hist(level);
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
        if (s_info[2] < tb.lvl_x0 || s_info[2] >= tb.lvl_x1) s_info[1] = b;  // not in the served batch: no rows
    }
    for (int i = threadIdx.x; i < 2 * bins.head_bins; i += kHistBlock) lds[i] = 0ull;
    __syncthreads();
    const int begin = s_info[0], end = s_info[1];
    unsigned long long *h = reinterpret_cast<unsigned long long *>(cur_q + (size_t)s_info[2] * tb.n_bins);
    const float scale_g = tb.quant->scale_g, scale_h = tb.quant->scale_h;
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    constexpr int NW = kHistBlock / 64;
    int pos = begin + w;
    GHPair s{0, 0};
    int e0 = 0, e1 = 0;
    if (pos < end) {
        const int r = DIRECT ? pos : ridx[pos];
        s = gh[r];
        e0 = bins.row_ptr[r];
        e1 = bins.row_ptr[r + 1];
    }
    while (pos < end) {
        const int npos = pos + NW;
        GHPair ns{0, 0};
        int ne0 = 0, ne1 = 0;
        if (npos < end) {  // requested before this row's atomics
            const int r = DIRECT ? npos : ridx[npos];
            ns = gh[r];
            ne0 = bins.row_ptr[r];
            ne1 = bins.row_ptr[r + 1];
        }
        const unsigned long long gq = (unsigned long long)__float2ll_rn(s.g * scale_g);
        const unsigned long long hq = (unsigned long long)__float2ll_rn(s.h * scale_h);
        for (int e = e0 + lane; e < e1; e += 64) {
            const int word = bins.hist_word[e];
            if (word < 0) {
                const int slot = ~word;
                atomicAdd(lds + 2 * slot, gq);
                atomicAdd(lds + 2 * slot + 1, hq);
            } else {
                atomicAdd(h + 2 * (size_t)word, gq);
                atomicAdd(h + 2 * (size_t)word + 1, hq);
            }
        }
        pos = npos;
        s = ns;
        e0 = ne0;
        e1 = ne1;
    }
    __syncthreads();
    for (int i = threadIdx.x; i < bins.head_bins; i += kHistBlock) {
        const unsigned long long g = lds[2 * i], hh = lds[2 * i + 1];
        if ((g | hh) != 0ull) {
            const size_t b = (size_t)bins.head_bin[i];
            atomicAdd(h + 2 * b, g);
            atomicAdd(h + 2 * b + 1, hh);
        }
    }
}

// Root histogram of the sparse layout from the bin-major copy: every row takes part at the root, so the sum of a
// bin is the sum over a contiguous run of the copy. A wavefront reduces 64 consecutive values by bin (segmented
// scan over sorted keys) and the last lane of every run adds it to the histogram: one pair of atomics per run
// and wavefront, to addresses that ascend with the position, instead of one pair per stored value to random
// lines of a histogram far larger than the caches (4.3 ms -> 1.1 ms at 69 M values, 6.3 M bins). Same integers
// as k_hist_csr, in another order: the histogram is bit-identical.
__global__ __launch_bounds__(kBlock) void k_hist_root_csc(TreeBuffers tb_all, CsrBins bins, const GHPair *__restrict__ gh) {
    const TreeBuffers tb = tb_all.for_class(blockIdx.z);
    gh += (size_t)blockIdx.z * tb.n;
    unsigned long long *h = reinterpret_cast<unsigned long long *>(tb.hist(0));
    const float scale_g = tb.quant->scale_g, scale_h = tb.quant->scale_h;
    const int lane = lane_id();
    const long n_tiles = (bins.nnz + 63) / 64;
    for (long tile = (long)blockIdx.x * kWaves + wave_id(); tile < n_tiles; tile += (long)gridDim.x * kWaves) {
        const long e = tile * 64 + lane;
        int b = -1;
        long long gq = 0, hq = 0;
        if (e < bins.nnz) {
            b = bins.csc_bin[e];
            const GHPair s = gh[bins.csc_row[e]];
            gq = __float2ll_rn(s.g * scale_g);
            hq = __float2ll_rn(s.h * scale_h);
        }
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const int ob = __shfl_up(b, d);
            const long long og = shfl_up_ll(gq, d), oh = shfl_up_ll(hq, d);
            if (lane >= d && ob == b) {  // sorted keys: equal ends mean one run in between
                gq += og;
                hq += oh;
            }
        }
        const int nb = __shfl_down(b, 1);
        if (b >= 0 && (lane == 63 || nb != b)) {
            atomicAdd(h + 2 * (size_t)b, (unsigned long long)gq);
            atomicAdd(h + 2 * (size_t)b + 1, (unsigned long long)hq);
        }
    }
}

template <bool DIRECT>
__global__ __launch_bounds__(kBlock) void k_part_count_csr(TreeBuffers tb_all, CsrBins bins, int level) {
    __shared__ int lds[kWaves];
    __shared__ int s_x;
    const TreeBuffers tb = tb_all.for_class(blockIdx.z);
    const int *__restrict__ ridx = tb.list(level);
    const int item = blockIdx.x;
    if (item >= tb.ctl[level].n_pitems) return;
    const int nl = 1 << level, off = nl - 1;
    if (threadIdx.x == 0) s_x = find_owner(tb.pbegin(level), nl, item);
    __syncthreads();
    const int x_in = s_x;
    const TreeNode &nd = tb.nodes[off + x_in];
    if (!node_splits(nd)) {
        if (threadIdx.x == 0) tb.pitem_nleft[item] = 0;
        return;
    }
    const int2 sg = tb.seg[off + x_in];
    const int pb = sg.x + (item - tb.pbegin(level)[x_in]) * kPartChunk;
    const int pe = min(sg.y, pb + kPartChunk);
    const int f = nd.split_feature_id;
    const int cb = tb.cut_row_ptr[f], ce = tb.cut_row_ptr[f + 1];
    const int sbid = cb + (tb.split_bin != nullptr ? tb.split_bin[off + x_in] : (int)nd.split_bid);
    const bool dr = nd.default_right;
    int nleft = 0;
    unsigned rights = 0;
#pragma unroll
    for (int k = 0; k < kPartChunk / kBlock; ++k) {
        int pos = pb + k * kBlock + threadIdx.x;
        if (pos < pe) {
            int row = DIRECT ? pos : ridx[pos];
            bool right = csr_goes_right(bins, row, cb, ce, sbid, dr);
            rights |= (right ? 1u : 0u) << k;
            nleft += right ? 0 : 1;
        }
    }
    tb.goes_right[(size_t)item * kBlock + threadIdx.x] = (uint8_t)rights;  // (see k_part_count_dense)
    int tot = block_sum(nleft, lds);
    if (threadIdx.x == 0) tb.pitem_nleft[item] = tot;
}

// ------------------------------------------------------------------------ split finding
// Split search. One wavefront scans one pack of whole features (at most 256 bins, 4 consecutive bins
// per lane) of one node with a segmented inclusive prefix sum over the exact 64-bit fixed-point
// histogram: integer sums are associative, so the parallel scan returns bit-for-bit what a
// sequential one would, and candidates separated only by empty bins tie exactly. Per candidate:
// left = sum of the feature's bins below it, missing = node sum - feature total, gain with missing
// values sent right and left (hist_tree_builder_single.cu:257-325 / :614-681 of the reference);
// the wavefront keeps its best candidate: largest |gain|, ties to the smaller bin index (:330-335).
// SUB (sparse layout, whose histograms are not merged from work-item partials): the node of a pair that
// was not built from rows is derived here as parent - built while it is scanned, and stored for the next
// level, instead of by a separate pass over the (very long) histograms.
template <bool SUB>
__global__ __launch_bounds__(kBlock) void k_eval_split(TreeBuffers tb_all, int level, float mcw, float lambda,
                                                      bool store_sibling) {
#pragma clang fp contract(off)
    const TreeBuffers tb = tb_all.for_class(blockIdx.z);
    longlong2 *__restrict__ hist_q = tb.hist(level);
    __shared__ GHPair s_miss[kWaves][kEvalPackBins];
    const int lane = lane_id(), w = wave_id();
    const int pack = blockIdx.x * kWaves + w;
    const int x_in = blockIdx.y + tb.lvl_x0;
    const int x = (1 << level) - 1 + x_in;
    const TreeNode nd = tb.nodes[x];
    const bool active = pack < tb.n_packs && nd.is_valid;
    int b_begin = 0, b_end = 0;
    if (active) {
        b_begin = tb.pack_begin[pack];
        b_end = tb.pack_begin[pack + 1];
    }
    const GHPair S = nd.sum_gh_pair;
    longlong2 *h = hist_q + (size_t)x_in * tb.n_bins;
    const double inv_g = tb.quant->inv_g, inv_h = tb.quant->inv_h;
    // SUB: is this node the sibling of the pair's built node?
    const longlong2 *h_par = nullptr, *h_built = nullptr;
    if (SUB && level > 0 && active && !tb.singles(level)) {
        const int built = tb.hpair_built[x_in >> 1];
        if (built >= 0 && built != x) {
            h_par = tb.hist(level + 1) + (size_t)(x_in >> 1) * tb.n_bins;
            h_built = hist_q + (size_t)(built - ((1 << level) - 1)) * tb.n_bins;
        }
    }

    // The pack's bins are read with consecutive lanes on consecutive bins (whole lines per load) and handed
    // over through LDS to the scan's layout of four consecutive bins per lane.
    __shared__ longlong2 s_v[kWaves][kEvalPackBins];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int b = b_begin + j * 64 + lane;
        if (b < b_end) {
            longlong2 v;
            if (SUB && h_par != nullptr) {
                const longlong2 pv = h_par[b], bv = h_built[b];
                v = make_longlong2(pv.x - bv.x, pv.y - bv.y);
                if (store_sibling) h[b] = v;
            } else {
                v = h[b];
            }
            s_v[w][j * 64 + lane] = v;
        }
    }
    __syncthreads();
    long long incg[4], inch[4];
    int lastb[4];  // pack-relative index of the last bin of the element's feature
    bool valid[4], head[4], last[4], ign[4];
    long long rung = 0, runh = 0;
    bool any_head = false;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        int b = b_begin + lane * 4 + j;
        valid[j] = b < b_end;
        lastb[j] = 0;
        head[j] = false;
        last[j] = false;
        ign[j] = false;
        incg[j] = inch[j] = 0;
        if (valid[j]) {
            const longlong2 v = s_v[w][lane * 4 + j];
            // one word per bin instead of the chain bin -> feature -> feature's bin range
            const unsigned meta = tb.bin_meta[b];  // low byte: bins up to the feature's last one, bit 8: first bin
            ign[j] = tb.ignored != nullptr && tb.ignored[tb.cut_fid[b]] != 0;
            const int to_last = (int)(meta & 0xffu);
            head[j] = (meta & 0x100u) != 0;
            last[j] = to_last == 0;
            lastb[j] = b + to_last - b_begin;
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
            if (ign[j]) score = 0.f;  // column sampling: hist_tree_builder_single.cu:304 / :663
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
    // wavefront arg-max: larger |score| wins, ties go to the smaller bin index. Only the key travels through the
    // butterfly; the lane that holds the winner writes its candidate itself.
    float win = best;
    int win_idx = best_idx;
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) {
        const float oa = __shfl_xor(win, d);
        const int oi = __shfl_xor(win_idx, d);
        if (oa > win || (oa == win && oi < win_idx)) {
            win = oa;
            win_idx = oi;
        }
    }
    // (without any candidate every lane still holds the initial key and the first one writes the empty record)
    const unsigned long long owners = __ballot(best == win && best_idx == win_idx);
    if (active && lane == __ffsll((long long)owners) - 1) {
        SplitCand c;
        c.score = best_score;
        c.index = best_idx;
        c.miss = best_miss;
        c.left = best_left;
        c.pad[0] = c.pad[1] = 0;
        tb.cand[(size_t)x_in * tb.n_packs + pack] = c;
    }
}

// Split search for features of any number of bins (max_num_bin above 255): one workgroup per (feature, node) walks the
// feature's bins in chunks of kBlock with a block-wide inclusive scan of the exact 64-bit sums and a carry from
// chunk to chunk. Same candidates, gains and tie rule as k_eval_split (whose wavefront holds a whole feature of at
// most 256 bins); one candidate per feature. In the CSR layout the node of a pair that was not built from rows is
// derived as parent - built while it is read (and stored for the next level); the dense layout's k_hist_merge has
// done that already.
__device__ __forceinline__ longlong2 wide_bin(const longlong2 *h, const longlong2 *h_par, const longlong2 *h_built, int b) {
    if (h_par == nullptr) return h[b];
    const longlong2 pv = h_par[b], bv = h_built[b];
    return make_longlong2(pv.x - bv.x, pv.y - bv.y);
}

__global__ __launch_bounds__(kBlock) void k_eval_split_wide(TreeBuffers tb_all, int level, float mcw, float lambda,
                                                           bool store_sibling) {
#pragma clang fp contract(off)
    __shared__ long long s_g[kWaves], s_h[kWaves];
    __shared__ float s_abs[kWaves];
    __shared__ int s_idx[kWaves];
    const TreeBuffers tb = tb_all.for_class(blockIdx.z);
    const int f = blockIdx.x;
    const int x_in = blockIdx.y + tb.lvl_x0;
    const int x = (1 << level) - 1 + x_in;
    const TreeNode nd = tb.nodes[x];
    if (!nd.is_valid) return;  // (nobody reads the candidates of an invalid node)
    const int cb = tb.cut_row_ptr[f], ce = tb.cut_row_ptr[f + 1];
    SplitCand *out = &tb.cand[(size_t)x_in * tb.n_packs + f];
    if (cb == ce) {
        if (threadIdx.x == 0) out->index = 0x7fffffff;  // a feature without bins has no candidate
        return;
    }
    const int lane = lane_id(), w = wave_id();
    longlong2 *h = tb.hist(level) + (size_t)x_in * tb.n_bins;
    const longlong2 *h_par = nullptr, *h_built = nullptr;
    if (tb.sparse && level > 0 && !tb.singles(level)) {  // (the dense layout's k_hist_merge has derived the siblings)
        const int built = tb.hpair_built[x_in >> 1];
        if (built >= 0 && built != x) {
            h_par = tb.hist(level + 1) + (size_t)(x_in >> 1) * tb.n_bins;
            h_built = tb.hist(level) + (size_t)(built - ((1 << level) - 1)) * tb.n_bins;
        }
    }
    const GHPair S = nd.sum_gh_pair;
    const double inv_g = tb.quant->inv_g, inv_h = tb.quant->inv_h;
    const bool ign = tb.ignored != nullptr && tb.ignored[f] != 0;
    // ---- the feature's total (missing = node sum - total), the derived sibling stored on the way
    long long tg = 0, th = 0;
    for (int b = cb + threadIdx.x; b < ce; b += kBlock) {
        const longlong2 v = wide_bin(h, h_par, h_built, b);
        if (h_par != nullptr && store_sibling) h[b] = v;
        tg += v.x;
        th += v.y;
    }
    tg = wave_sum_ll(tg);
    th = wave_sum_ll(th);
    if (lane == 0) {
        s_g[w] = tg;
        s_h[w] = th;
    }
    __syncthreads();
    tg = th = 0;
    for (int i = 0; i < kWaves; ++i) {
        tg += s_g[i];
        th += s_h[i];
    }
    __syncthreads();
    const GHPair m{S.g - (float)((double)tg * inv_g), S.h - (float)((double)th * inv_h)};
    // ---- candidates, chunk by chunk
    long long carry_g = 0, carry_h = 0;
    float best = -1.f, best_score = 0.f;
    int best_idx = 0x7fffffff;
    GHPair best_left{0, 0};
    for (int base = cb; base < ce; base += kBlock) {
        const int b = base + threadIdx.x;
        longlong2 v = make_longlong2(0, 0);
        if (b < ce) v = (h_par != nullptr && !store_sibling) ? wide_bin(h, h_par, h_built, b) : h[b];
        long long ig = v.x, ih = v.y;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const long long pg = shfl_up_ll(ig, d), ph = shfl_up_ll(ih, d);
            if (lane >= d) {
                ig += pg;
                ih += ph;
            }
        }
        if (lane == 63) {
            s_g[w] = ig;
            s_h[w] = ih;
        }
        __syncthreads();
        long long wg = 0, wh = 0, cg = 0, ch = 0;
        for (int i = 0; i < kWaves; ++i) {
            if (i < w) {
                wg += s_g[i];
                wh += s_h[i];
            }
            cg += s_g[i];
            ch += s_h[i];
        }
        __syncthreads();
        if (b < ce) {
            const long long exg = carry_g + wg + ig - v.x, exh = carry_h + wh + ih - v.y;  // bins below b
            const GHPair l{(float)((double)exg * inv_g), (float)((double)exh * inv_h)};
            const float gr = split_gain(S, l, mcw, lambda);
            const GHPair l2{l.g + m.g, l.h + m.h};
            const float gl = split_gain(S, l2, mcw, lambda);
            float score = (gl > gr) ? gl : -gr;
            if (ign) score = 0.f;  // column sampling: hist_tree_builder_single.cu:304 / :663
            const float a = fabsf(score);
            if (a > best) {  // (a thread's bins ascend: the first maximum is the one with the smallest index)
                best = a;
                best_score = score;
                best_idx = b;
                best_left = l;
            }
        }
        carry_g += cg;
        carry_h += ch;
    }
    // workgroup arg-max: larger |score| wins, ties go to the smaller bin index (hist_tree_builder_single.cu:330-335)
    float win = best;
    int win_idx = best_idx;
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) {
        const float oa = __shfl_xor(win, d);
        const int oi = __shfl_xor(win_idx, d);
        if (oa > win || (oa == win && oi < win_idx)) {
            win = oa;
            win_idx = oi;
        }
    }
    if (lane == 0) {
        s_abs[w] = win;
        s_idx[w] = win_idx;
    }
    __syncthreads();
    for (int i = 0; i < kWaves; ++i) {
        if (s_abs[i] > win || (s_abs[i] == win && s_idx[i] < win_idx)) {
            win = s_abs[i];
            win_idx = s_idx[i];
        }
    }
    if (best == win && best_idx == win_idx) {  // exactly one thread: bin indices are distinct
        SplitCand c;
        c.score = best_score;
        c.index = best_idx;
        c.miss = m;
        c.left = best_left;
        c.pad[0] = c.pad[1] = 0;
        *out = c;
    }
}

// Per node: reduce the wavefront candidates, fill the split record (hist_tree_builder_single.cu
// :365-389) and apply it to the tree (update_tree, :860-899). One workgroup per node of the level.
__global__ __launch_bounds__(kBlock) void k_best_update(TreeBuffers tb_all, int level, float rt_eps, float lambda) {
    const TreeBuffers tb = tb_all.for_class(blockIdx.z);
    __shared__ float s_abs[kWaves];
    __shared__ int s_idx[kWaves];
    __shared__ int s_pack[kWaves];
    const int x_in = blockIdx.x + tb.lvl_x0;
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
    if (tb.best_key != nullptr) {
        // sparse level pass: the tasks have already reduced their candidates to one key per node (larger |gain|,
        // then smaller bin index); the record sits in the slot of the task that searches the winning bin's feature
        if (threadIdx.x == 0) {
            const unsigned long long key = tb.best_key[x_in];
            tb.best_key[x_in] = 0ull;  // ready for the next level
            if (key != 0ull) {
                best_idx = (int)(0xffffffffu - (unsigned)key);
                best_pack = tb.feat_slot[tb.cut_fid[best_idx]];
                best = __uint_as_float((unsigned)(key >> 32));
            }
        }
    } else
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
    if (best_pack < 0) {  // no candidate at all (a node none of whose rows stores a value): a leaf
        SplitPoint z{};
        z.nid = x;
        z.split_fea_id = -1;
        sp = z;
        node.is_leaf = true;
        tb.nodes[node.lch_index].is_valid = false;
        tb.nodes[node.rch_index].is_valid = false;
        return;
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
        if (tb.split_bin != nullptr) tb.split_bin[x] = c.index - fbegin;
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

// Partition work items: every node of a level that holds rows owns ceil(rows / kPartChunk) items, planned one level
// ahead (k_tree_init for the root, k_part_scan_plan for the children it creates) so that no planning step sits
// between the split search and the partition; the items of a node that did not split return at once.
// Decide left/right for every row of a work item from the split feature's column of the bin matrix
// (missing -> default direction, else right iff bin >= split bin; the reference's rule at
// hist_tree_builder_single.cu:986-1011) and count the rows that go left.
template <bool DIRECT, typename BinT>
__global__ __launch_bounds__(kBlock) void k_part_count_dense(TreeBuffers tb_all, DenseBins bins, int level) {
    __shared__ int lds[kWaves];
    __shared__ int s_x;
    const TreeBuffers tb = tb_all.for_class(blockIdx.z);
    const int *__restrict__ ridx = tb.list(level);
    const int item = blockIdx.x;
    if (item >= tb.ctl[level].n_pitems) return;
    const int nl = 1 << level, off = nl - 1;
    if (threadIdx.x == 0) s_x = find_owner(tb.pbegin(level), nl, item);
    __syncthreads();
    const int x_in = s_x;
    const TreeNode &nd = tb.nodes[off + x_in];
    if (!node_splits(nd)) {
        if (threadIdx.x == 0) tb.pitem_nleft[item] = 0;
        return;
    }
    const int2 sg = tb.seg[off + x_in];
    const int pb = sg.x + (item - tb.pbegin(level)[x_in]) * kPartChunk;
    const int pe = min(sg.y, pb + kPartChunk);
    const int f = nd.split_feature_id;
    // (features of more than 255 bins keep their split bin in a side array: TreeNode::split_bid is a byte)
    const int sbid = tb.split_bin != nullptr ? tb.split_bin[off + x_in] : (int)nd.split_bid;
    const bool dr = nd.default_right;
    // A stored bin outside [lo, lo + span) means that the row has no value of the feature: the missing sentinel, or
    // (a feature that shares its column with others, DenseBins::feat_col) a bin of another feature of the bundle.
    int c = f, lo = 0, span = sizeof(BinT) == 2 ? kMissingBin16 : kMissingBin;
    if (sizeof(BinT) == 1 && bins.feat_col != nullptr) {
        c = bins.feat_col[f];
        lo = bins.feat_lo[f];
        span = tb.cut_row_ptr[f + 1] - tb.cut_row_ptr[f];
    }
    const BinT *column = reinterpret_cast<const BinT *>(bins.col) + (size_t)c * bins.col_stride;
    int nleft = 0;
    // All row ids first, then all bins, then the decisions, then the stores. Every load is unconditional (positions
    // past the item's end are clamped to its last row), so each phase's loads are issued back to back and a thread's
    // eight gathers are in flight together; a conditional load would make the compiler wait for everything
    // outstanding, the previous store included, before the next one.
    constexpr int R = kPartChunk / kBlock;
    int row[R], b[R];
#pragma unroll
    for (int k = 0; k < R; ++k) {
        const int pos = min(pb + k * kBlock + (int)threadIdx.x, pe - 1);
        row[k] = DIRECT ? pos : ridx[pos];
    }
#pragma unroll
    for (int k = 0; k < R; ++k) b[k] = column[row[k]];
    unsigned rights = 0;
#pragma unroll
    for (int k = 0; k < R; ++k) {
        const int t = b[k] - lo;
        const bool right = ((unsigned)t >= (unsigned)span) ? dr : (t >= sbid);
        rights |= (right ? 1u : 0u) << k;
        if (pb + k * kBlock + (int)threadIdx.x < pe) nleft += right ? 0 : 1;
    }
    // the decisions of a thread's eight rows as one byte (k_part_scatter gives the same rows to the same thread)
    static_assert(R <= 8, "a byte per thread holds the decisions of its rows");
    tb.goes_right[(size_t)item * kBlock + threadIdx.x] = (uint8_t)rights;
    int tot = block_sum(nleft, lds);
    if (threadIdx.x == 0) tb.pitem_nleft[item] = tot;
}

// Scan the per-item left counts, publish the children's row segments and plan the histogram work
// of the next level: per sibling pair the child with fewer rows is built (ties: the left one, as
// hist_tree_builder_single.cu:466-467), the other one comes from subtraction. One workgroup.
constexpr int kScanLdsItems = 12 * 1024;  // item offsets that k_part_scan_plan keeps in LDS (25 M rows)
__global__ __launch_bounds__(kBlock) void k_part_scan_plan(TreeBuffers tb_all, int level) {
    const TreeBuffers tb = tb_all.for_class(blockIdx.z);
    __shared__ int lds[kWaves];
    __shared__ int s_loff[kScanLdsItems + 1];
    const int nl = 1 << level, off = nl - 1;
    const int n_p = tb.ctl[level].n_pitems;
    const int *pb_cur = tb.pbegin(level);
    int *pb_next = tb.pbegin(level + 1);
    // the offsets of the items also stay in LDS when they fit, so that the per-node step below does not wait for
    // its own global stores
    const bool in_lds = n_p <= kScanLdsItems;
    // (what the per-node step needs from global memory is requested here, next to the item counts: one round trip)
    TreeNode my_node{};
    int2 my_seg = make_int2(0, 0);
    int my_pb0 = 0, my_pb1 = 0;
    const bool fast = nl <= kBlock && !tb.singles(level + 1) && (int)threadIdx.x < nl;
    if (fast) {
        my_node = tb.nodes[off + threadIdx.x];
        my_seg = tb.seg[off + threadIdx.x];
        my_pb0 = pb_cur[threadIdx.x];
        my_pb1 = pb_cur[threadIdx.x + 1];
    }
    int carry = 0;
    constexpr int IPT = 20;  // items per thread and step (10 M rows are 4 883 items: one step)
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
            if (i0 + j < n_p) {
                tb.pitem_loff[i0 + j] = run;
                if (in_lds) s_loff[i0 + j] = run;
            }
            run += v[j];
        }
        carry += tot;
    }
    if (threadIdx.x == 0) {
        tb.pitem_loff[n_p] = carry;
        if (in_lds) s_loff[n_p] = carry;
    }
    __syncthreads();
    if (tb.singles(level + 1)) {
        // No parent histograms below this level (the arena is smaller than the level): every child of a split node
        // is built from its own rows; the plan's "pairs" are the 2 nl single nodes of the next level.
        int rows_sum = 0, n_built = 0;
        for (int x_in = threadIdx.x; x_in < nl; x_in += kBlock) {
            const TreeNode &nd = tb.nodes[off + x_in];
            const int2 sg = tb.seg[off + x_in];
            if (node_splits(nd)) {
                const int nleft = tb.pitem_loff[pb_cur[x_in + 1]] - tb.pitem_loff[pb_cur[x_in]];
                tb.node_nleft[x_in] = nleft;
                tb.seg[nd.lch_index] = make_int2(sg.x, sg.x + nleft);
                tb.seg[nd.rch_index] = make_int2(sg.x + nleft, sg.y);
                tb.hpair_built[2 * x_in] = nd.lch_index;
                tb.hpair_built[2 * x_in + 1] = nd.rch_index;
                rows_sum += sg.y - sg.x;
                n_built += 2;
            } else {
                tb.node_nleft[x_in] = 0;
                tb.seg[nd.lch_index] = make_int2(0, 0);
                tb.seg[nd.rch_index] = make_int2(0, 0);
                tb.hpair_built[2 * x_in] = -1;
                tb.hpair_built[2 * x_in + 1] = -1;
            }
        }
        const int total_rows = block_sum(rows_sum, lds);
        n_built = block_sum(n_built, lds);
        const int room = max(tb.target_hitems / 4, tb.target_hitems - n_built);
        int chunk = (total_rows + room - 1) / room;
        chunk = max(kHistMinChunk, (chunk + 255) / 256 * 256);
        int hcarry = 0, pcarry = 0;
        for (int base = 0; base < 2 * nl; base += kBlock) {
            const int c_in = base + threadIdx.x;
            int cnt = 0, pc = 0;
            if (c_in < 2 * nl) {
                const int2 sg = tb.seg[2 * nl - 1 + c_in];  // the child's heap id: (2 nl - 1) + c_in
                if (tb.hpair_built[c_in] >= 0) cnt = (sg.y - sg.x + chunk - 1) / chunk;
                pc = (sg.y - sg.x + kPartChunk - 1) / kPartChunk;
            }
            int tot, ptot;
            const int ex = block_excl_scan(cnt, lds, &tot);
            const int pex = block_excl_scan(pc, lds, &ptot);
            if (c_in < 2 * nl) {
                tb.hpair_begin[c_in] = hcarry + ex;
                pb_next[c_in] = pcarry + pex;
            }
            hcarry += tot;
            pcarry += ptot;
        }
        if (threadIdx.x == 0) {
            tb.hpair_begin[2 * nl] = hcarry;
            pb_next[2 * nl] = pcarry;
            LevelCtl c;
            c.hchunk = chunk;
            c.n_hitems = hcarry;
            c.n_pitems = pcarry;
            c.rows_built = total_rows;
            tb.ctl[level + 1] = c;
        }
        return;
    }
    if (nl <= kBlock) {
        // the usual case (levels up to 8): one node per thread, everything after the scan stays in registers
        const int x_in = threadIdx.x;
        int built = -1, rows = 0;
        int pl = 0, pr = 0;  // partition items of the two children
        if (x_in < nl) {
            const TreeNode &nd = my_node;
            const int2 sg = my_seg;
            if (node_splits(nd)) {
                const int nleft = in_lds ? s_loff[my_pb1] - s_loff[my_pb0] : tb.pitem_loff[my_pb1] - tb.pitem_loff[my_pb0];
                const int nright = (sg.y - sg.x) - nleft;
                tb.node_nleft[x_in] = nleft;
                tb.seg[nd.lch_index] = make_int2(sg.x, sg.x + nleft);
                tb.seg[nd.rch_index] = make_int2(sg.x + nleft, sg.y);
                built = (nleft <= nright) ? nd.lch_index : nd.rch_index;
                rows = min(nleft, nright);
                pl = (nleft + kPartChunk - 1) / kPartChunk;
                pr = (nright + kPartChunk - 1) / kPartChunk;
            } else {
                tb.node_nleft[x_in] = 0;
                tb.seg[nd.lch_index] = make_int2(0, 0);
                tb.seg[nd.rch_index] = make_int2(0, 0);
            }
            tb.hpair_built[x_in] = built;
        }
        const int total_rows = block_sum(rows, lds);
        const int n_built = block_sum(built >= 0 ? 1 : 0, lds);
        const int room = max(tb.target_hitems / 4, tb.target_hitems - n_built);
        int chunk = (total_rows + room - 1) / room;
        chunk = max(kHistMinChunk, (chunk + 255) / 256 * 256);
        const int cnt = built >= 0 ? (rows + chunk - 1) / chunk : 0;
        int tot, ptot;
        const int ex = block_excl_scan(cnt, lds, &tot);
        const int pex = block_excl_scan(pl + pr, lds, &ptot);
        if (x_in < nl) {
            tb.hpair_begin[x_in] = ex;
            pb_next[2 * x_in] = pex;
            pb_next[2 * x_in + 1] = pex + pl;
        }
        if (threadIdx.x == 0) {
            tb.hpair_begin[nl] = tot;
            pb_next[2 * nl] = ptot;
            LevelCtl c;
            c.hchunk = chunk;
            c.n_hitems = tot;
            c.n_pitems = ptot;
            c.rows_built = total_rows;
            tb.ctl[level + 1] = c;
        }
        return;
    }
    // children segments + rows of the built child of every pair
    int rows_sum = 0;
    for (int x_in = threadIdx.x; x_in < nl; x_in += kBlock) {
        const TreeNode &nd = tb.nodes[off + x_in];
        const int2 sg = tb.seg[off + x_in];
        int built = -1;
        if (node_splits(nd)) {
            int nleft = tb.pitem_loff[pb_cur[x_in + 1]] - tb.pitem_loff[pb_cur[x_in]];
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
    int n_built = 0;
    for (int x_in = threadIdx.x; x_in < nl; x_in += kBlock) n_built += tb.hpair_built[x_in] >= 0 ? 1 : 0;
    n_built = block_sum(n_built, lds);
    // every built node adds up to one partly filled item: size the items so that their number stays
    // within target_hitems (= the workgroups the chip holds at once; one more would run as a second round)
    const int room = max(tb.target_hitems / 4, tb.target_hitems - n_built);
    int chunk = (total_rows + room - 1) / room;
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
    // partition items of the next level: every child that received rows
    int pcarry = 0;
    for (int base = 0; base < nl; base += kBlock) {
        const int x_in = base + threadIdx.x;
        int pl = 0, pr = 0;
        if (x_in < nl) {
            const TreeNode &nd = tb.nodes[off + x_in];
            const int2 sl = tb.seg[nd.lch_index], sr = tb.seg[nd.rch_index];
            pl = (sl.y - sl.x + kPartChunk - 1) / kPartChunk;
            pr = (sr.y - sr.x + kPartChunk - 1) / kPartChunk;
        }
        int ptot;
        const int pex = block_excl_scan(pl + pr, lds, &ptot);
        if (x_in < nl) {
            pb_next[2 * x_in] = pcarry + pex;
            pb_next[2 * x_in + 1] = pcarry + pex + pl;
        }
        pcarry += ptot;
    }
    if (threadIdx.x == 0) {
        tb.hpair_begin[nl] = carry;
        pb_next[2 * nl] = pcarry;
        LevelCtl c;
        c.hchunk = chunk;
        c.n_hitems = carry;
        c.n_pitems = pcarry;
        c.rows_built = total_rows;
        tb.ctl[level + 1] = c;
    }
}

// Stable two-way compaction of a work item's rows into the children's segments with wavefront
// ballots and popcounts. (Moving the gradient pairs along with the row ids was measured: it makes
// the histogram's gradient reads sequential but costs more in this kernel than it saves there.)
// The row -> node map is not touched here; k_end_bounds / k_tree_end derive it from the row lists
// when it is needed.
template <bool DIRECT>
__global__ __launch_bounds__(kBlock) void k_part_scatter(TreeBuffers tb_all, int level) {
    __shared__ int s_x;
    __shared__ int s_cnt[kPartChunk / kBlock][2][kWaves];
    const TreeBuffers tb = tb_all.for_class(blockIdx.z);
    const int *__restrict__ ridx_cur = tb.list(level);
    int *__restrict__ ridx_next = tb.list(level + 1);
    const int item = blockIdx.x;
    if (item >= tb.ctl[level].n_pitems) return;
    const int nl = 1 << level, off = nl - 1;
    if (threadIdx.x == 0) s_x = find_owner(tb.pbegin(level), nl, item);
    __syncthreads();
    const int x_in = s_x;
    if (!node_splits(tb.nodes[off + x_in])) return;
    const int2 sg = tb.seg[off + x_in];
    const int first_item = tb.pbegin(level)[x_in];
    const int pb = sg.x + (item - first_item) * kPartChunk;
    const int pe = min(sg.y, pb + kPartChunk);
    const int loff = tb.pitem_loff[item] - tb.pitem_loff[first_item];
    int left_base = sg.x + loff;
    int right_base = sg.x + tb.node_nleft[x_in] + ((pb - sg.x) - loff);
    const int lane = lane_id(), w = wave_id();
    // all loads of the item first (unconditional, clamped positions), one barrier for the wavefront counts of all
    // eight steps, then all stores
    constexpr int R = kPartChunk / kBlock;
    int row[R];
    const unsigned rights = tb.goes_right[(size_t)item * kBlock + threadIdx.x];  // bit k: the thread's k-th row goes right
#pragma unroll
    for (int k = 0; k < R; ++k) {
        const int pos = min(pb + k * kBlock + (int)threadIdx.x, pe - 1);
        row[k] = DIRECT ? pos : ridx_cur[pos];
    }
#pragma unroll
    for (int k = 0; k < R; ++k) {
        const bool valid = pb + k * kBlock + (int)threadIdx.x < pe;
        const bool right = (rights >> k) & 1u;
        const unsigned long long mL = __ballot(valid && !right), mR = __ballot(valid && right);
        if (lane == 0) {
            s_cnt[k][0][w] = __popcll(mL);
            s_cnt[k][1][w] = __popcll(mR);
        }
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < R; ++k) {
        const bool valid = pb + k * kBlock + (int)threadIdx.x < pe;
        const bool right = (rights >> k) & 1u;
        const unsigned long long mL = __ballot(valid && !right), mR = __ballot(valid && right);
        int bL = 0, bR = 0, tL = 0, tR = 0;
#pragma unroll
        for (int i = 0; i < kWaves; ++i) {
            const int cl = s_cnt[k][0][i], cr = s_cnt[k][1][i];
            if (i < w) {
                bL += cl;
                bR += cr;
            }
            tL += cl;
            tR += cr;
        }
        if (valid) {
            const int dest = right ? right_base + bR + lanes_below(mR) : left_base + bL + lanes_below(mL);
            ridx_next[dest] = row[k];
        }
        left_base += tL;
        right_base += tR;
    }
}

// ---------------------------------------------------------------------------------- prune
// Bottom-up, level-parallel form of the reference's Tree::prune_self (src/thundergbm/tree.cu:96-128):
// a node whose two children are valid leaves and whose gain is below gamma becomes a leaf and its
// children are marked pruned; then final ids are renumbered over valid, unpruned nodes.
__device__ void prune_tree(const TreeBuffers &tb, float gamma) {  // every thread of a kBlock-wide workgroup
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
    // value a row adds to its prediction when it ended in node i: the weight of the first ancestor that
    // was not pruned (what predict_in_training finds by climbing, tree_builder.cu:62-74)
    for (int i = threadIdx.x; i < tb.n_nodes; i += kBlock) {
        int x = i;
        while (x != -1 && tb.nodes[x].is_pruned) x = tb.nodes[x].parent_index;
        tb.leaf_value[i] = x >= 0 ? tb.nodes[x].base_weight : 0.f;
    }
}

__global__ __launch_bounds__(kBlock) void k_prune(TreeBuffers tb_all, float gamma) {
    prune_tree(tb_all.for_class(blockIdx.z), gamma);
}

// -------------------------------------------------------------------------- end of a tree
// The trainer keeps rows as per-node lists; everything that happens per row after the last split
// search wants row order: the row -> node map (the reference's ins2node_id), the prediction update
// (tree_builder.cu:62-74), the training metric (pointwise_metric.cu:13-20, multiclass_metric.cu:39-44)
// and the next round's gradients (regression_obj.h:130-154). Scattering node ids from the lists into
// a row-ordered array costs one partial 128-byte line per row, so this kernel goes the other way:
// a workgroup owns kRowBlock consecutive rows, finds for every node that still holds rows the part of
// its (ascending) row list that falls into the block by binary search, drops the node ids into LDS
// and then walks its rows in order with coalesced accesses only.
//   A node holds rows if it is valid and was not split; a split node of level `lookup_level` still
// holds the rows of its children (the last level of a tree is never partitioned into lists: nobody
// reads those lists), each row's child follows from the split feature's bin as in
// hist_tree_builder_single.cu:986-1011.
// MODE 0: write the row -> node map only. 1: prediction update of one tree. 2: prediction update,
// metric partials, next gradients and their block statistics (objectives with one tree per round;
// same arithmetic and order as k_gradient_pointwise, k_sum_gh and k_metric_partial).
__device__ __forceinline__ void metric_row(int kind, int n, int K, int i, float yi, const float *__restrict__ yp,
                                           float p0, double &acc, float &accf);

struct TreeEndArgs {
    int lookup_level;
    const float *y;
    float *yp;
    float lr;
    int objective, metric_kind;
    GHPair *gh;
    GradStats *stats;
    double *metric_partial;
    int with_prune;  // prune the tree first (prune_self with `gamma`)
    float gamma;
    unsigned *gh_words;  // MODE 2: where the rows' gradient words go (word_from_row; nullptr: nowhere)
};

constexpr int kEndInline = 8;                        // shorter sub-ranges are handled by the finding thread
constexpr int kEndListCap = kRowBlock / kEndInline;  // so at most this many longer ones exist per block

// First position p of the ascending run list[sx, sy) with list[p] >= r, given first = list[sx] < r and
// last = list[sy - 1] >= r. A node's rows are spread roughly evenly over the matrix, so the search
// starts at the interpolated position, brackets the answer by doubling steps and bisects the bracket:
// a handful of probes that (unlike a bisection of the whole run) all fall into a few neighbouring lines.
__device__ int list_lower_bound(const int *__restrict__ list, int sx, int sy, int first, int last, int r) {
    int g = sx + (int)((long long)(r - first) * (sy - 1 - sx) / (last - first));
    g = min(max(g, sx + 1), sy - 1);
    int lo, hi;  // invariant: list[lo] < r <= list[hi]
    if (list[g] < r) {
        lo = g;
        int step = 16;
        while (lo + step < sy - 1 && list[lo + step] < r) {
            lo += step;
            step *= 2;
        }
        hi = min(lo + step, sy - 1);
    } else {
        hi = g;
        int step = 16;
        while (hi - step > sx && list[hi - step] >= r) {
            hi -= step;
            step *= 2;
        }
        lo = max(hi - step, sx);
    }
    while (hi - lo > 1) {
        int mid = lo + (hi - lo) / 2;
        if (list[mid] < r) lo = mid; else hi = mid;
    }
    return hi;
}

template <bool SPARSE>
__device__ __forceinline__ int end_child_of(const TreeBuffers &tb, const DenseBins &dbins, const CsrBins &cbins,
                                            const TreeNode &nd, int row) {
    bool right;
    if (SPARSE) {
        const int cb = tb.cut_row_ptr[nd.split_feature_id], ce = tb.cut_row_ptr[nd.split_feature_id + 1];
        // (the node's own heap id is its children's parent index; wide features keep their split bin in a side array)
        const int sb = tb.split_bin != nullptr ? tb.split_bin[(nd.lch_index - 1) / 2] : (int)nd.split_bid;
        right = csr_goes_right(cbins, row, cb, ce, cb + sb, nd.default_right);
    } else if (dbins.bin_bytes == 2) {
        const int b = reinterpret_cast<const uint16_t *>(dbins.col)[(size_t)nd.split_feature_id * dbins.col_stride + row];
        const int sb = tb.split_bin != nullptr ? tb.split_bin[(nd.lch_index - 1) / 2] : (int)nd.split_bid;
        right = (b == kMissingBin16) ? nd.default_right : (b >= sb);
    } else if (dbins.feat_col != nullptr) {
        const int f = nd.split_feature_id;
        const int t = (int)dbins.col[(size_t)dbins.feat_col[f] * dbins.col_stride + row] - (int)dbins.feat_lo[f];
        right = ((unsigned)t >= (unsigned)(tb.cut_row_ptr[f + 1] - tb.cut_row_ptr[f])) ? nd.default_right
                                                                                     : (t >= (int)nd.split_bid);
    } else {
        const int b = dbins.col[(size_t)nd.split_feature_id * dbins.col_stride + row];
        right = (b == kMissingBin) ? nd.default_right : (b >= nd.split_bid);
    }
    return right ? nd.rch_index : nd.lch_index;
}

// bound[b * n_holders + x] = first position of node x's row list whose row is >= b * kRowBlock (b = 0 ..
// n_blocks), 0 everywhere for nodes that hold no rows: row block b then owns positions [bound[b][x],
// bound[b + 1][x]) of every list. One thread per entry; neighbouring threads search neighbouring
// boundaries of the same list.
// with_prune: the launch has one workgroup more, which prunes the tree meanwhile (the searches read fields of the
// nodes that pruning does not touch; what both produce is first read by k_tree_end).
__global__ __launch_bounds__(kBlock) void k_end_bounds(TreeBuffers tb_all, int lookup_level, int n_blocks,
                                                      int with_prune, float gamma) {
    const TreeBuffers tb = tb_all.for_class(blockIdx.z);
    const int search_blocks = gridDim.x - (with_prune ? 1 : 0);
    if (with_prune && blockIdx.x == search_blocks) {
        prune_tree(tb, gamma);
        return;
    }
    const int n_holders = (1 << tb.depth) - 1;
    const size_t total = (size_t)n_holders * (n_blocks + 1);
    for (size_t idx = (size_t)blockIdx.x * kBlock + threadIdx.x; idx < total; idx += (size_t)search_blocks * kBlock) {
        const int x = (int)(idx / (n_blocks + 1)), b = (int)(idx % (n_blocks + 1));
        const TreeNode &nd = tb.nodes[x];
        const int level = 31 - __clz(x + 1);
        int pos = 0;
        if (nd.is_valid && (nd.split_feature_id < 0 || level == lookup_level)) {
            const int2 sg = tb.seg[x];
            if (sg.y > sg.x) {
                const long long r = (long long)b * kRowBlock;
                if (level == 0) {  // the root's list is the identity
                    pos = (int)min(max(r, (long long)sg.x), (long long)sg.y);
                } else {
                    const int *list = tb.list(level);
                    const int first = list[sg.x], last = list[sg.y - 1];
                    pos = r <= first ? sg.x : (r > last ? sg.y : list_lower_bound(list, sg.x, sg.y, first, last, (int)r));
                }
            }
        }
        tb.end_bound[(size_t)b * n_holders + x] = pos;
    }
}

// The row-ordered part of the end of a tree: s_leaf holds the node of every row of the block.
template <int MODE>
__device__ __forceinline__ void tree_end_rows(const TreeBuffers &tb, const TreeEndArgs &a, const short *s_leaf, int r0, int r1) {
    __shared__ float s_f[kStatsLds];
    __shared__ double s_d[kWaves];
    constexpr int U = 4;
    if (MODE == 0) {
        for (int i = r0 + threadIdx.x; i < r1; i += kBlock) {
            const int x = s_leaf[i - r0];
            if (x >= 0) tb.nid[i] = x;
        }
        return;
    }
    // rows in order; thread t takes rows t, t + kBlock, ... (the order every row-blocked reduction uses)
    const float *__restrict__ y = a.y;
    float *__restrict__ yp = a.yp;
    GHPair *__restrict__ gh = a.gh;
    const float *__restrict__ leaf_value = tb.leaf_value;
    RowStats st;
    double acc = 0;
    float accf = 0;
    for (int i0 = r0 + threadIdx.x; i0 < r1; i0 += kBlock * U) {
        float p[U], w[U], yi[U];
        bool ok[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int i = i0 + u * kBlock;
            ok[u] = i < r1;
            const int x = ok[u] ? s_leaf[i - r0] : -1;
            p[u] = ok[u] ? yp[i] : 0.f;
            yi[u] = (MODE == 2 && ok[u]) ? y[i] : 0.f;
            w[u] = x >= 0 ? leaf_value[x] : 0.f;
            ok[u] = ok[u] && (MODE == 2 || x >= 0);
            if (x >= 0) p[u] += a.lr * w[u];
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (!ok[u]) continue;
            const int i = i0 + u * kBlock;
            yp[i] = p[u];
            if (MODE == 2) {
                metric_row(a.metric_kind, tb.n, 1, i, yi[u], yp, p[u], acc, accf);
                const GHPair o = pointwise_gradient(a.objective, yi[u], p[u]);
                if (gh != nullptr) gh[i] = o;  // (nullptr: the next tree reads the words only)
                if (a.gh_words != nullptr) a.gh_words[i] = word_from_row(a.objective, yi[u], p[u]);
                st.add(o);
            }
        }
    }
    if (MODE == 2) {
        store_block_stats(st, s_f, a.stats + blockIdx.x);
        acc += (double)accf;
        store_block_sum_d(acc, s_d, a.metric_partial + blockIdx.x);
    }
}


template <int MODE, bool SPARSE>
__global__ __launch_bounds__(kBlock) void k_tree_end(TreeBuffers tb_all, DenseBins dbins, CsrBins cbins, TreeEndArgs a) {
    __shared__ short s_leaf[kRowBlock];  // node of every row of the block (depth <= 14: ids below 2^15), -1: none
    const TreeBuffers tb = tb_all.for_class(blockIdx.z);
    if (MODE == 1) a.yp += (size_t)blockIdx.z * tb.n;  // class-major predictions
    __shared__ int s_list[kEndListCap][3];  // node, first and one-past-last list position
    __shared__ int s_split[kEndListCap];    // -1: the rows stay in the node; else feature | bin << 16 | default_right << 24
    __shared__ int s_off[kEndListCap];
    __shared__ int s_scan[kWaves];
    __shared__ int s_n;
    const int r0 = blockIdx.x * kRowBlock, r1 = min(tb.n, r0 + kRowBlock);
    constexpr int U = 4;
    if (tb.nid16 != nullptr) {
        // sparse level pass: the row -> node map is kept per row, nothing to look up
        for (int i = threadIdx.x; i < kRowBlock; i += kBlock) s_leaf[i] = r0 + i < r1 ? (short)tb.nid16[r0 + i] : (short)-1;
    } else {
    for (int i = threadIdx.x; i < kRowBlock; i += kBlock) s_leaf[i] = -1;
    if (threadIdx.x == 0) s_n = 0;
    __syncthreads();
    const int n_holders = (1 << tb.depth) - 1;  // nodes of the levels that own row lists
    const int *b_lo = tb.end_bound + (size_t)blockIdx.x * n_holders, *b_hi = b_lo + n_holders;
    for (int x = threadIdx.x; x < n_holders; x += kBlock) {
        const int pa = b_lo[x], pb = b_hi[x];
        if (pb <= pa) continue;
        const TreeNode &nd = tb.nodes[x];
        // (trees of up to kEndListCap row-holding nodes list every sub-range: the inline walk is a chain of
        // dependent loads)
        if (pb - pa > kEndInline || n_holders <= kEndListCap) {
            int e = atomicAdd(&s_n, 1);
            s_list[e][0] = x;
            s_list[e][1] = pa;
            s_list[e][2] = pb;
            s_split[e] = nd.split_feature_id < 0
                             ? -1
                             : (nd.split_feature_id | (int)nd.split_bid << 16 | (nd.default_right ? 1 : 0) << 24);
        } else {
            const int *list = tb.list(31 - __clz(x + 1));
            for (int p = pa; p < pb; ++p) {
                const int row = x == 0 ? p : list[p];
                s_leaf[row - r0] = nd.split_feature_id >= 0 ? end_child_of<SPARSE>(tb, dbins, cbins, nd, row) : x;
            }
        }
    }
    __syncthreads();
    // The listed sub-ranges are walked as one flat index space spread over all threads (independent
    // loads in flight instead of one dependent chain per sub-range): s_off = exclusive scan of the lengths.
    const int n_list = s_n;
    int total = 0;
    for (int base = 0; base < n_list; base += kBlock) {
        const int e = base + threadIdx.x;
        const int len = e < n_list ? s_list[e][2] - s_list[e][1] : 0;
        int tot;
        const int ex = block_excl_scan(len, s_scan, &tot);
        if (e < n_list) s_off[e] = total + ex;
        total += tot;
    }
    __syncthreads();
    for (int j0 = threadIdx.x; j0 < total; j0 += kBlock * U) {
        // (every load is unconditional - entries past the end repeat the last one and are skipped when the results
        // are stored -, so a thread's four list entries, then its four bins, are in flight together)
        int node[U], row[U], split[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int j = min(j0 + u * kBlock, total - 1);
            int lo = 0, hi = n_list;  // last entry with s_off <= j
            while (hi - lo > 1) {
                const int mid = (lo + hi) / 2;
                if (s_off[mid] <= j) lo = mid; else hi = mid;
            }
            node[u] = s_list[lo][0];
            split[u] = s_split[lo];
            const int p = s_list[lo][1] + (j - s_off[lo]);
            const int listed = tb.list(31 - __clz(node[u] + 1))[p];  // (the root's list is the identity and not stored)
            row[u] = node[u] == 0 ? p : listed;
        }
        // (16-bit bins and bundled columns: the packed split word has no room for what the decision needs)
        if (SPARSE || dbins.bin_bytes == 2 || dbins.feat_col != nullptr) {
#pragma unroll
            for (int u = 0; u < U; ++u) {
                if (j0 + u * kBlock >= total) continue;
                s_leaf[row[u] - r0] =
                    split[u] >= 0 ? end_child_of<SPARSE>(tb, dbins, cbins, tb.nodes[node[u]], row[u]) : node[u];
            }
        } else {
            int bin[U];
#pragma unroll
            for (int u = 0; u < U; ++u)  // (feature 0 for the entries of nodes that did not split)
                bin[u] = dbins.col[(size_t)(split[u] >= 0 ? split[u] & 0xffff : 0) * dbins.col_stride + row[u]];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                if (j0 + u * kBlock >= total) continue;
                int leaf = node[u];
                if (split[u] >= 0) {
                    const bool right = bin[u] == kMissingBin ? (split[u] >> 24) != 0 : bin[u] >= ((split[u] >> 16) & 0xff);
                    leaf = 2 * node[u] + (right ? 2 : 1);  // heap order: children of x are 2x + 1 and 2x + 2
                }
                s_leaf[row[u] - r0] = leaf;
            }
        }
    }
    }  // row lists
    __syncthreads();
    tree_end_rows<MODE>(tb, a, s_leaf, r0, r1);
}

// ---------------------------------------------------------------------------------- metric
// kind 0: sum of squared errors; 1: correct binary decisions (sigmoid > 0.5 in double, like
// multiclass_metric.cu:40); 2: correct arg-max decisions (first maximum wins, :17-29).
__device__ __forceinline__ void metric_row(int kind, int n, int K, int i, float yi, const float *__restrict__ yp,
                                           float p0, double &acc, float &accf) {
    if (kind == 0) {
        float e = p0 - yi;
        accf += e * e;
    } else if (kind == 1) {
        // sigmoid(p) > 0.5 evaluated in double as in the reference; away from zero that is the sign of p
        int k = fabsf(p0) > 1e-6f ? (p0 > 0.f ? 1 : 0) : ((1.0 / (1.0 + exp(-(double)p0)) > 0.5) ? 1 : 0);
        acc += (k == yi) ? 1 : 0;
    } else {
        int mk = 0;
        float mp = p0;
        for (int k = 1; k < K; ++k) {
            float v = yp[(size_t)k * n + i];
            if (v > mp) {
                mp = v;
                mk = k;
            }
        }
        acc += (mk == yi) ? 1 : 0;
    }
}

__global__ __launch_bounds__(kBlock) void k_metric_partial(int kind, int n, int K, const float *__restrict__ y,
                                                          const float *__restrict__ yp, double *__restrict__ out) {
    __shared__ double sd[kWaves];
    double acc = 0;
    float accf = 0;
    const int r0 = blockIdx.x * kRowBlock, r1 = min(n, r0 + kRowBlock);
    for (int i = r0 + threadIdx.x; i < r1; i += kBlock) metric_row(kind, n, K, i, y[i], yp, yp[i], acc, accf);
    acc += (double)accf;
    store_block_sum_d(acc, sd, out + blockIdx.x);
}

// The counting metrics (kind 1 and 2) do not depend on the order of their additions, so their partials come from
// four times the threads per row block: the class predictions of a row are a chain of dependent-latency loads that
// 256 threads per 4096 rows do not hide.
constexpr int kCountBlock = 1024;
__global__ __launch_bounds__(kCountBlock) void k_metric_count(int kind, int n, int K, const float *__restrict__ y,
                                                             const float *__restrict__ yp, double *__restrict__ out) {
    __shared__ double sd[kCountBlock / 64];
    double acc = 0;
    float accf = 0;
    const int r0 = blockIdx.x * kRowBlock, r1 = min(n, r0 + kRowBlock);
    for (int i = r0 + threadIdx.x; i < r1; i += kCountBlock) metric_row(kind, n, K, i, y[i], yp, yp[i], acc, accf);
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) acc += __shfl_xor(acc, d);
    if (lane_id() == 0) sd[threadIdx.x / 64] = acc;
    __syncthreads();
    if (threadIdx.x == 0) {
        double t = 0;
        for (int i = 0; i < kCountBlock / 64; ++i) t += sd[i];
        out[blockIdx.x] = t;
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

int grid_for(size_t n, int cap = 4096) {
    size_t b = (n + kBlock - 1) / kBlock;
    if (b < 1) b = 1;
    if (b > (size_t)cap) b = cap;
    return (int)b;
}

}  // namespace

// =================================================================================== launchers
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

void launch_bagging(hipStream_t s, int N, unsigned seed, int *count, GHPair *gh, const int *perm, int n_rows) {
    k_bagging_draw<<<grid_for(N), kBlock, 0, s>>>(N, seed, count);
    k_bagging_apply<<<grid_for(N), kBlock, 0, s>>>(N, count, gh, perm, n_rows);
}

// Launchers: `tb` is the first buffer set to use, `n_class` consecutive sets (class trees of one round)
// are served by the same launch through blockIdx.z; gradient and prediction pointers address the
// first of those classes.
void launch_tree_init(hipStream_t s, const TreeBuffers &tb, const GHPair *gh_class, float lambda, bool stats_ready,
                      int n_class) {
    if (!stats_ready)  // n_grad_blocks == row_blocks(n)
        k_sum_gh<<<dim3(tb.n_grad_blocks, 1, n_class), kBlock, 0, s>>>(tb.n, gh_class, tb.root_partial);
    k_tree_init<<<dim3(1, 1, n_class), kBlock, 0, s>>>(tb, lambda);
    if (tb.nid16 != nullptr) {
        // sparse level pass: every row starts in the root (the n_class maps lie back to back)
        const size_t words = ((size_t)tb.n + 2) / 2 * (size_t)n_class;
        k_fill_u32<<<grid_for(words), kBlock, 0, s>>>(reinterpret_cast<unsigned *>(tb.nid16), 0u, words);
    }
}

template <int LPR, int SLOTS, bool BIN16>
static void hist_dense_launch(hipStream_t s, const TreeBuffers &tb, const DenseBins &bins, const GHPair *gh,
                              int level, int n_class) {
    const int n_pairs = tb.n_hpairs(level);
    dim3 grid(bins.n_blocks, tb.max_hitems, n_class);
    size_t lds = (size_t)tb.max_block_bins * sizeof(unsigned long long);
    if (lds > 64 * 1024) {
        // more than the default dynamic LDS window: opt in once per kernel instance and size
        static size_t opted = 0;
        if (lds > opted) {
            HIP_CHECK(hipFuncSetAttribute(
                reinterpret_cast<const void *>(&k_hist_dense<LPR, true, kHistBlock, SLOTS, BIN16>),
                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
            HIP_CHECK(hipFuncSetAttribute(
                reinterpret_cast<const void *>(&k_hist_dense<LPR, false, kHistBlock, SLOTS, BIN16>),
                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
            opted = lds;
        }
    }
    if constexpr (!BIN16 && LPR >= 4) {
        if (bins.gh_lane >= 0 && bins.gh_fresh) {
            if (lds > 64 * 1024) {
                static size_t opted_w = 0;
                if (lds > opted_w) {
                    HIP_CHECK(hipFuncSetAttribute(
                        reinterpret_cast<const void *>(&k_hist_dense<LPR, true, kHistBlock, SLOTS, BIN16, true>),
                        hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
                    HIP_CHECK(hipFuncSetAttribute(
                        reinterpret_cast<const void *>(&k_hist_dense<LPR, false, kHistBlock, SLOTS, BIN16, true>),
                        hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
                    opted_w = lds;
                }
            }
            if (level == 0)
                k_hist_dense<LPR, true, kHistBlock, SLOTS, BIN16, true><<<grid, kHistBlock, lds, s>>>(tb, bins, gh, level, n_pairs);
            else
                k_hist_dense<LPR, false, kHistBlock, SLOTS, BIN16, true><<<grid, kHistBlock, lds, s>>>(tb, bins, gh, level, n_pairs);
            return;
        }
    }
    if (level == 0)
        k_hist_dense<LPR, true, kHistBlock, SLOTS, BIN16><<<grid, kHistBlock, lds, s>>>(tb, bins, gh, level, n_pairs);
    else
        k_hist_dense<LPR, false, kHistBlock, SLOTS, BIN16><<<grid, kHistBlock, lds, s>>>(tb, bins, gh, level, n_pairs);
}

template <int LPR>
static void hist_dense_dispatch(hipStream_t s, const TreeBuffers &tb, const DenseBins &bins, const GHPair *gh,
                                int level, int n_class) {
    const int slots = (tb.max_block_bins + kHistBlock - 1) / kHistBlock;  // bins drained per thread
    if (bins.bin_bytes == 2) {  // (fewer variants: the blocks of 16-bit bins are sized to fill the LDS)
        if (slots <= 4) hist_dense_launch<LPR, 4, true>(s, tb, bins, gh, level, n_class);
        else if (slots <= 8) hist_dense_launch<LPR, 8, true>(s, tb, bins, gh, level, n_class);
        else if (slots <= 20) hist_dense_launch<LPR, 20, true>(s, tb, bins, gh, level, n_class);
        else fatal("feature block with %d bins does not fit the histogram kernel", tb.max_block_bins);
        return;
    }
    if (slots <= 1) hist_dense_launch<LPR, 1, false>(s, tb, bins, gh, level, n_class);
    else if (slots <= 2) hist_dense_launch<LPR, 2, false>(s, tb, bins, gh, level, n_class);
    else if (slots <= 3) hist_dense_launch<LPR, 3, false>(s, tb, bins, gh, level, n_class);
    else if (slots <= 4) hist_dense_launch<LPR, 4, false>(s, tb, bins, gh, level, n_class);
    else if (slots <= 6) hist_dense_launch<LPR, 6, false>(s, tb, bins, gh, level, n_class);
    else if (slots <= 7) hist_dense_launch<LPR, 7, false>(s, tb, bins, gh, level, n_class);  // fewer accumulator registers
    else if (slots <= 8) hist_dense_launch<LPR, 8, false>(s, tb, bins, gh, level, n_class);
    else if (slots <= 16) hist_dense_launch<LPR, 16, false>(s, tb, bins, gh, level, n_class);
    else if (slots <= 20) hist_dense_launch<LPR, 20, false>(s, tb, bins, gh, level, n_class);
    else fatal("feature block with %d bins does not fit the histogram kernel", tb.max_block_bins);
}

void launch_hist_dense(hipStream_t s, const TreeBuffers &tb, const DenseBins &bins, const GHPair *gh, int level,
                       int n_class) {
    switch (bins.W * bins.bin_bytes) {  // bytes per row of a block = 4 x lanes per row
        case 4: hist_dense_dispatch<1>(s, tb, bins, gh, level, n_class); break;
        case 8: hist_dense_dispatch<2>(s, tb, bins, gh, level, n_class); break;
        case 16: hist_dense_dispatch<4>(s, tb, bins, gh, level, n_class); break;
        case 32: hist_dense_dispatch<8>(s, tb, bins, gh, level, n_class); break;
        case 64: hist_dense_dispatch<16>(s, tb, bins, gh, level, n_class); break;
        default: fatal("unsupported dense block width %d x %d bytes", bins.W, bins.bin_bytes);
    }
}

void launch_hist_merge(hipStream_t s, const TreeBuffers &tb, int level, int n_class) {
    const int n_pairs = tb.hpair_hi(level) - tb.hpair_lo(level);  // of the served nodes
    if (tb.target_hitems <= 16) {
        // wide data: many feature blocks, so a node has only a handful of work items and very long histograms;
        // one thread per bin walks them (a block of 8 bins would leave most of its 32 groups without an item)
        dim3 grid((tb.n_bins + kBlock - 1) / kBlock, n_pairs, n_class);
        k_hist_merge<kBlock><<<grid, kBlock, 0, s>>>(tb, level);
    } else if (n_pairs * n_class <= 4) {
        dim3 grid((tb.n_bins + 7) / 8, n_pairs, n_class);
        k_hist_merge<8><<<grid, kBlock, 0, s>>>(tb, level);
    } else {
        dim3 grid((tb.n_bins + 31) / 32, n_pairs, n_class);
        k_hist_merge<32><<<grid, kBlock, 0, s>>>(tb, level);
    }
}

void launch_root_sum(hipStream_t s, const TreeBuffers &tb, const GHPair *gh_class, float lambda, int n_class) {
    if (tb.complete_feature >= 0) {
        k_root_sum_bins<<<dim3(1, 1, n_class), kBlock, 0, s>>>(tb, lambda);
    } else {
        const int blocks = std::max(1, std::min(kRootSumBlocks, (tb.n + kBlock - 1) / kBlock));
        k_root_sum_rows<<<dim3(blocks, 1, n_class), kBlock, 0, s>>>(tb, gh_class);
        k_root_sum_final<<<dim3(1, 1, n_class), kBlock, 0, s>>>(tb, blocks, lambda);
    }
}

long device_count_bytes(hipStream_t s, const uint8_t *d_v, size_t n, uint8_t value) {
    unsigned long long *d_out = nullptr, h = 0;
    HIP_CHECK(hipMalloc(&d_out, sizeof(unsigned long long)));
    HIP_CHECK(hipMemsetAsync(d_out, 0, sizeof(unsigned long long), s));
    k_count_bytes<<<grid_for(n, 2048), kBlock, 0, s>>>(d_v, n, value, d_out);
    HIP_CHECK(hipMemcpyAsync(&h, d_out, sizeof(h), hipMemcpyDeviceToHost, s));
    HIP_CHECK(hipStreamSynchronize(s));
    HIP_CHECK(hipFree(d_out));
    return (long)h;
}

long device_count_u16(hipStream_t s, const uint16_t *d_v, size_t n, uint16_t value) {
    unsigned long long *d_out = nullptr, h = 0;
    HIP_CHECK(hipMalloc(&d_out, sizeof(unsigned long long)));
    HIP_CHECK(hipMemsetAsync(d_out, 0, sizeof(unsigned long long), s));
    k_count_u16<<<grid_for(n, 2048), kBlock, 0, s>>>(d_v, n, value, d_out);
    HIP_CHECK(hipMemcpyAsync(&h, d_out, sizeof(h), hipMemcpyDeviceToHost, s));
    HIP_CHECK(hipStreamSynchronize(s));
    HIP_CHECK(hipFree(d_out));
    return (long)h;
}

void launch_hist_csr(hipStream_t s, const TreeBuffers &tb, const CsrBins &bins, const GHPair *gh, int level,
                     int n_class) {
    const int n_pairs = tb.n_hpairs(level);
    const int zgrid = std::min(1024, (tb.n_bins + kBlock - 1) / kBlock);
    k_hist_zero_built<<<dim3(zgrid, tb.hpair_hi(level) - tb.hpair_lo(level), n_class), kBlock, 0, s>>>(tb, level);
    const size_t lds = (size_t)bins.head_bins * 2 * sizeof(unsigned long long);
    if (bins.hist_word != nullptr && lds > 64 * 1024) {
        static size_t opted = 0;  // more than the default dynamic LDS window: opt in once
        if (lds > opted) {
            HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(&k_hist_csr_head<true>),
                                          hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
            HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(&k_hist_csr_head<false>),
                                          hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
            opted = lds;
        }
    }
    if (level == 0 && bins.csc_row != nullptr) {
        const long tiles = (bins.nnz + 63) / 64;
        const int blocks = (int)std::min<long>(8192, (tiles + kWaves - 1) / kWaves);
        if (blocks > 0) k_hist_root_csc<<<dim3(blocks, 1, n_class), kBlock, 0, s>>>(tb, bins, gh);
        return;
    }
    const dim3 grid(tb.max_hitems, 1, n_class);
    if (bins.hist_word != nullptr) {
        if (level == 0) k_hist_csr_head<true><<<grid, kHistBlock, lds, s>>>(tb, bins, gh, n_pairs, level);
        else k_hist_csr_head<false><<<grid, kHistBlock, lds, s>>>(tb, bins, gh, n_pairs, level);
    } else {
        if (level == 0) k_hist_csr<true><<<grid, kBlock, 0, s>>>(tb, bins, gh, n_pairs, level);
        else k_hist_csr<false><<<grid, kBlock, 0, s>>>(tb, bins, gh, n_pairs, level);
    }
    // the sibling histograms (parent - built) are produced by k_eval_split<true>
}

void launch_eval_split(hipStream_t s, const TreeBuffers &tb, int level, float mcw, float lambda, int n_class,
                       bool store_sibling) {
    dim3 grid((tb.n_packs + kWaves - 1) / kWaves, tb.nodes_served(level), n_class);
    if (tb.sparse) k_eval_split<true><<<grid, kBlock, 0, s>>>(tb, level, mcw, lambda, store_sibling);
    else k_eval_split<false><<<grid, kBlock, 0, s>>>(tb, level, mcw, lambda, true);
}

void launch_eval_split_wide(hipStream_t s, const TreeBuffers &tb, int level, float mcw, float lambda, int n_class,
                            bool store_sibling) {
    dim3 grid(tb.F, tb.nodes_served(level), n_class);
    k_eval_split_wide<<<grid, kBlock, 0, s>>>(tb, level, mcw, lambda, store_sibling);
}

void launch_best_update(hipStream_t s, const TreeBuffers &tb, int level, float rt_eps, float lambda, int n_class) {
    k_best_update<<<dim3(tb.nodes_served(level), 1, n_class), kBlock, 0, s>>>(tb, level, rt_eps, lambda);
}

void launch_partition_dense(hipStream_t s, const TreeBuffers &tb, const DenseBins &bins, int level, int n_class) {
    if (level == tb.depth - 1) return;  // the last level's children never get row lists (see k_tree_end)
    const dim3 one(1, 1, n_class), items(tb.max_pitems, 1, n_class);
    const bool b16 = bins.bin_bytes == 2;
    if (level == 0) {
        if (b16) k_part_count_dense<true, uint16_t><<<items, kBlock, 0, s>>>(tb, bins, level);
        else k_part_count_dense<true, uint8_t><<<items, kBlock, 0, s>>>(tb, bins, level);
        k_part_scan_plan<<<one, kBlock, 0, s>>>(tb, level);
        k_part_scatter<true><<<items, kBlock, 0, s>>>(tb, level);
    } else {
        if (b16) k_part_count_dense<false, uint16_t><<<items, kBlock, 0, s>>>(tb, bins, level);
        else k_part_count_dense<false, uint8_t><<<items, kBlock, 0, s>>>(tb, bins, level);
        k_part_scan_plan<<<one, kBlock, 0, s>>>(tb, level);
        k_part_scatter<false><<<items, kBlock, 0, s>>>(tb, level);
    }
}

void launch_partition_csr(hipStream_t s, const TreeBuffers &tb, const CsrBins &bins, int level, int n_class) {
    if (level == tb.depth - 1) return;
    const dim3 one(1, 1, n_class), items(tb.max_pitems, 1, n_class);
    if (level == 0) {
        k_part_count_csr<true><<<items, kBlock, 0, s>>>(tb, bins, level);
        k_part_scan_plan<<<one, kBlock, 0, s>>>(tb, level);
        k_part_scatter<true><<<items, kBlock, 0, s>>>(tb, level);
    } else {
        k_part_count_csr<false><<<items, kBlock, 0, s>>>(tb, bins, level);
        k_part_scan_plan<<<one, kBlock, 0, s>>>(tb, level);
        k_part_scatter<false><<<items, kBlock, 0, s>>>(tb, level);
    }
}

template <bool SPARSE>
static void tree_end_launch(hipStream_t s, const TreeBuffers &tb, const DenseBins &d, const CsrBins &c, int mode,
                            const TreeEndArgs &a, int n_class) {
    const dim3 grid(row_blocks(tb.n), 1, n_class);
    if (mode == 0) k_tree_end<0, SPARSE><<<grid, kBlock, 0, s>>>(tb, d, c, a);
    else if (mode == 1) k_tree_end<1, SPARSE><<<grid, kBlock, 0, s>>>(tb, d, c, a);
    else k_tree_end<2, SPARSE><<<grid, kBlock, 0, s>>>(tb, d, c, a);
}

static void tree_end(hipStream_t s, const TreeBuffers &tb, const DenseBins *dbins, const CsrBins *cbins, int mode,
                     const TreeEndArgs &a, int n_class = 1) {
    const int n_blocks = row_blocks(tb.n);
    const size_t entries = (size_t)((1 << tb.depth) - 1) * (n_blocks + 1);
    if (tb.nid16 == nullptr)
        k_end_bounds<<<dim3(grid_for(entries, 8192) + (a.with_prune ? 1 : 0), 1, n_class), kBlock, 0, s>>>(
            tb, a.lookup_level, n_blocks, a.with_prune, a.gamma);
    else if (a.with_prune)
        k_prune<<<dim3(1, 1, n_class), kBlock, 0, s>>>(tb, a.gamma);
    if (tb.sparse) tree_end_launch<true>(s, tb, DenseBins{}, *cbins, mode, a, n_class);
    else tree_end_launch<false>(s, tb, *dbins, CsrBins{}, mode, a, n_class);
}

void launch_nid_rebuild(hipStream_t s, const TreeBuffers &tb, const DenseBins *dbins, const CsrBins *cbins,
                        int lookup_level) {
    TreeEndArgs a{};
    a.lookup_level = lookup_level;
    tree_end(s, tb, dbins, cbins, 0, a);
}

void launch_predict_in_training(hipStream_t s, const TreeBuffers &tb, const DenseBins *dbins, const CsrBins *cbins,
                                int lookup_level, float *yp_class, float lr, int n_class, const float *prune_gamma) {
    TreeEndArgs a{};
    a.lookup_level = lookup_level;
    a.yp = yp_class;
    a.lr = lr;
    a.with_prune = prune_gamma != nullptr;
    a.gamma = prune_gamma != nullptr ? *prune_gamma : 0.f;
    tree_end(s, tb, dbins, cbins, 1, a, n_class);
}

void launch_round_end(hipStream_t s, const TreeBuffers &tb, const DenseBins *dbins, const CsrBins *cbins,
                      int lookup_level, int objective, int metric_kind, const float *y, float *yp, float lr,
                      GHPair *gh, double *metric_scratch, float *metric_out, const float *prune_gamma,
                      unsigned *gh_words) {
    TreeEndArgs a{};
    a.gh_words = gh_words;
    a.with_prune = prune_gamma != nullptr;
    a.gamma = prune_gamma != nullptr ? *prune_gamma : 0.f;
    a.lookup_level = lookup_level;
    a.y = y;
    a.yp = yp;
    a.lr = lr;
    a.objective = objective;
    a.metric_kind = metric_kind;
    a.gh = gh;
    a.stats = tb.root_partial;
    a.metric_partial = metric_scratch;
    tree_end(s, tb, dbins, cbins, 2, a);
    k_metric_final<<<1, kBlock, 0, s>>>(metric_kind, tb.n, row_blocks(tb.n), metric_scratch, metric_out);
}

void launch_gh_words(hipStream_t s, int objective, int n, const float *y, const float *yp, unsigned *words) {
    if (n <= 0) return;
    k_gh_words<<<std::min(4096, (n + kBlock - 1) / kBlock), kBlock, 0, s>>>(objective, n, y, yp, words);
}

void launch_metric(hipStream_t s, int kind, int n, int num_class, const float *y, const float *yp, double *scratch,
                   float *out) {
    int blocks = row_blocks(n);  // scratch: one double per block
    if (kind == 0)
        k_metric_partial<<<blocks, kBlock, 0, s>>>(kind, n, num_class, y, yp, scratch);
    else
        k_metric_count<<<blocks, kCountBlock, 0, s>>>(kind, n, num_class, y, yp, scratch);
    k_metric_final<<<1, kBlock, 0, s>>>(kind, n, blocks, scratch, out);
}

}  // namespace tgbm
