// Sparse layout, level pass: histogram build and split search of one tree level in a single pass over the
// bin-major copy of the stored values (sorted by global bin id, rows ascending inside a bin).
//
// The reference (hist_tree_builder_single.cu:203-216, :485-505, :257-350, :614-752) keeps one histogram of all
// cut points per node and scans every bin of every node. With 100 000 features that is ~100 MB per node of which a
// deep node touches a few percent. Here a workgroup owns a run of features: it adds the fixed-point gradient pair
// of every stored value to an LDS table cell (bin, node of the value's row), then searches the tables of its
// features for the best candidate of every node (same prefix sums, missing-value term, gain formula and tie rule as
// the dense split search) and hands one candidate per node to k_best_update. Nothing per-node lives in HBM, nothing
// has to be zeroed or subtracted, and a (feature, node) pair without stored values costs one look at its cells.
// Sums are 64-bit integers at the tree's scales: exact, so the candidates are the very numbers a per-node histogram
// would give.
#include <algorithm>
#include <cstdlib>

#include "device_api.h"
#include "kernel_common.h"

namespace tgbm {
namespace {

constexpr int kSpBlock = 1024;
constexpr int kSpWaves = kSpBlock / 64;

struct SegResult {
    float win;     // |score| of the segment's best candidate, -1: none
    int win_idx;   // its global bin index
    float score;   // owner lane only: signed score, missing sums, left sums
    GHPair miss, left;
    bool owner;
};

// Best candidate of one (feature, node) segment; one wavefront, lane l looks at ceil(kf / 64) consecutive bins of the
// feature's kf <= 256 bins. cell(b) = cells[b * stride]. The arithmetic is that of k_eval_split: exact integer prefix sums,
// missing = node sum - feature total, gain with the missing rows sent right and left
// (hist_tree_builder_single.cu:300-323), largest |gain| wins, ties go to the smaller bin index (:330-335).
// `force`: evaluate even when the segment holds no value (the feature owning global bin 0: when no candidate of a
// node has a positive gain the arg-max of the reference ends on bin 0).
__device__ SegResult eval_segment(const longlong2 *cells, int stride, int kf, int gbin0, GHPair S, double inv_g,
                                  double inv_h, float mcw, float lambda, bool ignored, bool force) {
#pragma clang fp contract(off)
    const int lane = lane_id();
    const int bpl = (kf + 63) >> 6;  // bins per lane: 1 for the usual <= 64 bins, so that every lane has a candidate
    long long incg[4], inch[4];
    long long rung = 0, runh = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int b = lane * bpl + j;
        if (j < bpl && b < kf) {
            const longlong2 v = cells[(size_t)b * stride];
            rung += v.x;
            runh += v.y;
        }
        incg[j] = rung;
        inch[j] = runh;
    }
    long long aggg = rung, aggh = runh;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const long long pg = shfl_up_ll(aggg, d), ph = shfl_up_ll(aggh, d);
        if (lane >= d) {
            aggg += pg;
            aggh += ph;
        }
    }
    // totals: the last lane's inclusive sum
    const long long totg = (long long)(((unsigned long long)(unsigned)__shfl((int)((unsigned long long)aggg >> 32), 63) << 32) |
                                       (unsigned)__shfl((int)(unsigned)(unsigned long long)aggg, 63));
    const long long toth = (long long)(((unsigned long long)(unsigned)__shfl((int)((unsigned long long)aggh >> 32), 63) << 32) |
                                       (unsigned)__shfl((int)(unsigned)(unsigned long long)aggh, 63));
    SegResult r;
    r.win = -1.f;
    r.win_idx = 0x7fffffff;
    r.owner = false;
    r.score = 0.f;
    r.miss = r.left = GHPair{0, 0};
    if (!force && totg == 0 && toth == 0) return r;
    const long long carryg = aggg - rung, carryh = aggh - runh;  // exclusive prefix of the lane
    const GHPair m{S.g - (float)((double)totg * inv_g), S.h - (float)((double)toth * inv_h)};
    float best = -1.f, best_score = 0.f;
    int best_idx = 0x7fffffff;
    GHPair best_left{0, 0};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        if (j >= bpl) break;
        const int b = lane * bpl + j;
        if (b < kf) {
            const long long exg = carryg + (j == 0 ? 0 : incg[j > 0 ? j - 1 : 0]);
            const long long exh = carryh + (j == 0 ? 0 : inch[j > 0 ? j - 1 : 0]);
            const GHPair l{(float)((double)exg * inv_g), (float)((double)exh * inv_h)};
            const float gr = split_gain(S, l, mcw, lambda);
            const GHPair l2{l.g + m.g, l.h + m.h};
            const float gl = split_gain(S, l2, mcw, lambda);
            float score = (gl > gr) ? gl : -gr;
            if (ignored) score = 0.f;  // column sampling: hist_tree_builder_single.cu:304 / :663
            const float a = fabsf(score);
            if (a > best) {
                best = a;
                best_score = score;
                best_idx = gbin0 + b;
                best_left = l;
            }
        }
    }
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
    r.win = win;
    r.win_idx = win_idx;
    r.owner = best == win && best_idx == win_idx && best >= 0.f;
    r.score = best_score;
    r.miss = m;
    r.left = best_left;
    return r;
}

// key that orders candidates like the reference's arg-max: larger |gain| first, then the smaller bin index
__device__ __forceinline__ unsigned long long cand_key(float abs_gain, int index) {
    return ((unsigned long long)__float_as_uint(abs_gain) << 32) | (unsigned long long)(0xffffffffu - (unsigned)index);
}
__device__ __forceinline__ int key_index(unsigned long long key) { return (int)(0xffffffffu - (unsigned)key); }

struct SpShared {
    GHPair S[kSparseMaxLevelNodes];              // node sums of the level
    unsigned long long key[kSparseMaxLevelNodes];  // best candidate of every node over the task's features so far
    unsigned char ok[kSparseMaxLevelNodes];        // node is valid
    int fbin[kSparseBatchFeatures + 2];            // first bin (relative to the batch) of every feature of the batch
    int ctl[8];  // batch: first feature, end feature, first bin, bins, node range begin, nodes in range, first value, end value
};

// Level-wide state every task starts from: node sums and validity into LDS, keys cleared.
__device__ void sp_begin(const TreeBuffers &tb, SpShared &sh, int level) {
    const int nl = 1 << level, off = nl - 1;
    for (int x = threadIdx.x; x < nl; x += kSpBlock) {
        const TreeNode &nd = tb.nodes[off + x];
        sh.S[x] = nd.sum_gh_pair;
        sh.ok[x] = nd.is_valid ? 1 : 0;
        sh.key[x] = 0ull;
    }
}

// End of a task: its best key of every node competes with the other tasks' (the record already sits in the task's
// candidate slot, where k_best_update finds it through the winning bin's feature).
__device__ void sp_publish(const TreeBuffers &tb, SpShared &sh, int level) {
    const int nl = 1 << level;
    __syncthreads();
    for (int x = threadIdx.x; x < nl; x += kSpBlock) {
        const unsigned long long k = sh.key[x];
        if (k != 0ull && k > __hip_atomic_load(&tb.best_key[x], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))
            atomicMax(&tb.best_key[x], k);
    }
}

// Split search over the tables of one batch: features [fa, fa + nf) x nodes [n0, n0 + nn) of the level, cells at
// (node - n0) * bins + (bin - bin0): the bins of a (feature, node) segment lie next to each other. Phase 1 raises every node's key; after a barrier the wavefronts whose segment holds
// a node's current best write that candidate's details to the task's slot (a later batch with a better candidate
// overwrites them). `dump`: also store the cells into the level's per-node histograms.
__device__ void sp_search_batch(const TreeBuffers &tb, SpShared &sh, const longlong2 *cells, int level, int fa, int nf,
                                int bin0, int n0, int nn, int cand_slot, float mcw, float lambda, longlong2 *dump) {
    const int w = threadIdx.x >> 6, lane = lane_id();
    const double inv_g = tb.quant->inv_g, inv_h = tb.quant->inv_h;
    const int n_seg = nf * nn;
    const int bins = sh.fbin[nf];
    for (int seg = w; seg < n_seg; seg += kSpWaves) {
        const int fi = seg / nn, x = seg - fi * nn;
        const int node = n0 + x;
        if (!sh.ok[node]) continue;
        const int b0 = sh.fbin[fi], kf = sh.fbin[fi + 1] - b0;
        if (kf <= 0) continue;
        const bool ign = tb.ignored != nullptr && tb.ignored[fa + fi] != 0;
        const SegResult r = eval_segment(cells + (size_t)x * bins + b0, 1, kf, bin0 + b0, sh.S[node], inv_g, inv_h, mcw,
                                         lambda, ign, bin0 + b0 == 0);
        if (r.win >= 0.f && lane == 0) atomicMax(&sh.key[node], cand_key(r.win, r.win_idx));
    }
    __syncthreads();
    for (int x = w; x < nn; x += kSpWaves) {
        const int node = n0 + x;
        const unsigned long long key = sh.key[node];
        if (key == 0ull) continue;
        const int idx = key_index(key);
        if (idx < bin0 || idx >= bin0 + bins) continue;  // the node's best comes from an earlier batch
        // the feature of that bin: last feature of the batch whose first bin is <= idx - bin0
        int lo = 0, hi = nf;
        while (hi - lo > 1) {
            const int mid = (lo + hi) >> 1;
            if (sh.fbin[mid] <= idx - bin0) lo = mid; else hi = mid;
        }
        const int b0 = sh.fbin[lo], kf = sh.fbin[lo + 1] - b0;
        const bool ign = tb.ignored != nullptr && tb.ignored[fa + lo] != 0;
        const SegResult r = eval_segment(cells + (size_t)x * bins + b0, 1, kf, bin0 + b0, sh.S[node], inv_g, inv_h, mcw,
                                         lambda, ign, true);
        if (r.owner && r.win_idx == idx) {
            SplitCand c;
            c.score = r.score;
            c.index = idx;
            c.miss = r.miss;
            c.left = r.left;
            c.pad[0] = c.pad[1] = 0;
            tb.cand[(size_t)node * tb.n_packs + cand_slot] = c;
        }
    }
    if (dump != nullptr) {
        const int total = bins * nn;
        for (int c = threadIdx.x; c < total; c += kSpBlock) {
            const int x = c / bins, b = c - x * bins;
            dump[(size_t)(n0 + x) * tb.n_bins + bin0 + b] = cells[c];
        }
    }
}

// One task = a run of whole features (batched so that their tables fit the LDS) or one chunk of a big feature (its
// table goes to the partial buffer, k_sparse_big adds the chunks up and searches them).
__global__ __launch_bounds__(kSpBlock) void k_sparse_level(TreeBuffers tb_all, CsrBins bins, SparsePass sp,
                                                          const GHPair *__restrict__ gh, int level, float mcw,
                                                          float lambda, int dump_hist, int n_cells) {
    extern __shared__ longlong2 cells[];  // [n_cells]
    __shared__ SpShared sh;
    const TreeBuffers tb = tb_all.for_class(blockIdx.z);
    gh += (size_t)blockIdx.z * tb.n;
    const SparseTask task = sp.tasks[blockIdx.x];
    const int nl = 1 << level, off = nl - 1;
    const unsigned short *__restrict__ nid16 = tb.nid16;
    const int *__restrict__ crp = tb.cut_row_ptr;
    const float scale_g = tb.quant->scale_g, scale_h = tb.quant->scale_h;
    const GHPair *__restrict__ csc_gh = sp.csc_gh != nullptr ? sp.csc_gh + (size_t)blockIdx.z * sp.nnz : nullptr;
    sp_begin(tb, sh, level);
    longlong2 *dump = (dump_hist && task.cand_slot >= 0) ? tb.hist(level) : nullptr;
    longlong2 *partial = task.partial_slot >= 0
                             ? sp.partial + ((size_t)blockIdx.z * sp.n_partial_slots + task.partial_slot) * sp.partial_stride
                             : nullptr;
    int f = task.f_begin;
    while (f < task.f_end) {
        __syncthreads();
        if (threadIdx.x == 0) {
            // next batch: as many whole features as fit with all nodes of the level, or one feature with a node range
            int kf = crp[f + 1] - crp[f];
            int fb = f + 1, nn = nl;
            if ((long)kf * nl <= n_cells) {
                int total = kf;
                while (fb < task.f_end && fb - f < kSparseBatchFeatures) {
                    const int k = crp[fb + 1] - crp[fb];
                    if ((long)(total + k) * nl > n_cells) break;
                    total += k;
                    ++fb;
                }
                kf = total;
            } else {
                nn = n_cells / kf;
            }
            sh.ctl[0] = f;
            sh.ctl[1] = fb;
            sh.ctl[2] = crp[f];
            sh.ctl[3] = kf;
            sh.ctl[5] = nn;
            sh.ctl[6] = max(task.v_begin, sp.feat_val_begin[f]);
            sh.ctl[7] = min(task.v_end, sp.feat_val_begin[fb]);
        }
        __syncthreads();
        const int fa = sh.ctl[0], fb = sh.ctl[1], bin0 = sh.ctl[2], nbins = sh.ctl[3], nn_max = sh.ctl[5];
        const int v0 = sh.ctl[6], v1 = sh.ctl[7];
        const int nf = fb - fa;
        for (int i = threadIdx.x; i <= nf; i += kSpBlock) sh.fbin[i] = crp[fa + i] - bin0;
        for (int n0 = 0; n0 < nl; n0 += nn_max) {
            const int nn = min(nn_max, nl - n0);
            const int n_cells = nbins * nn;
            __syncthreads();
            for (int c = threadIdx.x; c < n_cells; c += kSpBlock) cells[c] = make_longlong2(0, 0);
            __syncthreads();
            // accumulate: four values in flight per thread (row -> node from the cache-resident map, then the pair)
            constexpr int U = 8;
            for (int e0 = v0 + threadIdx.x; e0 < v1; e0 += kSpBlock * U) {
                // (every load is unconditional - a value index past the end repeats the last value and is skipped
                // below -, so each stage's eight loads are issued together instead of one after the other)
                int gb[U], row[U], x[U];
                GHPair s[U];
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const int e = min(e0 + u * kSpBlock, v1 - 1);
                    gb[u] = bins.csc_bin[e];
                    row[u] = bins.csc_row[e];
                    if (csc_gh != nullptr) s[u] = csc_gh[e];
                }
#pragma unroll
                for (int u = 0; u < U; ++u) x[u] = (int)nid16[row[u]] - off - n0;
                if (csc_gh == nullptr) {
#pragma unroll
                    for (int u = 0; u < U; ++u) s[u] = gh[row[u]];
                }
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    if (e0 + u * kSpBlock < v1 && (unsigned)x[u] < (unsigned)nn) {
                        const long long gq = round_to_ll(s[u].g * scale_g), hq = round_to_ll(s[u].h * scale_h);
                        unsigned long long *cell = reinterpret_cast<unsigned long long *>(cells + (size_t)x[u] * nbins + (gb[u] - bin0));
                        atomicAdd(cell, (unsigned long long)gq);
                        atomicAdd(cell + 1, (unsigned long long)hq);
                    }
                }
            }
            __syncthreads();
            if (partial != nullptr) {
                // (node, bin) cells of the whole level, this node range's part
                for (int c = threadIdx.x; c < n_cells; c += kSpBlock) {
                    const int xx = c / nbins, b = c - xx * nbins;
                    partial[(size_t)(n0 + xx) * nbins + b] = cells[c];
                }
            } else {
                sp_search_batch(tb, sh, cells, level, fa, nf, bin0, n0, nn, task.cand_slot, mcw, lambda, dump);
            }
        }
        f = fb;
    }
    if (partial == nullptr) sp_publish(tb, sh, level);
}

// A big feature: the tables of its chunks are added up (node range by node range) and searched.
__global__ __launch_bounds__(kSpBlock) void k_sparse_big(TreeBuffers tb_all, SparsePass sp, int level, float mcw,
                                                        float lambda, int dump_hist, int n_cells) {
    extern __shared__ longlong2 cells[];
    __shared__ SpShared sh;
    const TreeBuffers tb = tb_all.for_class(blockIdx.z);
    const SparseBig big = sp.big[blockIdx.x];
    const int nl = 1 << level;
    const int f = big.feature;
    const int bin0 = tb.cut_row_ptr[f], kf = tb.cut_row_ptr[f + 1] - bin0;
    sp_begin(tb, sh, level);
    if (threadIdx.x == 0) {
        sh.fbin[0] = 0;
        sh.fbin[1] = kf;
    }
    const longlong2 *base = sp.partial + (size_t)blockIdx.z * sp.n_partial_slots * sp.partial_stride;
    longlong2 *dump = dump_hist ? tb.hist(level) : nullptr;
    // the level's nodes are shared out over gridDim.y workgroups (a feature of many chunks would otherwise add up
    // megabytes of tables in one workgroup)
    const int per = (nl + (int)gridDim.y - 1) / (int)gridDim.y;
    const int ny0 = min(nl, (int)blockIdx.y * per), ny1 = min(nl, ny0 + per);
    const int nn_max = (long)kf * per <= n_cells ? per : n_cells / kf;
    for (int n0 = ny0; n0 < ny1; n0 += nn_max) {
        const int nn = min(nn_max, ny1 - n0);
        const int n_cells = kf * nn;
        __syncthreads();
        for (int c = threadIdx.x; c < n_cells; c += kSpBlock) {
            long long g = 0, h = 0;
#pragma unroll 4
            for (int slot = big.slot_begin; slot < big.slot_end; ++slot) {
                const longlong2 v = base[(size_t)slot * sp.partial_stride + (size_t)n0 * kf + c];
                g += v.x;
                h += v.y;
            }
            cells[c] = make_longlong2(g, h);
        }
        __syncthreads();
        sp_search_batch(tb, sh, cells, level, f, 1, bin0, n0, nn, big.cand_slot, mcw, lambda, dump);
    }
    sp_publish(tb, sh, level);
}

// ------------------------------------------------------------------------------------ sorted pass
// Features with at most kSortedTile stored values. A task (one workgroup) owns a run of whole features and a tile of
// the sorted-pass arrays; the tile holds the features' values in the order (feature, node of the level, bin), rows
// in arrival order inside a bin. A level reads the previous level's order, looks up the node every value's row has
// moved to, and partitions every (feature, node) run stably into the values of the left and of the right child;
// the runs of nodes that did not split drop out (all rows of a node split or none, so a run is all live or all
// dead). The new order goes back to HBM for the next level and is scanned right away: a forward and a backward
// segmented sum per (feature, node) run give every position the run's sum up to it and after it, hence the left
// sum and the feature's total in the node (missing = node sum - total). Candidates exist only where the left sum
// changes: the feature's first bin (left side empty) and the bin after every bin that holds a value - the bins in
// between repeat the previous candidate's gain and lose the tie on the smaller index - so the result is what the
// scan of a complete (bin, node) table gives. The root level reads the static order and fetches the gradient pairs.
constexpr int kSoV = kSortedPerThread;
constexpr int kSoWaves = kSortedBlock / 64;
constexpr unsigned kSoNodeMask = 0xfffu << kSortedNodeShift;
// LDS position of tile position i: one element of padding after every 32, so that neither the lanes of a wavefront
// that each own eight consecutive positions nor lanes at consecutive positions collide in a bank
constexpr int kSoLds = kSortedTile + kSortedTile / 32;
__device__ __forceinline__ int so_phys(int i) { return i + (i >> 5); }

struct SoCount {
    int seg;    // since the run began: values << 16 | values that go left
    int plain;  // over the whole tile: dead values
};
struct SoSum {
    long long g, h;
};
__device__ __forceinline__ void so_zero_seg(SoCount &a) { a.seg = 0; }
__device__ __forceinline__ void so_add_seg(SoCount &a, const SoCount &b) { a.seg += b.seg; }
__device__ __forceinline__ void so_add_plain(SoCount &a, const SoCount &b) { a.plain += b.plain; }
__device__ __forceinline__ void so_zero_seg(SoSum &a) { a.g = a.h = 0; }
__device__ __forceinline__ void so_add_seg(SoSum &a, const SoSum &b) {
    a.g += b.g;
    a.h += b.h;
}
__device__ __forceinline__ void so_add_plain(SoSum &, const SoSum &) {}

template <bool FWD>
__device__ __forceinline__ int so_shfl(int v, int d) {
    return FWD ? __shfl_up(v, d) : __shfl_down(v, d);
}
template <bool FWD>
__device__ __forceinline__ long long so_shfl(long long v, int d) {
    const int lo = so_shfl<FWD>((int)(unsigned)(unsigned long long)v, d);
    const int hi = so_shfl<FWD>((int)((unsigned long long)v >> 32), d);
    return (long long)(((unsigned long long)(unsigned)hi << 32) | (unsigned)lo);
}
template <bool FWD>
__device__ __forceinline__ SoCount so_shfl(SoCount v, int d) {
    return SoCount{so_shfl<FWD>(v.seg, d), so_shfl<FWD>(v.plain, d)};
}
template <bool FWD>
__device__ __forceinline__ SoSum so_shfl(SoSum v, int d) {
    return SoSum{so_shfl<FWD>(v.g, d), so_shfl<FWD>(v.h, d)};
}

// Inclusive segmented scan over the tile (thread t owns positions t * kSoV ..). FWD: v[j] becomes the sum from the
// start of its run (brk = a run starts here) up to j; !FWD: from j to the end of its run (brk = a run ends here).
// The `plain` part of T ignores the breaks. Two barriers; s_agg / s_flag are free again afterwards.
template <typename T, bool FWD>
__device__ void so_block_scan(T (&v)[kSoV], const bool (&brk)[kSoV], T *s_agg, int *s_flag) {
    const int lane = lane_id(), w = wave_id();
    T run{};
    bool any = false;
#pragma unroll
    for (int jj = 0; jj < kSoV; ++jj) {
        const int j = FWD ? jj : kSoV - 1 - jj;
        if (brk[j]) {
            so_zero_seg(run);
            any = true;
        }
        so_add_seg(run, v[j]);
        so_add_plain(run, v[j]);
        v[j] = run;
    }
    T agg = run;
    int flag = any ? 1 : 0;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const T o = so_shfl<FWD>(agg, d);
        const int of = so_shfl<FWD>(flag, d);
        const bool has = FWD ? lane >= d : lane + d < 64;
        if (has) {
            if (!flag) so_add_seg(agg, o);
            so_add_plain(agg, o);
            flag |= of;
        }
    }
    T carry = so_shfl<FWD>(agg, 1);
    int cflag = so_shfl<FWD>(flag, 1);
    if (FWD ? lane == 0 : lane == 63) {
        carry = T{};
        cflag = 0;
    }
    if (FWD ? lane == 63 : lane == 0) {
        s_agg[w] = agg;
        s_flag[w] = flag;
    }
    __syncthreads();
    T wc{};
    if (FWD) {
        for (int u = 0; u < w; ++u) {
            if (s_flag[u]) so_zero_seg(wc);
            so_add_seg(wc, s_agg[u]);
            so_add_plain(wc, s_agg[u]);
        }
    } else {
        for (int u = kSoWaves - 1; u > w; --u) {
            if (s_flag[u]) so_zero_seg(wc);
            so_add_seg(wc, s_agg[u]);
            so_add_plain(wc, s_agg[u]);
        }
    }
    if (!cflag) so_add_seg(carry, wc);
    so_add_plain(carry, wc);
    bool open = true;
#pragma unroll
    for (int jj = 0; jj < kSoV; ++jj) {
        const int j = FWD ? jj : kSoV - 1 - jj;
        if (brk[j]) open = false;
        if (open) so_add_seg(v[j], carry);
        so_add_plain(v[j], carry);
    }
    __syncthreads();
}

// split_gain with the node's own term (f.g^2 / (f.h + lambda), the same for every candidate of the node) taken from
// a table: the same operations in the same order, hence the same bits
__device__ __forceinline__ float so_gain(GHPair f, float fterm, GHPair l, float mcw, float lambda) {
#pragma clang fp contract(off)
    const GHPair r{f.g - l.g, f.h - l.h};
    float gain = 0.f;
    if (l.h >= mcw && r.h >= mcw) gain = (l.g * l.g) / (l.h + lambda) + (r.g * r.g) / (r.h + lambda) - fterm;
    return fmaxf(0.f, gain);
}

// Upper estimate of so_gain from the hardware reciprocal (1 ulp) instead of divisions; -1: the weight gate closes
__device__ __forceinline__ float so_gain_estimate(GHPair f, float fterm, GHPair l, float mcw, float lambda) {
    const GHPair r{f.g - l.g, f.h - l.h};
    if (!(l.h >= mcw && r.h >= mcw)) return -1.f;
    const float a = l.g * l.g * __builtin_amdgcn_rcpf(l.h + lambda), b = r.g * r.g * __builtin_amdgcn_rcpf(r.h + lambda);
    return (a + b - fterm) + (a + b + fabsf(fterm)) * 3.8146973e-6f;  // + 2^-18 of the terms: far above the roundings
}

// Signed score of a candidate (> 0: missing values go left), hist_tree_builder_single.cu:300-323. `floor`: the
// largest |score| the candidate's node has seen so far; a candidate whose estimate stays below it cannot become the
// node's best and is not evaluated (0 = no candidate).
__device__ __forceinline__ float so_score(GHPair S, float fterm, GHPair m, GHPair l, bool ignored, float mcw,
                                          float lambda, float floor) {
#pragma clang fp contract(off)
    const GHPair l2{l.g + m.g, l.h + m.h};
    const float er = so_gain_estimate(S, fterm, l, mcw, lambda), el = so_gain_estimate(S, fterm, l2, mcw, lambda);
    if (fmaxf(er, el) < floor || ignored) return 0.f;  // (column sampling: hist_tree_builder_single.cu:304 / :663)
    const float gr = so_gain(S, fterm, l, mcw, lambda);
    const float gl = so_gain(S, fterm, l2, mcw, lambda);
    return (gl > gr) ? gl : -gr;
}

template <bool LEVEL0>
__global__ __launch_bounds__(kSortedBlock) void k_sparse_sorted(TreeBuffers tb_all, SparsePass sp,
                                                               const GHPair *__restrict__ gh, int level, float mcw,
                                                               float lambda, int dump_hist, int last_level) {
#pragma clang fp contract(off)
    extern __shared__ unsigned char so_dyn[];  // per node of the level: best key (8 bytes), sums (8), own gain term (4)
    __shared__ int s_row[kSoLds];
    __shared__ unsigned s_key[kSoLds];
    __shared__ GHPair s_gh[kSoLds];
    __shared__ unsigned short s_aux[kSoLds];  // first the left counts of the old runs, then the start of every value's run
    __shared__ SoSum s_agg_sum[kSoWaves];
    __shared__ SoCount s_agg_cnt[kSoWaves];
    __shared__ int s_flag[kSoWaves];
    __shared__ int s_dead;
    const TreeBuffers tb = tb_all.for_class(blockIdx.z);
    const SortedTask task = sp.sorted_tasks[blockIdx.x];
    const int nl = 1 << level, off = nl - 1;
    unsigned long long *s_best = reinterpret_cast<unsigned long long *>(so_dyn);
    GHPair *s_S = reinterpret_cast<GHPair *>(s_best + nl);
    float *s_P = reinterpret_cast<float *>(s_S + nl);
    const size_t base = (size_t)blockIdx.z * (size_t)sp.n_sorted + (size_t)task.v_begin;
    int *live = sp.sorted_live + ((size_t)blockIdx.z * kSortedLevels + level) * sp.n_sorted_tasks;
    const int M = LEVEL0 ? task.count : live[(long)blockIdx.x - sp.n_sorted_tasks];
    gh += (size_t)blockIdx.z * tb.n;
    const int *__restrict__ in_row = LEVEL0 ? sp.sorted_row0 + task.v_begin : sp.srow(level - 1) + base;
    const unsigned *__restrict__ in_key = LEVEL0 ? sp.sorted_key0 + task.v_begin : sp.skey(level - 1) + base;
    const GHPair *__restrict__ in_gh = LEVEL0 ? nullptr : sp.sgh(level - 1) + base;
    int *__restrict__ out_row = sp.srow(level) + base;
    unsigned *__restrict__ out_key = sp.skey(level) + base;
    GHPair *__restrict__ out_gh = sp.sgh(level) + base;
    if (M == 0) {
        if (threadIdx.x == 0) live[blockIdx.x] = 0;
        return;
    }
    for (int x = threadIdx.x; x < nl; x += kSortedBlock) {
        const GHPair S = tb.nodes[off + x].sum_gh_pair;
        // what the other tasks have published so far: a candidate below it need not be looked at
        s_best[x] = __hip_atomic_load(&tb.best_key[x], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        s_S[x] = S;
        s_P[x] = (S.g * S.g) / (S.h + lambda);
    }
    // ---- the previous order into LDS with coalesced loads (position q = k * block + thread), every load of the
    // thread in flight before the first one is used; the root level also fetches the gradient pair of every value's
    // row here and takes the run starts (= feature starts) from the static arrays
    {
        int lrow[kSoV];
        unsigned lkey[kSoV];
        GHPair lgh[kSoV];
        unsigned short lst[kSoV];
#pragma unroll
        for (int k = 0; k < kSoV; ++k) {
            const int q = k * kSortedBlock + threadIdx.x;
            lrow[k] = q < M ? in_row[q] : 0;
            lkey[k] = q < M ? in_key[q] : 0u;
            if (!LEVEL0) lgh[k] = q < M ? in_gh[q] : GHPair{0, 0};
            if (LEVEL0) lst[k] = q < M ? sp.sorted_start0[task.v_begin + q] : (unsigned short)0;
        }
        if (LEVEL0) {
#pragma unroll
            for (int k = 0; k < kSoV; ++k) lgh[k] = gh[lrow[k]];  // (row 0 for the positions past the end)
        }
#pragma unroll
        for (int k = 0; k < kSoV; ++k) {
            const int q = k * kSortedBlock + threadIdx.x;
            if (q < M) {
                s_row[so_phys(q)] = lrow[k];
                s_key[so_phys(q)] = lkey[k];
                s_gh[so_phys(q)] = lgh[k];
                if (LEVEL0) s_aux[so_phys(q)] = lst[k];
            }
        }
    }
    __syncthreads();
    const int i0 = threadIdx.x * kSoV;
    static_assert(32 % kSoV == 0, "a thread's positions must not straddle a padding element");
    const int pb = so_phys(i0);  // so_phys(i0 + j) = pb + j: a thread's positions share one padding count
    int Mn = M;  // values of the new order
    if (!LEVEL0) {
        const uint8_t *__restrict__ row_move = tb.row_move;
        int row[kSoV];
        unsigned key[kSoV];
        GHPair pair[kSoV];
#pragma unroll
        for (int j = 0; j < kSoV; ++j) {
            const int i = i0 + j;
            row[j] = i < M ? s_row[pb + j] : -1;
            key[j] = i < M ? s_key[pb + j] : 0xffffffffu;
            pair[j] = i < M ? s_gh[pb + j] : GHPair{0, 0};
        }
        const unsigned prevk = (i0 > 0 && i0 - 1 < M) ? s_key[so_phys(i0 - 1)] : 0xffffffffu;
        const unsigned nextk = (i0 + kSoV < M) ? s_key[so_phys(i0 + kSoV)] : 0xffffffffu;
        // the value's node of the level above is in its key; the row -> node update left two bits per row: did the
        // node split, and did the row go right (all of a thread's look-ups are issued before the first is used)
        unsigned mv[kSoV];
#pragma unroll
        for (int j = 0; j < kSoV; ++j) mv[j] = row_move[max(row[j], 0)];
        int xn[kSoV];
#pragma unroll
        for (int j = 0; j < kSoV; ++j) {
            xn[j] = -1;  // the node is a leaf, or the run left the pass at the level above (mark in the key)
            if (row[j] >= 0 && (key[j] & kSoNodeMask) != kSoNodeMask && (mv[j] & 1u))
                xn[j] = 2 * (int)((key[j] >> kSortedNodeShift) & 0xfffu) + (int)(mv[j] >> 1);
        }
        SoCount fw[kSoV];
        bool head[kSoV], tail[kSoV];
#pragma unroll
        for (int j = 0; j < kSoV; ++j) {
            const int i = i0 + j;
            const bool valid = i < M;
            const unsigned pk = j == 0 ? prevk : key[j > 0 ? j - 1 : 0];
            const unsigned nk = j == kSoV - 1 ? nextk : key[j < kSoV - 1 ? j + 1 : 0];
            head[j] = valid && (i == 0 || (pk >> kSortedNodeShift) != (key[j] >> kSortedNodeShift));
            tail[j] = valid && (i == M - 1 || (nk >> kSortedNodeShift) != (key[j] >> kSortedNodeShift));
            const bool alive = valid && xn[j] >= 0;
            fw[j].seg = alive ? ((1 << 16) | ((xn[j] & 1) ? 0 : 1)) : 0;
            fw[j].plain = (valid && !alive) ? 1 : 0;
        }
        // (the scan's barriers also make sure that every thread has taken its values out of the LDS arrays before
        // the new order is written over them)
        so_block_scan<SoCount, true>(fw, head, s_agg_cnt, s_flag);
        if (threadIdx.x == kSortedBlock - 1) s_dead = fw[kSoV - 1].plain;  // (positions past the end add nothing)
        // the last value of a run knows how many of the run go left: it leaves the count at the run's start
#pragma unroll
        for (int j = 0; j < kSoV; ++j)
            if (tail[j] && xn[j] >= 0)
                s_aux[so_phys(i0 + j - ((fw[j].seg >> 16) - 1))] = (unsigned short)(fw[j].seg & 0xffff);
        __syncthreads();
        Mn = M - s_dead;
        int pos[kSoV], start[kSoV];
#pragma unroll
        for (int j = 0; j < kSoV; ++j) {
            pos[j] = -1;
            const int i = i0 + j;
            if (i < M && xn[j] >= 0) {
                const int cnt = fw[j].seg >> 16, lefts = fw[j].seg & 0xffff;  // inclusive
                const int nleft = s_aux[so_phys(i - (cnt - 1))];               // of the whole run
                const int s_new = i - (cnt - 1) - fw[j].plain;                 // the run's start once the dead are gone
                const bool l = !(xn[j] & 1);
                start[j] = l ? s_new : s_new + nleft;
                pos[j] = l ? s_new + lefts - 1 : s_new + nleft + (cnt - 1) - lefts;
            }
        }
        __syncthreads();  // every left count has been read: s_aux takes the run starts of the new order
#pragma unroll
        for (int j = 0; j < kSoV; ++j) {
            if (pos[j] >= 0) {
                const int pp = so_phys(pos[j]);
                s_row[pp] = row[j];
                s_key[pp] = (key[j] & ~kSoNodeMask) | ((unsigned)xn[j] << kSortedNodeShift);
                s_gh[pp] = pair[j];
                s_aux[pp] = (unsigned short)start[j];
            }
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) live[blockIdx.x] = Mn;
    if (Mn == 0) return;
    // ---- rows and gradient pairs of the new order back to HBM (coalesced); the keys follow once the runs that leave
    // the pass are marked
    // (no level reads the order of the tree's last level)
    if (!last_level) {
        for (int q = threadIdx.x; q < Mn; q += kSortedBlock) {
            out_row[q] = s_row[so_phys(q)];
            out_gh[q] = s_gh[so_phys(q)];
        }
    }
    unsigned key[kSoV];
    SoSum fs[kSoV];
    bool head[kSoV], tail[kSoV], last_of_bin[kSoV];
    const float scale_g = tb.quant->scale_g, scale_h = tb.quant->scale_h;
    const double inv_g = tb.quant->inv_g, inv_h = tb.quant->inv_h;
#pragma unroll
    for (int j = 0; j < kSoV; ++j) {
        const int p = i0 + j;
        const bool in = p < Mn;
        key[j] = in ? s_key[pb + j] : 0xffffffffu;
        fs[j] = SoSum{0, 0};
        if (in) {
            const GHPair s = s_gh[pb + j];
            fs[j].g = round_to_ll(s.g * scale_g);
            fs[j].h = round_to_ll(s.h * scale_h);
        }
    }
    {
        const unsigned prevk = (i0 > 0 && i0 - 1 < Mn) ? s_key[so_phys(i0 - 1)] : 0xffffffffu;
        const unsigned nextk = (i0 + kSoV < Mn) ? s_key[so_phys(i0 + kSoV)] : 0xffffffffu;
#pragma unroll
        for (int j = 0; j < kSoV; ++j) {
            const int p = i0 + j;
            const bool in = p < Mn;
            const unsigned pk = j == 0 ? prevk : key[j > 0 ? j - 1 : 0];
            const unsigned nk = j == kSoV - 1 ? nextk : key[j < kSoV - 1 ? j + 1 : 0];
            head[j] = in && (p == 0 || (pk >> kSortedNodeShift) != (key[j] >> kSortedNodeShift));
            tail[j] = in && (p + 1 == Mn || (nk >> kSortedNodeShift) != (key[j] >> kSortedNodeShift));
            last_of_bin[j] = in && (p + 1 == Mn || nk != key[j]);
        }
    }
    if (dump_hist) {
        // stage-wise inspection: the per-node histograms of the level (zeroed before the launch) get the values
        unsigned long long *hist = reinterpret_cast<unsigned long long *>(tb.hist(level));
#pragma unroll
        for (int j = 0; j < kSoV; ++j) {
            if (i0 + j < Mn) {
                const int x = (int)((key[j] >> kSortedNodeShift) & 0xfffu), lb = (int)(key[j] & 0xffu);
                const int fbegin = sp.sorted_meta[task.meta_begin + (int)(key[j] >> kSortedFeatShift)].x;
                unsigned long long *cell = hist + 2 * ((size_t)x * tb.n_bins + fbegin + lb);
                atomicAdd(cell, (unsigned long long)fs[j].g);
                atomicAdd(cell + 1, (unsigned long long)fs[j].h);
            }
        }
    }
    // (the scan's barriers: the stores above have read s_gh, which now takes the run totals)
    so_block_scan<SoSum, true>(fs, head, s_agg_sum, s_flag);
    // the last value of a run holds the run's sums = the feature's total in the node: as floats to the run's start.
    // It also decides whether the run can matter at this level at all. Every candidate of the run splits a subset A
    // of the run's values off the node (a prefix when the missing rows go right, a suffix when they go left), with
    // A.h >= min_child_weight, |A.g| <= (values of the run) x (largest |g| of the tree) =: ga and A.h <= the run's
    // hessian sum th, so its gain is at most
    //   ga^2 / (mcw + lambda) + (|S.g| + ga)^2 / (max(mcw, S.h - th) + lambda) - S.g^2 / (S.h + lambda).
    // A run whose bound (plus 2^-18 of its terms, far above the float roundings of the bound and of the gains it
    // stands for) stays below the best gain the node has seen so far has no candidate worth evaluating: it is
    // marked in the sign of the hessian total (which is never negative). On 2 M x 100 k data that is 85 % of the
    // values at every level.
    int start[kSoV];
    const float g_max = tb.quant->gq_max * tb.quant->inv_g;
#pragma unroll
    for (int j = 0; j < kSoV; ++j) {
        start[j] = (i0 + j < Mn) ? (int)s_aux[pb + j] : 0;
        if (tail[j]) {
            const float tg = (float)((double)fs[j].g * inv_g), th = (float)((double)fs[j].h * inv_h);
            const int x = (int)((key[j] >> kSortedNodeShift) & 0xfffu);
            const GHPair S = s_S[x];
            const float P = s_P[x];
            const float floor = __uint_as_float((unsigned)(s_best[x] >> 32));
            const float ga = g_max * (float)(i0 + j - start[j] + 1);
            const float sa = fabsf(S.g) + ga;
            const float t1 = ga * ga / (mcw + lambda), t2 = sa * sa / (fmaxf(mcw, S.h - th) + lambda);
            const bool hopeless = (t1 + t2 - P) + (t1 + t2 + fabsf(P)) * 3.8146973e-6f < floor;
            s_gh[so_phys(start[j])] = GHPair{tg, hopeless ? -th : th};
        }
    }
    __syncthreads();
    // ---- A (feature, node) run whose hessians add up to less than min_child_weight cannot yield a split, here or
    // in any node below (hessians are not negative, so every left or right side taken from the run's values, and
    // every run of a child node, weighs less still; the margin covers the float roundings of the missing-value
    // arithmetic, a few ulps of the node's hessian sum). Such runs leave the pass: their keys get the node field's
    // all-ones mark, which the next level reads as "dead". Not when the per-node histograms are being recorded.
    GHPair tot[kSoV];
    bool drop[kSoV], hopeless[kSoV];
#pragma unroll
    for (int j = 0; j < kSoV; ++j) {
        drop[j] = hopeless[j] = false;
        tot[j] = GHPair{0, 0};
        const int p = i0 + j;
        if (p < Mn) {
            tot[j] = s_gh[so_phys(start[j])];
            hopeless[j] = (__float_as_uint(tot[j].h) >> 31) != 0u;
            tot[j].h = fabsf(tot[j].h);
            const float Sh = s_S[(key[j] >> kSortedNodeShift) & 0xfffu].h;
            drop[j] = !dump_hist && tot[j].h + Sh * 4.76837158e-7f < mcw;  // 2^-21
            if (drop[j]) s_key[pb + j] = key[j] | kSoNodeMask;
        }
    }
    __syncthreads();
    if (!last_level)
        for (int q = threadIdx.x; q < Mn; q += kSortedBlock) out_key[q] = s_key[so_phys(q)];
    // ---- candidates: raise the node's key in LDS, then the winners publish. A candidate without gain never
    // competes: the node's candidate at global bin 0 (a table feature's) has at least its key.
    float sc_head[kSoV], sc_bin[kSoV];
#pragma unroll
    for (int j = 0; j < kSoV; ++j) {
        sc_head[j] = sc_bin[j] = 0.f;
        if (!(head[j] || last_of_bin[j]) || drop[j] || hopeless[j]) continue;
        const int x = (int)((key[j] >> kSortedNodeShift) & 0xfffu), lb = (int)(key[j] & 0xffu);
        const int fi = task.meta_begin + (int)(key[j] >> kSortedFeatShift);
        const int2 meta = sp.sorted_meta[fi];
        const bool ign = tb.ignored != nullptr && tb.ignored[sp.sorted_fid[fi]] != 0;
        const GHPair S = s_S[x];
        const float P = s_P[x];
        const GHPair mm{S.g - tot[j].g, S.h - tot[j].h};
        const float floor = __uint_as_float((unsigned)(s_best[x] >> 32));
        if (head[j]) {
            sc_head[j] = so_score(S, P, mm, GHPair{0, 0}, ign, mcw, lambda, floor);
            if (sc_head[j] != 0.f) atomicMax(&s_best[x], cand_key(fabsf(sc_head[j]), meta.x));
        }
        if (last_of_bin[j] && lb < meta.y - 1) {
            const GHPair l{(float)((double)fs[j].g * inv_g), (float)((double)fs[j].h * inv_h)};
            sc_bin[j] = so_score(S, P, mm, l, ign, mcw, lambda, floor);
            if (sc_bin[j] != 0.f) atomicMax(&s_best[x], cand_key(fabsf(sc_bin[j]), meta.x + lb + 1));
        }
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < kSoV; ++j) {
        if (sc_head[j] == 0.f && sc_bin[j] == 0.f) continue;
        const int x = (int)((key[j] >> kSortedNodeShift) & 0xfffu), lb = (int)(key[j] & 0xffu);
        const int fbegin = sp.sorted_meta[task.meta_begin + (int)(key[j] >> kSortedFeatShift)].x;
        const unsigned long long best = s_best[x];
        const bool win_head = sc_head[j] != 0.f && best == cand_key(fabsf(sc_head[j]), fbegin);
        const bool win_bin = sc_bin[j] != 0.f && best == cand_key(fabsf(sc_bin[j]), fbegin + lb + 1);
        if (!(win_head || win_bin)) continue;
        // the tile's best of the node: worth publishing only if it beats what other tasks have published so far
        if (best <= __hip_atomic_load(&tb.best_key[x], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) continue;
        const GHPair S = s_S[x];
        SplitCand o;
        o.miss = GHPair{S.g - tot[j].g, S.h - tot[j].h};
        o.pad[0] = o.pad[1] = 0;
        if (win_head) {
            o.score = sc_head[j];
            o.index = fbegin;
            o.left = GHPair{0, 0};  // the first bin records an empty left side (hist_tree_builder_single.cu:378)
        } else {
            o.score = sc_bin[j];
            o.index = fbegin + lb + 1;
            o.left = GHPair{(float)((double)fs[j].g * inv_g), (float)((double)fs[j].h * inv_h)};
        }
        tb.cand[(size_t)x * tb.n_packs + task.cand_slot] = o;
        atomicMax(&tb.best_key[x], best);
    }
}

// Row -> node update of a level (update_ins2node_id, hist_tree_builder_single.cu:908-1020): a row whose node was
// split moves to the left or right child by the reference's rule (binary search of the row's ascending bin ids for
// one inside the split feature's range; none = missing -> default direction). Rows per child are counted on the way.
__global__ __launch_bounds__(kSpBlock) void k_sparse_partition(TreeBuffers tb_all, CsrBins bins, int level) {
    __shared__ int cnt[2 * kSparseMaxLevelNodes];
    const TreeBuffers tb = tb_all.for_class(blockIdx.z);
    const int nl = 1 << level, off = nl - 1;
    for (int i = threadIdx.x; i < 2 * nl; i += kSpBlock) cnt[i] = 0;
    __syncthreads();
    const int n64 = (tb.n + 63) & ~63;
    for (int r = blockIdx.x * kSpBlock + threadIdx.x; r < n64; r += gridDim.x * kSpBlock) {
        bool moved = false, right = false;
        if (r < tb.n) {
            const int node = tb.nid16[r];
            if (node >= off) {  // (else the row stays in a leaf of an earlier level)
                const TreeNode &nd = tb.nodes[node];
                if (node_splits(nd)) {
                    moved = true;
                    const int col = bins.col_of_feature != nullptr ? bins.col_of_feature[nd.split_feature_id] : -1;
                    if (col >= 0) {
                        // a frequent feature: the row's local bin id is one byte away (same rule: missing -> default
                        // direction, else right iff the bin is not below the split bin)
                        const int b = bins.colbin[(size_t)col * bins.col_stride + r];
                        right = b == kMissingBin ? (bool)nd.default_right : (b >= (int)nd.split_bid);
                    } else {
                        const int cb = tb.cut_row_ptr[nd.split_feature_id], ce = tb.cut_row_ptr[nd.split_feature_id + 1];
                        right = csr_goes_right(bins, r, cb, ce, cb + nd.split_bid, nd.default_right);
                    }
                    tb.nid16[r] = (unsigned short)(right ? nd.rch_index : nd.lch_index);
                    atomicAdd(&cnt[2 * (node - off) + (right ? 1 : 0)], 1);
                }
            }
        }
        tb.row_move[r] = (uint8_t)((moved ? 1 : 0) | (moved && right ? 2 : 0));  // (r < n rounded up to 64: allocated)
    }
    __syncthreads();
    for (int i = threadIdx.x; i < 2 * nl; i += kSpBlock)
        if (cnt[i] != 0) atomicAdd(&tb.node_rows[2 * off + 1 + i], cnt[i]);  // children of level node x: 2 (off + x) + 1, + 2
}

// csc_gh[e] = gh[csc_row[e]] for the stored values of the table tasks (the sorted pass fetches its pairs itself)
__global__ __launch_bounds__(256) void k_sparse_gh_refresh(int n, SparsePass sp, const int *__restrict__ csc_row,
                                                          const GHPair *__restrict__ gh) {
    gh += (size_t)blockIdx.z * n;
    GHPair *__restrict__ out = sp.csc_gh + (size_t)blockIdx.z * sp.nnz;
    const SparseTask task = sp.tasks[blockIdx.x];
    for (int e = task.v_begin + threadIdx.x; e < task.v_end; e += 256) out[e] = gh[csc_row[e]];
}

__global__ __launch_bounds__(256) void k_sparse_cols(long nnz, const int *__restrict__ csc_bin,
                                                    const int *__restrict__ csc_row, const int *__restrict__ cut_fid,
                                                    const int *__restrict__ cut_row_ptr,
                                                    const int *__restrict__ col_of_feature, uint8_t *__restrict__ colbin,
                                                    size_t col_stride) {
    for (long e = (long)blockIdx.x * 256 + threadIdx.x; e < nnz; e += (long)gridDim.x * 256) {
        const int b = csc_bin[e];
        const int f = cut_fid[b];
        const int c = col_of_feature[f];
        if (c >= 0) colbin[(size_t)c * col_stride + csc_row[e]] = (uint8_t)(b - cut_row_ptr[f]);
    }
}

// Static order of a sorted task's tile: its features one after the other, each in the order of the bin-major copy.
__global__ __launch_bounds__(256) void k_sorted_setup(SparsePass sp, CsrBins bins, const int *__restrict__ cut_row_ptr,
                                                     int *__restrict__ row0, unsigned *__restrict__ key0,
                                                     unsigned short *__restrict__ start0) {
    const SortedTask task = sp.sorted_tasks[blockIdx.x];
    int dst = task.v_begin;
    for (int fi = 0; fi < task.n_feat; ++fi) {
        const int f = sp.sorted_fid[task.meta_begin + fi];
        const int v0 = sp.feat_val_begin[f], m = sp.feat_val_begin[f + 1] - v0;
        const int fbegin = cut_row_ptr[f];
        for (int a = threadIdx.x; a < m; a += 256) {
            row0[dst + a] = bins.csc_row[v0 + a];
            key0[dst + a] = ((unsigned)fi << kSortedFeatShift) | (unsigned)(bins.csc_bin[v0 + a] - fbegin);
            start0[dst + a] = (unsigned short)(dst - task.v_begin);
        }
        dst += m;
    }
}

}  // namespace

void launch_sparse_cols(hipStream_t s, long nnz, const int *csc_bin, const int *csc_row, const int *cut_fid,
                        const int *cut_row_ptr, const int *col_of_feature, uint8_t *colbin, size_t col_stride) {
    if (nnz == 0) return;
    const int grid = (int)std::min<long>(16384, (nnz + 255) / 256);
    k_sparse_cols<<<grid, 256, 0, s>>>(nnz, csc_bin, csc_row, cut_fid, cut_row_ptr, col_of_feature, colbin, col_stride);
}

void launch_sorted_setup(hipStream_t s, const TreeBuffers &tb, const CsrBins &bins, const SparsePass &sp, int *row0,
                         unsigned *key0, unsigned short *start0) {
    if (sp.n_sorted_tasks == 0) return;
    k_sorted_setup<<<sp.n_sorted_tasks, 256, 0, s>>>(sp, bins, tb.cut_row_ptr, row0, key0, start0);
}

void launch_sparse_gh_refresh(hipStream_t s, const TreeBuffers &tb, const CsrBins &bins, const SparsePass &sp,
                              const GHPair *gh, int n_class) {
    if (sp.csc_gh == nullptr || sp.n_tasks == 0) return;
    k_sparse_gh_refresh<<<dim3(sp.n_tasks, 1, n_class), 256, 0, s>>>(tb.n, sp, bins.csc_row, gh);
}

void launch_sparse_level(hipStream_t s, const TreeBuffers &tb, const CsrBins &bins, const SparsePass &sp,
                         const GHPair *gh, int level, float mcw, float lambda, bool dump_hist, int n_class,
                         bool last_level) {
    // LDS table of a table task: room for one feature of 255 bins with every node of the level, at least 2048 and at
    // most kSparseCells cells (shallow levels: small tables, two workgroups per CU; deep levels: node ranges)
    int n_cells = 2048;
    while (n_cells < kSparseCells && n_cells < 256 * (1 << level)) n_cells *= 2;
    const size_t lds = sizeof(longlong2) * (size_t)n_cells;
    if (dump_hist) {
        // the table kernels store the cells of their features, the sorted pass adds its values: start from zero
        for (int k = 0; k < n_class; ++k)
            launch_fill_f32(s, reinterpret_cast<float *>(tb.for_class(k).hist(level)), 0.f,
                            (size_t)(1 << level) * tb.n_bins * 4);
    }
    static bool opted = false;
    if (!opted) {  // more than the default dynamic LDS window: opt in once
        const size_t lds_max = sizeof(longlong2) * (size_t)kSparseCells;
        HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(&k_sparse_level),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_max));
        HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(&k_sparse_big),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_max));
        opted = true;
    }
    if (sp.n_tasks > 0)
        k_sparse_level<<<dim3(sp.n_tasks, 1, n_class), kSpBlock, lds, s>>>(tb, bins, sp, gh, level, mcw, lambda,
                                                                          dump_hist ? 1 : 0, n_cells);
    if (sp.n_big > 0)
        k_sparse_big<<<dim3(sp.n_big, std::min(1 << level, 16), n_class), kSpBlock, lds, s>>>(
            tb, sp, level, mcw, lambda, dump_hist ? 1 : 0, n_cells);
    if (sp.n_sorted_tasks > 0) {
        const int dh = dump_hist ? 1 : 0;
        const size_t so_lds = (size_t)(1 << level) * 20;
        if (level == 0)
            k_sparse_sorted<true><<<dim3(sp.n_sorted_tasks, 1, n_class), kSortedBlock, so_lds, s>>>(
                tb, sp, gh, level, mcw, lambda, dh, last_level ? 1 : 0);
        else
            k_sparse_sorted<false><<<dim3(sp.n_sorted_tasks, 1, n_class), kSortedBlock, so_lds, s>>>(
                tb, sp, gh, level, mcw, lambda, dh, last_level ? 1 : 0);
    }
}

void launch_sparse_partition(hipStream_t s, const TreeBuffers &tb, const CsrBins &bins, int level, int n_class) {
    const int grid = std::max(1, std::min(1024, (tb.n + kSpBlock - 1) / kSpBlock));
    k_sparse_partition<<<dim3(grid, 1, n_class), kSpBlock, 0, s>>>(tb, bins, level);
}

}  // namespace tgbm
