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

// Level-wide state every task starts from: node sums and validity into LDS, keys cleared, the task's candidate slot
// marked empty for every node.
__device__ void sp_begin(const TreeBuffers &tb, SpShared &sh, int level, int cand_slot) {
    const int nl = 1 << level, off = nl - 1;
    for (int x = threadIdx.x; x < nl; x += kSpBlock) {
        const TreeNode &nd = tb.nodes[off + x];
        sh.S[x] = nd.sum_gh_pair;
        sh.ok[x] = nd.is_valid ? 1 : 0;
        sh.key[x] = 0ull;
        if (cand_slot >= 0) tb.cand[(size_t)x * tb.n_packs + cand_slot].index = 0x7fffffff;
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
                                                          float lambda, int dump_hist) {
    extern __shared__ longlong2 cells[];  // [kSparseCells]
    __shared__ SpShared sh;
    const TreeBuffers tb = tb_all.for_class(blockIdx.z);
    gh += (size_t)blockIdx.z * tb.n;
    const SparseTask task = sp.tasks[blockIdx.x];
    const int nl = 1 << level, off = nl - 1;
    const unsigned short *__restrict__ nid16 = tb.nid16;
    const int *__restrict__ crp = tb.cut_row_ptr;
    const float scale_g = tb.quant->scale_g, scale_h = tb.quant->scale_h;
    const GHPair *__restrict__ csc_gh = sp.csc_gh != nullptr ? sp.csc_gh + (size_t)blockIdx.z * sp.nnz : nullptr;
    sp_begin(tb, sh, level, task.cand_slot);
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
            if ((long)kf * nl <= kSparseCells) {
                int total = kf;
                while (fb < task.f_end && fb - f < kSparseBatchFeatures) {
                    const int k = crp[fb + 1] - crp[fb];
                    if ((long)(total + k) * nl > kSparseCells) break;
                    total += k;
                    ++fb;
                }
                kf = total;
            } else {
                nn = kSparseCells / kf;
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
            constexpr int U = 4;
            for (int e0 = v0 + threadIdx.x; e0 < v1; e0 += kSpBlock * U) {
                int gb[U], row[U], x[U];
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const int e = e0 + u * kSpBlock;
                    const bool in = e < v1;
                    gb[u] = in ? bins.csc_bin[e] : 0;
                    row[u] = in ? bins.csc_row[e] : -1;
                }
#pragma unroll
                for (int u = 0; u < U; ++u) x[u] = row[u] >= 0 ? (int)nid16[row[u]] - off - n0 : -1;
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    if ((unsigned)x[u] < (unsigned)nn) {
                        const GHPair s = csc_gh != nullptr ? csc_gh[e0 + u * kSpBlock] : gh[row[u]];
                        const long long gq = __float2ll_rn(s.g * scale_g), hq = __float2ll_rn(s.h * scale_h);
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
}

// A big feature: the tables of its chunks are added up (node range by node range) and searched.
__global__ __launch_bounds__(kSpBlock) void k_sparse_big(TreeBuffers tb_all, SparsePass sp, int level, float mcw,
                                                        float lambda, int dump_hist) {
    extern __shared__ longlong2 cells[];
    __shared__ SpShared sh;
    const TreeBuffers tb = tb_all.for_class(blockIdx.z);
    const SparseBig big = sp.big[blockIdx.x];
    const int nl = 1 << level;
    const int f = big.feature;
    const int bin0 = tb.cut_row_ptr[f], kf = tb.cut_row_ptr[f + 1] - bin0;
    sp_begin(tb, sh, level, big.cand_slot);
    if (threadIdx.x == 0) {
        sh.fbin[0] = 0;
        sh.fbin[1] = kf;
    }
    const longlong2 *base = sp.partial + (size_t)blockIdx.z * sp.n_partial_slots * sp.partial_stride;
    longlong2 *dump = dump_hist ? tb.hist(level) : nullptr;
    const int nn_max = (long)kf * nl <= kSparseCells ? nl : kSparseCells / kf;
    for (int n0 = 0; n0 < nl; n0 += nn_max) {
        const int nn = min(nn_max, nl - n0);
        const int n_cells = kf * nn;
        __syncthreads();
        for (int c = threadIdx.x; c < n_cells; c += kSpBlock) {
            long long g = 0, h = 0;
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
}

// ------------------------------------------------------------------------------------ tail features
// A feature with a few hundred stored values touches a few hundred (bin, node) cells of the thousands a table of
// a deep level has. One wavefront takes such a feature: it loads the values (already ascending by bin), sorts them
// stably by the node of their row (counting sort in LDS, ranks from ballots), and scans the sorted run: a forward
// and a backward segmented sum per node give every position the node's sum up to it and after it, hence the left
// sum and the feature total (missing = node sum - total). Candidates exist only where the left sum changes: the
// feature's first bin (left empty) and the bin after every bin that holds a value - all bins in between repeat the
// previous candidate's gain and lose the tie on the smaller index - so the result is what the scan of a complete
// (bin, node) table gives. Every wavefront keeps its best key per node in LDS and owns one candidate slot in HBM.
constexpr int kTailBlock = 64 * kSparseTailWaves;
constexpr int kTailR = kSparseTailValues / 64;  // values per lane

__device__ __forceinline__ long long shfl_down_ll(long long v, int d) {
    int lo = __shfl_down((int)(unsigned)(unsigned long long)v, d);
    int hi = __shfl_down((int)((unsigned long long)v >> 32), d);
    return (long long)(((unsigned long long)(unsigned)hi << 32) | (unsigned)lo);
}

struct TailCand {
    float score;
    int index;
    GHPair left;
    unsigned long long key;
};

__device__ __forceinline__ TailCand tail_candidate(GHPair S, GHPair m, GHPair l, int index, bool ignored, float mcw,
                                                   float lambda) {
#pragma clang fp contract(off)
    const float gr = split_gain(S, l, mcw, lambda);
    const GHPair l2{l.g + m.g, l.h + m.h};
    const float gl = split_gain(S, l2, mcw, lambda);
    TailCand c;
    c.score = (gl > gr) ? gl : -gr;
    if (ignored) c.score = 0.f;
    c.index = index;
    c.left = l;
    c.key = cand_key(fabsf(c.score), index);
    return c;
}

__global__ __launch_bounds__(kTailBlock) void k_sparse_tail(TreeBuffers tb_all, CsrBins bins, SparsePass sp,
                                                          const GHPair *__restrict__ gh, int level, float mcw,
                                                          float lambda, int dump_hist) {
#pragma clang fp contract(off)
    extern __shared__ unsigned char dyn[];
    __shared__ GHPair s_S[kSparseMaxLevelNodes];
    const TreeBuffers tb = tb_all.for_class(blockIdx.z);
    gh += (size_t)blockIdx.z * tb.n;
    const SparseTailTask task = sp.tail_tasks[blockIdx.x];
    const int nl = 1 << level, off = nl - 1;
    const int w = threadIdx.x >> 6, lane = lane_id();
    // per wavefront: sorted sums (2 x 8 B), sorted (node << 8 | bin) keys, node counters, best keys
    const size_t wave_bytes = (size_t)kSparseTailValues * 20 + (size_t)nl * 12;
    unsigned char *base = dyn + (size_t)w * ((wave_bytes + 15) / 16 * 16);
    long long *s_g = reinterpret_cast<long long *>(base);
    long long *s_h = s_g + kSparseTailValues;
    unsigned long long *s_key = reinterpret_cast<unsigned long long *>(s_h + kSparseTailValues);  // [nl]
    unsigned *s_k = reinterpret_cast<unsigned *>(s_key + nl);                                   // [kSparseTailValues]
    int *s_cnt = reinterpret_cast<int *>(s_k + kSparseTailValues);                              // [nl]
    const int slot = task.cand_slot + w;
    for (int x = threadIdx.x; x < nl; x += kTailBlock) s_S[x] = tb.nodes[off + x].sum_gh_pair;
    for (int x = lane; x < nl; x += 64) {
        s_key[x] = 0ull;
        tb.cand[(size_t)x * tb.n_packs + slot].index = 0x7fffffff;
    }
    __syncthreads();
    const unsigned short *__restrict__ nid16 = tb.nid16;
    const float scale_g = tb.quant->scale_g, scale_h = tb.quant->scale_h;
    const double inv_g = tb.quant->inv_g, inv_h = tb.quant->inv_h;
    const unsigned long long below = lane == 0 ? 0ull : (~0ull >> (64 - lane));
    const GHPair *__restrict__ csc_gh = sp.csc_gh != nullptr ? sp.csc_gh + (size_t)blockIdx.z * sp.nnz : nullptr;
    for (int fi = task.i_begin + w; fi < task.i_end; fi += kSparseTailWaves) {
        const int f = sp.tail_feat[fi];
        const int v0 = sp.feat_val_begin[f], m = sp.feat_val_begin[f + 1] - v0;
        const int fbegin = tb.cut_row_ptr[f], kf = tb.cut_row_ptr[f + 1] - fbegin;
        const bool ign = tb.ignored != nullptr && tb.ignored[f] != 0;
        const int R = (m + 63) >> 6;  // rounds that hold values (the loops below stop there)
        // ---- load: value a = r * 64 + lane of the feature, ascending by bin
        int xs[kTailR], lbs[kTailR], posn[kTailR];
        long long gq[kTailR], hq[kTailR];
        {
            int row[kTailR];
#pragma unroll
            for (int r = 0; r < kTailR; ++r) {
                const int a = r * 64 + lane;
                const bool in = r < R && a < m;
                lbs[r] = in ? bins.csc_bin[v0 + a] - fbegin : 0;
                row[r] = in ? bins.csc_row[v0 + a] : -1;
            }
#pragma unroll
            for (int r = 0; r < kTailR; ++r) {
                xs[r] = -1;
                if (r < R && row[r] >= 0) xs[r] = (int)nid16[row[r]] - off;  // < 0: a leaf above
            }
#pragma unroll
            for (int r = 0; r < kTailR; ++r) {
                gq[r] = hq[r] = 0;
                if (r < R && xs[r] >= 0) {
                    const GHPair s = csc_gh != nullptr ? csc_gh[v0 + r * 64 + lane] : gh[row[r]];
                    gq[r] = __float2ll_rn(s.g * scale_g);
                    hq[r] = __float2ll_rn(s.h * scale_h);
                }
            }
        }
        if (dump_hist) {
            // stage-wise inspection: the per-node histograms of the level (zeroed before the launch) get the values
            unsigned long long *hist = reinterpret_cast<unsigned long long *>(tb.hist(level));
#pragma unroll
            for (int r = 0; r < kTailR; ++r) {
                if (xs[r] >= 0) {
                    unsigned long long *cell = hist + 2 * ((size_t)xs[r] * tb.n_bins + fbegin + lbs[r]);
                    atomicAdd(cell, (unsigned long long)gq[r]);
                    atomicAdd(cell + 1, (unsigned long long)hq[r]);
                }
            }
        }
        // ---- stable counting sort by node: rank inside the node from ballots, in arrival order
        for (int x = lane; x < nl; x += 64) s_cnt[x] = 0;
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int r = 0; r < kTailR; ++r) {
            if (r >= R) break;
            const bool act = xs[r] >= 0;
            unsigned long long mask = __ballot(act);
            for (int bit = 0; bit < level; ++bit) {
                const bool b = (xs[r] >> bit) & 1;
                const unsigned long long bm = __ballot(act && b);
                mask &= b ? bm : ~bm;
            }
            int first = 0;
            if (act) {
                const int rank = __popcll(mask & below);
                if (rank == 0) {
                    first = s_cnt[xs[r]];
                    s_cnt[xs[r]] = first + __popcll(mask);
                }
                posn[r] = rank;
            }
            const int leader = act ? __ffsll((long long)mask) - 1 : lane;
            first = __shfl(first, leader);
            if (act) posn[r] += first;
            __builtin_amdgcn_wave_barrier();
        }
        // exclusive scan of the node counters (a run of counters per lane)
        int M;
        {
            const int per = (nl + 63) / 64;
            const int i0 = lane * per, i1 = min(nl, i0 + per);
            int local = 0;
            for (int i = i0; i < i1; ++i) local += s_cnt[i];
            int inc = local;
#pragma unroll
            for (int d = 1; d < 64; d <<= 1) {
                const int t = __shfl_up(inc, d);
                if (lane >= d) inc += t;
            }
            M = __shfl(inc, 63);
            int run = inc - local;
            for (int i = i0; i < i1; ++i) {
                const int c = s_cnt[i];
                s_cnt[i] = run;
                run += c;
            }
        }
        if (M == 0) continue;  // every value sits in a row that stopped in a leaf above this level
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int r = 0; r < kTailR; ++r) {
            if (r >= R) break;
            if (xs[r] >= 0) {
                const int d = s_cnt[xs[r]] + posn[r];
                s_g[d] = gq[r];
                s_h[d] = hq[r];
                s_k[d] = ((unsigned)xs[r] << 8) | (unsigned)lbs[r];
            }
        }
        __builtin_amdgcn_wave_barrier();
        // ---- scans over the sorted run: lane l owns positions [l * Rm, (l + 1) * Rm)
        const int Rm = (M + 63) / 64;
        const int p0 = lane * Rm;
        unsigned k[kTailR];
        long long Ig[kTailR], Ih[kTailR], Bg[kTailR], Bh[kTailR];
        bool head[kTailR], tail[kTailR], last_of_bin[kTailR];
        {
            long long rg = 0, rh = 0;
            bool any_head = false;
#pragma unroll
            for (int j = 0; j < kTailR; ++j) {
                const int p = p0 + j;
                const bool in = j < Rm && p < M;
                k[j] = in ? s_k[p] : 0xffffffffu;
                gq[j] = in ? s_g[p] : 0;
                hq[j] = in ? s_h[p] : 0;
                const unsigned prev = (in && p > 0) ? s_k[p - 1] : 0xffffffffu;
                const unsigned next = (in && p + 1 < M) ? s_k[p + 1] : 0xffffffffu;
                head[j] = in && (p == 0 || (prev >> 8) != (k[j] >> 8));
                tail[j] = in && (p + 1 == M || (next >> 8) != (k[j] >> 8));
                last_of_bin[j] = in && (p + 1 == M || next != k[j]);
                if (head[j]) {
                    rg = rh = 0;
                    any_head = true;
                }
                rg += gq[j];
                rh += hq[j];
                Ig[j] = rg;
                Ih[j] = rh;
            }
            long long ag = rg, ah = rh;
            int flag = any_head ? 1 : 0;
#pragma unroll
            for (int d = 1; d < 64; d <<= 1) {
                const long long pg = shfl_up_ll(ag, d), ph = shfl_up_ll(ah, d);
                const int pf = __shfl_up(flag, d);
                if (lane >= d) {
                    if (!flag) {
                        ag += pg;
                        ah += ph;
                    }
                    flag |= pf;
                }
            }
            long long cg = shfl_up_ll(ag, 1), ch = shfl_up_ll(ah, 1);
            if (lane == 0) cg = ch = 0;
            bool seen = false;
#pragma unroll
            for (int j = 0; j < kTailR; ++j) {
                if (head[j]) seen = true;
                if (!seen) {
                    Ig[j] += cg;
                    Ih[j] += ch;
                }
            }
        }
        {
            long long rg = 0, rh = 0;
            bool any_tail = false;
#pragma unroll
            for (int j = kTailR - 1; j >= 0; --j) {
                if (tail[j]) {
                    rg = rh = 0;
                    any_tail = true;
                }
                Bg[j] = rg;
                Bh[j] = rh;
                rg += gq[j];
                rh += hq[j];
            }
            long long ag = rg, ah = rh;
            int flag = any_tail ? 1 : 0;
#pragma unroll
            for (int d = 1; d < 64; d <<= 1) {
                const long long pg = shfl_down_ll(ag, d), ph = shfl_down_ll(ah, d);
                const int pf = __shfl_down(flag, d);
                if (lane + d < 64) {
                    if (!flag) {
                        ag += pg;
                        ah += ph;
                    }
                    flag |= pf;
                }
            }
            long long cg = shfl_down_ll(ag, 1), ch = shfl_down_ll(ah, 1);
            if (lane == 63) cg = ch = 0;
            bool seen = false;
#pragma unroll
            for (int j = kTailR - 1; j >= 0; --j) {
                if (tail[j]) seen = true;
                if (!seen) {
                    Bg[j] += cg;
                    Bh[j] += ch;
                }
            }
        }
        // ---- candidates: raise the wavefront's key of the node, then the winners write their record. A candidate
        // without gain never wins: the node's candidate at global bin 0 (a table feature's) has at least its key.
        float sc_head[kTailR], sc_bin[kTailR];
#pragma unroll
        for (int j = 0; j < kTailR; ++j) {
            sc_head[j] = sc_bin[j] = 0.f;
            if (j >= Rm) break;
            if (!(head[j] || last_of_bin[j])) continue;
            const int x = (int)(k[j] >> 8), lb = (int)(k[j] & 0xffu);
            const GHPair S = s_S[x];
            const GHPair mm{S.g - (float)((double)(Ig[j] + Bg[j]) * inv_g), S.h - (float)((double)(Ih[j] + Bh[j]) * inv_h)};
            if (head[j]) {
                const TailCand c = tail_candidate(S, mm, GHPair{0, 0}, fbegin, ign, mcw, lambda);
                sc_head[j] = c.score;
                if (c.score != 0.f) atomicMax(&s_key[x], c.key);
            }
            if (last_of_bin[j] && lb < kf - 1) {
                const GHPair l{(float)((double)Ig[j] * inv_g), (float)((double)Ih[j] * inv_h)};
                const TailCand c = tail_candidate(S, mm, l, fbegin + lb + 1, ign, mcw, lambda);
                sc_bin[j] = c.score;
                if (c.score != 0.f) atomicMax(&s_key[x], c.key);
            }
        }
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int j = 0; j < kTailR; ++j) {
            if (j >= Rm) break;
            if (sc_head[j] == 0.f && sc_bin[j] == 0.f) continue;
            const int x = (int)(k[j] >> 8), lb = (int)(k[j] & 0xffu);
            const unsigned long long best = s_key[x];
            const bool win_head = sc_head[j] != 0.f && best == cand_key(fabsf(sc_head[j]), fbegin);
            const bool win_bin = sc_bin[j] != 0.f && best == cand_key(fabsf(sc_bin[j]), fbegin + lb + 1);
            if (!(win_head || win_bin)) continue;
            const GHPair S = s_S[x];
            SplitCand o;
            o.miss = GHPair{S.g - (float)((double)(Ig[j] + Bg[j]) * inv_g), S.h - (float)((double)(Ih[j] + Bh[j]) * inv_h)};
            o.pad[0] = o.pad[1] = 0;
            if (win_head) {
                o.score = sc_head[j];
                o.index = fbegin;
                o.left = GHPair{0, 0};  // the first bin records an empty left side (hist_tree_builder_single.cu:378)
            } else {
                o.score = sc_bin[j];
                o.index = fbegin + lb + 1;
                o.left = GHPair{(float)((double)Ig[j] * inv_g), (float)((double)Ih[j] * inv_h)};
            }
            tb.cand[(size_t)x * tb.n_packs + slot] = o;
        }
        __builtin_amdgcn_wave_barrier();
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
    for (int r = blockIdx.x * kSpBlock + threadIdx.x; r < tb.n; r += gridDim.x * kSpBlock) {
        const int node = tb.nid16[r];
        if (node < off) continue;  // the row stays in a leaf of an earlier level
        const TreeNode &nd = tb.nodes[node];
        if (!node_splits(nd)) continue;
        const int cb = tb.cut_row_ptr[nd.split_feature_id], ce = tb.cut_row_ptr[nd.split_feature_id + 1];
        const bool right = csr_goes_right(bins, r, cb, ce, cb + nd.split_bid, nd.default_right);
        tb.nid16[r] = (unsigned short)(right ? nd.rch_index : nd.lch_index);
        atomicAdd(&cnt[2 * (node - off) + (right ? 1 : 0)], 1);
    }
    __syncthreads();
    for (int i = threadIdx.x; i < 2 * nl; i += kSpBlock)
        if (cnt[i] != 0) atomicAdd(&tb.node_rows[2 * off + 1 + i], cnt[i]);  // children of level node x: 2 (off + x) + 1, + 2
}

__global__ __launch_bounds__(256) void k_sparse_gh_refresh(int n, long nnz, const int *__restrict__ csc_row,
                                                          const GHPair *__restrict__ gh, GHPair *__restrict__ out) {
    gh += (size_t)blockIdx.z * n;
    out += (size_t)blockIdx.z * nnz;
    for (long e = (long)blockIdx.x * 256 + threadIdx.x; e < nnz; e += (long)gridDim.x * 256) out[e] = gh[csc_row[e]];
}

}  // namespace

void launch_sparse_gh_refresh(hipStream_t s, const TreeBuffers &tb, const CsrBins &bins, const SparsePass &sp,
                              const GHPair *gh, int n_class) {
    if (sp.csc_gh == nullptr || sp.nnz == 0) return;
    const int grid = (int)std::min<long>(16384, (sp.nnz + 255) / 256);
    k_sparse_gh_refresh<<<dim3(grid, 1, n_class), 256, 0, s>>>(tb.n, sp.nnz, bins.csc_row, gh, sp.csc_gh);
}

void launch_sparse_level(hipStream_t s, const TreeBuffers &tb, const CsrBins &bins, const SparsePass &sp,
                         const GHPair *gh, int level, float mcw, float lambda, bool dump_hist, int n_class) {
    const size_t lds = sizeof(longlong2) * (size_t)kSparseCells;
    if (dump_hist) {
        // the table kernels store the cells of their features, the tail kernel adds its values: start from zero
        for (int k = 0; k < n_class; ++k)
            launch_fill_f32(s, reinterpret_cast<float *>(tb.for_class(k).hist(level)), 0.f,
                            (size_t)(1 << level) * tb.n_bins * 4);
    }
    static bool opted = false;
    if (!opted) {  // more than the default dynamic LDS window: opt in once
        HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(&k_sparse_level),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(&k_sparse_big),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        opted = true;
    }
    if (sp.n_tasks > 0)
        k_sparse_level<<<dim3(sp.n_tasks, 1, n_class), kSpBlock, lds, s>>>(tb, bins, sp, gh, level, mcw, lambda,
                                                                          dump_hist ? 1 : 0);
    if (sp.n_big > 0)
        k_sparse_big<<<dim3(sp.n_big, 1, n_class), kSpBlock, lds, s>>>(tb, sp, level, mcw, lambda, dump_hist ? 1 : 0);
    if (sp.n_tail_tasks > 0) {
        const int nl = 1 << level;
        const size_t wave_bytes = ((size_t)kSparseTailValues * 20 + (size_t)nl * 12 + 15) / 16 * 16;
        const size_t tail_lds = wave_bytes * kSparseTailWaves;
        static size_t tail_opted = 0;
        if (tail_lds > 64 * 1024 && tail_lds > tail_opted) {
            HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(&k_sparse_tail),
                                          hipFuncAttributeMaxDynamicSharedMemorySize, (int)tail_lds));
            tail_opted = tail_lds;
        }
        k_sparse_tail<<<dim3(sp.n_tail_tasks, 1, n_class), kTailBlock, tail_lds, s>>>(tb, bins, sp, gh, level, mcw, lambda,
                                                                                     dump_hist ? 1 : 0);
    }
}

void launch_sparse_partition(hipStream_t s, const TreeBuffers &tb, const CsrBins &bins, int level, int n_class) {
    const int grid = std::max(1, std::min(1024, (tb.n + kSpBlock - 1) / kSpBlock));
    k_sparse_partition<<<dim3(grid, 1, n_class), kSpBlock, 0, s>>>(tb, bins, level);
}

}  // namespace tgbm
