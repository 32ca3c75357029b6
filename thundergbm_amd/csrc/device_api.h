// Host-callable launchers of the HIP kernels (gfx950). All launches are stream-ordered and never
// synchronise; sizes are validated by the callers in trainer.hip / predictor.hip.
#pragma once
#include <hip/hip_runtime.h>

#include <vector>

#include "common.h"

#define HIP_CHECK(expr)                                                                              \
    do {                                                                                             \
        hipError_t e_ = (expr);                                                                      \
        if (e_ != hipSuccess) ::tgbm::fatal("%s:%d HIP error %s: %s", __FILE__, __LINE__, #expr,     \
                                            hipGetErrorString(e_));                                  \
    } while (0)

// A kernel launch reports a bad configuration (too much LDS, an empty or oversized grid) only through
// hipGetLastError; the host stages call this after their launches so that such a failure aborts with the
// stage's name instead of leaving stale results behind.
#define HIP_CHECK_LAUNCHES(stage)                                                                    \
    do {                                                                                             \
        hipError_t e_ = hipGetLastError();                                                           \
        if (e_ != hipSuccess) ::tgbm::fatal("kernel launch failed in %s: %s", stage, hipGetErrorString(e_)); \
    } while (0)

namespace tgbm {

constexpr int kMissingBin = 255;   // dense matrix sentinel: the feature has no stored value in this row
constexpr int kMissingBin16 = 65535;  // the same for 16-bit bins
// 16-bit bins: bins of a feature block that leave the LDS room for two histogram workgroups per CU, and the most a
// block may hold at all (160 KB of 8-byte bins)
constexpr int kDense16BlockBins = 8192;
constexpr int kDense16MaxBlockBins = 20480;
constexpr int kPartChunk = 2048;   // rows per partition work item (256 threads x 8 rounds)
constexpr int kEvalPackBins = 256; // bins scanned by one wavefront in split finding (4 per lane)
constexpr int kCsrHeadBins = 4864;  // head slots of the sparse histogram: 2 x 8 bytes each, two workgroups per CU
// Rows a packed LDS bin may absorb before it is drained (QuantCtl::flush_rows). With float hessians (32 + 32-bit
// fields) 8192: a row of a large node is then counted at 2^-17 of the tree's largest |g|, and even rows that all
// round the same way (the first logistic tree has two gradient values) stay within 4e-6 of the sum of |g|; 32768
// measured 1.2 % faster on 10 M rows (root items never drained) and put the root sum of that tree beyond the 1e-5
// bound. With integer hessians the gradient field has 47 bits and 32768 rows cost no precision that matters: the
// 500 k x 2000 regression builds a tree in 1.90 instead of 2.00 ms.
constexpr int kHistFlushRows = 8192;
constexpr int kHistFlushRowsInt = 32768;
constexpr int kRowBlock = 4096;    // rows owned by one workgroup of the row-ordered passes and reductions
inline int row_blocks(int n) { return n <= 0 ? 1 : (n + kRowBlock - 1) / kRowBlock; }

// Per-level control block written by the planning kernels and read by the worker kernels.
struct LevelCtl {
    int hchunk;      // rows per histogram work item
    int n_hitems;    // histogram work items of the level
    int n_pitems;    // partition work items of the level
    int rows_built;  // rows visited by the histogram build of the level
};

// Fixed-point plan of one tree. Histograms are exact 64-bit integer sums of round(g * scale_g), round(h * scale_h);
// the scales are the largest powers of two that keep the sum over all n rows below 2^62, so the quantum is about
// max|g| * n / 2^62 (2^-38 of the largest gradient at 10 M rows).
//   Dense layout: a work item (a run of rows of one node) accumulates in LDS with one 64-bit integer atomic per
// (row, feature) - gfx950 executes those about 15x faster than float LDS atomics - into a packed bin: gradient in
// the high 64 - h_bits bits (signed), hessian in the low h_bits bits. The fields must hold the sum of the
// rows added between two drains of the LDS bins into 64-bit registers, at most min(rows of the node,
// flush_rows), so the items of a node coarsen the tree's scales by a power of two (shift) that depends on the
// node's row count only: the fewer rows a node has, the finer it counts, and what a row adds to a node does not
// depend on the order of the rows;
// k_hist_merge shifts every item's sums back to the tree's scale. h_bits: 32 in general; when every hessian of the
// tree is a small non-negative integer (squared loss: 1, or the draw count under bagging) the hessian field gets
// exactly the bits that flush_rows * max h needs and the gradient field the rest (47 bits for h = 1), which
// is what keeps heavy-tailed regression residuals at float-like resolution (2^-32 of the largest |g| per row).
// All sums after the LDS stage are 64-bit integers: exact, order-independent, bit-reproducible.
struct QuantCtl {
    float scale_g, scale_h;  // value -> integer of the tree's histograms (powers of two)
    float inv_g, inv_h;      // integer -> value
    float gq_max, hq_max;    // max|g| * scale_g, max h * scale_h: the most one row can add
    int h_bits;              // width of the hessian field of a packed LDS bin
    int h_integer;           // 1: every hessian is an integer, scale_h = 1 and no item shifts it
    int flush_rows;          // rows a packed LDS bin absorbs between two drains (kHistFlushRows / kHistFlushRowsInt)
};

// Block result of the per-tree gradient reduction.
struct GradStats {
    float g, h;        // sums
    float gmax, hmax;  // max |g|, max h
    float hfrac;       // max |h - round(h)|: 0 when every hessian is an integer
};

// Candidate produced by one wavefront of the split finder.
struct SplitCand {
    float score;  // signed gain: > 0 missing goes left, <= 0 missing goes right
    int index;    // global bin index
    GHPair miss;
    GHPair left;  // sum of the bins strictly below the candidate, within its feature
    int pad[2];
};

// Dense column-blocked bin matrix: block b holds features [b*W, (b+1)*W) as n rows of W bytes.
struct DenseBins {
    const uint8_t *data = nullptr;
    int W = 0;          // features per row of a block (a row of a block is W * bin_bytes bytes, a multiple of 4)
    int n_blocks = 0;
    size_t block_stride = 0;  // bytes between blocks = n * W * bin_bytes
    // Column-major copy (feature f = n consecutive bins at col + f * col_stride * bin_bytes): the partition reads
    // one feature of many rows, which costs one bin per row here instead of one sector per row.
    const uint8_t *col = nullptr;
    size_t col_stride = 0;  // in bins
    // 1: byte bins (at most 255 bins per feature, 255 = no stored value); 2: 16-bit bins for max_num_bin above 255
    // (65535 = no stored value)
    int bin_bytes = 1;
    // Bundles (byte bins only; nullptr: every feature has a column of its own). Consecutive features of which no row
    // stores more than one (one-hot groups) share one column of the matrix: feature f sits in column feat_col[f] and
    // its local bin b is stored as feat_lo[f] + b, where feat_lo[f] counts the bins of the bundle's features before
    // f - the byte is the bin's distance from the bundle's first global bin, which is all the histogram kernel needs.
    // A byte outside [feat_lo[f], feat_lo[f] + bins of f) means that f has no stored value in the row.
    const int *feat_col = nullptr;
    const uint8_t *feat_lo = nullptr;
    int n_cols = 0;  // columns of the matrix (= features when nothing is bundled)
    // Lane (dword) of a row's record that is kept free of bins for the row's gradient word (the last lane of the
    // row), -1: none. gh_fresh: gh_words[row] (launch_gh_words) matches the gradient array of this launch; the root
    // level's histogram launch then decodes the words (gh_objective says how) instead of reading the pairs and copies
    // them into the records, and the launches below the root take them from the records instead of gathering the
    // pairs. That lane never adds bins either way.
    int gh_lane = -1;
    int gh_fresh = 0;
    int gh_objective = 0;
    const unsigned *gh_words = nullptr;  // [n]
};

// Sparse layout for wide, mostly-missing data: the reference's own representation, CSR rows of global
// bin ids (hist_tree_builder_single.cu:49-130).
struct CsrBins {
    const int *row_ptr = nullptr;  // [n + 1]
    const int *bin = nullptr;      // [nnz] global bin id, ascending within a row
    // Histogram addressing of the same stored values: the bins of the most frequent features (the
    // "head", at most kCsrHeadBins of them) are accumulated in LDS. word >= 0: global bin id,
    // word < 0: ~word is the head slot. nullptr: no head (every value goes to HBM).
    const int *hist_word = nullptr;  // [nnz]
    const int *head_bin = nullptr;   // [head_bins] global bin id of every head slot
    int head_bins = 0;
    // The same stored values sorted by global bin id (rows ascending inside a bin): the root histogram, where
    // every row takes part, is a segmented sum over this copy instead of atomics to random bins. nullptr: none.
    const int *csc_bin = nullptr;  // [nnz]
    const int *csc_row = nullptr;  // [nnz]
    long nnz = 0;
    // Sparse level pass: byte columns of the frequent features (local bin id of the row, kMissingBin = no stored
    // value), column col_of_feature[f] at colbin + col * col_stride; col_of_feature[f] < 0: the feature has none
    const uint8_t *colbin = nullptr;
    const int *col_of_feature = nullptr;  // [F]
    size_t col_stride = 0;
};

// Sparse layout, level pass: one pass per level over the bin-major copy of the stored values (sorted by global bin,
// rows ascending inside a bin). A task is a run of whole features, or a chunk of one feature that has too many
// values for one workgroup ("big" feature); a task accumulates (node, bin) tables of its features in LDS and
// searches them for every node's best candidate right there, so no per-node histogram exists in HBM.
constexpr int kSparseCells = 8192;      // (node, bin) cells of 16 bytes an LDS table holds
constexpr int kSparseMaxLevelNodes = 1024;  // deepest level the pass serves (depth <= 11)
constexpr int kSparseBatchFeatures = 2047;  // features whose tables share one LDS batch at most
constexpr int kSparseTaskValues = 32768;    // stored values per task (and per chunk of a big feature)
struct SparseTask {
    int f_begin, f_end;  // features [f_begin, f_end) (a chunk task: one feature)
    int v_begin, v_end;  // positions of the bin-major copy
    int cand_slot;       // candidate slot the task fills, -1: a chunk (its feature's slot is filled by k_sparse_big)
    int partial_slot;    // chunk: where its table goes in SparsePass::partial, else -1
};
// Features with at most kSortedTile stored values are not searched through tables: their values are kept sorted by
// (feature, node, bin) from level to level - a stable two-way partition of every (feature, node) run when the node
// splits - and the split search is a segmented scan of that order, so the work follows the stored values and not
// the (bin, node) cells. A task is a run of whole features whose values fit one workgroup tile.
constexpr int kSortedBlock = 512;                        // threads of a sorted-pass workgroup
constexpr int kSortedPerThread = 8;                      // consecutive values a thread owns
constexpr int kSortedTile = kSortedBlock * kSortedPerThread;  // values per task at most
constexpr int kSortedLevels = 12;                        // levels the pass serves (depth <= 11, one spare)
struct SortedTask {
    int v_begin;     // first position of the task's tile in the sorted-pass arrays
    int count;       // stored values of its features (= live values at the root)
    int meta_begin;  // first entry of its features in SparsePass::sorted_meta / sorted_fid
    int n_feat;      // features of the task
    int cand_slot;   // candidate slot the task fills
};
// Key of a stored value in the sorted pass: feature (index inside its task) << 20 | node of the level << 8 | local bin
constexpr int kSortedNodeShift = 8, kSortedFeatShift = 20;
struct SparseBig {
    int feature;
    int slot_begin, slot_end;  // partial slots of its chunks
    int cand_slot;
};
struct SparsePass {
    const SparseTask *tasks = nullptr;
    int n_tasks = 0;
    const SparseBig *big = nullptr;
    int n_big = 0;
    // sorted pass (features of at most kSortedTile values)
    const SortedTask *sorted_tasks = nullptr;
    int n_sorted_tasks = 0;
    const int2 *sorted_meta = nullptr;    // per feature of a task: (first global bin, number of bins)
    const int *sorted_fid = nullptr;      // its feature id
    const int *sorted_row0 = nullptr;     // [n_sorted] rows and keys in the static order (feature, bin, row): the
    const unsigned *sorted_key0 = nullptr;  // root level's input
    const unsigned short *sorted_start0 = nullptr;  // [n_sorted] tile position where the value's feature starts
    long n_sorted = 0;
    // per set: the order of the previous and of the current level, ping-pong by level parity
    int *sorted_row[2] = {nullptr, nullptr};
    unsigned *sorted_key[2] = {nullptr, nullptr};
    GHPair *sorted_gh[2] = {nullptr, nullptr};
    int *sorted_live = nullptr;           // [n_sets][kSortedLevels][n_sorted_tasks] live values of a tile after a level
    const int *feat_val_begin = nullptr;  // [F + 1] first position of every feature in the bin-major copy
    // [n_sets][nnz] the gradient pair of every stored value's row, in the order of the bin-major copy, refreshed once
    // per tree: the level passes then stream it instead of fetching a cache line per value (nullptr: no room, gather)
    GHPair *csc_gh = nullptr;
    long nnz = 0;
    longlong2 *partial = nullptr;         // [n_sets][n_partial_slots][partial_stride] chunk tables, (bin, node) cells
    size_t partial_stride = 0;            // cells per slot: most bins of a big feature x kSparseMaxLevelNodes at most
    int n_partial_slots = 0;
    int n_cand_slots = 0;

    // the sorted pass's order of a level (selected without indexing an array member dynamically)
    __host__ __device__ int *srow(int level) const { return (level & 1) ? sorted_row[1] : sorted_row[0]; }
    __host__ __device__ unsigned *skey(int level) const { return (level & 1) ? sorted_key[1] : sorted_key[0]; }
    __host__ __device__ GHPair *sgh(int level) const { return (level & 1) ? sorted_gh[1] : sorted_gh[0]; }
};

struct TreeBuffers {
    int n = 0, n_bins = 0, F = 0, depth = 0, n_nodes = 0;
    int sparse = 0;                // 1: CSR layout, histograms accumulated directly in hist_q
    TreeNode *nodes = nullptr;     // [n_nodes]
    int2 *seg = nullptr;           // [n_nodes] row-list segment [x, y) of every node
    int *nid = nullptr;            // [n]
    int *ridx[2] = {nullptr, nullptr};  // [n] row lists, ping-pong by level parity
    uint8_t *goes_right = nullptr; // [max_pitems * 256] per partition item and thread: bit k = its k-th row goes right
    longlong2 *hist_q[2] = {nullptr, nullptr};  // [max_level_nodes * n_bins] exact fixed-point histograms (g, h)
                                                // of the nodes of a level, ping-pong by level parity
    longlong2 *partial = nullptr;  // [max_hitems * n_bins] per-item fixed-point sums (g, h)
    QuantCtl *quant = nullptr;     // scales of the current tree
    int2 *hitem_shift = nullptr;   // [max_hitems] powers of two by which a dense work item (its node) coarsened (g, h)
    // Root sums as exact integers at the tree's scales (what a row order cannot change), from the gradients when no
    // feature is stored in every row: [2 i], [2 i + 1] the sums of workgroup i of k_root_sum_rows (up to 256)
    // sparse level pass only (else nullptr): node every row has reached (heap id) and rows per node
    unsigned short *nid16 = nullptr;  // [n + 2]
    int *node_rows = nullptr;         // [n_nodes]
    // what the last row -> node update did with every row: bit 0 = the row moved to a child (its node split), bit 1 =
    // to the right child. A byte per row instead of the 16-bit node: the sorted pass, which knows a value's previous
    // node from its key, looks its rows up here with one-byte loads, eight of them in flight per thread (the whole
    // map stays in every L2).
    uint8_t *row_move = nullptr;      // [n rounded up to 64]
    // sparse level pass: best candidate key of every node of the level over all tasks, and the candidate slot of
    // the task that searches a feature (k_best_update reads the winner's record from that slot)
    unsigned long long *best_key = nullptr;  // [max_level_nodes]
    const int *feat_slot = nullptr;          // [F]
    long long *root_total = nullptr;
    int complete_feature = -1;     // dense layout: a feature stored in every row (its bins add up to the root), or -1
    int max_hitems = 0, target_hitems = 0, max_pitems = 0;
    float *leaf_value = nullptr;   // [n_nodes] prediction increment of a row that ended in the node (after pruning)
    int *end_bound = nullptr;      // [(row_blocks(n) + 1) x (2^depth - 1)] list positions of the row block boundaries
    int *hpair_begin = nullptr;    // [max_pairs + 1] first histogram item of every sibling pair
    int *hpair_built = nullptr;    // [max_pairs] heap id of the node built from rows, -1 = inactive pair
    int *pitem_begin = nullptr;    // [2][max_level_nodes + 1] first partition item of every node of a level, by level parity
    int *pitem_nleft = nullptr;    // [max_pitems]
    int *pitem_loff = nullptr;     // [max_pitems]
    int *node_nleft = nullptr;     // [max_level_nodes]
    LevelCtl *ctl = nullptr;       // [depth + 1]
    SplitPoint *sp = nullptr;      // [max_level_nodes]
    SplitCand *cand = nullptr;     // [max_level_nodes * n_packs]
    GradStats *root_partial = nullptr;  // [n_grad_blocks] block results of the per-tree gradient reduction
    int n_grad_blocks = 0;
    // split finder packing: wavefront w scans global bins [pack_begin[w], pack_begin[w+1]) (whole features)
    const int *pack_begin = nullptr;
    // per bin: distance to the last bin of its feature (low byte) and whether it is the feature's first bin (bit 8)
    const unsigned short *bin_meta = nullptr;  // [n_bins]
    int n_packs = 0;
    const uint8_t *ignored = nullptr;  // [F] columns whose candidates score 0 this round (nullptr: none)
    // Features with more than 255 cut points (max_num_bin up to 65 535; CSR layout, per-node path): the node's split
    // bin does not fit TreeNode::split_bid, a byte as in the reference's model format, so the row -> node update
    // reads it from here. nullptr: every feature has at most 255 bins.
    int *split_bin = nullptr;          // [n_nodes] local bin id of the node's split
    const int *cut_row_ptr = nullptr;
    const int *cut_fid = nullptr;
    const float *cut_val = nullptr;
    // dense block tables
    const int *blk_bin_begin = nullptr;  // [n_blocks + 1] first global bin of every block
    const int *feat_lds_off = nullptr;   // [n_blocks * W] bin offset of a feature inside its block
    int max_block_bins = 0;
    // Every per-tree array above is allocated n_sets times back to back (one set per class tree of a
    // boosting round, so that the trees of a round can be built by the same launches, class = blockIdx.z).
    int n_sets = 1;
    int max_level_nodes = 0;
    // Histogram arena smaller than the deepest level (it is sized against the free memory; the reference does the
    // same with its last_hist buffer and builds both siblings from rows beyond the depth that fits,
    // hist_tree_builder_single.cu:811-832, :544-570): hist_nodes node histograms per buffer. A level with more nodes
    // is served in batches of nodes [lvl_x0, lvl_x1) (the buffer pointer is shifted so that node x still sits at
    // x * n_bins); from level singles_from on no parent histogram exists any more, so every child of a split node
    // is built from its own rows and the "pairs" of the work-item plan are single nodes.
    int hist_nodes = 0;
    int lvl_x0 = 0, lvl_x1 = 1 << 30;
    int singles_from = 1 << 30;
    __host__ __device__ bool singles(int level) const { return level >= singles_from; }
    __host__ __device__ int n_hpairs(int level) const {
        return level == 0 ? 1 : (singles(level) ? (1 << level) : (1 << (level - 1)));
    }
    __host__ __device__ int hpair_lo(int level) const { return singles(level) ? lvl_x0 : (lvl_x0 >> 1); }
    __host__ __device__ int hpair_hi(int level) const {  // end of the pairs of the served nodes
        const int n = n_hpairs(level);
        const long hi = singles(level) ? (long)lvl_x1 : (((long)lvl_x1 + 1) >> 1);
        return hi < n ? (int)hi : n;
    }
    __host__ __device__ int nodes_served(int level) const {
        const int nl = 1 << level;
        return (lvl_x1 < nl ? lvl_x1 : nl) - lvl_x0;
    }
    size_t n_end_bound = 0, n_partial = 0;

    // Row list / histogram buffer of a level (selected without indexing an array member dynamically: a
    // kernel's local copy of this struct would otherwise be placed in scratch memory).
    __host__ __device__ int *list(int level) const { return (level & 1) ? ridx[1] : ridx[0]; }
    __host__ __device__ longlong2 *hist(int level) const { return (level & 1) ? hist_q[1] : hist_q[0]; }
    __host__ __device__ int *pbegin(int level) const { return pitem_begin + (level & 1) * (max_level_nodes + 1); }

    // The buffers of set k (k = 0: this object itself).
    __host__ __device__ TreeBuffers for_class(int k) const {
        TreeBuffers t = *this;
        if (k == 0) return t;
        const size_t K = (size_t)k;
        t.nodes += K * n_nodes;
        t.seg += K * n_nodes;
        t.nid += K * n;
        t.ridx[0] += K * n;
        t.ridx[1] += K * n;
        t.goes_right += K * (size_t)max_pitems * 256;
        t.hist_q[0] += K * hist_nodes * n_bins;
        t.hist_q[1] += K * hist_nodes * n_bins;
        t.partial += K * n_partial;
        t.quant += K;
        t.hitem_shift += K * max_hitems;
        t.root_total += K * 512;
        if (nid16 != nullptr) {
            t.nid16 += K * (((size_t)n + 2) / 2 * 2);
            t.node_rows += K * n_nodes;
            t.row_move += K * (((size_t)n + 63) / 64 * 64);
            t.best_key += K * max_level_nodes;
        }
        t.leaf_value += K * n_nodes;
        t.end_bound += K * n_end_bound;
        t.hpair_begin += K * (max_level_nodes + 1);
        t.hpair_built += K * max_level_nodes;
        t.pitem_begin += K * 2 * (max_level_nodes + 1);
        t.pitem_nleft += K * ((size_t)max_pitems + 1);
        t.pitem_loff += K * ((size_t)max_pitems + 1);
        t.node_nleft += K * max_level_nodes;
        t.ctl += K * (depth + 2);
        t.sp += K * max_level_nodes;
        t.cand += K * max_level_nodes * n_packs;
        t.root_partial += K * n_grad_blocks;
        if (split_bin != nullptr) t.split_bin += K * n_nodes;
        return t;
    }
};

// objective codes
enum Objective { OBJ_SQUARE = 0, OBJ_LOGISTIC = 1, OBJ_SOFTMAX = 2, OBJ_RANK = 3 };

void launch_gradient(hipStream_t s, int objective, int n, int num_class, const float *y, const float *yp, GHPair *gh,
                     GHPair *block_sums, int n_blocks);
// RowSampler::do_bagging over the N gradient pairs; `count` holds N zeroed ints and is left zeroed. perm (may
// be null): original row of each of the n_rows physical positions; the N entries are planes of n_rows rows
void launch_bagging(hipStream_t s, int N, unsigned seed, int *count, GHPair *gh, const int *perm = nullptr,
                    int n_rows = 0);
// Tree-building launchers: `tb` is the first buffer set, `n_class` consecutive sets (the class trees of one
// round) are served by one launch; gradient / prediction pointers address the first of those classes.
// stats_ready: tb.root_partial already holds the block statistics of gh_class (fused round end)
void launch_tree_init(hipStream_t s, const TreeBuffers &tb, const GHPair *gh_class, float lambda,
                      bool stats_ready = false, int n_class = 1);
void launch_hist_dense(hipStream_t s, const TreeBuffers &tb, const DenseBins &bins, const GHPair *gh, int level,
                       int n_class = 1);
void launch_hist_merge(hipStream_t s, const TreeBuffers &tb, int level, int n_class = 1);
// After the root histogram exists: replaces the root's float sums (whose last bits depend on the order of the rows)
// by the exact fixed-point totals, from the bins of tb.complete_feature or, without one, from the gradients.
void launch_root_sum(hipStream_t s, const TreeBuffers &tb, const GHPair *gh_class, float lambda, int n_class = 1);
// Number of bytes equal to `value` among n bytes in device memory (synchronises).
long device_count_bytes(hipStream_t s, const uint8_t *d_v, size_t n, uint8_t value);
long device_count_u16(hipStream_t s, const uint16_t *d_v, size_t n, uint16_t value);
void launch_hist_csr(hipStream_t s, const TreeBuffers &tb, const CsrBins &bins, const GHPair *gh, int level,
                     int n_class = 1);
void launch_partition_csr(hipStream_t s, const TreeBuffers &tb, const CsrBins &bins, int level, int n_class = 1);
// store_sibling (sparse layout only): keep the derived sibling histograms; nobody reads those of a tree's
// last level
void launch_eval_split(hipStream_t s, const TreeBuffers &tb, int level, float mcw, float lambda, int n_class = 1,
                       bool store_sibling = true);
// Split search with one workgroup per (feature, node): any number of bins per feature (n_packs = F candidates per node)
void launch_eval_split_wide(hipStream_t s, const TreeBuffers &tb, int level, float mcw, float lambda, int n_class = 1,
                            bool store_sibling = true);
void launch_best_update(hipStream_t s, const TreeBuffers &tb, int level, float rt_eps, float lambda, int n_class = 1);
void launch_partition_dense(hipStream_t s, const TreeBuffers &tb, const DenseBins &bins, int level, int n_class = 1);
// Sparse level pass (tb.nid16 set): split search of a level (candidates into tb.cand, one slot per task / big
// feature; launch_best_update follows) and the row -> node update. dump_hist: also store the (node, bin) tables
// into tb.hist(level) (stage-wise driving and tests; needs tb.hist_q). last_level: the tree's deepest level (the
// sorted pass then keeps its new order to itself: no level reads it).
void launch_sparse_level(hipStream_t s, const TreeBuffers &tb, const CsrBins &bins, const SparsePass &sp,
                         const GHPair *gh, int level, float mcw, float lambda, bool dump_hist, int n_class = 1,
                         bool last_level = false);
void launch_sparse_partition(hipStream_t s, const TreeBuffers &tb, const CsrBins &bins, int level, int n_class = 1);
// Byte columns of the frequent features (CsrBins::colbin, pre-filled with kMissingBin) from the bin-major copy.
void launch_sparse_cols(hipStream_t s, long nnz, const int *csc_bin, const int *csc_row, const int *cut_fid,
                        const int *cut_row_ptr, const int *col_of_feature, uint8_t *colbin, size_t col_stride);
// Fills the static order of the sorted pass (row0 / key0, sp.n_sorted entries) from the bin-major copy.
void launch_sorted_setup(hipStream_t s, const TreeBuffers &tb, const CsrBins &bins, const SparsePass &sp, int *row0,
                         unsigned *key0, unsigned short *start0);
// csc_gh[e] = gh[csc_row[e]] for the values of the table tasks, n_class gradient planes (once per tree)
void launch_sparse_gh_refresh(hipStream_t s, const TreeBuffers &tb, const CsrBins &bins, const SparsePass &sp,
                              const GHPair *gh, int n_class = 1);
// Row-ordered passes over the row lists (one of dbins / cbins by tb.sparse). lookup_level: the level
// whose split nodes still hold their children's rows (-1: none).
void launch_nid_rebuild(hipStream_t s, const TreeBuffers &tb, const DenseBins *dbins, const CsrBins *cbins,
                        int lookup_level);
// (prune_gamma, here and below: prune the tree with this gamma first - launch_prune's work inside the same launches)
void launch_predict_in_training(hipStream_t s, const TreeBuffers &tb, const DenseBins *dbins, const CsrBins *cbins,
                                int lookup_level, float *yp_class, float lr, int n_class = 1,
                                const float *prune_gamma = nullptr);
// prediction update + metric + next gradients + their block statistics (tb.root_partial); metric_scratch
// holds row_blocks(n) doubles
void launch_round_end(hipStream_t s, const TreeBuffers &tb, const DenseBins *dbins, const CsrBins *cbins,
                      int lookup_level, int objective, int metric_kind, const float *y, float *yp, float lr,
                      GHPair *gh, double *metric_scratch, float *metric_out, const float *prune_gamma = nullptr,
                      unsigned *gh_words = nullptr);
// words[i] = the gradient word of row i (the pair of a squared or 0/1-label logistic loss in 32 bits, which the
// histogram kernels decode to the very pair launch_gradient computes; see DenseBins::gh_lane)
void launch_gh_words(hipStream_t s, int objective, int n, const float *y, const float *yp, unsigned *words);
// scratch: row_blocks(n) doubles
void launch_metric(hipStream_t s, int objective_metric, int n, int num_class, const float *y, const float *yp,
                   double *scratch, float *out);
void launch_fill_f32(hipStream_t s, float *p, float v, size_t n);
void launch_fill_u8(hipStream_t s, uint8_t *p, uint8_t v, size_t n);

// data preparation
// F: columns of the matrix; feat_col / feat_lo: DenseBins' bundle tables or nullptr
void launch_bin_dense(hipStream_t s, int n, const int *row_ptr, const int *col, const float *val, const float *cut_val,
                      const int *cut_row_ptr, uint8_t *binmat, int W, size_t block_stride, uint8_t *colmat,
                      size_t col_stride, int bin_bytes, int F, const int *feat_col = nullptr,
                      const uint8_t *feat_lo = nullptr, bool rows_ascend = true);
// false when some row holds a column index below its predecessor's
bool device_rows_ascend(hipStream_t s, int n, const int *row_ptr, const int *col);
// min_next[c] (pre-filled with INT_MAX) = smallest column index that follows column c in a row (equal neighbours, a
// column stored twice, do not count); *descending is set when a row's columns do not ascend
void launch_min_next_col(hipStream_t s, int n, const int *row_ptr, const int *col, int *min_next, int *descending);
// feat_slot (may be nullptr): first head slot of a feature or -1; then hist_word is written as well
void launch_bin_csr(hipStream_t s, long nnz, const int *col, const float *val, const float *cut_val,
                    const int *cut_row_ptr, int *bin_id, const int *feat_slot = nullptr, int *hist_word = nullptr);
// cut points on device: returns the device arrays through out parameters allocated by the callee
struct DeviceCuts {
    float *cut_val = nullptr;
    int *cut_row_ptr = nullptr;
    int *cut_fid = nullptr;
    int n_bins = 0;
    std::vector<long> feature_nnz;  // host: stored values per feature
};
DeviceCuts build_cut_points(hipStream_t s, int F, long nnz, const float *d_val, const int *d_col, int max_num_bin);

// Tile sums of the device-wide exclusive scan, one pair of arrays per recursion level (grown on demand).
struct ScanScratch {
    struct Level {
        unsigned *sums = nullptr, *scanned = nullptr;
        size_t cap = 0;
    };
    std::vector<Level> levels;
    void release();
};

// out[i] = in[0] + ... + in[i-1] over n 32-bit counters, *d_total (device) = the sum of all of them.
void device_exclusive_scan(hipStream_t s, const unsigned *in, unsigned *out, long n, unsigned *d_total,
                           ScanScratch &sc);

// Buffers of sort_pairs for up to `cap` (64-bit key, 32-bit payload) pairs; allocated once, reused per call.
struct PairSorter {
    long cap = 0, n_tiles = 0;
    unsigned long long *keys[2] = {nullptr, nullptr};
    int *vals[2] = {nullptr, nullptr};
    unsigned *counts = nullptr, *offsets = nullptr, *d_total = nullptr;
    ScanScratch scan;
    void alloc(long n);
    void release();
};
// Stable LSD radix sort (8 bits per pass) of the n pairs in keys[0] / vals[0] by the key bits [0, key_bits),
// ascending. Returns which of the two buffer pairs (0 or 1) holds the result. Stream-ordered; allocates only
// when the scan scratch has to grow (first call).
int sort_pairs(hipStream_t s, PairSorter &ps, long n, int key_bits);

// Bin-major copy of CSR bin ids: sort keys (global bin, payload = row) of every stored value, and the sorted
// pairs split into the two int arrays the root histogram reads. sort_key (may be null): the key a bin sorts by
// (the bin itself stays in the key's high half and is what csc_bin receives).
void launch_csc_keys(hipStream_t s, int n_rows, const int *row_ptr, const int *bin, const int *sort_key,
                     unsigned long long *keys, int *vals);
void launch_csc_unpack(hipStream_t s, long nnz, const unsigned long long *keys, const int *vals, int *csc_bin,
                       int *csc_row);

// Pieces of the physical re-ordering of the rows: sort keys (node of a row, payload = its position), gathers
// dst[p] = src[from[p]] of whole rows, the row permutation, and the column-major copy rebuilt from the
// row-major blocks.
void launch_reorder_keys(hipStream_t s, int n, int depth, const int *nid, unsigned long long *keys, int *vals);
void launch_gather_rows(hipStream_t s, int n, int bytes_per_row, const int *from, const void *src, void *dst);
void launch_gather_perm(hipStream_t s, int n, const int *from, const int *perm_old, int *perm_new);
void launch_cols_from_rows(hipStream_t s, int n, int W, int F, int n_blocks, const uint8_t *binmat, size_t block_stride,
                           uint8_t *colmat, size_t col_stride, int bin_bytes);

// Largest of n ints in device memory (synchronises; 0 for n == 0); aborts when one of them is negative.
int device_max_int(hipStream_t s, const int *d_v, long n);

// Host -> device copy of a pageable array on stream s; large ones go through pinned staging buffers and are
// complete on return, small ones (< 128 MB) are a plain stream-ordered hipMemcpyAsync.
void upload_large(hipStream_t s, void *dst, const void *src, size_t bytes);

// prediction of the n rows that row_ptr addresses (entry offsets into col / val); out[t * out_stride + i] for
// class tree t and row i, out_stride = 0 means n (a slice of a larger row set passes the whole set's size)
// `packed` (optional): the same nodes as 16-byte records (launch_pack_model); with them the trees are walked from LDS
void launch_predict(hipStream_t s, int n, int F, const int *row_ptr, const int *col, const float *val,
                    const TreeNode *model, int n_iter, int n_class_trees, int n_nodes, float lr, float base_score,
                    float *out, size_t out_stride = 0, const struct PackedNode *packed = nullptr,
                    const uint2 *compact = nullptr, int compact_depth = 0);
// What a traversal reads of a node, in one 16-byte record.
struct PackedNode {
    float split_value, base_weight;
    unsigned children;  // left | right << 16 (a tree has at most 2^15 - 1 nodes)
    unsigned meta;      // split feature (24 bits, all ones: not a feature of the data) | default_right << 30 | leaf << 31
};
void launch_pack_model(hipStream_t s, const TreeNode *model, long n_total, int n_nodes, PackedNode *packed);
// `compact` of launch_predict: eight-byte records (threshold or leaf weight; left child | address of the split feature's
// values | flags) for a model and data of F features that compact_records_apply() accepts; `compact_depth`: what it
// returned. The records depend on F (features the data lacks, rows per workgroup), so they are packed per data set.
void launch_pack_compact(hipStream_t s, const TreeNode *model, int n_iter, int n_class_trees, int n_nodes, int F,
                         uint2 *packed);
// Do the eight-byte records describe this model on data of F features? Every split node keeps its children side by
// side (right = left + 1) and below itself - then a walk needs one child index and ends after at most `depth` steps,
// the number returned (0: they do not apply) -, and one tree fits the LDS next to the rows' dense vectors.
int compact_records_apply(const TreeNode *model, size_t n_total, int n_nodes, int F);
int compact_rows_per_group(int F);  // rows per workgroup of the kernel that walks the eight-byte records
void launch_predict_transform(hipStream_t s, int kind, int n, int num_class, const float *label, float *y);

}  // namespace tgbm
