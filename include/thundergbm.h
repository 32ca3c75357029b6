/*
 * C ABI of libthundergbm.so (MI355X build).
 *
 * Part 1 is the drop-in boundary: the nine entry points that the reference's Python wrapper
 * (python/thundergbm/thundergbm.py) binds with ctypes, with the argument order, types and
 * ownership rules of src/thundergbm/scikit_tgbm.cpp, plus the two file-based entry points of the R
 * interface (src/thundergbm/gbm_R_interface.cpp). Where the reference declares `Tree *&model`
 * the ABI passes the address of an 8-byte slot; it is spelled `tgbm_model **` here. The model is
 * opaque, owned by the library and released only by model_free().
 *
 * Part 2 is a session API over the same trainer for callers that keep data resident in HBM between
 * calls (the benchmark) or drive the stages one by one (the parity tests).
 *
 * Failures abort the process after printing a FATAL line, as the reference's CHECK macros do.
 * One call trains on one GPU and blocks until done. The training and prediction calls of part 1 hold a
 * process-wide lock (the reference serialises Booster::boost with a global mutex, booster.h:17,78), so calls
 * from several threads run one after the other; a session of part 2 belongs to one thread at a time.
 */
#ifndef THUNDERGBM_H
#define THUNDERGBM_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct tgbm_model tgbm_model;

/* ---------------------------------------------------------------- Part 1: reference boundary */

/* scikit_tgbm.cpp:13-23. verbose 0 = silent, 1 = info, 2 = debug. */
void set_logger(int verbose);

/* scikit_tgbm.cpp:26-80. CSR input (float32 values, int32 indices, ascending columns per row).
 * num_class is in/out, group_label receives the distinct labels (caller allocates one float per
 * distinct label), tree_per_iter and *model are outputs. column_sampling_rate < 1 samples columns per
 * round as the reference does (see tgbm_trainer_set_option). group / num_group are the query group sizes
 * of the ranking objectives (rank:pairwise, rank:ndcg; dataset.cpp:64-68) and ignored otherwise. bagging != 0
 * resamples the gradients every round (RowSampler::do_bagging, row_sampler.cu:9-38, booster.h:84). n_device
 * and n_parallel_trees (never read by the reference either) are accepted for signature compatibility and
 * ignored. */
void sparse_train_scikit(int row_size, float *val, int *row_ptr, int *col_ptr, float *label, int depth, int n_trees,
                         int n_device, float min_child_weight, float lambda, float gamma, int max_num_bin,
                         int verbose, float column_sampling_rate, int bagging, int n_parallel_trees,
                         float learning_rate, char *obj_type, int *num_class, char *tree_method, tgbm_model **model,
                         int *tree_per_iter, float *group_label, int *group, int num_group);

/* scikit_tgbm.cpp:83-121. y_pred: row_size floats, or row_size * num_class (class-major) for
 * multi:softprob. As in the reference the base score is not part of this path. group / num_group: query
 * groups of the rows for a ranking objective; they only feed the metric line of the log and may be absent. */
void sparse_predict_scikit(int row_size, float *val, int *row_ptr, int *col_ptr, float *y_pred, tgbm_model **model,
                           int n_trees, int trees_per_iter, char *objective, int num_class, float learning_rate,
                           float *group_label, int *group, int num_group, int verbose);

/* scikit_tgbm.cpp:123-147 / parser.cpp:146-171: raw binary model file. */
void save(char *model_path, char *objective, float learning_rate, int num_class, int n_trees, int trees_per_iter,
          tgbm_model **model, float *group_label);

/* scikit_tgbm.cpp:148-172 / parser.cpp:102-145. */
void load_model(char *model_path, float *learning_rate, int *num_class, int *n_trees, int *trees_per_iter,
                tgbm_model **model);

/* scikit_tgbm.cpp:173-182: the label table of a model file. */
void load_config(char *model_path, float *group_label);

/* scikit_tgbm.cpp:184-197: node count of every tree (all 2^(depth+1)-1 heap slots). */
void get_n_nodes(tgbm_model **model, int *n_nodes, int n_trees, int tree_per_iter);

/* scikit_tgbm.cpp:199-248: one tree as parallel arrays in heap order. */
void get_a_tree(tgbm_model **model, int tree_id, int n_nodes, int *children_left, int *children_right,
                int *children_default, int *features, float *thresholds, float *values,
                float *node_sample_weights);

/* scikit_tgbm.cpp:250-254. */
void model_free(tgbm_model **model);

/* gbm_R_interface.cpp:10-61 and :63-86, the two symbols R/gbm.R reaches with .C(): every argument is a
 * pointer, strings are char**. train_R loads the LIBSVM file data[0] (plus data[0].group for a ranking
 * objective), trains and writes the model file model_out[0]; predict_R loads model_in[0] and the file
 * data[0], predicts and logs the metric. min_child_weight is an int here, as in the reference. */
void train_R(int *depth, int *n_trees, int *n_gpus, int *verbose, int *profiling, char **data, int *max_num_bin,
             double *column_sampling_rate, int *bagging, int *n_parallel_trees, double *learning_rate,
             char **objective, int *num_class, int *min_child_weight, double *lambda_tgbm, double *gamma,
             char **tree_method, char **model_out);
void predict_R(char **data, char **model_in, int *verbose);

/* ------------------------------------------------------------------- Part 2: session API */

typedef struct tgbm_trainer tgbm_trainer;

/* DataSet::load_from_sparse + HistTreeBuilder_single::init + Booster::init
 * (dataset.cpp:20-63, hist_tree_builder_single.cu:783-844, booster.h:36-74): copies the CSR input
 * to the GPU, builds cut points, the bin matrix and the base score. */
tgbm_trainer *tgbm_trainer_create(int row_size, const float *val, const int *row_ptr, const int *col_ptr,
                                  const float *label, int depth, int n_trees, float min_child_weight, float lambda,
                                  float gamma, int max_num_bin, float learning_rate, const char *objective,
                                  int num_class, int verbose);
/* The same with query groups for the ranking objectives rank:pairwise / rank:ndcg (LambdaRank,
 * LambdaRankNDCG: objective/ranking_obj.cpp:11-18, :100-103): `group` holds num_group sizes of consecutive
 * runs of rows that sum to row_size, as in the group / num_group arguments of sparse_train_scikit
 * (scikit_tgbm.cpp:31, dataset.cpp:64-68). Other objectives ignore them. */
tgbm_trainer *tgbm_trainer_create_grouped(int row_size, const float *val, const int *row_ptr, const int *col_ptr,
                                          const float *label, int depth, int n_trees, float min_child_weight,
                                          float lambda, float gamma, int max_num_bin, float learning_rate,
                                          const char *objective, int num_class, int verbose, const int *group,
                                          int num_group);
void tgbm_trainer_destroy(tgbm_trainer *t);

/* Options that tgbm_trainer_create has no argument for. "column_sampling_rate" (GBMParam, common.h:92):
 * below 1 every boosting round ignores max(1, int(n_features * rate)) randomly chosen columns in its split
 * search (Shard::column_sampling, builder/shard.cu:8-22; the shuffle draws from the process-wide rand()).
 * "bagging" (common.h:97): non-zero makes every gradient pass multiply the gradient pairs by bootstrap draw
 * counts (RowSampler::do_bagging, row_sampler.cu:9-38; seeded with one rand() per pass).
 * "reorder_first", "reorder_burst", "reorder_every", "reorder_min_rows" (no counterpart in the reference):
 * tgbm_trainer_boost physically re-orders the rows by the leaves of the tree just built after each of the
 * trees `reorder_first` .. `reorder_first + reorder_burst - 1` and then every `reorder_every` trees
 * (defaults 1, 3 and 32; reorder_first 0 = never) when the dataset has at least
 * `reorder_min_rows` rows (default 2^20), the layout is dense and the objective is not a ranking one. Results do not
 * depend on it beyond float round-off, and all per-row buffers keep the caller's row order. */
void tgbm_trainer_set_option(tgbm_trainer *t, const char *key, double value);
/* The column sampling of one round for stage-wise driving (tgbm_trainer_boost does it itself). */
void tgbm_trainer_sample_columns(tgbm_trainer *t);

/* `rounds` iterations of Booster::boost (booster.h:76-93); returns after the GPU finished. */
void tgbm_trainer_boost(tgbm_trainer *t, int rounds);

/* Stage-wise driving; each call returns after enqueueing (tgbm_trainer_get synchronises).
 * gradient = ObjectiveFunction::get_gradient (then do_bagging when the option is on); tree_init = Tree::init2; find_split = find_split +
 * update_tree of the level; partition = update_ins2node_id; finish_tree = prune_self +
 * predict_in_training. */
void tgbm_trainer_gradient(tgbm_trainer *t);
void tgbm_trainer_tree_init(tgbm_trainer *t, int class_id);
void tgbm_trainer_find_split(tgbm_trainer *t, int level);
void tgbm_trainer_partition(tgbm_trainer *t, int level);
void tgbm_trainer_finish_tree(tgbm_trainer *t, int class_id);
float tgbm_trainer_metric(tgbm_trainer *t);

/* Integer facts: n, n_features, n_bins, num_class, tree_per_rounds, n_nodes, dense_W,
 * dense_blocks, dense_cols (columns of the dense bin matrix: fewer than n_features when runs of features
 * that never meet in a row share a column), trees_built, rounds_done, n_packs, depth, y_pred_size, max_hitems, n_sets (class trees
 * of a round built by common launches), reorders_done, device_free_mb (free device memory in MiB). */
int tgbm_trainer_info(tgbm_trainer *t, const char *key);
float tgbm_trainer_base_score(tgbm_trainer *t);

/* Copies a device buffer to `out` when `cap` is large enough; always returns its size in bytes.
 * Names: cut_val, cut_row_ptr, cut_fid, binmat (dense layout: [dense_blocks][n][dense_W] bins of the matrix's
 * columns; with dense_cols < n_features feature f is column feat_col[f] and its local bin b is stored as
 * feat_lo[f] + b), feat_col (int per feature), feat_lo (byte per feature), nid, gh, y_pred, y, nodes, sp, hist_q0, hist_q1,
 * quant, ctl, seg, ridx0, ridx1, model, metric_log, labels, rank_order (ranking objectives: the rows in
 * the order of the last gradient or metric pass). After tgbm_trainer_boost `gh` may already
 * hold the gradients of the next round (single-tree objectives compute them in the round's last pass). */
size_t tgbm_trainer_get(tgbm_trainer *t, const char *name, void *out, size_t cap);
/* Overwrites gh or y_pred (lock-step tests feed both implementations the same state). */
void tgbm_trainer_set(tgbm_trainer *t, const char *name, const void *in, size_t bytes);

/* Histogram-build timing with HIP events on the trainer's stream. get_profile fills
 * out[0] = summed kernel milliseconds, out[1] = launches, out[2] = rows visited,
 * out[3] = algorithmic bytes (rows x (features + 8 [+4 below the root])). */
void tgbm_trainer_set_profiling(tgbm_trainer *t, int on);
void tgbm_trainer_get_profile(tgbm_trainer *t, double *out4);
/* Per-stage timing of the rounds boosted while profiling was on (the reference accumulates host timers for histogram
 * build, evaluation and data partitioning under its `profiling` switch, hist_tree_builder_single.cu:19-27, :196-219,
 * :392, :400-418; thundergbm_train.cpp:28-30). HIP events on the trainer's stream close every stage. Fills up to
 * `cap` of: out[0] rounds; milliseconds of out[1] gradients + tree init, [2] histogram build, [3] merge + sibling
 * subtraction + root sums, [4] split search + tree update, [5] partition, [6] end of tree (prune, prediction update,
 * fused metric and next gradients), [7] metric as a pass of its own, [8] row re-ordering; then the histogram launches
 * of the root level: [9] milliseconds, [10] launches, [11] algorithmic bytes; and of the levels below it: [12], [13],
 * [14]. Returns the number of values it knows (15). */
int tgbm_trainer_get_phase_profile(tgbm_trainer *t, double *out, int cap);

/* Moves the trees built so far into a model handle usable with the Part 1 functions. */
tgbm_model *tgbm_trainer_export_model(tgbm_trainer *t);

/* Predictor::predict_raw (predictor.cu:32-189) with an explicit base score: class-major raw scores,
 * row_size * trees_per_iter floats. */
void tgbm_predict_raw(int row_size, const float *val, const int *row_ptr, const int *col_ptr, tgbm_model *model,
                      int n_trees, int trees_per_iter, float learning_rate, float base_score, float *out);

/* tgbm_predict_raw for callers that cannot allocate device memory (tight serving loops, harnesses that forbid
 * hipMalloc). It has no counterpart in the reference. Same arguments, same scores bit for bit, but no hipMalloc /
 * hipFree / stream creation: the device copies of the rows, the model and the scores live in a file-scope device
 * array of about 34 MiB that every GPU used by the library holds until the process ends (its address is resolved on
 * the first call on a device). Limits per call: row_size <= 65536, stored values <= 2^20,
 * row_size * trees_per_iter <= 2^19, nodes of the trees used <= 2^19 (e.g. 800 trees of depth 8). Returns 0, or 1
 * with a message on stderr when a limit is exceeded (nothing is computed then); malformed input (a null model, a
 * row_ptr that does not ascend, a negative column index) aborts the process with a message, as in every other entry
 * point. Calls share the device's array, which keeps the last call's contents; they are serialised inside one
 * process, and calls from several processes on one GPU do not interfere (every process has its own copy). The work
 * runs on the default stream with synchronous host copies (the call cannot be recorded into a HIP graph) and returns
 * after the scores were copied to `out`. The trees are walked in their 48-byte node form (the packed LDS form of
 * tgbm_predict_raw needs an allocation), so a call takes about twice the device time of tgbm_predict_raw. */
int tgbm_predict_raw_noalloc(int row_size, const float *val, const int *row_ptr, const int *col_ptr,
                             tgbm_model *model, int n_trees, int trees_per_iter, float learning_rate,
                             float base_score, float *out);

/* Cut points and global bin ids of a CSR matrix (HistCut::get_cut_points_single, hist_cut.cu:232-286;
 * get_bin_ids, hist_tree_builder_single.cu:49-130), computed on the GPU. cut_val / cut_fid need one
 * slot per stored value at most (row_ptr[row_size]); returns the number of cut points. */
int tgbm_cut_points(int row_size, int n_features, const float *val, const int *row_ptr, const int *col_ptr,
                    int max_num_bin, float *cut_val, int *cut_row_ptr, int *cut_fid, int *bin_id);

#ifdef __cplusplus
}
#endif
#endif /* THUNDERGBM_H */
