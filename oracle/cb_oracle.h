/*
 * CPU oracle for the CatBoost model-evaluation path (binarize -> tree evaluation).
 *
 * TEST INFRASTRUCTURE ONLY. This is a plain-C restatement of the reference CPU evaluator
 * (catboost/libs/model/cpu) used as the checker for the HIP evaluator and as the timed
 * "port" CPU baseline. Nothing in the shipped library links, loads or calls it.
 *
 * Model tables arrive as flat arrays that mirror the TModelTrees flatbuffer table
 * (catboost/libs/model/flatbuffers/model.fbs:22-46, features.fbs:11-59).
 */
#ifndef CB_ORACLE_H
#define CB_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { CBO_NAN_AS_IS = 0, CBO_NAN_AS_FALSE = 1, CBO_NAN_AS_TRUE = 2 };

typedef struct cbo_model_desc {
    int32_t approx_dim;

    /* trees: TreeSplits / TreeSizes / TreeStartOffsets (model.h:97-141) */
    int32_t n_trees;
    const int32_t* tree_sizes;
    const int32_t* tree_start_offsets;
    int32_t n_tree_splits;
    const int32_t* tree_splits;

    /* float features, in model order (features.h:50-94) */
    int32_t n_float;
    const int32_t* ff_index;
    const int32_t* ff_flat_index;
    const int32_t* ff_has_nans;
    const int32_t* ff_nan_treatment;
    const int32_t* ff_border_offsets; /* n_float + 1 */
    const float* ff_borders;

    /* categorical features (features.h:104-140) */
    int32_t n_cat;
    const int32_t* cf_index;
    const int32_t* cf_flat_index;
    const int32_t* cf_used;

    /* one-hot features (features.h:142-160) */
    int32_t n_onehot;
    const int32_t* oh_cat_index;
    const int32_t* oh_value_offsets; /* n_onehot + 1 */
    const int32_t* oh_values;

    /* leaves: [tree][leaf * approx_dim + k] */
    uint64_t n_leaf_values;
    const double* leaf_values;

    /* non-symmetric trees (model.h:78-95); both empty for oblivious models */
    int32_t n_step_nodes;
    const uint16_t* step_nodes; /* pairs (LeftSubtreeDiff, RightSubtreeDiff) */
    const uint32_t* node_id_to_leaf_id;

    double scale;
    const double* bias; /* approx_dim values */

    /* CTR features in model order (features.h:306-323, online_ctr.h:108-316); n_ctr = 0 without them.
     * A projection = categorical features (by feature Index), float splits (feature Index, border)
     * and one-hot splits (cat feature Index, value). */
    int32_t n_ctr;
    const int32_t* ctr_border_offsets; /* n_ctr + 1 */
    const float* ctr_borders;
    const int32_t* ctr_cat_offsets; /* n_ctr + 1 */
    const int32_t* ctr_cats;
    const int32_t* ctr_float_offsets; /* n_ctr + 1 */
    const int32_t* ctr_float_feature;
    const float* ctr_float_border;
    const int32_t* ctr_onehot_offsets; /* n_ctr + 1 */
    const int32_t* ctr_onehot_cat;
    const int32_t* ctr_onehot_value;
    const int32_t* ctr_type; /* ECtrType, ctr_data.fbs:5-12 */
    const int32_t* ctr_target_border_idx;
    const float* ctr_prior_num;
    const float* ctr_prior_denom;
    const float* ctr_shift;
    const float* ctr_scale;
    const int32_t* ctr_table; /* value table of the CTR's base */
    /* value tables of the static CTR provider (ctr_value_table.h:17-109) */
    int32_t n_ctr_tables;
    const uint64_t* table_bucket_offsets; /* n_ctr_tables + 1, counted in 12-byte buckets */
    const uint8_t* table_buckets;         /* {u64 hash, u32 row} packed, dense_hash_view.h:12-26 */
    const uint64_t* table_blob_offsets;   /* n_ctr_tables + 1, in bytes */
    const uint8_t* table_blobs;
    const int32_t* table_counter_denominator;
    const int32_t* table_target_classes_count;
} cbo_model_desc;

typedef struct cbo_model cbo_model;

/* Copies the arrays and derives the runtime tables. Returns NULL and fills err on failure. */
cbo_model* cbo_model_create(const cbo_model_desc* desc, char* err, size_t err_len);
void cbo_model_free(cbo_model* m);

int32_t cbo_bucket_count(const cbo_model* m);
int32_t cbo_is_oblivious(const cbo_model* m);
int32_t cbo_tree_count(const cbo_model* m);
int32_t cbo_approx_dim(const cbo_model* m);
size_t cbo_flat_vector_expected_size(const cbo_model* m);
size_t cbo_min_float_vector_size(const cbo_model* m);
size_t cbo_min_cat_vector_size(const cbo_model* m);
size_t cbo_used_cat_count(const cbo_model* m);
/* out: n_tree_splits entries of (feature_index u16, xor_mask u8, split_idx u8) packed as
 * feature_index | xor_mask << 16 | split_idx << 24 */
void cbo_repacked_bins(const cbo_model* m, uint32_t* out);
void cbo_first_leaf_offsets(const cbo_model* m, uint64_t* out);

/* Feature access modes, as the accessor lambdas of TCpuEvaluator (formula_evaluator.cpp). */
typedef struct cbo_features {
    /* layout 0: flat rows       feats[doc * stride + FlatIndex], cats bit-cast from the same row
     * layout 1: flat transposed feats[FlatIndex * stride + doc]
     * layout 2: split rows      floats[doc * stride + Index], cats[doc * cat_stride + Index] */
    int32_t layout;
    const float* floats;
    size_t stride;
    const int32_t* cats;
    size_t cat_stride;
} cbo_features;

/* Bins in the reference layout: blocks of 128 docs, [block][bucket][doc in block], the
 * last block packed with its own doc count (quantization.h:333-365). */
void cbo_binarize(const cbo_model* m, const cbo_features* f, size_t n_docs, uint8_t* bins);

/* Raw formula values, out[doc * dim + k] = Scale * sum + Bias (bias only when tree_start == 0). */
void cbo_calc(const cbo_model* m, const cbo_features* f, size_t n_docs,
              size_t tree_start, size_t tree_end, double* out);
/* Same, doc blocks fanned over n_threads threads. */
void cbo_calc_mt(const cbo_model* m, const cbo_features* f, size_t n_docs,
                 size_t tree_start, size_t tree_end, double* out, int n_threads);
/* Leaf indexes, out[doc * (tree_end - tree_start) + t]. */
void cbo_calc_leaf_indexes(const cbo_model* m, const cbo_features* f, size_t n_docs,
                           size_t tree_start, size_t tree_end, uint32_t* out);

/* Independent brute force that never touches repacked bins: evaluates each split from the
 * raw (feature, border) / (cat feature, value) definition, one doc at a time. */
void cbo_calc_bruteforce(const cbo_model* m, const cbo_features* f, size_t n_docs,
                         size_t tree_start, size_t tree_end, double* out, uint32_t* leaf_indexes);

/* CTR values of the model's CTR features, out[ctr * n_docs + doc], computed per document from the
 * raw features (TStaticCtrProvider::CalcCtrs, static_ctr_provider.cpp:14-131). */
void cbo_calc_ctrs(const cbo_model* m, const cbo_features* f, size_t n_docs, float* out);

/* CalcCatFeatureHash (catboost/libs/cat_feature/cat_feature.cpp:6-8). */
uint64_t cbo_city_hash64(const char* s, size_t len);
uint32_t cbo_cat_feature_hash(const char* s, size_t len);
/* GetIntegerCatFeatureHash (catboost/libs/model_interface/c_api.cpp:944-949). */
int32_t cbo_integer_cat_feature_hash(long long v);

/* The exponent of the prediction types: NCB::FastExpWithInfInplace on an AVX2 host
 * (catboost/libs/helpers/math_utils.cpp:14-27) = fmath::expd_v (contrib/libs/fmath/fmath.hpp:565-648):
 * the first n & ~3 values take the vector path, the rest fmath::expd (:474-512). */
void cbo_fast_exp_inplace(double* x, size_t n);

/* TEvalResultProcessor::PostprocessBlock over blocks of min(128, n_docs) documents
 * (catboost/libs/model/eval_processing.h:174-240, cpu/formula_evaluator.cpp:27). raw[doc * dim + k]
 * -> out; out holds n_docs values for CBO_CLASS, n_docs * dim otherwise. Returns 0, or -1 for a
 * prediction type the dimension does not support. */
enum { CBO_RAW = 0, CBO_EXPONENT = 1, CBO_RMSE_WITH_UNCERTAINTY = 2, CBO_PROBABILITY = 3, CBO_CLASS = 4,
       CBO_MULTI_PROBABILITY = 5 };
int cbo_apply_prediction_type(int type, size_t dim, size_t n_docs, const double* raw, double* out);

#ifdef __cplusplus
}
#endif
#endif
