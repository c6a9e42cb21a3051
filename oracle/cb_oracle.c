/*
 * CPU oracle for the CatBoost model-evaluation path. TEST INFRASTRUCTURE ONLY: it is the
 * checker for the HIP evaluator and the timed CPU "port" baseline; the shipped library never
 * links or calls it.
 *
 * Every function restates a piece of the reference (paths relative to the CatBoost tree):
 *   derive tables        catboost/libs/model/model.cpp:471-577 (CalcBinFeatures), :586-624
 *   binarize             catboost/libs/model/cpu/quantization.h:54-141, 333-529
 *   oblivious trees      catboost/libs/model/cpu/evaluator_impl.cpp:16-52, 154-172, 246-361
 *   non-symmetric trees  catboost/libs/model/cpu/evaluator_impl.cpp:462-493, 661-705
 *   block driver         catboost/libs/model/cpu/formula_evaluator.cpp:10-81, cpu/evaluator.h:95-155
 *   scale and bias       catboost/libs/model/scale_and_bias.cpp:4-50
 *   cat feature hash     catboost/libs/cat_feature/cat_feature.cpp:6-8, util/digest/city.cpp:58-200
 *   prediction types     catboost/libs/model/eval_processing.h:15-99, 174-240,
 *                        contrib/libs/fmath/fmath.hpp:150-185, 474-512, 565-648 (the exponent)
 *   CTR features         catboost/libs/model/static_ctr_provider.cpp:14-178, ctr_provider.h:64-123,
 *                        online_ctr.h:290-293, hash.h:11-14, catboost/libs/helpers/dense_hash_view.h:46-56,
 *                        cpu/quantization.h:263-327
 *
 * Pinned by (see tests/test_oracle.py, tests/test_ref_vectors.py): the reference's own
 * standalone evaluator and its own fmath exponent, both built from the reference tree by
 * oracle/build_ref.sh (vectors under tests/golden/), the reference unit-test closed forms
 * (catboost/libs/model/ut/formula_evaluator_ut.cpp:76-146, 284-307), the .cbm fixtures with
 * golden predictions of the JVM / Rust / .NET binding tests, the JVM hash known answers, the
 * numpy searchsorted invariant for binarize, the oblivious -> non-symmetric equivalence and the
 * raw-split brute force below. CTR features: the golden predictions of the JVM, Rust and node
 * binding tests for models with CTRs of kinds Borders and Counter (reproduced to the last bit) and
 * the .NET mushroom test (8124 labels; projections of up to four categorical features, some with
 * a one-hot split); and, for all six CTR kinds, tables with up to five target classes and
 * projections with float splits (also past a feature's first 254 borders) and one-hot splits, the
 * CTR calculator that the reference ships for exported models (model_export/resources/ctr_structs.cpp
 * + ctr_calcer.cpp, built where they lie by oracle/build_ref.sh into oracle/_ref/ctr_calc): its values
 * on the seeded models of tests/ctr_models.py are stored in tests/golden/ctr_ref_vectors.npz and
 * reproduced bit for bit. That calculator answers an unknown hash with Calc(0, 0) for every kind,
 * the evaluator's TStaticCtrProvider with Calc(0, denominator) for Counter and FeatureFreq
 * (static_ctr_provider.cpp:63-75); this one case rests on the adult goldens (Counter CTRs, unknown
 * categories) alone. Whole models: the two trained models that the reference keeps as exported C++
 * code, tables and applier in one file (python-package/ut/medium/canondata/test.test_cpp_export_*;
 * built where they lie into oracle/_ref/export_{cat,nocat}): that applier's predictions on 3000
 * seeded documents each (tests/golden/cpp_export_vectors.npz) are reproduced bit for bit, and the
 * (bucket, split index, xor mask) derived here per tree split equal the arrays in that code.
 * Parity unpinned (followed by reading only, cross-checked by the brute force): the NaN gating
 * "HasNans && treatment != AsIs", >254-border buckets combined with one-hot XorMask, the
 * leaf numbering of non-symmetric multi-dimensional models, and for CTR projections the table
 * TStaticCtrProvider::SetupBinFeatureIndexes builds from a split to its (bin, value)
 * (static_ctr_provider.cpp:139-170; the fixture generator restates it a second time in Python).
 */
#include "cb_oracle.h"

#include <math.h>
#include <pthread.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#define CBO_BLOCK 128         /* FORMULA_EVALUATION_BLOCK_SIZE, cpu/quantization.h:16 */
#define CBO_MAX_VALUES_PER_BIN 254 /* model.h:72 */

/* ------------------------------------------------------------------ CityHash64 v1.0 ---- */
/* util/digest/city.cpp: the Yandex tree pins CityHash version 1 (util/digest/city.h:8-9). */

static const uint64_t K0 = 0xc3a5c85c97cb3127ULL;
static const uint64_t K1 = 0xb492b66fbe98f273ULL;
static const uint64_t K2 = 0x9ae16a3b2f90404fULL;
static const uint64_t K3 = 0xc949d7c7509e6557ULL;

static uint64_t ld64(const char* p) { uint64_t v; memcpy(&v, p, 8); return v; }
static uint32_t ld32(const char* p) { uint32_t v; memcpy(&v, p, 4); return v; }
static uint64_t rotr(uint64_t v, int s) { return s == 0 ? v : ((v >> s) | (v << (64 - s))); }
static uint64_t shift_mix(uint64_t v) { return v ^ (v >> 47); }

/* util/digest/city.h:36-45 */
static uint64_t hash128to64(uint64_t lo, uint64_t hi) {
    const uint64_t kMul = 0x9ddfea08eb382d69ULL;
    uint64_t a = (lo ^ hi) * kMul;
    a ^= (a >> 47);
    uint64_t b = (hi ^ a) * kMul;
    b ^= (b >> 47);
    b *= kMul;
    return b;
}

/* city.cpp:78-100 */
static uint64_t hash_len_0_16(const char* s, size_t len) {
    if (len > 8) {
        uint64_t a = ld64(s);
        uint64_t b = ld64(s + len - 8);
        return hash128to64(a, rotr(b + len, (int)len)) ^ b;
    }
    if (len >= 4) {
        uint64_t a = ld32(s);
        return hash128to64(len + (a << 3), ld32(s + len - 4));
    }
    if (len > 0) {
        uint8_t a = (uint8_t)s[0];
        uint8_t b = (uint8_t)s[len >> 1];
        uint8_t c = (uint8_t)s[len - 1];
        uint32_t y = (uint32_t)a + ((uint32_t)b << 8);
        uint32_t z = (uint32_t)len + ((uint32_t)c << 2);
        return shift_mix(y * K2 ^ z * K3) * K2;
    }
    return K2;
}

/* city.cpp:104-111 */
static uint64_t hash_len_17_32(const char* s, size_t len) {
    uint64_t a = ld64(s) * K1;
    uint64_t b = ld64(s + 8);
    uint64_t c = ld64(s + len - 8) * K2;
    uint64_t d = ld64(s + len - 16) * K0;
    return hash128to64(rotr(a - b, 43) + rotr(c, 30) + d, a + rotr(b ^ K3, 20) - c + len);
}

typedef struct { uint64_t first, second; } u64pair;

/* city.cpp:115-136 */
static u64pair weak_hash_32_seeds6(uint64_t w, uint64_t x, uint64_t y, uint64_t z, uint64_t a, uint64_t b) {
    a += w;
    b = rotr(b + a + z, 21);
    uint64_t c = a;
    a += x;
    a += y;
    b += rotr(a, 44);
    u64pair r = {a + z, b + c};
    return r;
}
static u64pair weak_hash_32_seeds(const char* s, uint64_t a, uint64_t b) {
    return weak_hash_32_seeds6(ld64(s), ld64(s + 8), ld64(s + 16), ld64(s + 24), a, b);
}

/* city.cpp:139-162 */
static uint64_t hash_len_33_64(const char* s, size_t len) {
    uint64_t z = ld64(s + 24);
    uint64_t a = ld64(s) + (len + ld64(s + len - 16)) * K0;
    uint64_t b = rotr(a + z, 52);
    uint64_t c = rotr(a, 37);
    a += ld64(s + 8);
    c += rotr(a, 7);
    a += ld64(s + 16);
    uint64_t vf = a + z;
    uint64_t vs = b + rotr(a, 31) + c;
    a = ld64(s + 16) + ld64(s + len - 32);
    z = ld64(s + len - 8);
    b = rotr(a + z, 52);
    c = rotr(a, 37);
    a += ld64(s + len - 24);
    c += rotr(a, 7);
    a += ld64(s + len - 16);
    uint64_t wf = a + z;
    uint64_t ws = b + rotr(a, 31) + c;
    uint64_t r = shift_mix((vf + ws) * K2 + (wf + vs) * K0);
    return shift_mix(r * K0 + vs) * K2;
}

/* city.cpp:164-200 */
uint64_t cbo_city_hash64(const char* s, size_t len) {
    if (len <= 32) {
        return len <= 16 ? hash_len_0_16(s, len) : hash_len_17_32(s, len);
    } else if (len <= 64) {
        return hash_len_33_64(s, len);
    }
    uint64_t x = ld64(s);
    uint64_t y = ld64(s + len - 16) ^ K1;
    uint64_t z = ld64(s + len - 56) ^ K0;
    u64pair v = weak_hash_32_seeds(s + len - 64, len, y);
    u64pair w = weak_hash_32_seeds(s + len - 32, len * K1, K0);
    z += shift_mix(v.second) * K1;
    x = rotr(z + x, 39) * K1;
    y = rotr(y, 33) * K1;
    len = (len - 1) & ~(size_t)63;
    do {
        x = rotr(x + y + v.first + ld64(s + 16), 37) * K1;
        y = rotr(y + v.second + ld64(s + 48), 42) * K1;
        x ^= w.second;
        y ^= v.first;
        z = rotr(z ^ w.first, 33);
        v = weak_hash_32_seeds(s, v.second * K1, x + w.first);
        w = weak_hash_32_seeds(s + 32, z + w.second, y);
        uint64_t t = z; z = x; x = t;
        s += 64;
        len -= 64;
    } while (len != 0);
    return hash128to64(hash128to64(v.first, w.first) + shift_mix(y) * K1 + z,
                       hash128to64(v.second, w.second) + x);
}

uint32_t cbo_cat_feature_hash(const char* s, size_t len) {
    return (uint32_t)(cbo_city_hash64(s, len) & 0xffffffffULL);
}

int32_t cbo_integer_cat_feature_hash(long long v) {
    char buf[32];
    int n = snprintf(buf, sizeof(buf), "%lld", v);
    uint32_t h = cbo_cat_feature_hash(buf, (size_t)n);
    int32_t r;
    memcpy(&r, &h, 4);
    return r;
}

/* ------------------------------------------------------------------------ model -------- */

typedef struct { uint16_t feature_index; uint8_t xor_mask; uint8_t split_idx; } cbo_repacked_bin;

/* one entry per binary feature (TModelSplit), in CalcBinFeatures order */
typedef struct {
    int32_t is_onehot;
    int32_t is_ctr;
    int32_t feature;   /* index into float features / one-hot features / CTR features of the model */
    float border;
    int32_t value;
} cbo_bin_feature;

/* a bin of the quantized block that a CTR projection looks at (TBinFeatureIndexValue, ctr_provider.h:80-92) */
typedef struct {
    uint32_t bin_index;
    int32_t check_value_equal;
    uint8_t value;
} cbo_bin_index_value;

struct cbo_model {
    int32_t approx_dim, n_trees, n_tree_splits, n_float, n_cat, n_onehot, n_step_nodes;
    int32_t *tree_sizes, *tree_start_offsets, *tree_splits;
    int32_t *ff_index, *ff_flat_index, *ff_has_nans, *ff_nan_treatment, *ff_border_offsets;
    float* ff_borders;
    int32_t *cf_index, *cf_flat_index, *cf_used;
    int32_t *oh_cat_index, *oh_value_offsets, *oh_values;
    uint64_t n_leaf_values;
    double* leaf_values;
    uint16_t* step_nodes;
    uint32_t* node_id_to_leaf_id;
    double scale;
    double* bias;
    /* derived */
    int32_t oblivious;
    int32_t bucket_count;
    int32_t n_bin_features;
    cbo_bin_feature* bin_features;
    cbo_repacked_bin* repacked;
    uint64_t* first_leaf_offsets;
    int32_t used_float, used_cat;
    size_t min_float_size, min_cat_size, flat_expected;
    int32_t* oh_packed_cat; /* per one-hot feature: packed index among used cat features */
    int32_t has_onehot;
    /* CTR features and their tables */
    int32_t n_ctr, n_ctr_tables;
    int32_t *ctr_border_offsets, *ctr_cat_offsets, *ctr_cats, *ctr_float_offsets, *ctr_float_feature;
    int32_t *ctr_onehot_offsets, *ctr_onehot_cat, *ctr_onehot_value, *ctr_type, *ctr_target_border_idx, *ctr_table;
    float *ctr_borders, *ctr_float_border, *ctr_prior_num, *ctr_prior_denom, *ctr_shift, *ctr_scale;
    uint64_t *table_bucket_offsets, *table_blob_offsets;
    uint8_t *table_buckets, *table_blobs;
    int32_t *table_counter_denominator, *table_target_classes_count;
    /* derived, TStaticCtrProvider::SetupBinFeatureIndexes (static_ctr_provider.cpp:142-178) */
    int32_t* ctr_packed_cats;             /* per projection cat feature: row of the transposed hashes */
    cbo_bin_index_value* ctr_bin_indexes; /* per projection float split, then per one-hot split */
    int32_t *ctr_float_raw, *ctr_onehot_raw; /* position of the split's feature in the model's lists */
};

static void* dup_mem(const void* p, size_t n) {
    void* r = malloc(n ? n : 1);
    if (n && p) memcpy(r, p, n);
    return r;
}

void cbo_model_free(cbo_model* m) {
    if (!m) return;
    free(m->tree_sizes); free(m->tree_start_offsets); free(m->tree_splits);
    free(m->ff_index); free(m->ff_flat_index); free(m->ff_has_nans); free(m->ff_nan_treatment);
    free(m->ff_border_offsets); free(m->ff_borders);
    free(m->cf_index); free(m->cf_flat_index); free(m->cf_used);
    free(m->oh_cat_index); free(m->oh_value_offsets); free(m->oh_values);
    free(m->leaf_values); free(m->step_nodes); free(m->node_id_to_leaf_id); free(m->bias);
    free(m->bin_features); free(m->repacked); free(m->first_leaf_offsets); free(m->oh_packed_cat);
    free(m->ctr_border_offsets); free(m->ctr_cat_offsets); free(m->ctr_cats); free(m->ctr_float_offsets);
    free(m->ctr_float_feature); free(m->ctr_onehot_offsets); free(m->ctr_onehot_cat); free(m->ctr_onehot_value);
    free(m->ctr_type); free(m->ctr_target_border_idx); free(m->ctr_table); free(m->ctr_borders);
    free(m->ctr_float_border); free(m->ctr_prior_num); free(m->ctr_prior_denom); free(m->ctr_shift);
    free(m->ctr_scale); free(m->table_bucket_offsets); free(m->table_blob_offsets); free(m->table_buckets);
    free(m->table_blobs); free(m->table_counter_denominator); free(m->table_target_classes_count);
    free(m->ctr_packed_cats); free(m->ctr_bin_indexes); free(m->ctr_float_raw); free(m->ctr_onehot_raw);
    free(m);
}

#define FAIL(...) do { if (err) snprintf(err, err_len, __VA_ARGS__); cbo_model_free(m); return NULL; } while (0)

cbo_model* cbo_model_create(const cbo_model_desc* d, char* err, size_t err_len) {
    cbo_model* m = (cbo_model*)calloc(1, sizeof(cbo_model));
    m->approx_dim = d->approx_dim;
    m->n_trees = d->n_trees;
    m->n_tree_splits = d->n_tree_splits;
    m->n_float = d->n_float;
    m->n_cat = d->n_cat;
    m->n_onehot = d->n_onehot;
    m->n_step_nodes = d->n_step_nodes;
    m->n_leaf_values = d->n_leaf_values;
    m->scale = d->scale;
    m->tree_sizes = dup_mem(d->tree_sizes, sizeof(int32_t) * d->n_trees);
    m->tree_start_offsets = dup_mem(d->tree_start_offsets, sizeof(int32_t) * d->n_trees);
    m->tree_splits = dup_mem(d->tree_splits, sizeof(int32_t) * d->n_tree_splits);
    m->ff_index = dup_mem(d->ff_index, sizeof(int32_t) * d->n_float);
    m->ff_flat_index = dup_mem(d->ff_flat_index, sizeof(int32_t) * d->n_float);
    m->ff_has_nans = dup_mem(d->ff_has_nans, sizeof(int32_t) * d->n_float);
    m->ff_nan_treatment = dup_mem(d->ff_nan_treatment, sizeof(int32_t) * d->n_float);
    m->ff_border_offsets = dup_mem(d->ff_border_offsets, sizeof(int32_t) * (d->n_float + 1));
    int32_t n_borders = d->n_float ? d->ff_border_offsets[d->n_float] : 0;
    m->ff_borders = dup_mem(d->ff_borders, sizeof(float) * n_borders);
    m->cf_index = dup_mem(d->cf_index, sizeof(int32_t) * d->n_cat);
    m->cf_flat_index = dup_mem(d->cf_flat_index, sizeof(int32_t) * d->n_cat);
    m->cf_used = dup_mem(d->cf_used, sizeof(int32_t) * d->n_cat);
    m->oh_cat_index = dup_mem(d->oh_cat_index, sizeof(int32_t) * d->n_onehot);
    m->oh_value_offsets = dup_mem(d->oh_value_offsets, sizeof(int32_t) * (d->n_onehot + 1));
    int32_t n_values = d->n_onehot ? d->oh_value_offsets[d->n_onehot] : 0;
    m->oh_values = dup_mem(d->oh_values, sizeof(int32_t) * n_values);
    m->leaf_values = dup_mem(d->leaf_values, sizeof(double) * d->n_leaf_values);
    m->step_nodes = dup_mem(d->step_nodes, sizeof(uint16_t) * 2 * d->n_step_nodes);
    m->node_id_to_leaf_id = dup_mem(d->node_id_to_leaf_id, sizeof(uint32_t) * d->n_step_nodes);
    m->bias = dup_mem(d->bias, sizeof(double) * d->approx_dim);
    m->has_onehot = d->n_onehot > 0;
    m->n_ctr = d->n_ctr;
    m->n_ctr_tables = d->n_ctr_tables;
    int32_t n_ctr_borders = 0;
    if (d->n_ctr > 0) {
        const int n = d->n_ctr;
        m->ctr_border_offsets = dup_mem(d->ctr_border_offsets, sizeof(int32_t) * (n + 1));
        m->ctr_cat_offsets = dup_mem(d->ctr_cat_offsets, sizeof(int32_t) * (n + 1));
        m->ctr_float_offsets = dup_mem(d->ctr_float_offsets, sizeof(int32_t) * (n + 1));
        m->ctr_onehot_offsets = dup_mem(d->ctr_onehot_offsets, sizeof(int32_t) * (n + 1));
        n_ctr_borders = d->ctr_border_offsets[n];
        m->ctr_borders = dup_mem(d->ctr_borders, sizeof(float) * n_ctr_borders);
        m->ctr_cats = dup_mem(d->ctr_cats, sizeof(int32_t) * d->ctr_cat_offsets[n]);
        m->ctr_float_feature = dup_mem(d->ctr_float_feature, sizeof(int32_t) * d->ctr_float_offsets[n]);
        m->ctr_float_border = dup_mem(d->ctr_float_border, sizeof(float) * d->ctr_float_offsets[n]);
        m->ctr_onehot_cat = dup_mem(d->ctr_onehot_cat, sizeof(int32_t) * d->ctr_onehot_offsets[n]);
        m->ctr_onehot_value = dup_mem(d->ctr_onehot_value, sizeof(int32_t) * d->ctr_onehot_offsets[n]);
        m->ctr_type = dup_mem(d->ctr_type, sizeof(int32_t) * n);
        m->ctr_target_border_idx = dup_mem(d->ctr_target_border_idx, sizeof(int32_t) * n);
        m->ctr_prior_num = dup_mem(d->ctr_prior_num, sizeof(float) * n);
        m->ctr_prior_denom = dup_mem(d->ctr_prior_denom, sizeof(float) * n);
        m->ctr_shift = dup_mem(d->ctr_shift, sizeof(float) * n);
        m->ctr_scale = dup_mem(d->ctr_scale, sizeof(float) * n);
        m->ctr_table = dup_mem(d->ctr_table, sizeof(int32_t) * n);
        const int nt = d->n_ctr_tables;
        m->table_bucket_offsets = dup_mem(d->table_bucket_offsets, sizeof(uint64_t) * (nt + 1));
        m->table_blob_offsets = dup_mem(d->table_blob_offsets, sizeof(uint64_t) * (nt + 1));
        m->table_buckets = dup_mem(d->table_buckets, 12 * (size_t)d->table_bucket_offsets[nt]);
        m->table_blobs = dup_mem(d->table_blobs, (size_t)d->table_blob_offsets[nt]);
        m->table_counter_denominator = dup_mem(d->table_counter_denominator, sizeof(int32_t) * nt);
        m->table_target_classes_count = dup_mem(d->table_target_classes_count, sizeof(int32_t) * nt);
    }
    /* IsOblivious, model.h:271-273 */
    m->oblivious = (d->n_step_nodes == 0);

    if (d->approx_dim < 1) FAIL("approx dimension must be positive");

    /* used-feature statistics, model.cpp:431-449 */
    for (int i = 0; i < m->n_float; ++i) {
        if (m->ff_border_offsets[i + 1] > m->ff_border_offsets[i]) {
            ++m->used_float;
            m->min_float_size = (size_t)m->ff_index[i] + 1;
        }
    }
    for (int i = 0; i < m->n_cat; ++i) {
        if (m->cf_used[i]) {
            ++m->used_cat;
            m->min_cat_size = (size_t)m->cf_index[i] + 1;
        }
    }
    /* GetFlatFeatureVectorExpectedSize, model.h:534-541 */
    m->flat_expected = 0;
    if (m->n_cat && (size_t)(m->cf_flat_index[m->n_cat - 1] + 1) > m->flat_expected)
        m->flat_expected = (size_t)(m->cf_flat_index[m->n_cat - 1] + 1);
    if (m->n_float && (size_t)(m->ff_flat_index[m->n_float - 1] + 1) > m->flat_expected)
        m->flat_expected = (size_t)(m->ff_flat_index[m->n_float - 1] + 1);

    /* CalcBinFeatures, model.cpp:471-577 */
    int32_t total = n_borders + n_values + n_ctr_borders;
    m->bin_features = (cbo_bin_feature*)calloc(total ? total : 1, sizeof(cbo_bin_feature));
    uint32_t* split_bucket = (uint32_t*)calloc(total ? total : 1, sizeof(uint32_t));
    uint32_t* split_idx = (uint32_t*)calloc(total ? total : 1, sizeof(uint32_t));
    int32_t nb = 0;
    uint32_t buckets = 0;
    for (int i = 0; i < m->n_float; ++i) {
        int32_t cnt = m->ff_border_offsets[i + 1] - m->ff_border_offsets[i];
        if (cnt == 0) continue;
        for (int b = 0; b < cnt; ++b) {
            m->bin_features[nb].is_onehot = 0;
            m->bin_features[nb].feature = i;
            m->bin_features[nb].border = m->ff_borders[m->ff_border_offsets[i] + b];
            split_bucket[nb] = buckets + b / CBO_MAX_VALUES_PER_BIN;
            split_idx[nb] = (b % CBO_MAX_VALUES_PER_BIN) + 1;
            ++nb;
        }
        buckets += (cnt + CBO_MAX_VALUES_PER_BIN - 1) / CBO_MAX_VALUES_PER_BIN;
    }
    for (int i = 0; i < m->n_onehot; ++i) {
        int32_t cnt = m->oh_value_offsets[i + 1] - m->oh_value_offsets[i];
        for (int v = 0; v < cnt; ++v) {
            m->bin_features[nb].is_onehot = 1;
            m->bin_features[nb].feature = i;
            m->bin_features[nb].value = m->oh_values[m->oh_value_offsets[i] + v];
            split_bucket[nb] = buckets + v / CBO_MAX_VALUES_PER_BIN;
            split_idx[nb] = (v % CBO_MAX_VALUES_PER_BIN) + 1;
            ++nb;
        }
        buckets += (cnt + CBO_MAX_VALUES_PER_BIN - 1) / CBO_MAX_VALUES_PER_BIN;
    }
    for (int i = 0; i < m->n_ctr; ++i) {
        int32_t cnt = m->ctr_border_offsets[i + 1] - m->ctr_border_offsets[i];
        for (int b = 0; b < cnt; ++b) {
            m->bin_features[nb].is_ctr = 1;
            m->bin_features[nb].feature = i;
            m->bin_features[nb].border = m->ctr_borders[m->ctr_border_offsets[i] + b];
            split_bucket[nb] = buckets + b / CBO_MAX_VALUES_PER_BIN;
            split_idx[nb] = (b % CBO_MAX_VALUES_PER_BIN) + 1;
            ++nb;
        }
        buckets += (cnt + CBO_MAX_VALUES_PER_BIN - 1) / CBO_MAX_VALUES_PER_BIN;
    }
    m->n_bin_features = nb;
    m->bucket_count = (int32_t)buckets;

    m->repacked = (cbo_repacked_bin*)calloc(m->n_tree_splits ? m->n_tree_splits : 1, sizeof(cbo_repacked_bin));
    if (nb == 0 && m->n_tree_splits > 0) {
        /* trees without conditions: only valid for non-symmetric models, model.cpp:545-556 */
        for (int i = 0; i < m->n_tree_splits; ++i) {
            if (m->tree_splits[i] != 0) { free(split_bucket); free(split_idx); FAIL("expected 0 as empty nodes marker"); }
        }
        if (m->oblivious) { free(split_bucket); free(split_idx); FAIL("split ids present but there are no splits in the model"); }
    } else {
        for (int i = 0; i < m->n_tree_splits; ++i) {
            int32_t s = m->tree_splits[i];
            if (s < 0 || s >= nb) { free(split_bucket); free(split_idx); FAIL("tree split %d out of range", s); }
            if (split_bucket[s] > 0xffff) { free(split_bucket); free(split_idx); FAIL("too many features in model"); }
            m->repacked[i].feature_index = (uint16_t)split_bucket[s];
            if (!m->bin_features[s].is_onehot) {
                m->repacked[i].split_idx = (uint8_t)split_idx[s];
                m->repacked[i].xor_mask = 0;
            } else {
                m->repacked[i].xor_mask = (uint8_t)((~split_idx[s]) & 0xff);
                m->repacked[i].split_idx = 0xff;
            }
        }
    }
    free(split_bucket);
    free(split_idx);

    /* CalcFirstLeafOffsets, model.cpp:586-624 */
    m->first_leaf_offsets = (uint64_t*)calloc(m->n_trees ? m->n_trees : 1, sizeof(uint64_t));
    if (m->oblivious) {
        uint64_t cur = 0;
        for (int t = 0; t < m->n_trees; ++t) {
            m->first_leaf_offsets[t] = cur;
            cur += ((uint64_t)1 << m->tree_sizes[t]) * (uint64_t)m->approx_dim;
        }
        if (cur > m->n_leaf_values) FAIL("leaf values vector too short");
    } else {
        for (int t = 0; t < m->n_trees; ++t) {
            int32_t b = m->tree_start_offsets[t], e = b + m->tree_sizes[t];
            uint32_t mn = 0xffffffffu;
            if (e > m->n_step_nodes) FAIL("tree nodes out of range");
            for (int n = b; n < e; ++n) {
                if (m->step_nodes[2 * n] == 0 || m->step_nodes[2 * n + 1] == 0) {
                    uint32_t li = m->node_id_to_leaf_id[n];
                    if (li % (uint32_t)m->approx_dim != 0) FAIL("expect that leaf values are aligned");
                    if (li < mn) mn = li;
                }
            }
            m->first_leaf_offsets[t] = mn;
        }
    }

    /* packed cat indexes, quantization.h:277-296 */
    m->oh_packed_cat = (int32_t*)calloc(m->n_onehot ? m->n_onehot : 1, sizeof(int32_t));
    for (int i = 0; i < m->n_onehot; ++i) {
        int32_t packed = 0, found = -1;
        for (int c = 0; c < m->n_cat; ++c) {
            if (!m->cf_used[c]) continue;
            if (m->cf_index[c] == m->oh_cat_index[i]) found = packed;
            ++packed;
        }
        if (found < 0) FAIL("one-hot feature refers to an unused categorical feature");
        m->oh_packed_cat[i] = found;
    }

    /* TStaticCtrProvider::SetupBinFeatureIndexes, static_ctr_provider.cpp:142-178: where a projection's
     * splits sit in the quantized block, and which row of the transposed hashes a cat feature is */
    if (m->n_ctr > 0) {
        const int n = m->n_ctr;
        const int32_t nc = m->ctr_cat_offsets[n], nf = m->ctr_float_offsets[n], no = m->ctr_onehot_offsets[n];
        m->ctr_packed_cats = (int32_t*)calloc(nc ? nc : 1, sizeof(int32_t));
        m->ctr_bin_indexes = (cbo_bin_index_value*)calloc((nf + no) ? (nf + no) : 1, sizeof(cbo_bin_index_value));
        m->ctr_float_raw = (int32_t*)calloc(nf ? nf : 1, sizeof(int32_t));
        m->ctr_onehot_raw = (int32_t*)calloc(no ? no : 1, sizeof(int32_t));
        for (int i = 0; i < nc; ++i) {
            int32_t packed = 0, found = -1;
            for (int c = 0; c < m->n_cat; ++c) {
                if (!m->cf_used[c]) continue;
                if (m->cf_index[c] == m->ctr_cats[i]) found = packed;
                ++packed;
            }
            if (found < 0) FAIL("CTR projection refers to an unused categorical feature");
            m->ctr_packed_cats[i] = found;
        }
        for (int i = 0; i < nf; ++i) {
            uint32_t current = 0;
            int found = 0;
            for (int ff = 0; ff < m->n_float && !found; ++ff) {
                const int32_t b0 = m->ff_border_offsets[ff], b1 = m->ff_border_offsets[ff + 1];
                if (b1 == b0) continue;
                if (m->ff_index[ff] == m->ctr_float_feature[i]) {
                    for (int32_t b = b0; b < b1; ++b) {
                        if (m->ff_borders[b] == m->ctr_float_border[i]) {
                            m->ctr_bin_indexes[i].bin_index = current + (uint32_t)(b - b0) / CBO_MAX_VALUES_PER_BIN;
                            m->ctr_bin_indexes[i].check_value_equal = 0;
                            m->ctr_bin_indexes[i].value = (uint8_t)((b - b0) % CBO_MAX_VALUES_PER_BIN + 1);
                            m->ctr_float_raw[i] = ff;
                            found = 1;
                            break;
                        }
                    }
                }
                current += (uint32_t)(b1 - b0 + CBO_MAX_VALUES_PER_BIN - 1) / CBO_MAX_VALUES_PER_BIN;
            }
            if (!found) FAIL("CTR projection refers to a float split the model does not have");
        }
        uint32_t float_buckets = 0;
        for (int ff = 0; ff < m->n_float; ++ff)
            float_buckets += (uint32_t)(m->ff_border_offsets[ff + 1] - m->ff_border_offsets[ff] + CBO_MAX_VALUES_PER_BIN - 1) /
                             CBO_MAX_VALUES_PER_BIN;
        for (int i = 0; i < no; ++i) {
            uint32_t current = float_buckets;
            int found = 0;
            for (int oh = 0; oh < m->n_onehot && !found; ++oh) {
                const int32_t v0 = m->oh_value_offsets[oh], v1 = m->oh_value_offsets[oh + 1];
                if (m->oh_cat_index[oh] == m->ctr_onehot_cat[i]) {
                    for (int32_t v = v0; v < v1; ++v) {
                        if (m->oh_values[v] == m->ctr_onehot_value[i]) {
                            m->ctr_bin_indexes[nf + i].bin_index = current + (uint32_t)(v - v0) / CBO_MAX_VALUES_PER_BIN;
                            m->ctr_bin_indexes[nf + i].check_value_equal = 1;
                            m->ctr_bin_indexes[nf + i].value = (uint8_t)((v - v0) % CBO_MAX_VALUES_PER_BIN + 1);
                            m->ctr_onehot_raw[i] = oh;
                            found = 1;
                            break;
                        }
                    }
                }
                current += (uint32_t)(v1 - v0 + CBO_MAX_VALUES_PER_BIN - 1) / CBO_MAX_VALUES_PER_BIN;
            }
            if (!found) FAIL("CTR projection refers to a one-hot split the model does not have");
        }
        for (int i = 0; i < n; ++i) {
            const int32_t t = m->ctr_table[i];
            if (t < 0 || t >= m->n_ctr_tables) FAIL("CTR feature without a value table");
            const uint64_t buckets_in_table = m->table_bucket_offsets[t + 1] - m->table_bucket_offsets[t];
            if (buckets_in_table == 0 || (buckets_in_table & (buckets_in_table - 1)) != 0)
                FAIL("dense hash view must have 2^k buckets");
        }
    }
    return m;
}

int32_t cbo_bucket_count(const cbo_model* m) { return m->bucket_count; }
int32_t cbo_is_oblivious(const cbo_model* m) { return m->oblivious; }
int32_t cbo_tree_count(const cbo_model* m) { return m->n_trees; }
int32_t cbo_approx_dim(const cbo_model* m) { return m->approx_dim; }
size_t cbo_flat_vector_expected_size(const cbo_model* m) { return m->flat_expected; }
size_t cbo_min_float_vector_size(const cbo_model* m) { return m->min_float_size; }
size_t cbo_min_cat_vector_size(const cbo_model* m) { return m->min_cat_size; }
size_t cbo_used_cat_count(const cbo_model* m) { return (size_t)m->used_cat; }

void cbo_repacked_bins(const cbo_model* m, uint32_t* out) {
    for (int i = 0; i < m->n_tree_splits; ++i) {
        out[i] = (uint32_t)m->repacked[i].feature_index | ((uint32_t)m->repacked[i].xor_mask << 16) |
                 ((uint32_t)m->repacked[i].split_idx << 24);
    }
}
void cbo_first_leaf_offsets(const cbo_model* m, uint64_t* out) {
    memcpy(out, m->first_leaf_offsets, sizeof(uint64_t) * m->n_trees);
}

/* --------------------------------------------------------------------- accessors -------- */

static inline float get_float(const cbo_model* m, const cbo_features* f, int feat, size_t doc) {
    switch (f->layout) {
        case 0: return f->floats[doc * f->stride + (size_t)m->ff_flat_index[feat]];
        case 1: return f->floats[(size_t)m->ff_flat_index[feat] * f->stride + doc];
        default: return f->floats[doc * f->stride + (size_t)m->ff_index[feat]];
    }
}

/* hashed categorical value; flat layouts bit-cast the float slot (cat_feature.h:19-21) */
static inline uint32_t get_cat(const cbo_model* m, const cbo_features* f, int cat, size_t doc) {
    float v;
    uint32_t u;
    switch (f->layout) {
        case 0: v = f->floats[doc * f->stride + (size_t)m->cf_flat_index[cat]]; memcpy(&u, &v, 4); return u;
        case 1: v = f->floats[(size_t)m->cf_flat_index[cat] * f->stride + doc]; memcpy(&u, &v, 4); return u;
        default: return (uint32_t)f->cats[doc * f->cat_stride + (size_t)m->cf_index[cat]];
    }
}

/* -------------------------------------------------------------------------- CTRs -------- */

/* CalcHash, catboost/libs/model/hash.h:11-14 */
static inline uint64_t ctr_calc_hash(uint64_t a, uint64_t b) {
    const uint64_t magic = 0x4906ba494954cb65ULL;
    return magic * (a + magic * b);
}

/* TDenseIndexHashView::GetIndex, catboost/libs/helpers/dense_hash_view.h:46-56 */
#define CBO_NOT_FOUND 0xffffffffu
static uint32_t ctr_table_index(const cbo_model* m, int table, uint64_t hash) {
    const uint8_t* buckets = m->table_buckets + 12 * (size_t)m->table_bucket_offsets[table];
    const uint64_t mask = m->table_bucket_offsets[table + 1] - m->table_bucket_offsets[table] - 1;
    for (uint64_t zz = hash & mask;; zz = (zz + 1) & mask) {
        uint64_t h;
        memcpy(&h, buckets + 12 * zz, 8);
        if (h == 0xffffffffffffffffULL) return CBO_NOT_FOUND;
        if (h == hash) {
            uint32_t v;
            memcpy(&v, buckets + 12 * zz + 8, 4);
            return v;
        }
    }
}

/* TModelCtr::Calc, online_ctr.h:290-293 */
static inline float ctr_calc(const cbo_model* m, int ctr, float count_in_class, float total_count) {
    float v = (count_in_class + m->ctr_prior_num[ctr]) / (total_count + m->ctr_prior_denom[ctr]);
    return (v + m->ctr_shift[ctr]) * m->ctr_scale[ctr];
}

/* The value of CTR `ctr` for a row of its table (or CBO_NOT_FOUND): the per-type branches of
 * TStaticCtrProvider::CalcCtrs, static_ctr_provider.cpp:52-126. */
static float ctr_value(const cbo_model* m, int ctr, uint32_t row) {
    const int table = m->ctr_table[ctr];
    const uint8_t* blob = m->table_blobs + m->table_blob_offsets[table];
    const int type = m->ctr_type[ctr];
    if (type == 2 || type == 3) { /* BinarizedTargetMeanValue, FloatTargetMeanValue: {float Sum; int Count} */
        if (row == CBO_NOT_FOUND) return ctr_calc(m, ctr, 0.f, 0.f);
        float sum;
        int32_t count;
        memcpy(&sum, blob + 8 * (size_t)row, 4);
        memcpy(&count, blob + 8 * (size_t)row + 4, 4);
        return ctr_calc(m, ctr, sum, (float)count);
    }
    const int32_t* ints = (const int32_t*)blob;
    if (type == 4 || type == 5) { /* Counter, FeatureFreq */
        const int32_t denominator = m->table_counter_denominator[table];
        if (row == CBO_NOT_FOUND) return ctr_calc(m, ctr, 0.f, (float)denominator);
        return ctr_calc(m, ctr, (float)ints[row], (float)denominator);
    }
    const int32_t classes = m->table_target_classes_count[table];
    const int32_t target_border = m->ctr_target_border_idx[ctr];
    if (type == 1) { /* Buckets */
        if (row == CBO_NOT_FOUND) return ctr_calc(m, ctr, 0.f, 0.f);
        const int32_t* history = ints + (size_t)row * (size_t)classes;
        int32_t good = history[target_border], total = 0;
        for (int32_t c = 0; c < classes; ++c) total += history[c];
        return ctr_calc(m, ctr, (float)good, (float)total);
    }
    /* Borders */
    if (classes > 2) {
        int32_t good = 0, total = 0;
        if (row != CBO_NOT_FOUND) {
            const int32_t* history = ints + (size_t)row * (size_t)classes;
            for (int32_t c = 0; c < target_border + 1; ++c) total += history[c];
            for (int32_t c = target_border + 1; c < classes; ++c) good += history[c];
            total += good;
        }
        return ctr_calc(m, ctr, (float)good, (float)total);
    }
    if (row == CBO_NOT_FOUND) return ctr_calc(m, ctr, 0.f, 0.f);
    const int32_t* history = ints + 2 * (size_t)row;
    return ctr_calc(m, ctr, (float)history[1], (float)(history[0] + history[1]));
}

/* CalcCtrs over one quantized block (static_ctr_provider.cpp:14-131, CalcHashes of ctr_provider.h:94-123):
 * bins = [bucket][doc_count] of the float and one-hot features, hashes = [used cat][doc_count];
 * ctrs = [ctr][doc_count]. Consecutive CTRs with one projection share their hashes in the reference; the
 * hash does not depend on that, so every CTR computes its own here. */
static void calc_ctrs_block(const cbo_model* m, const uint8_t* bins, const uint32_t* transposed_hash,
                            size_t doc_count, float* ctrs) {
    uint64_t hashes[CBO_BLOCK];
    const int32_t nf_all = m->ctr_float_offsets[m->n_ctr];
    for (int ctr = 0; ctr < m->n_ctr; ++ctr) {
        for (size_t d = 0; d < doc_count; ++d) hashes[d] = 0;
        for (int32_t i = m->ctr_cat_offsets[ctr]; i < m->ctr_cat_offsets[ctr + 1]; ++i) {
            const uint32_t* vals = transposed_hash + (size_t)m->ctr_packed_cats[i] * doc_count;
            for (size_t d = 0; d < doc_count; ++d)
                hashes[d] = ctr_calc_hash(hashes[d], (uint64_t)(int64_t)(int32_t)vals[d]);
        }
        for (int pass = 0; pass < 2; ++pass) {
            const int32_t b = pass == 0 ? m->ctr_float_offsets[ctr] : nf_all + m->ctr_onehot_offsets[ctr];
            const int32_t e = pass == 0 ? m->ctr_float_offsets[ctr + 1] : nf_all + m->ctr_onehot_offsets[ctr + 1];
            for (int32_t i = b; i < e; ++i) {
                const cbo_bin_index_value* bi = &m->ctr_bin_indexes[i];
                const uint8_t* col = bins + (size_t)bi->bin_index * doc_count;
                if (!bi->check_value_equal) {
                    for (size_t d = 0; d < doc_count; ++d)
                        hashes[d] = ctr_calc_hash(hashes[d], (uint64_t)(col[d] >= bi->value));
                } else {
                    for (size_t d = 0; d < doc_count; ++d)
                        hashes[d] = ctr_calc_hash(hashes[d], (uint64_t)(col[d] == bi->value));
                }
            }
        }
        for (size_t d = 0; d < doc_count; ++d)
            ctrs[(size_t)ctr * doc_count + d] = ctr_value(m, ctr, ctr_table_index(m, m->ctr_table[ctr], hashes[d]));
    }
}

/* ---------------------------------------------------------------------- binarize -------- */

/* One block of <= 128 docs; result is [bucket][doc_count] (quantization.h:333-529). */
static void binarize_block(const cbo_model* m, const cbo_features* f, size_t start, size_t doc_count,
                           uint8_t* result, uint32_t* transposed_hash) {
    float vals[CBO_BLOCK];
    memset(result, 0, (size_t)m->bucket_count * doc_count);
    uint8_t* out = result;
    for (int i = 0; i < m->n_float; ++i) {
        const int32_t b0 = m->ff_border_offsets[i], b1 = m->ff_border_offsets[i + 1];
        if (b1 == b0) continue; /* !UsedInModel, quantization.h:368-370 */
        const int substitute = m->ff_has_nans[i] && m->ff_nan_treatment[i] != CBO_NAN_AS_IS;
        const float subst = (m->ff_nan_treatment[i] == CBO_NAN_AS_FALSE) ? -INFINITY : INFINITY;
        for (size_t d = 0; d < doc_count; ++d) {
            float v = get_float(m, f, i, start + d);
            if (substitute && isnan(v)) v = subst;
            vals[d] = v;
        }
        for (int32_t bs = b0; bs < b1; bs += CBO_MAX_VALUES_PER_BIN) {
            const int32_t be = (bs + CBO_MAX_VALUES_PER_BIN < b1) ? bs + CBO_MAX_VALUES_PER_BIN : b1;
            for (int32_t b = bs; b < be; ++b) {
                const float border = m->ff_borders[b];
                for (size_t d = 0; d < doc_count; ++d) out[d] += (uint8_t)(vals[d] > border);
            }
            out += doc_count;
        }
    }
    if (m->used_cat != 0) {
        /* ComputeOneHotAndCtrFeaturesForBlock, quantization.h:263-327 */
        int packed = 0;
        for (int c = 0; c < m->n_cat; ++c) {
            if (!m->cf_used[c]) continue;
            for (size_t d = 0; d < doc_count; ++d)
                transposed_hash[(size_t)packed * doc_count + d] = get_cat(m, f, c, start + d);
            ++packed;
        }
        /* OneHotBinsFromTransposedCatFeatures, quantization.h:54-79 */
        for (int i = 0; i < m->n_onehot; ++i) {
            const int32_t v0 = m->oh_value_offsets[i], v1 = m->oh_value_offsets[i + 1];
            const uint32_t* hashes = transposed_hash + (size_t)m->oh_packed_cat[i] * doc_count;
            for (size_t d = 0; d < doc_count; ++d) {
                int32_t val;
                memcpy(&val, &hashes[d], 4);
                uint8_t* wp = out + d;
                for (int32_t bs = v0; bs < v1; bs += CBO_MAX_VALUES_PER_BIN) {
                    const int32_t be = (bs + CBO_MAX_VALUES_PER_BIN < v1) ? bs + CBO_MAX_VALUES_PER_BIN : v1;
                    for (int32_t b = bs; b < be; ++b)
                        *wp |= (uint8_t)((uint8_t)(val == m->oh_values[b]) * (uint8_t)(b - bs + 1));
                    wp += doc_count;
                }
            }
            out += doc_count * (size_t)((v1 - v0 + CBO_MAX_VALUES_PER_BIN - 1) / CBO_MAX_VALUES_PER_BIN);
        }
        if (m->n_ctr > 0) {
            /* quantization.h:304-325: CTR values of the block, binarized like float features without
             * a NaN policy */
            float* ctrs = (float*)malloc(sizeof(float) * (size_t)m->n_ctr * doc_count);
            calc_ctrs_block(m, result, transposed_hash, doc_count, ctrs);
            for (int i = 0; i < m->n_ctr; ++i) {
                const float* v = ctrs + (size_t)i * doc_count;
                const int32_t b0 = m->ctr_border_offsets[i], b1 = m->ctr_border_offsets[i + 1];
                for (int32_t bs = b0; bs < b1; bs += CBO_MAX_VALUES_PER_BIN) {
                    const int32_t be = (bs + CBO_MAX_VALUES_PER_BIN < b1) ? bs + CBO_MAX_VALUES_PER_BIN : b1;
                    for (int32_t b = bs; b < be; ++b) {
                        const float border = m->ctr_borders[b];
                        for (size_t d = 0; d < doc_count; ++d) out[d] += (uint8_t)(v[d] > border);
                    }
                    out += doc_count;
                }
            }
            free(ctrs);
        }
    }
}

void cbo_calc_ctrs(const cbo_model* m, const cbo_features* f, size_t n_docs, float* out) {
    if (m->n_ctr == 0) return;
    uint8_t* bins = (uint8_t*)malloc((size_t)(m->bucket_count ? m->bucket_count : 1) * CBO_BLOCK);
    uint32_t* th = (uint32_t*)malloc(sizeof(uint32_t) * CBO_BLOCK * (size_t)(m->used_cat ? m->used_cat : 1));
    float* ctrs = (float*)malloc(sizeof(float) * (size_t)m->n_ctr * CBO_BLOCK);
    for (size_t start = 0; start < n_docs; start += CBO_BLOCK) {
        const size_t dc = n_docs - start < CBO_BLOCK ? n_docs - start : CBO_BLOCK;
        binarize_block(m, f, start, dc, bins, th);
        calc_ctrs_block(m, bins, th, dc, ctrs);
        for (int i = 0; i < m->n_ctr; ++i)
            for (size_t d = 0; d < dc; ++d) out[(size_t)i * n_docs + start + d] = ctrs[(size_t)i * dc + d];
    }
    free(bins); free(th); free(ctrs);
}

void cbo_binarize(const cbo_model* m, const cbo_features* f, size_t n_docs, uint8_t* bins) {
    uint32_t* th = (uint32_t*)malloc(sizeof(uint32_t) * CBO_BLOCK * (size_t)(m->used_cat ? m->used_cat : 1));
    for (size_t start = 0; start < n_docs; start += CBO_BLOCK) {
        size_t dc = n_docs - start < CBO_BLOCK ? n_docs - start : CBO_BLOCK;
        binarize_block(m, f, start, dc, bins + start * (size_t)m->bucket_count, th);
    }
    free(th);
}

/* ------------------------------------------------------------------------- trees -------- */

/* CalcIndexesBasic, evaluator_impl.cpp:16-52: bit `depth` <- split `depth` of the tree. */
static void calc_indexes_oblivious(const cbo_model* m, const uint8_t* bins, size_t dc, int tree, uint32_t* idx) {
    const cbo_repacked_bin* sp = m->repacked + m->tree_start_offsets[tree];
    const int depth_n = m->tree_sizes[tree];
    memset(idx, 0, sizeof(uint32_t) * dc);
    for (int depth = 0; depth < depth_n; ++depth) {
        const uint8_t border = sp[depth].split_idx;
        const uint8_t x = sp[depth].xor_mask;
        const uint8_t* col = bins + (size_t)sp[depth].feature_index * dc;
        for (size_t d = 0; d < dc; ++d) idx[d] |= (uint32_t)((uint8_t)(col[d] ^ x) >= border) << depth;
    }
}

/* CalcIndexesNonSymmetric, evaluator_impl.cpp:462-493: returns the final node id per doc. */
static void calc_indexes_nonsym(const cbo_model* m, const uint8_t* bins, size_t dc, int tree, uint32_t* idx) {
    for (size_t d = 0; d < dc; ++d) {
        uint32_t node = (uint32_t)m->tree_start_offsets[tree];
        if (m->bucket_count != 0) {
            for (;;) {
                const cbo_repacked_bin sp = m->repacked[node];
                const uint8_t v = (uint8_t)(bins[(size_t)sp.feature_index * dc + d] ^ sp.xor_mask);
                const uint16_t diff = (v >= sp.split_idx) ? m->step_nodes[2 * node + 1] : m->step_nodes[2 * node];
                node += diff;
                if (diff == 0) break;
            }
        }
        idx[d] = node;
    }
}

/* One block: adds raw leaf sums into res[doc * dim + k] (CalcTreesBlockedImpl :257-361,
 * CalcNonSymmetricTrees :661-705); leaf indexes go to li[(t - tree_start) * dc + doc]. */
static void calc_trees_block(const cbo_model* m, const uint8_t* bins, size_t dc, size_t tree_start, size_t tree_end,
                             double* res, uint32_t* li, uint32_t* idx) {
    const int dim = m->approx_dim;
    for (size_t t = tree_start; t < tree_end; ++t) {
        if (m->oblivious) {
            calc_indexes_oblivious(m, bins, dc, (int)t, idx);
            if (li) {
                memcpy(li + (t - tree_start) * dc, idx, sizeof(uint32_t) * dc);
            } else {
                const double* leaf = m->leaf_values + m->first_leaf_offsets[t];
                if (dim == 1) {
                    for (size_t d = 0; d < dc; ++d) res[d] += leaf[idx[d]];
                } else {
                    for (size_t d = 0; d < dc; ++d)
                        for (int k = 0; k < dim; ++k) res[d * dim + k] += leaf[(size_t)idx[d] * dim + k];
                }
            }
        } else {
            calc_indexes_nonsym(m, bins, dc, (int)t, idx);
            for (size_t d = 0; d < dc; ++d) idx[d] = m->node_id_to_leaf_id[idx[d]];
            if (li) {
                for (size_t d = 0; d < dc; ++d)
                    li[(t - tree_start) * dc + d] = (uint32_t)((idx[d] - m->first_leaf_offsets[t]) / (uint64_t)dim);
            } else if (dim == 1) {
                for (size_t d = 0; d < dc; ++d) res[d] += m->leaf_values[idx[d]];
            } else {
                for (size_t d = 0; d < dc; ++d)
                    for (int k = 0; k < dim; ++k) res[d * dim + k] += m->leaf_values[(size_t)idx[d] + k];
            }
        }
    }
}

/* ApplyScaleAndBias, scale_and_bias.cpp:4-50 */
static void apply_scale_and_bias(const cbo_model* m, double* data, size_t n_items, size_t tree_start) {
    const int dim = m->approx_dim;
    int zero_bias = 1;
    for (int k = 0; k < dim; ++k) if (m->bias[k] != 0.0) zero_bias = 0;
    if (m->scale == 1.0 && zero_bias) return;
    if (dim == 1 || zero_bias) {
        const double bias = zero_bias ? 0.0 : m->bias[0];
        if (m->scale != 1.0 || zero_bias) {
            if (zero_bias || tree_start > 0) {
                for (size_t i = 0; i < n_items; ++i) data[i] *= m->scale;
            } else {
                for (size_t i = 0; i < n_items; ++i) data[i] = m->scale * data[i] + bias;
            }
        } else if (tree_start == 0) {
            for (size_t i = 0; i < n_items; ++i) data[i] += bias;
        }
    } else {
        if (m->scale != 1.0) {
            if (tree_start > 0) {
                for (size_t i = 0; i < n_items; ++i) data[i] = m->scale * data[i];
            } else {
                for (size_t i = 0; i < n_items;)
                    for (int k = 0; k < dim; ++k, ++i) data[i] = m->scale * data[i] + m->bias[k];
            }
        } else if (tree_start == 0) {
            for (size_t i = 0; i < n_items;)
                for (int k = 0; k < dim; ++k, ++i) data[i] += m->bias[k];
        }
    }
}

static void calc_range(const cbo_model* m, const cbo_features* f, size_t doc_begin, size_t doc_end,
                       size_t tree_start, size_t tree_end, double* out, uint32_t* leaf_out) {
    const int dim = m->approx_dim;
    const size_t n_tr = tree_end - tree_start;
    uint8_t* bins = (uint8_t*)malloc((size_t)CBO_BLOCK * (size_t)(m->bucket_count ? m->bucket_count : 1));
    uint32_t* th = (uint32_t*)malloc(sizeof(uint32_t) * CBO_BLOCK * (size_t)(m->used_cat ? m->used_cat : 1));
    uint32_t idx[CBO_BLOCK];
    uint32_t* li = leaf_out ? (uint32_t*)malloc(sizeof(uint32_t) * CBO_BLOCK * (n_tr ? n_tr : 1)) : NULL;
    for (size_t start = doc_begin; start < doc_end; start += CBO_BLOCK) {
        const size_t dc = doc_end - start < CBO_BLOCK ? doc_end - start : CBO_BLOCK;
        binarize_block(m, f, start, dc, bins, th);
        if (leaf_out) {
            calc_trees_block(m, bins, dc, tree_start, tree_end, NULL, li, idx);
            /* Transpose2DArray, cpu/evaluator.h:157-172: [tree][doc] -> [doc][tree] */
            for (size_t t = 0; t < n_tr; ++t)
                for (size_t d = 0; d < dc; ++d) leaf_out[(start + d) * n_tr + t] = li[t * dc + d];
        } else {
            double* res = out + start * (size_t)dim;
            memset(res, 0, sizeof(double) * dc * (size_t)dim);
            calc_trees_block(m, bins, dc, tree_start, tree_end, res, NULL, idx);
            apply_scale_and_bias(m, res, dc * (size_t)dim, tree_start);
        }
    }
    free(bins);
    free(th);
    free(li);
}

void cbo_calc(const cbo_model* m, const cbo_features* f, size_t n_docs,
              size_t tree_start, size_t tree_end, double* out) {
    if (m->n_trees == 0) {
        /* formula_evaluator.cpp:29-41 */
        for (size_t i = 0; i < n_docs * (size_t)m->approx_dim; ++i) out[i] = m->bias[i % (size_t)m->approx_dim];
        return;
    }
    calc_range(m, f, 0, n_docs, tree_start, tree_end, out, NULL);
}

void cbo_calc_leaf_indexes(const cbo_model* m, const cbo_features* f, size_t n_docs,
                           size_t tree_start, size_t tree_end, uint32_t* out) {
    calc_range(m, f, 0, n_docs, tree_start, tree_end, NULL, out);
}

typedef struct {
    const cbo_model* m; const cbo_features* f; size_t b, e, ts, te; double* out;
} cbo_job;

static void* job_main(void* p) {
    cbo_job* j = (cbo_job*)p;
    calc_range(j->m, j->f, j->b, j->e, j->ts, j->te, j->out, NULL);
    return NULL;
}

void cbo_calc_mt(const cbo_model* m, const cbo_features* f, size_t n_docs,
                 size_t tree_start, size_t tree_end, double* out, int n_threads) {
    if (n_threads <= 1 || m->n_trees == 0 || n_docs < 2 * CBO_BLOCK) {
        cbo_calc(m, f, n_docs, tree_start, tree_end, out);
        return;
    }
    size_t n_blocks = (n_docs + CBO_BLOCK - 1) / CBO_BLOCK;
    if ((size_t)n_threads > n_blocks) n_threads = (int)n_blocks;
    pthread_t* th = (pthread_t*)malloc(sizeof(pthread_t) * n_threads);
    cbo_job* jobs = (cbo_job*)malloc(sizeof(cbo_job) * n_threads);
    for (int i = 0; i < n_threads; ++i) {
        size_t b = n_blocks * (size_t)i / (size_t)n_threads * CBO_BLOCK;
        size_t e = n_blocks * (size_t)(i + 1) / (size_t)n_threads * CBO_BLOCK;
        if (e > n_docs) e = n_docs;
        cbo_job j = {m, f, b, e, tree_start, tree_end, out};
        jobs[i] = j;
        pthread_create(&th[i], NULL, job_main, &jobs[i]);
    }
    for (int i = 0; i < n_threads; ++i) pthread_join(th[i], NULL);
    free(th);
    free(jobs);
}

/* -------------------------------------------------------------------- brute force -------- */

/* Truth value of binary feature `bf` for one doc straight from its definition:
 * float split  <=> value > border after the NaN policy of quantization.h:375-409,
 * one-hot split <=> hashed value == Value (split.h:17-19). */
static float raw_float(const cbo_model* m, const cbo_features* f, int feature, size_t doc) {
    float v = get_float(m, f, feature, doc);
    if (isnan(v) && m->ff_has_nans[feature] && m->ff_nan_treatment[feature] != CBO_NAN_AS_IS)
        v = (m->ff_nan_treatment[feature] == CBO_NAN_AS_FALSE) ? -INFINITY : INFINITY;
    return v;
}

/* CTR of one document from the raw features: the projection's hash folds the categorical hashes, then
 * "value > border" per float split and "hash == value" per one-hot split (ctr_provider.h:64-78 with the
 * bins replaced by what they stand for). */
static float raw_ctr(const cbo_model* m, const cbo_features* f, int ctr, size_t doc) {
    uint64_t h = 0;
    for (int32_t i = m->ctr_cat_offsets[ctr]; i < m->ctr_cat_offsets[ctr + 1]; ++i) {
        for (int c = 0; c < m->n_cat; ++c)
            if (m->cf_index[c] == m->ctr_cats[i])
                h = ctr_calc_hash(h, (uint64_t)(int64_t)(int32_t)get_cat(m, f, c, doc));
    }
    for (int32_t i = m->ctr_float_offsets[ctr]; i < m->ctr_float_offsets[ctr + 1]; ++i)
        h = ctr_calc_hash(h, (uint64_t)(raw_float(m, f, m->ctr_float_raw[i], doc) > m->ctr_float_border[i]));
    for (int32_t i = m->ctr_onehot_offsets[ctr]; i < m->ctr_onehot_offsets[ctr + 1]; ++i) {
        for (int c = 0; c < m->n_cat; ++c)
            if (m->cf_index[c] == m->ctr_onehot_cat[i])
                h = ctr_calc_hash(h, (uint64_t)((int32_t)get_cat(m, f, c, doc) == m->ctr_onehot_value[i]));
    }
    return ctr_value(m, ctr, ctr_table_index(m, m->ctr_table[ctr], h));
}

static int raw_condition(const cbo_model* m, const cbo_features* f, int bf, size_t doc) {
    const cbo_bin_feature* b = &m->bin_features[bf];
    if (b->is_ctr) return raw_ctr(m, f, b->feature, doc) > b->border;
    if (!b->is_onehot) {
        float v = get_float(m, f, b->feature, doc);
        if (isnan(v) && m->ff_has_nans[b->feature] && m->ff_nan_treatment[b->feature] != CBO_NAN_AS_IS)
            v = (m->ff_nan_treatment[b->feature] == CBO_NAN_AS_FALSE) ? -INFINITY : INFINITY;
        return v > b->border;
    }
    int cat = -1;
    for (int c = 0; c < m->n_cat; ++c)
        if (m->cf_index[c] == m->oh_cat_index[b->feature]) cat = c;
    int32_t hv;
    uint32_t h = get_cat(m, f, cat, doc);
    memcpy(&hv, &h, 4);
    return hv == b->value;
}

void cbo_calc_bruteforce(const cbo_model* m, const cbo_features* f, size_t n_docs,
                         size_t tree_start, size_t tree_end, double* out, uint32_t* leaf_indexes) {
    const int dim = m->approx_dim;
    const size_t n_tr = tree_end - tree_start;
    for (size_t d = 0; d < n_docs; ++d) {
        double* res = out + d * (size_t)dim;
        for (int k = 0; k < dim; ++k) res[k] = 0.0;
        for (size_t t = tree_start; t < tree_end; ++t) {
            uint64_t value_idx;
            if (m->oblivious) {
                uint32_t idx = 0;
                for (int depth = 0; depth < m->tree_sizes[t]; ++depth)
                    idx |= (uint32_t)raw_condition(m, f, m->tree_splits[m->tree_start_offsets[t] + depth], d) << depth;
                value_idx = m->first_leaf_offsets[t] + (uint64_t)idx * (uint64_t)dim;
            } else {
                uint32_t node = (uint32_t)m->tree_start_offsets[t];
                for (;;) {
                    const uint16_t l = m->step_nodes[2 * node], r = m->step_nodes[2 * node + 1];
                    if (l == 0 && r == 0) break;
                    const uint16_t diff = raw_condition(m, f, m->tree_splits[node], d) ? r : l;
                    if (diff == 0) break;
                    node += diff;
                }
                value_idx = m->node_id_to_leaf_id[node];
            }
            for (int k = 0; k < dim; ++k) res[k] += m->leaf_values[value_idx + (uint64_t)k];
            if (leaf_indexes)
                leaf_indexes[d * n_tr + (t - tree_start)] = (uint32_t)((value_idx - m->first_leaf_offsets[t]) / (uint64_t)dim);
        }
        for (int k = 0; k < dim; ++k) {
            double v = m->scale * res[k];
            if (tree_start == 0) v += m->bias[k];
            res[k] = v;
        }
    }
}

/* ---- prediction types ---------------------------------------------------------------- */

/* fmath's table-based exponent, double precision: ExpdVar (fmath.hpp:150-185). The table and the
 * scale come from the C library's pow / log exactly as the reference computes them at start-up. */
#define CBO_EXPD_SBIT 11
static uint64_t g_expd_tbl[1 << CBO_EXPD_SBIT];
static double g_expd_a, g_expd_ra;
static pthread_once_t g_expd_once = PTHREAD_ONCE_INIT;

static void expd_init(void) {
    const int s = 1 << CBO_EXPD_SBIT;
    g_expd_a = s / log(2.0);
    g_expd_ra = 1 / g_expd_a;
    for (int i = 0; i < s; i++) {
        const double d = pow(2.0, i * (1.0 / s));
        uint64_t bits;
        memcpy(&bits, &d, 8);
        g_expd_tbl[i] = bits & ((1ULL << 52) - 1);
    }
}

/* One value through the arithmetic both paths share (fmath.hpp:587-600 / :484-495): every
 * multiply, add and subtract is a separate rounding. `di` is the integer the table index and the
 * exponent are taken from: all 64 bits of d on the vector path, its sign-extended low half on the
 * scalar path (only bits 0..22 matter). */
static double expd_core(double x, uint64_t (*index_bits)(double)) {
    const double b = (double)(3ULL << 51);
    const uint64_t adj = (1ULL << (CBO_EXPD_SBIT + 10)) - (1ULL << CBO_EXPD_SBIT);
    const double C1 = 1.0, C2 = 0.16666666685227835064, C3 = 3.0000000027955394;
    double d = x * g_expd_a;
    d = d + b;
    const uint64_t di = index_bits(d);
    const uint64_t iax = g_expd_tbl[di & ((1u << CBO_EXPD_SBIT) - 1)];
    double t = d - b;
    t = t * g_expd_ra;
    t = t - x;
    const uint64_t u = (((di + adj) >> CBO_EXPD_SBIT) << 52) | iax;
    double y = C3 - t;
    const double tt = t * t;
    y = y * tt;
    y = y * C2;
    y = y - t;
    y = y + C1;
    double scale;
    memcpy(&scale, &u, 8);
    return y * scale;
}

static uint64_t expd_bits_all(double d) {
    uint64_t bits;
    memcpy(&bits, &d, 8);
    return bits;
}

static uint64_t expd_bits_low(double d) {
    uint64_t bits;
    memcpy(&bits, &d, 8);
    return (uint64_t)(int64_t)(int32_t)(uint32_t)bits;
}

void cbo_fast_exp_inplace(double* x, size_t n) {
    pthread_once(&g_expd_once, expd_init);
    const size_t vec = n & ~(size_t)3;
    for (size_t i = 0; i < vec; i++) {
        /* _mm256_min_pd / _mm256_max_pd hand back their second operand unless the compare holds,
         * so a NaN becomes the upper clamp */
        double v = x[i];
        v = (v < 709.78272569338397) ? v : 709.78272569338397;
        v = (v > -708.39641853226408) ? v : -708.39641853226408;
        x[i] = expd_core(v, expd_bits_all);
    }
    for (size_t i = vec; i < n; i++) {
        const double v = x[i];
        if (v <= -708.39641853226408) {
            x[i] = 0;
        } else if (v >= 709.78271289338397) {
            x[i] = INFINITY;
        } else {
            x[i] = expd_core(v, expd_bits_low);
        }
    }
}

int cbo_apply_prediction_type(int type, size_t dim, size_t n_docs, const double* raw, double* out) {
    const size_t block = n_docs < 128 ? n_docs : 128;
    if (type == CBO_RAW) {
        memcpy(out, raw, n_docs * dim * sizeof(double));
        return 0;
    }
    for (size_t begin = 0; begin < n_docs; begin += block) {
        const size_t n = n_docs - begin < block ? n_docs - begin : block;
        const double* r = raw + begin * dim;
        if (type == CBO_CLASS) {
            double* o = out + begin;
            for (size_t i = 0; i < n; i++) {
                if (dim == 1) {
                    o[i] = r[i] > 0.0;
                } else {
                    size_t best = 0;  /* first maximum, as MaxElement */
                    for (size_t k = 1; k < dim; k++) {
                        if (r[i * dim + best] < r[i * dim + k]) {
                            best = k;
                        }
                    }
                    o[i] = (double)best;
                }
            }
            continue;
        }
        double* o = out + begin * dim;
        memcpy(o, r, n * dim * sizeof(double));
        if (dim == 1) {
            if (type == CBO_PROBABILITY) {           /* CalcSigmoid over the block */
                for (size_t i = 0; i < n; i++) {
                    o[i] = -o[i];
                }
                cbo_fast_exp_inplace(o, n);
                for (size_t i = 0; i < n; i++) {
                    o[i] = 1. / (1. + o[i]);
                }
            } else if (type == CBO_EXPONENT) {
                cbo_fast_exp_inplace(o, n);
            } else {
                return -1;
            }
        } else if (type == CBO_RMSE_WITH_UNCERTAINTY) {  /* exp(2 x) of the second value of a document */
            for (size_t i = 1; i < n * dim; i += dim) {
                o[i] *= 2.0f;
                cbo_fast_exp_inplace(o + i, 1);
            }
        } else if (type == CBO_PROBABILITY) {            /* CalcSoftmax per document */
            for (size_t i = 0; i < n; i++) {
                double* v = o + i * dim;
                double mx = v[0];
                for (size_t k = 1; k < dim; k++) {
                    if (mx < v[k]) {
                        mx = v[k];
                    }
                }
                for (size_t k = 0; k < dim; k++) {
                    v[k] = v[k] - mx;
                }
                cbo_fast_exp_inplace(v, dim);
                double sum = 0;
                for (size_t k = 0; k < dim; k++) {
                    sum += v[k];
                }
                for (size_t k = 0; k < dim; k++) {
                    v[k] /= sum;
                }
            }
        } else if (type == CBO_MULTI_PROBABILITY) {      /* CalcSigmoid over the block's values */
            for (size_t i = 0; i < n * dim; i++) {
                o[i] = -o[i];
            }
            cbo_fast_exp_inplace(o, n * dim);
            for (size_t i = 0; i < n * dim; i++) {
                o[i] = 1. / (1. + o[i]);
            }
        } else {
            return -1;
        }
    }
    return 0;
}
