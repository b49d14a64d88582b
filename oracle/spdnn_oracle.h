/*
 * CPU oracle for the Sparse DNN Graph Challenge inference path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing under graphchallenge21_amd/ links, loads or
 * calls this file; it is the checker the HIP path is compared with (tests, the smoke
 * check and the CPU-baseline leg of the benchmark).
 *
 * Every function restates, in plain C, what the reference computes on the CPU; the
 * reference location each one follows is cited at its definition in spdnn_oracle.c.
 */
#ifndef SPDNN_ORACLE_H
#define SPDNN_ORACLE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- seeded synthetic inputs (the build's own definition; see spdnn_oracle.c) ---- */
uint64_t orc_splitmix64(uint64_t x);
void orc_gen_layer_params(uint64_t seed, int layer, int neuron, int* perm, int* offset, int* stride);
int  orc_gen_layer_csr(uint64_t seed, int layer, int neuron, int nnz_per_row, float value,
                       int* rowptr, int* col, float* val);
void orc_gen_features(uint64_t seed, int neuron, int64_t row_begin, int64_t nrows,
                      float dmin, float dmax, float* out_rowmajor);
uint32_t orc_feature_threshold(uint64_t seed, int64_t row, float dmin, float dmax);

/* ---- reference host data layer ---- */
int  orc_hash_reorder(int v, int buckets, int max_domain);
int64_t orc_count_tsv_triples(const char* path);
int64_t orc_read_weight_tsv(const char* path, int begin_idx, int64_t cap,
                            int* row, int* col, float* val, int* n_rows, int* n_cols);
int  orc_coo_to_csr(int64_t nnz, int n_rows, const int* row, const int* col, const float* val,
                    int* rowptr, int* csr_col, float* csr_val);
int64_t orc_read_features_tsv(const char* path, int neuron, int batch, float* dense_rowmajor);

/* ---- arithmetic ---- */
float orc_relu_clamp(float x);
void  orc_set_threads(int n);
int   orc_get_threads(void);
void  orc_layer(const float* yin, int64_t nrows, int neuron,
                const int* rowptr, const int* col, const float* val,
                float bias, float* yout, int* active);
int64_t orc_compact(const float* y, int64_t nrows, int neuron, const int* active,
                    const int* gid_in, float* y_out, int* gid_out);

/* ---- fusion analysis ---- */
void orc_need_access(int neuron, const int* rowptr, const int* col, const unsigned char* out_flags,
                     unsigned char* in_flags);

#ifdef __cplusplus
}
#endif
#endif
