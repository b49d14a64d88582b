// TSV loaders in the challenge's file formats, the host data layer of the reference driver
// (COOMatrix(file, 1, false), src/utils/matrix.h:255-282; read_input, src/network.cpp:33-54),
// re-done as a single pass over the file bytes instead of iostream extraction.
#pragma once
#include <cstdint>
#include <string>
#include <vector>

namespace spdnn {

struct Triple { int32_t a, b; float v; };

// Reads whitespace-separated "int int float" triples.  Returns false and sets err on failure.
bool read_triples(const std::string& path, std::vector<Triple>& out, std::string& err);

// Weight file "in out value" (1-based) -> CSR of an N x N layer with row = output neuron,
// col = input neuron, entries of a row in ascending input index (file order among duplicates).
bool read_weight_tsv_csr(const std::string& path, int N, std::vector<int32_t>& rowptr,
                         std::vector<int32_t>& col, std::vector<float>& val, std::string& err);

// Feature file "row neuron value" (1-based) -> dense row-major batch x N; rows beyond batch are
// skipped like the reference does, of an entry that occurs twice the last line counts.  *kept
// receives the number of lines stored.  The file is parsed by up to `threads` threads.
bool read_features_tsv_dense(const std::string& path, int N, int batch, std::vector<float>& dense,
                             int64_t* kept, std::string& err, int threads = 1);
// the same into memory of the caller (batch * N floats)
bool read_features_tsv_into(const std::string& path, int N, int batch, float* dense, int64_t* kept,
                            std::string& err, int threads = 1);

// Packed binary files as the reference's library benchmarks consume them
// (benchmark/cusparse/cusparse.cu:318-383): "neuron{N}.bin" holds one record per layer of
// int32 row[nnz], int32 col[nnz], float32 val[nnz] (1-based; row = OUTPUT neuron = CSR row,
// col = input neuron, nnz = 32 N in the reference); "sparse-images-{N}.bin" holds int32 row[] (neuron),
// int32 col[] (image), float32 val[] over the whole file.  `layer` selects the record.
bool read_weight_bin_csr(const std::string& path, int N, int layer, int64_t nnz, std::vector<int32_t>& rowptr,
                         std::vector<int32_t>& col, std::vector<float>& val, std::string& err);
bool read_features_bin_dense(const std::string& path, int N, int batch, std::vector<float>& dense,
                             int64_t* kept, std::string& err);

}  // namespace spdnn
