#include "tsv_io.hpp"

#include <cstdio>
#include <cstdlib>
#include <cstring>

namespace spdnn {

bool read_triples(const std::string& path, std::vector<Triple>& out, std::string& err) {
    FILE* f = fopen(path.c_str(), "rb");
    if (!f) { err = "FILE:" + path + " does not exists."; return false; }
    fseek(f, 0, SEEK_END);
    const long sz = ftell(f);
    fseek(f, 0, SEEK_SET);
    std::vector<char> buf((size_t)sz + 1);
    if (sz > 0 && fread(buf.data(), 1, (size_t)sz, f) != (size_t)sz) { fclose(f); err = "short read: " + path; return false; }
    fclose(f);
    buf[(size_t)sz] = 0;
    out.clear();
    char* p = buf.data();
    char* end = buf.data() + sz;
    while (p < end) {
        char* q;
        const long a = strtol(p, &q, 10);
        if (q == p) break;  // no more numbers (trailing whitespace) - like a failed stream extraction
        p = q;
        const long b = strtol(p, &q, 10);
        if (q == p) { err = "malformed line in " + path; return false; }
        p = q;
        const float v = strtof(p, &q);
        if (q == p) { err = "malformed line in " + path; return false; }
        p = q;
        out.push_back(Triple{(int32_t)a, (int32_t)b, v});
    }
    return true;
}

bool read_weight_tsv_csr(const std::string& path, int N, std::vector<int32_t>& rowptr,
                         std::vector<int32_t>& col, std::vector<float>& val, std::string& err) {
    std::vector<Triple> t;
    if (!read_triples(path, t, err)) return false;
    rowptr.assign((size_t)N + 1, 0);
    for (const Triple& e : t) {
        const int in = e.a - 1, out = e.b - 1;
        if (in < 0 || in >= N || out < 0 || out >= N) { err = "neuron index out of range in " + path; return false; }
        rowptr[(size_t)out + 1]++;
    }
    for (int j = 0; j < N; ++j) rowptr[j + 1] += rowptr[j];
    col.resize(t.size());
    val.resize(t.size());
    std::vector<int32_t> fill(rowptr.begin(), rowptr.end() - 1);
    for (const Triple& e : t) {
        const int out = e.b - 1;
        col[(size_t)fill[out]] = e.a - 1;
        val[(size_t)fill[out]] = e.v;
        fill[out]++;
    }
    // rows are sorted by input index later (normalize_csr); file order is kept among duplicates
    return true;
}

bool read_features_tsv_dense(const std::string& path, int N, int batch, std::vector<float>& dense,
                             int64_t* kept, std::string& err) {
    std::vector<Triple> t;
    if (!read_triples(path, t, err)) return false;
    dense.assign((size_t)batch * (size_t)N, 0.0f);
    int64_t k = 0;
    for (const Triple& e : t) {
        if (e.a > batch) continue;  // network.cpp:46: rows beyond the batch are skipped
        if (e.a < 1 || e.b < 1 || e.b > N) { err = "feature index out of range in " + path; return false; }
        dense[(size_t)(e.a - 1) * (size_t)N + (size_t)(e.b - 1)] = e.v;
        ++k;
    }
    if (kept) *kept = k;
    return true;
}

// ---- packed binary files (benchmark/cusparse/cusparse.cu:318-383) ---------------------------

static bool read_exact(FILE* f, void* dst, size_t bytes) { return bytes == 0 || fread(dst, 1, bytes, f) == bytes; }

bool read_weight_bin_csr(const std::string& path, int N, int layer, int64_t nnz, std::vector<int32_t>& rowptr,
                         std::vector<int32_t>& col, std::vector<float>& val, std::string& err) {
    FILE* f = fopen(path.c_str(), "rb");
    if (!f) { err = "FILE:" + path + " does not exists."; return false; }
    const int64_t rec = nnz * 12;
    if (fseeko(f, (off_t)(rec * layer), SEEK_SET) != 0) { fclose(f); err = "seek failed: " + path; return false; }
    std::vector<int32_t> r((size_t)nnz), c((size_t)nnz);
    std::vector<float> v((size_t)nnz);
    const bool ok = read_exact(f, r.data(), (size_t)nnz * 4) && read_exact(f, c.data(), (size_t)nnz * 4) &&
                    read_exact(f, v.data(), (size_t)nnz * 4);
    fclose(f);
    if (!ok) { err = "short read (layer record " + std::to_string(layer) + "): " + path; return false; }
    rowptr.assign((size_t)N + 1, 0);
    for (int64_t e = 0; e < nnz; ++e) {
        const int out = r[(size_t)e] - 1, in = c[(size_t)e] - 1;
        if (in < 0 || in >= N || out < 0 || out >= N) { err = "neuron index out of range in " + path; return false; }
        rowptr[(size_t)out + 1]++;
    }
    for (int j = 0; j < N; ++j) rowptr[j + 1] += rowptr[j];
    col.resize((size_t)nnz);
    val.resize((size_t)nnz);
    std::vector<int32_t> fill(rowptr.begin(), rowptr.end() - 1);
    for (int64_t e = 0; e < nnz; ++e) {
        const int out = r[(size_t)e] - 1;
        col[(size_t)fill[out]] = c[(size_t)e] - 1;
        val[(size_t)fill[out]] = v[(size_t)e];
        fill[out]++;
    }
    return true;
}

bool read_features_bin_dense(const std::string& path, int N, int batch, std::vector<float>& dense,
                             int64_t* kept, std::string& err) {
    FILE* f = fopen(path.c_str(), "rb");
    if (!f) { err = "FILE:" + path + " does not exists."; return false; }
    fseeko(f, 0, SEEK_END);
    const int64_t sz = (int64_t)ftello(f);
    fseeko(f, 0, SEEK_SET);
    if (sz % 12 != 0) { fclose(f); err = "size is not a multiple of 12 bytes: " + path; return false; }
    const int64_t nnz = sz / 12;
    std::vector<int32_t> r((size_t)nnz), c((size_t)nnz);
    std::vector<float> v((size_t)nnz);
    const bool ok = read_exact(f, r.data(), (size_t)nnz * 4) && read_exact(f, c.data(), (size_t)nnz * 4) &&
                    read_exact(f, v.data(), (size_t)nnz * 4);
    fclose(f);
    if (!ok) { err = "short read: " + path; return false; }
    dense.assign((size_t)batch * (size_t)N, 0.0f);
    int64_t k = 0;
    for (int64_t e = 0; e < nnz; ++e) {
        const int neuron = r[(size_t)e], image = c[(size_t)e];
        if (image > batch) continue;  // cusparse.cu:376: images beyond the batch are skipped
        if (image < 1 || neuron < 1 || neuron > N) { err = "feature index out of range in " + path; return false; }
        dense[(size_t)(image - 1) * (size_t)N + (size_t)(neuron - 1)] = v[(size_t)e];
        ++k;
    }
    if (kept) *kept = k;
    return true;
}

}  // namespace spdnn
