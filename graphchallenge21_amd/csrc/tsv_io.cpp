#include "tsv_io.hpp"

#include <algorithm>
#include <atomic>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <thread>

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
        // an index beyond 32 bits stays out of range for every width instead of wrapping into it
        const long lo = INT32_MIN, hi = INT32_MAX;
        out.push_back(Triple{(int32_t)std::min(std::max(a, lo), hi), (int32_t)std::min(std::max(b, lo), hi), v});
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

namespace {

// One "int int float" line starting at p (leading whitespace skipped).  Returns 1 and advances p,
// 0 at the end of the data, -1 on a malformed line.  Plain decimal integers in the value column
// (the challenge's feature files hold 1s) skip strtof.
inline int parse_triple(const char*& p, const char* end, long& a, long& b, float& v) {
    auto skip = [&] { while (p < end && (*p == ' ' || *p == '\t' || *p == '\n' || *p == '\r')) ++p; };
    auto integer = [&](long& out) -> bool {
        skip();
        const char* q = p;
        bool neg = false;
        if (q < end && (*q == '-' || *q == '+')) { neg = *q == '-'; ++q; }
        const char* d0 = q;
        long x = 0;
        while (q < end && *q >= '0' && *q <= '9' && q - d0 < 18) { x = x * 10 + (*q - '0'); ++q; }
        if (q == d0) return false;
        out = neg ? -x : x;
        p = q;
        return true;
    };
    skip();
    if (p >= end) return 0;
    if (!integer(a)) return -1;
    if (!integer(b)) return -1;
    skip();
    const char* q = p;
    long iv = 0;
    const char* save = p;
    if (integer(iv) && (p >= end || *p == '\n' || *p == '\r' || *p == ' ' || *p == '\t') && p - save <= 7) {
        v = (float)iv;   // up to 6 digits and a sign: exact in fp32
        return 1;
    }
    p = q;
    char* e;
    v = strtof(p, &e);   // the buffer ends in a 0 byte, so this stops inside it
    if (e == p) return -1;
    p = e;
    return 1;
}

}  // namespace

bool read_features_tsv_dense(const std::string& path, int N, int batch, std::vector<float>& dense,
                             int64_t* kept, std::string& err, int threads) {
    dense.resize((size_t)batch * (size_t)N);
    return read_features_tsv_into(path, N, batch, dense.data(), kept, err, threads);
}

bool read_features_tsv_into(const std::string& path, int N, int batch, float* dense, int64_t* kept,
                            std::string& err, int threads) {
    FILE* f = fopen(path.c_str(), "rb");
    if (!f) { err = "FILE:" + path + " does not exists."; return false; }
    fseeko(f, 0, SEEK_END);
    const int64_t sz = (int64_t)ftello(f);
    fseeko(f, 0, SEEK_SET);
    std::vector<char> buf((size_t)sz + 1);
    if (sz > 0 && fread(buf.data(), 1, (size_t)sz, f) != (size_t)sz) { fclose(f); err = "short read: " + path; return false; }
    fclose(f);
    buf[(size_t)sz] = 0;
    const char* base = buf.data();
    const char* end = base + sz;

    // Parts of the file, cut at line starts, are parsed side by side and stored straight into the
    // dense matrix.  The reference keeps the LAST line of an entry that occurs twice
    // (network.cpp:47); the parts cannot know each other's order, so a bitmap notes which entries
    // were stored and, should any entry come twice, the file is gone through again in order.
    const int T = (int)std::max<int64_t>(1, std::min<int64_t>(threads, sz / (1 << 20) + 1));
    std::vector<const char*> cut((size_t)T + 1, end);
    cut[0] = base;
    for (int t = 1; t < T; ++t) {
        const char* p = base + sz / T * t;
        while (p < end && *p != '\n') ++p;
        cut[(size_t)t] = p < end ? p + 1 : end;
    }
    const size_t total = (size_t)batch * (size_t)N;
    std::fill(dense, dense + total, 0.0f);
    std::vector<std::atomic<uint64_t>> seen(T > 1 ? (total + 63) / 64 : 0);
    for (auto& w : seen) w.store(0, std::memory_order_relaxed);
    std::vector<int64_t> kept_t((size_t)T, 0);
    std::vector<int> state((size_t)T, 0);  // 1 = malformed, 2 = index out of range
    std::atomic<bool> twice{false};
    auto parse_range = [&](const char* p, const char* e, bool mark, int64_t& k_out, int& state_out) {
        int64_t k = 0;
        long a, b;
        float v;
        state_out = 0;
        for (;;) {
            const int r = parse_triple(p, e, a, b, v);
            if (r == 0) break;
            if (r < 0) { state_out = 1; break; }
            if (a > batch) continue;  // network.cpp:46: rows beyond the batch are skipped
            if (a < 1 || b < 1 || b > N) { state_out = 2; break; }
            const size_t at = (size_t)(a - 1) * (size_t)N + (size_t)(b - 1);
            dense[at] = v;
            if (mark) {
                const uint64_t bit = 1ull << (at & 63);
                if (seen[at >> 6].fetch_or(bit, std::memory_order_relaxed) & bit) twice.store(true, std::memory_order_relaxed);
            }
            ++k;
        }
        k_out = k;
    };
    {
        std::vector<std::thread> th;
        for (int t = 1; t < T; ++t)
            th.emplace_back([&, t] { parse_range(cut[(size_t)t], cut[(size_t)t + 1], true, kept_t[(size_t)t], state[(size_t)t]); });
        parse_range(cut[0], cut[1], T > 1, kept_t[0], state[0]);
        for (std::thread& x : th) x.join();
    }
    bool again = twice.load();
    for (int t = 0; t < T; ++t) again |= state[(size_t)t] != 0;
    if (again && T > 1) {
        // an entry set twice, or a part that did not parse (a triple may straddle a line end, which
        // the reference's stream extraction accepts): the whole file once more, in order, as one part
        for (int t = 1; t < T; ++t) kept_t[(size_t)t] = 0;
        parse_range(base, end, false, kept_t[0], state[0]);
        for (int t = 1; t < T; ++t) state[(size_t)t] = 0;
    }
    // every other part's state is clear here: either nothing was wrong or the file was gone through as one part
    if (state[0] == 1) { err = "malformed line in " + path; return false; }
    if (state[0] == 2) { err = "feature index out of range in " + path; return false; }
    int64_t k = 0;
    for (int t = 0; t < T; ++t) k += kept_t[(size_t)t];
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
