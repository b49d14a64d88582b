#include "synth.hpp"

#include <numeric>

namespace spdnn {

uint64_t sm64(uint64_t x) {
    uint64_t z = x + 0x9E3779B97F4A7C15ULL;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ULL;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBULL;
    return z ^ (z >> 31);
}

static int gcd_i(int a, int b) { while (b) { int t = a % b; a = b; b = t; } return a; }

bool synth_layer_csr(uint64_t seed, int layer, int N, int K, float value, std::vector<int32_t>& rowptr,
                     std::vector<int32_t>& col, std::vector<float>& val) {
    if (N < 1 || K < 1 || K > N) return false;
    const uint64_t kl = sm64(sm64(seed ^ 0x4C41594552ULL) + (uint64_t)layer);
    const int o = (int)(sm64(kl) % (uint64_t)N);
    int s = (int)(sm64(kl + 1) % (uint64_t)N);
    if (s == 0) s = 1;
    while (gcd_i(s, N) != 1) { if (++s >= N) s = 1; }
    std::vector<int32_t> pi((size_t)N);
    std::iota(pi.begin(), pi.end(), 0);
    for (int i = N - 1; i >= 1; --i) {
        const uint64_t r = sm64(kl + 2 + (uint64_t)(N - 1 - i)) >> 32;
        const int j = (int)((r * (uint64_t)(i + 1)) >> 32);
        std::swap(pi[i], pi[j]);
    }
    rowptr.resize((size_t)N + 1);
    for (int j = 0; j <= N; ++j) rowptr[j] = j * K;
    col.resize((size_t)N * K);
    val.assign((size_t)N * K, value);
    // inputs are visited in ascending order, so every output row fills in ascending input index
    std::vector<int32_t> fill((size_t)N, 0);
    for (int i = 0; i < N; ++i) {
        int64_t j = ((int64_t)pi[i] + o) % N;
        for (int k = 0; k < K; ++k) {
            col[(size_t)j * K + fill[j]++] = i;
            j += s;
            if (j >= N) j -= N;
        }
    }
    return true;
}

void synth_features_host(uint64_t seed, int N, int64_t row_begin, int64_t nrows, float dmin, float dmax,
                         float* out) {
    const uint64_t kf = sm64(seed ^ 0x46454154ULL);
    const uint64_t lo = (uint64_t)((double)dmin * 4294967296.0);
    const uint64_t span = (uint64_t)(((double)dmax - (double)dmin) * 4294967296.0);
    for (int64_t r = 0; r < nrows; ++r) {
        const uint64_t rk = sm64(kf + (uint64_t)(row_begin + r));
        const uint64_t a = sm64(rk + 0xFFFFFFFF00000000ULL) >> 32;
        uint64_t thr = lo + ((a * span) >> 32);
        if (thr > 0xFFFFFFFFULL) thr = 0xFFFFFFFFULL;
        float* o = out + (size_t)r * (size_t)N;
        for (int c = 0; c < N; ++c) o[c] = (uint32_t)(sm64(rk + (uint64_t)c) >> 32) < (uint32_t)thr ? 1.0f : 0.0f;
    }
}

}  // namespace spdnn
