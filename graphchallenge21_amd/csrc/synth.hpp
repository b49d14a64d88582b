// Seeded synthetic inputs (host side): the permuted-stride layer generator and the Bernoulli
// feature rows.  The reference reads downloaded files and has no generator
// (src/microbenchmark/random.h:5-13 is an empty stub), so the definition is this library's own:
//
//   sm64(x)     SplitMix64 output function of x + 0x9E3779B97F4A7C15
//   layer l     key kl = sm64(sm64(seed ^ 0x4C41594552) + l), draw(n) = sm64(kl + n)
//               offset o = draw(0) mod N; stride s = draw(1) mod N (0 -> 1), incremented until
//               gcd(s, N) = 1; permutation pi by Fisher-Yates, i = N-1..1,
//               j = (hi32(draw(2 + N-1-i)) * (i+1)) >> 32
//               W_l[i, (pi(i) + o + k*s) mod N] = value, k = 0..K-1
//   features    key kf = sm64(seed ^ 0x46454154), row key rk = sm64(kf + row),
//               threshold thr = lo + ((hi32(sm64(rk + 0xFFFFFFFF00000000)) * span) >> 32),
//               lo = floor(dmin * 2^32), span = floor((dmax - dmin) * 2^32);
//               element (row, c) = hi32(sm64(rk + c)) < thr ? 1.0f : 0.0f
#pragma once
#include <cstdint>
#include <vector>

namespace spdnn {

uint64_t sm64(uint64_t x);

// CSR with row = output neuron, col = input neuron ascending.
bool synth_layer_csr(uint64_t seed, int layer, int N, int K, float value, std::vector<int32_t>& rowptr,
                     std::vector<int32_t>& col, std::vector<float>& val);

void synth_features_host(uint64_t seed, int N, int64_t row_begin, int64_t nrows, float dmin, float dmax,
                         float* rowmajor);

}  // namespace spdnn
