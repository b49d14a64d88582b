#include "inspector.hpp"

#include <algorithm>
#include <array>
#include <climits>
#include <cmath>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <numeric>
#include <stdexcept>

namespace spdnn {

std::string normalize_csr(int N, const int32_t* rowptr, const int32_t* col, const float* val,
                          std::vector<int32_t>& orp, std::vector<int32_t>& oc, std::vector<float>& ov) {
    if (!rowptr || rowptr[0] != 0) return "rowptr[0] must be 0";
    for (int j = 0; j < N; ++j)
        if (rowptr[j + 1] < rowptr[j]) return "rowptr must be non-decreasing";
    const int64_t nnz = rowptr[N];
    if (nnz > 0 && (!col || !val)) return "col/val missing";
    orp.assign(rowptr, rowptr + N + 1);
    oc.resize((size_t)nnz);
    ov.resize((size_t)nnz);
    std::vector<int32_t> order;
    for (int j = 0; j < N; ++j) {
        const int b = rowptr[j], e = rowptr[j + 1];
        bool sorted = true;
        for (int k = b; k < e; ++k) {
            if (col[k] < 0 || col[k] >= N) return "column index out of range";
            if (!std::isfinite(val[k])) return "non-finite weight";
            // with |w| <= 2^21 and activations <= 2^100 no sum of 32 products overflows, so no
            // infinity or NaN can arise inside the chain
            if (std::fabs(val[k]) > 2097152.0f) return "weight magnitude above 2^21";
            if (k > b && col[k] < col[k - 1]) sorted = false;
        }
        if (sorted) {
            std::copy(col + b, col + e, oc.begin() + b);
            std::copy(val + b, val + e, ov.begin() + b);
        } else {
            order.resize((size_t)(e - b));
            std::iota(order.begin(), order.end(), b);
            std::stable_sort(order.begin(), order.end(), [&](int32_t x, int32_t y) { return col[x] < col[y]; });
            for (int k = b; k < e; ++k) { oc[k] = col[order[k - b]]; ov[k] = val[order[k - b]]; }
        }
    }
    return std::string();
}

namespace {

// number of common elements of two ascending lists of length K; the common elements go to `common`
// (at most cap of them are stored)
inline int intersect_sorted(const int32_t* a, const int32_t* b, int K, int32_t* common, int cap) {
    int i = 0, j = 0, n = 0;
    while (i < K && j < K) {
        if (a[i] < b[j]) ++i;
        else if (a[i] > b[j]) ++j;
        else { if (n < cap) common[n] = a[i]; ++n; ++i; ++j; }
    }
    return n;
}

inline bool exact_weight(float w) {
    if (w == 0.0f) return true;
    int e = 0;
    const float m = std::frexp(std::fabs(w), &e);  // |w| = m * 2^e, m in [0.5, 1)
    return m == 0.5f && e >= -23 && e <= 25;
}

}  // namespace

bool discover_band(int N, int K, const std::vector<int32_t>& rowptr, const std::vector<int32_t>& col,
                   std::vector<int32_t>& in_pos, std::vector<int32_t>& out_at) {
    if (K < 2 || N < 4 * K) return false;
    // outputs of every input, ascending (counting pass over the rows in ascending output order)
    std::vector<int32_t> outs((size_t)N * K);
    std::vector<int32_t> fill((size_t)N, 0);
    for (int j = 0; j < N; ++j) {
        if (rowptr[j + 1] - rowptr[j] != K) return false;
        for (int e = rowptr[j]; e < rowptr[j + 1]; ++e) {
            const int i = col[e];
            if (fill[i] >= K) return false;
            outs[(size_t)i * K + fill[i]++] = j;
        }
    }
    for (int i = 0; i < N; ++i) if (fill[i] != K) return false;
    auto In = [&](int j) { return col.data() + rowptr[j]; };
    auto Out = [&](int i) { return outs.data() + (size_t)i * K; };
    int32_t tmp[4];

    // --- bootstrap: the 2K-1 inputs around input 0, ordered by how many outputs they share with it
    const int a0 = 0;
    std::vector<int32_t> cnt((size_t)N, 0);
    std::vector<int32_t> touched;
    for (int t = 0; t < K; ++t) {
        const int32_t* in = In(Out(a0)[t]);
        for (int k = 0; k < K; ++k) if (cnt[in[k]]++ == 0) touched.push_back(in[k]);
    }
    if (cnt[a0] != K || (int)touched.size() != 2 * K - 1) return false;
    std::vector<std::array<int32_t, 2>> by((size_t)K, std::array<int32_t, 2>{-1, -1});
    for (int32_t i : touched) {
        if (i == a0) continue;
        const int d = K - cnt[i];
        if (d < 1 || d > K - 1) return false;
        if (by[d][0] < 0) by[d][0] = i;
        else if (by[d][1] < 0) by[d][1] = i;
        else return false;
    }
    std::vector<int32_t> plus((size_t)K), minus((size_t)K);
    plus[0] = minus[0] = a0;
    for (int d = 1; d < K; ++d) {
        if (by[d][0] < 0 || by[d][1] < 0) return false;
        if (d == 1) { plus[1] = by[1][0]; minus[1] = by[1][1]; continue; }
        const int32_t c = by[d][0];
        if (intersect_sorted(Out(c), Out(plus[d - 1]), K, tmp, 0) == K - 1) { plus[d] = c; minus[d] = by[d][1]; }
        else { plus[d] = by[d][1]; minus[d] = c; }
        if (intersect_sorted(Out(plus[d]), Out(plus[d - 1]), K, tmp, 0) != K - 1) return false;
        if (intersect_sorted(Out(minus[d]), Out(minus[d - 1]), K, tmp, 0) != K - 1) return false;
    }

    // --- walk the band: positions 0..K-1 hold minus[K-1..1], a0; the output whose window is
    //     exactly those inputs sits at position K-1
    std::vector<int32_t> in_ext((size_t)N + 2 * K, -1), out_ext((size_t)N + 2 * K, -1);
    for (int d = 1; d < K; ++d) in_ext[K - 1 - d] = minus[d];
    in_ext[K - 1] = a0;
    {
        int found = -1, nfound = 0;
        const int32_t* oa = Out(a0);
        const int32_t* ob = Out(plus[1]);
        for (int t = 0; t < K; ++t)
            if (!std::binary_search(ob, ob + K, oa[t])) { found = oa[t]; ++nfound; }
        if (nfound != 1) return false;
        out_ext[K - 1] = found;
    }
    std::vector<uint8_t> mark((size_t)N, 0);
    for (int p = 0; p < K; ++p) mark[in_ext[p]] = 1;
    {
        const int32_t* in = In(out_ext[K - 1]);
        for (int k = 0; k < K; ++k) if (!mark[in[k]]) return false;
    }
    for (int v = K - 1; v < N + K - 1; ++v) {
        const int32_t a_hi = in_ext[v], a_lo2 = in_ext[v - K + 2];
        // outputs v and v+1 are the only ones reading both the newest and the second-oldest input
        int32_t next;
        if (a_hi == a_lo2) {  // K == 2
            const int32_t* o = Out(a_hi);
            if (o[0] == out_ext[v]) next = o[1];
            else if (o[1] == out_ext[v]) next = o[0];
            else return false;
        } else {
            if (intersect_sorted(Out(a_hi), Out(a_lo2), K, tmp, 4) != 2) return false;
            if (tmp[0] == out_ext[v]) next = tmp[1];
            else if (tmp[1] == out_ext[v]) next = tmp[0];
            else return false;
        }
        int32_t newi = -1;
        const int32_t* in = In(next);
        for (int k = 0; k < K; ++k)
            if (!mark[in[k]]) { if (newi >= 0) return false; newi = in[k]; }
        if (newi < 0) return false;
        mark[in_ext[v - K + 1]] = 0;
        mark[newi] = 1;
        in_ext[v + 1] = newi;
        out_ext[v + 1] = next;
    }
    // the walk went once around: it must close on itself
    for (int p = N; p < N + K; ++p) if (in_ext[p] != in_ext[p - N]) return false;
    if (out_ext[N + K - 1] != out_ext[K - 1]) return false;

    in_pos.assign((size_t)N, -1);
    out_at.assign((size_t)N, -1);
    for (int p = 0; p < N; ++p) {
        if (in_pos[in_ext[p]] >= 0) return false;
        in_pos[in_ext[p]] = p;
    }
    std::vector<uint8_t> seen((size_t)N, 0);
    for (int v = K - 1; v < N + K - 1; ++v) {
        const int j = out_ext[v];
        if (seen[j]) return false;
        seen[j] = 1;
        out_at[v % N] = j;
    }
    // final check, independent of the walk: every output reads exactly the window behind it
    for (int v = 0; v < N; ++v) {
        const int32_t* in = In(out_at[v]);
        for (int k = 0; k < K; ++k) {
            int d = v - in_pos[in[k]];
            if (d < 0) d += N;
            if (d >= K) return false;
        }
    }
    return true;
}

// A band labelling is fixed only up to a rotation and a reflection.  Where the layer is a band in
// ONE labelling of its neurons - neuron j sits at the same place of the band as an input and as an
// output, as in a chain of convolution-like layers over a common (possibly hidden) neuron order -
// that freedom is used up here, the same way for every such layer: reflected if need be so that
// position(j as output) == position(j as input), and rotated so that neuron 0 sits at position 0.
// Consecutive layers of this kind then agree on the labelling of the buffer between them (the
// first writes its outputs exactly where the second reads its inputs, dst = identity), which is
// what lets a pair of them run as one fused launch with the intermediate tile in LDS.  Other
// layers are left as discovered.  Returns whether the layer is of this kind.
bool canonicalize_self_aligned_band(int N, int K, std::vector<int32_t>& in_pos, std::vector<int32_t>& out_at) {
    std::vector<int32_t> out_pos((size_t)N);
    for (int v = 0; v < N; ++v) out_pos[(size_t)out_at[(size_t)v]] = v;
    auto delta = [&](int j) { return ((out_pos[(size_t)j] - in_pos[(size_t)j]) % N + N) % N; };
    const int d0 = delta(0);
    if (d0 != 0 && d0 != K - 1) return false;
    for (int j = 1; j < N; ++j) if (delta(j) != d0) return false;
    if (d0 == K - 1 && K > 1) {  // reflect: input p -> -p-(K-1), output v -> -v
        std::vector<int32_t> oa((size_t)N);
        for (int v = 0; v < N; ++v) oa[(size_t)((N - v) % N)] = out_at[(size_t)v];
        out_at.swap(oa);
        for (int i = 0; i < N; ++i) in_pos[(size_t)i] = (((-in_pos[(size_t)i] - (K - 1)) % N) + N) % N;
    }
    const int r = in_pos[0];
    if (r != 0) {
        for (int i = 0; i < N; ++i) in_pos[(size_t)i] = (in_pos[(size_t)i] - r + N) % N;
        std::vector<int32_t> oa((size_t)N);
        for (int v = 0; v < N; ++v) oa[(size_t)v] = out_at[(size_t)((v + r) % N)];
        out_at.swap(oa);
    }
    return true;
}

bool discover_blocks(int N, const std::vector<int32_t>& rowptr, const std::vector<int32_t>& col,
                     std::vector<std::vector<int32_t>>& groups) {
    groups.clear();
    for (int j = 0; j < N; ++j) {
        const int len = rowptr[j + 1] - rowptr[j];
        if (len < 1 || len > 32) return false;
    }
    // order the outputs by their input list; equal lists become neighbours
    std::vector<int32_t> order((size_t)N);
    std::iota(order.begin(), order.end(), 0);
    auto less = [&](int32_t a, int32_t b) {
        const int la = rowptr[a + 1] - rowptr[a], lb = rowptr[b + 1] - rowptr[b];
        if (la != lb) return la < lb;
        const int c = std::memcmp(col.data() + rowptr[a], col.data() + rowptr[b], (size_t)la * sizeof(int32_t));
        if (c != 0) return c < 0;
        return a < b;
    };
    auto same = [&](int32_t a, int32_t b) {
        const int la = rowptr[a + 1] - rowptr[a], lb = rowptr[b + 1] - rowptr[b];
        return la == lb && std::memcmp(col.data() + rowptr[a], col.data() + rowptr[b], (size_t)la * sizeof(int32_t)) == 0;
    };
    std::sort(order.begin(), order.end(), less);
    for (int i = 0; i < N;) {
        int e = i + 1;
        while (e < N && same(order[(size_t)i], order[(size_t)e])) ++e;
        for (int b = i; b < e; b += 16)
            groups.emplace_back(order.begin() + b, order.begin() + std::min(e, b + 16));
        i = e;
    }
    // worth it only if an input column loaded into registers is reused by several outputs
    if ((int64_t)groups.size() * 8 > (int64_t)N) return false;

    // Chain order: put groups that share inputs next to each other (greedy nearest neighbour on
    // the number of shared inputs), so that a wave walking consecutive groups finds the columns
    // it re-reads still in L2.
    const int ng = (int)groups.size();
    std::vector<std::vector<int32_t>> users((size_t)N);  // groups reading each input
    for (int g = 0; g < ng; ++g) {
        const int j0 = groups[(size_t)g][0];
        for (int e = rowptr[j0]; e < rowptr[j0 + 1]; ++e) users[(size_t)col[e]].push_back(g);
    }
    std::vector<uint8_t> placed((size_t)ng, 0);
    std::vector<int32_t> shared((size_t)ng, 0), touched;
    std::vector<std::vector<int32_t>> ordered;
    ordered.reserve((size_t)ng);
    int next_fresh = 0;
    for (int cur = 0, done = 0; done < ng; ++done) {
        if (done == 0 || cur < 0) {
            while (placed[(size_t)next_fresh]) ++next_fresh;
            cur = next_fresh;
        }
        placed[(size_t)cur] = 1;
        ordered.push_back(std::move(groups[(size_t)cur]));
        const int j0 = ordered.back()[0];
        touched.clear();
        for (int e = rowptr[j0]; e < rowptr[j0 + 1]; ++e)
            for (int32_t g : users[(size_t)col[e]])
                if (!placed[(size_t)g] && shared[(size_t)g]++ == 0) touched.push_back(g);
        int best = -1;
        for (int32_t g : touched) {
            if (best < 0 || shared[(size_t)g] > shared[(size_t)best] ||
                (shared[(size_t)g] == shared[(size_t)best] && g < best))
                best = g;
        }
        for (int32_t g : touched) shared[(size_t)g] = 0;
        cur = best;
    }
    groups.swap(ordered);
    return true;
}

bool discover_run_chains(int N, const std::vector<int32_t>& rowptr, const std::vector<int32_t>& col,
                         const std::vector<std::vector<int32_t>>& groups, std::vector<int32_t>& in_pos,
                         std::vector<int32_t>& out_at, int* cycles) {
    const int G = 16, K = 32, R = 16;
    int ncycles = 0;
    if (N % 256 != 0 || (int)groups.size() * G != N) return false;
    const int ng = N / G;
    for (const auto& g : groups)
        if ((int)g.size() != G || rowptr[g[0] + 1] - rowptr[g[0]] != K) return false;
    // the two groups reading every input
    std::vector<int32_t> user((size_t)N * 2, -1);
    for (int g = 0; g < ng; ++g) {
        const int j0 = groups[(size_t)g][0];
        for (int e = rowptr[j0]; e < rowptr[j0 + 1]; ++e) {
            int32_t* u = &user[(size_t)col[e] * 2];
            if (u[0] < 0) u[0] = g;
            else if (u[1] < 0) u[1] = g;
            else return false;
        }
    }
    for (int i = 0; i < N; ++i) if (user[(size_t)i * 2 + 1] < 0) return false;
    // neighbours of a group: the other reader of each of its inputs
    auto other = [&](int g, int input) {
        const int32_t* u = &user[(size_t)input * 2];
        return u[0] == g ? u[1] : u[0];
    };
    // inputs group g shares with group h, in ascending input index
    auto shared_with = [&](int g, int h, std::vector<int32_t>& out) {
        out.clear();
        const int j0 = groups[(size_t)g][0];
        for (int e = rowptr[j0]; e < rowptr[j0 + 1]; ++e)
            if (other(g, col[e]) == h) out.push_back(col[e]);
    };
    in_pos.assign((size_t)N, -1);
    out_at.assign((size_t)N, -1);
    std::vector<uint8_t> seen((size_t)ng, 0);
    std::vector<int32_t> cyc, run;
    int base = 0;  // run index of the first run of the current cycle
    for (int start = 0; start < ng; ++start) {
        if (seen[(size_t)start]) continue;
        // walk the cycle of groups start -> ... -> start, each sharing one run with the next
        cyc.clear();
        int prev = -1, cur = start;
        for (int steps = 0;; ++steps) {
            if (steps > ng || seen[(size_t)cur]) return false;
            seen[(size_t)cur] = 1;
            cyc.push_back(cur);
            const int j0 = groups[(size_t)cur][0];
            int a = -1, b = -1;  // the one or two groups this one shares inputs with
            for (int e = rowptr[j0]; e < rowptr[j0 + 1]; ++e) {
                const int o = other(cur, col[e]);
                if (o == cur) return false;
                if (a < 0 || o == a) a = o;
                else if (b < 0 || o == b) b = o;
                else return false;
            }
            int next;
            if (b < 0) {                 // both runs shared with the same group: a cycle of two
                if (prev >= 0 && a != prev) return false;
                if (prev >= 0) break;    // second group of the pair
                next = a;
            } else if (prev < 0) next = a;
            else if (a == prev) next = b;
            else if (b == prev) next = a;
            else return false;
            if (next == start) break;
            prev = cur;
            cur = next;
        }
        const int c = (int)cyc.size();
        if (c < 2) return false;
        // run i is what group i-1 and group i share; group i reads runs i and i+1 (mod c).
        // Fold the cycle (0, c-1, 1, c-2, ...) so that the two runs of every group lie at most two
        // run slots apart, and give group i the slot of its later run - or, for the one group
        // whose runs sit at the fold's end, the slot after it.
        auto fold = [&](int i) { return i < (c + 1) / 2 ? 2 * i : 2 * (c - 1 - i) + 1; };
        for (int i = 0; i < c; ++i) {
            const int gprev = cyc[(size_t)((i + c - 1) % c)], g = cyc[(size_t)i];
            shared_with(g, gprev, run);
            if (c == 2) {
                if ((int)run.size() != 2 * R) return false;
                if (i == 0) run.erase(run.begin(), run.begin() + R); else run.resize((size_t)R);
            }
            if ((int)run.size() != R) return false;
            const int slot = base + fold(i);
            for (int k = 0; k < R; ++k) {
                if (in_pos[(size_t)run[(size_t)k]] >= 0) return false;
                in_pos[(size_t)run[(size_t)k]] = slot * R + k;
            }
        }
        for (int i = 0; i < c; ++i) {
            const int fa = fold(i), fb = fold((i + 1) % c);
            const int lo = std::min(fa, fb), hi = std::max(fa, fb);
            int t;
            if (hi - lo == 2) t = hi;
            else if (lo == 0) t = 1;      // runs at fold slots 0 and 1
            else t = c;                   // runs at the last two fold slots
            if (c == 2) t = i == 0 ? 1 : 2;
            const int slot = (base + t) % ng;
            for (int o = 0; o < G; ++o) {
                if (out_at[(size_t)slot * G + o] >= 0) return false;
                out_at[(size_t)slot * G + o] = groups[(size_t)cyc[(size_t)i]][(size_t)o];
            }
        }
        base += c;
        ++ncycles;
    }
    if (base != ng) return false;
    if (cycles) *cycles = ncycles;
    // full check of what the kernel assumes: every entry of the output at position v lies in
    // [16*floor(v/16) - 32, 16*floor(v/16) + 15] (mod N)
    for (int v = 0; v < N; ++v) {
        const int j = out_at[(size_t)v];
        if (j < 0) return false;
        const int top = (v / G) * G + G - 1;
        for (int e = rowptr[j]; e < rowptr[j + 1]; ++e) {
            const int p = in_pos[(size_t)col[e]];
            if (p < 0) return false;
            const int back = ((top - p) % N + N) % N;
            if (back > 2 * R + G - 1) return false;
        }
    }
    return true;
}

bool common_run_order(int N, const std::vector<int32_t>& rowptr, const std::vector<int32_t>& col,
                      std::vector<int32_t>& pos) {
    const int G = 16;
    if (N % 256 != 0) return false;
    std::vector<std::vector<int32_t>> groups;
    if (!discover_blocks(N, rowptr, col, groups) || (int)groups.size() * G != N) return false;
    const int ng = N / G;
    std::vector<int32_t> group_of((size_t)N, -1);
    for (int g = 0; g < ng; ++g) {
        if ((int)groups[(size_t)g].size() != G) return false;
        for (int32_t j : groups[(size_t)g]) group_of[(size_t)j] = g;
    }
    // every group reads its own 16 neurons and the 16 neurons of one other group
    std::vector<int32_t> other((size_t)ng, -1);
    for (int g = 0; g < ng; ++g) {
        const int j0 = groups[(size_t)g][0];
        if (rowptr[j0 + 1] - rowptr[j0] != 2 * G) return false;
        int own = 0, far = 0;
        for (int e = rowptr[j0]; e < rowptr[j0 + 1]; ++e) {
            const int h = group_of[(size_t)col[e]];
            if (h == g) ++own;
            else if (other[(size_t)g] < 0 || other[(size_t)g] == h) { other[(size_t)g] = h; ++far; }
            else return false;
        }
        if (own != G || far != G) return false;
    }
    // one cycle through all groups; the group a slot reads lies one slot back
    std::vector<int32_t> slot((size_t)ng, -1);
    int g = 0;
    for (int t = 0; t < ng; ++t) {
        if (slot[(size_t)g] >= 0) return false;
        slot[(size_t)g] = (ng - t) % ng;
        g = other[(size_t)g];
    }
    if (g != 0) return false;
    pos.assign((size_t)N, -1);
    for (int h = 0; h < ng; ++h)
        for (int o = 0; o < G; ++o) pos[(size_t)groups[(size_t)h][(size_t)o]] = slot[(size_t)h] * G + o;
    return true;
}

int common_order_offset(int N, const std::vector<int32_t>& rowptr, const std::vector<int32_t>& col,
                        const std::vector<int32_t>& pos) {
    const int G = 16;
    if (N % 256 != 0 || (int)pos.size() != N) return 0;
    const int ng = N / G;
    int d = 0;
    for (int j = 0; j < N; ++j) {
        if (rowptr[j + 1] - rowptr[j] != 2 * G) return 0;
        const int t = pos[(size_t)j] / G;
        int own = 0, far = 0;
        for (int e = rowptr[j]; e < rowptr[j + 1]; ++e) {
            const int back = ((t - pos[(size_t)col[e]] / G) % ng + ng) % ng;
            if (back == 0) ++own;
            else if ((back == 1 || back == 2) && (d == 0 || d == back)) { d = back; ++far; }
            else return 0;
        }
        if (own != G || far != G) return 0;
    }
    return d;
}

// TILED plan (layers that are neither a band nor groups of identical rows).  Outputs are cut into
// tiles of 1024; a tile's input columns - the union over its outputs, ascending - are staged in LDS
// in panels of 512 columns and every output of the tile takes its inputs from there, so a column
// is read from memory once per tile instead of once per entry (the reference's general prototype
// stages a block's input list in shared memory the same way, src/microbenchmark/
// row-succ-no-transpose.cu:15-71).  A wave owns 64 outputs of the tile; per panel it works through
// `rounds` rounds of 2 entries per output (outputs with fewer entries in the panel are padded with
// weight -0), so the outputs of a tile are sorted by length before they are dealt to the waves.
// Accumulation order: an output's entries are ascending in input index, the union is ascending, so
// panel after panel, entry after entry is the order of the reference's CPU checker.
// Returns false (plan untouched) when staging would not pay: more than four reads per input column.
bool build_tiled_plan(int N, const std::vector<int32_t>& rowptr, const std::vector<int32_t>& col,
                      const std::vector<float>& val, LayerPlan& plan) {
    constexpr int TO = kTileOutputs, PC = kPanelCols, WO = 64, NWV = TO / WO;
    if (N < 64 || rowptr[N] == 0) return false;   // (a layer without any entry: nothing to stage)
    const int ntiles = (N + TO - 1) / TO;
    // outputs in the order of the middle of their input lists, so that a tile's union stays small
    // where the layer has locality; empty rows last
    std::vector<int32_t> order((size_t)N);
    std::iota(order.begin(), order.end(), 0);
    auto mid = [&](int j) { return rowptr[j + 1] > rowptr[j] ? col[(size_t)(rowptr[j] + rowptr[j + 1]) / 2] : INT32_MAX; };
    std::stable_sort(order.begin(), order.end(), [&](int32_t a, int32_t b) { return mid(a) < mid(b); });
    std::vector<int32_t> out_at((size_t)ntiles * TO, -1), cols, hdr((size_t)2 * ntiles, 0), wave_hdr;
    std::vector<float> ent;
    std::vector<int32_t> slot_of((size_t)N, -1);
    int64_t staged = 0;
    int gp = 0;  // panels so far
    for (int t = 0; t < ntiles; ++t) {
        const int o0 = t * TO, o1 = std::min(N, o0 + TO);
        std::vector<int32_t> outs(order.begin() + o0, order.begin() + o1);
        std::vector<int32_t> uni;
        for (int32_t j : outs) uni.insert(uni.end(), col.begin() + rowptr[j], col.begin() + rowptr[j + 1]);
        std::sort(uni.begin(), uni.end());
        uni.erase(std::unique(uni.begin(), uni.end()), uni.end());
        staged += (int64_t)uni.size();
        if (staged > 4 * (int64_t)N) return false;
        for (size_t k = 0; k < uni.size(); ++k) slot_of[(size_t)uni[k]] = (int32_t)k;
        const int np = (int)((uni.size() + PC - 1) / PC);
        // The 64 outputs of a wave pad, panel by panel, to the longest among them: deal the outputs to
        // the waves so that a wave's outputs are alike in the FIRST panel and, inside a quarter of the
        // tile, in the rest (on 1..24 random inputs per output of 1024: 19 000 entries with padding
        // instead of 22 700 when sorted by length alone; 13 200 are real).
        {
            auto first = [&](int32_t j) {
                int c = 0;
                for (int e = rowptr[j]; e < rowptr[j + 1] && slot_of[(size_t)col[e]] < PC; ++e) ++c;
                return c;
            };
            std::vector<std::pair<int, int>> cnt(outs.size());   // (entries in the first panel, in the others)
            std::vector<int32_t> idx(outs.size());
            for (size_t k = 0; k < outs.size(); ++k) {
                const int f = np > 1 ? first(outs[k]) : 0;
                cnt[k] = {f, rowptr[outs[k] + 1] - rowptr[outs[k]] - f};
                idx[k] = (int32_t)k;
            }
            std::stable_sort(idx.begin(), idx.end(), [&](int32_t a, int32_t b) { return cnt[(size_t)a].first > cnt[(size_t)b].first; });
            const size_t quarter = ((outs.size() + 3) / 4 + WO - 1) / WO * WO;
            for (size_t b0 = 0; b0 < idx.size(); b0 += quarter)
                std::stable_sort(idx.begin() + (long)b0, idx.begin() + (long)std::min(idx.size(), b0 + quarter),
                                 [&](int32_t a, int32_t b) { return cnt[(size_t)a].second > cnt[(size_t)b].second; });
            std::vector<int32_t> dealt(outs.size());
            for (size_t k = 0; k < outs.size(); ++k) dealt[k] = outs[(size_t)idx[k]];
            outs.swap(dealt);
        }
        hdr[(size_t)2 * t] = gp;
        hdr[(size_t)2 * t + 1] = np;
        for (size_t k = 0; k < outs.size(); ++k) out_at[(size_t)o0 + k] = outs[k];
        for (int p = 0; p < np; ++p) {
            for (int sl = 0; sl < PC; ++sl) {
                const size_t k = (size_t)p * PC + sl;
                cols.push_back(k < uni.size() ? uni[k] : uni[(size_t)p * PC]);  // padding: a column of this panel
            }
            for (int w = 0; w < NWV; ++w) {
                // entries of the wave's outputs that fall into this panel
                int maxc = 0;
                std::vector<std::pair<int, int>> rng((size_t)WO, {0, 0});
                for (int o = 0; o < WO; ++o) {
                    const size_t k = (size_t)w * WO + o;
                    if (k >= outs.size()) continue;
                    const int j = outs[k];
                    int b = rowptr[j], e = rowptr[j + 1];
                    while (b < e && slot_of[(size_t)col[b]] / PC < p) ++b;
                    int e2 = b;
                    while (e2 < e && slot_of[(size_t)col[e2]] / PC == p) ++e2;
                    rng[(size_t)o] = {b, e2};
                    maxc = std::max(maxc, e2 - b);
                }
                const int rounds = (maxc + 1) / 2;
                wave_hdr.push_back(rounds);
                wave_hdr.push_back((int32_t)(ent.size() / 256));
                for (int r = 0; r < rounds; ++r)
                    for (int o = 0; o < WO; ++o)
                        for (int k = 0; k < 2; ++k) {
                            const int e = rng[(size_t)o].first + r * 2 + k;
                            uint32_t off = 0;
                            float wgt = -0.0f;  // padding: adds an exact zero; the sign tells it from a stored zero weight
                            if (e < rng[(size_t)o].second) {
                                off = (uint32_t)(slot_of[(size_t)col[e]] % PC) * 256u;
                                wgt = val[e] == 0.0f ? 0.0f : val[e];
                            }
                            float f;
                            memcpy(&f, &off, 4);
                            ent.push_back(f);
                            ent.push_back(wgt);
                        }
            }
        }
        gp += np;
        if (ent.size() / 256 > (size_t)INT32_MAX / 2) return false;
    }
    plan.out_at.swap(out_at);
    plan.ell_col.swap(cols);
    plan.rowlen.swap(hdr);
    plan.rowlen.insert(plan.rowlen.end(), wave_hdr.begin(), wave_hdr.end());
    plan.wv.swap(ent);
    plan.ntiles = ntiles;
    return true;
}

// Longest merged step list over the pairs of neighbouring band positions (2u, 2u+1): the two outputs
// add their inputs in ascending input index, a shared input is one step.
static int merged_pair_steps(int N, int K, const std::vector<int32_t>& rowptr, const std::vector<int32_t>& col,
                             const std::vector<int32_t>& out_at) {
    int steps = K;
    for (int u = 0; u < N / 2; ++u) {
        const int j0 = out_at[(size_t)2 * u], j1 = out_at[(size_t)2 * u + 1];
        int a = rowptr[j0], b = rowptr[j1], m = 0;
        while (a < rowptr[j0 + 1] || b < rowptr[j1 + 1]) {
            const int ia = a < rowptr[j0 + 1] ? col[a] : INT32_MAX, ib = b < rowptr[j1 + 1] ? col[b] : INT32_MAX;
            if (ia <= ib) ++a;
            if (ib <= ia) ++b;
            ++m;
        }
        steps = std::max(steps, m);
    }
    return steps;
}

// The QUAD form of a BAND layer (see LayerPlan::quad_col): a four-way merge of the outputs' entry lists, which are
// sorted by input index.  Left empty when some quad merges to more than 36 steps.
static void build_quad_form(int N, const std::vector<int32_t>& rowptr, const std::vector<int32_t>& col,
                            const std::vector<float>& val, LayerPlan& plan) {
    const int nq = N / 4;
    int steps = 0;
    std::vector<int32_t> merged;
    auto merge_quad = [&](int c) {
        merged.clear();
        int at[4];
        for (int j = 0; j < 4; ++j) at[j] = rowptr[plan.out_at[(size_t)4 * c + j]];
        for (;;) {
            int32_t in = INT32_MAX;
            for (int j = 0; j < 4; ++j) {
                const int row = plan.out_at[(size_t)4 * c + j];
                if (at[j] < rowptr[row + 1]) in = std::min(in, col[at[j]]);
            }
            if (in == INT32_MAX) break;
            merged.push_back(in);
            for (int j = 0; j < 4; ++j) {
                const int row = plan.out_at[(size_t)4 * c + j];
                if (at[j] < rowptr[row + 1] && col[at[j]] == in) ++at[j];
            }
        }
    };
    for (int c = 0; c < nq; ++c) {
        merge_quad(c);
        steps = std::max(steps, (int)merged.size());
    }
    if (steps < 1 || steps > 36) return;
    const int ng = (steps + 3) / 4;
    plan.quad_groups = ng;
    plan.quad_col.assign((size_t)nq * ng * 4, 0u);
    plan.quad_w.assign((size_t)nq * ng * 16, 0.0f);
    for (int c = 0; c < nq; ++c) {
        merge_quad(c);
        int at[4];
        for (int j = 0; j < 4; ++j) at[j] = rowptr[plan.out_at[(size_t)4 * c + j]];
        const int m_used = (int)merged.size();
        for (int m = 0; m < ng * 4; ++m) {
            const size_t grp = (size_t)c * ng + (size_t)(m >> 2);
            const int32_t in = merged[(size_t)std::min(m, m_used - 1)];   // padding steps: the last column again, weights 0
            plan.quad_col[grp * 4 + (size_t)(m & 3)] = (uint32_t)plan.in_pos[(size_t)in] * (uint32_t)kQuadColumnBytes;
            if (m >= m_used) continue;
            for (int j = 0; j < 4; ++j) {
                const int row = plan.out_at[(size_t)4 * c + j];
                if (at[j] < rowptr[row + 1] && col[at[j]] == in) {
                    plan.quad_w[(grp * 4 + (size_t)(m & 3)) * 4 + (size_t)j] = val[at[j]];
                    ++at[j];
                }
            }
        }
    }
}

void inspect_layer(int N, const std::vector<int32_t>& rowptr, const std::vector<int32_t>& col,
                   const std::vector<float>& val, int force_kernel, bool fma_ok, LayerPlan& plan,
                   const std::vector<int32_t>* common_pos) {
    const int64_t nnz = rowptr[N];
    int kmax = 0;
    bool rows_regular = true, dup = false;
    for (int j = 0; j < N; ++j) {
        const int len = rowptr[j + 1] - rowptr[j];
        kmax = std::max(kmax, len);
        for (int e = rowptr[j] + 1; e < rowptr[j + 1]; ++e) if (col[e] == col[e - 1]) dup = true;
    }
    for (int j = 0; j < N; ++j) if (rowptr[j + 1] - rowptr[j] != kmax) rows_regular = false;
    bool cols_regular = rows_regular;
    if (rows_regular) {
        std::vector<int32_t> cc((size_t)N, 0);
        for (int64_t e = 0; e < nnz; ++e) cc[col[e]]++;
        for (int i = 0; i < N; ++i) if (cc[i] != kmax) { cols_regular = false; break; }
    }
    bool uniform = nnz > 0, exact = true;
    for (int64_t e = 0; e < nnz; ++e) {
        if (val[e] != val[0]) uniform = false;
        if (!exact_weight(val[e])) exact = false;
    }

    plan.kmax = kmax;
    plan.self_aligned = false;
    plan.pair_twins = false;
    plan.fuse_next = false;
    plan.info = spdnn_layer_plan{};
    plan.info.max_row_nnz = kmax;
    plan.info.regular = (rows_regular && cols_regular && !dup) ? 1 : 0;
    plan.info.uniform_value = uniform ? 1 : 0;
    plan.info.value = uniform ? val[0] : 0.0f;
    plan.info.exact_products = exact ? 1 : 0;
    // The fused multiply-add shortcut needs products that never underflow: power-of-two weights
    // AND activations that are zero or well above the denormal range (the caller decides).
    exact = exact && fma_ok;
    plan.info.band_halo = -1;
    plan.info.nnz = nnz;

    bool band = false;
    const int K = kmax;
    if (force_kernel != SPDNN_KERNEL_GATHER && plan.info.regular && K >= 4 && K <= 32 && (K % 4) == 0 &&
        (N % 256) == 0 && N >= 4 * K) {
        band = discover_band(N, K, rowptr, col, plan.in_pos, plan.out_at);
        if (band) plan.self_aligned = canonicalize_self_aligned_band(N, K, plan.in_pos, plan.out_at);
    }

    std::vector<std::vector<int32_t>> groups;
    bool block = !band && force_kernel != SPDNN_KERNEL_GATHER && !dup && discover_blocks(N, rowptr, col, groups);
    int halo = K - 1;
    // Walking the chains with the band kernel beats the BLOCK kernel from N = 4096 up (measured);
    // below that a row block's whole input sits in L2 and the BLOCK kernel's independent waves win.
    const char* chain_env = getenv("SPDNN_RUN_CHAINS_MIN_N");
    const int chain_min_n = chain_env ? atoi(chain_env) : 4096;   // 0 or negative: never
    const bool chains_ok = block && chain_min_n > 0 && N >= chain_min_n && plan.info.regular && K == 32;
    plan.info.common_order = 0;
    if (chains_ok && common_pos && uniform && exact && (plan.info.common_order = common_order_offset(N, rowptr, col, *common_pos)) > 0) {
        // the network's common neuron order is a run-chain labelling of this layer: inputs and outputs
        // both take it, so a neighbour laid out the same way finds the columns where it reads them
        plan.in_pos = *common_pos;
        plan.out_at.assign((size_t)N, 0);
        for (int i = 0; i < N; ++i) plan.out_at[(size_t)plan.in_pos[(size_t)i]] = i;
        band = true;
        block = false;
        halo = 32;
    } else if (chains_ok && discover_run_chains(N, rowptr, col, groups, plan.in_pos, plan.out_at, &plan.rc_cycles)) {
        band = true;    // 16-output groups chained through shared 16-input runs: walked like a band
        block = false;
        halo = 32;
    }

    if (band) {
        // A circulant pair merges to K + 1 steps, a pair inside a group of a run chain to 32; the kernel reads
        // fixed records of at most 36 steps.  A labelling whose pairs merge to more is not walked as a band:
        // the layer keeps its groups (BLOCK) if it has them, else it goes to the general classes.
        if (merged_pair_steps(N, K, rowptr, col, plan.out_at) > 36) {
            band = false;
            block = halo == 32;
            halo = K - 1;
        }
    }

    plan.ngroups = 0;
    plan.blk_cols.clear();
    plan.blk_cnt.clear();
    plan.alt_ngroups = 0;
    plan.alt_full = false;
    plan.alt_cols.clear();
    plan.alt_cnt.clear();
    plan.alt_out_at.clear();
    plan.alt_dst.clear();
    plan.alt_wv.clear();
    plan.rt_ent.clear();
    plan.alt_kmax = 0;
    plan.quad_col.clear();
    plan.quad_w.clear();
    plan.quad_groups = 0;
    if (band && halo == 32 && uniform && exact) {
        // the BLOCK form of a run-chain layer, its columns in the band's input labelling
        plan.alt_ngroups = (int)groups.size();
        plan.alt_full = true;
        plan.alt_cols.assign((size_t)plan.alt_ngroups * 32, 0);
        plan.alt_cnt.resize((size_t)plan.alt_ngroups);
        plan.alt_out_at.assign((size_t)plan.alt_ngroups * 16, -1);
        for (int g = 0; g < plan.alt_ngroups; ++g) {
            const int j0 = groups[(size_t)g][0];
            const int len = rowptr[j0 + 1] - rowptr[j0];
            plan.alt_cnt[(size_t)g] = len;
            if (len != 32) plan.alt_full = false;
            for (int k = 0; k < len; ++k) plan.alt_cols[(size_t)g * 32 + k] = plan.in_pos[(size_t)col[rowptr[j0] + k]];
            for (size_t o = 0; o < groups[(size_t)g].size(); ++o) plan.alt_out_at[(size_t)g * 16 + o] = groups[(size_t)g][o];
        }
    }
    if (block) {
        plan.kernel = SPDNN_KERNEL_BLOCK;
        plan.wmode = (uniform && exact) ? 0 : (exact ? 1 : 2);
        plan.ngroups = (int)groups.size();
        plan.kmax = kmax;
        plan.in_pos.resize((size_t)N);
        std::iota(plan.in_pos.begin(), plan.in_pos.end(), 0);
        plan.out_at.assign((size_t)plan.ngroups * 16, -1);
        plan.blk_cols.assign((size_t)plan.ngroups * 32, 0);
        plan.blk_cnt.resize((size_t)plan.ngroups);
        if (plan.wmode != 0) plan.wv.assign((size_t)plan.ngroups * 16 * 32, 0.0f); else plan.wv.clear();
        plan.blk_full = true;
        for (int g = 0; g < plan.ngroups; ++g) {
            const int j0 = groups[(size_t)g][0];
            const int len = rowptr[j0 + 1] - rowptr[j0];
            plan.blk_cnt[(size_t)g] = len;
            if (len != 32) plan.blk_full = false;
            for (int k = 0; k < len; ++k) plan.blk_cols[(size_t)g * 32 + k] = col[rowptr[j0] + k];
            for (size_t o = 0; o < groups[(size_t)g].size(); ++o) {
                const int j = groups[(size_t)g][o];
                plan.out_at[(size_t)g * 16 + o] = j;
                if (plan.wmode != 0)
                    for (int k = 0; k < len; ++k) plan.wv[((size_t)g * 16 + o) * 32 + k] = val[rowptr[j] + k];
            }
        }
        plan.sel.clear();
        plan.pairs.clear();
        plan.ell_col.clear();
        plan.rowlen.clear();
    } else if (band) {
        plan.kernel = SPDNN_KERNEL_BAND;
        plan.wmode = (uniform && exact) ? 0 : (exact ? 1 : 2);
        plan.info.band_halo = halo;
        plan.sel.resize((size_t)N * K);
        for (int v = 0; v < N; ++v) {
            const int j = plan.out_at[v];
            for (int k = 0; k < K; ++k)   // ascending input index = accumulation order
                plan.sel[(size_t)v * K + k] = (uint8_t)(plan.in_pos[col[rowptr[j] + k]] & 255);
        }
        // Pair records: the outputs at band positions 2u and 2u+1 add their inputs in ascending
        // input index, so the two lists merge into one list of steps in which shared inputs appear
        // once; per step a ring selector, a use bit per output and (unless the layer has one exact
        // value) a weight per output, 0 where the output does not use the step.
        const int npairs = N / 2;
        // (at most 36, checked above: the kernel reads fixed 16-dword records - two use masks, 36 one-byte
        // selectors - and 72 weights per pair)
        const int steps = merged_pair_steps(N, K, rowptr, col, plan.out_at);
        const int trips = 9;
        const int stride = 16;
        plan.pair_steps = steps;
        plan.pair_stride = stride;
        plan.pair_padded = trips * 4;
        plan.pairs.assign((size_t)npairs * stride, 0u);
        if (plan.wmode != 0) plan.wv.assign((size_t)npairs * trips * 8, 0.0f); else plan.wv.clear();
        bool twins = plan.wmode == 0;
        for (int u = 0; u < npairs; ++u) {
            const int j0 = plan.out_at[2 * u], j1 = plan.out_at[2 * u + 1];
            uint32_t* rec = &plan.pairs[(size_t)u * stride];
            uint8_t* slots = reinterpret_cast<uint8_t*>(rec + 4);
            float* w = plan.wmode != 0 ? &plan.wv[(size_t)u * trips * 8] : nullptr;
            uint64_t use0 = 0, use1 = 0;
            int a = rowptr[j0], b = rowptr[j1], m = 0;
            while (a < rowptr[j0 + 1] || b < rowptr[j1 + 1]) {
                const int ia = a < rowptr[j0 + 1] ? col[a] : INT32_MAX, ib = b < rowptr[j1 + 1] ? col[b] : INT32_MAX;
                const int in = std::min(ia, ib);
                slots[m] = (uint8_t)(plan.in_pos[(size_t)in] & 255);
                if (ia == in) { use0 |= 1ull << m; if (w) w[2 * m] = val[a]; ++a; }
                if (ib == in) { use1 |= 1ull << m; if (w) w[2 * m + 1] = val[b]; ++b; }
                ++m;
            }
            // padding steps read a column this pair reads anyway (a live ring slot), with weight 0
            for (int t = m; t < trips * 4; ++t) slots[t] = slots[m - 1];
            rec[0] = (uint32_t)use0; rec[1] = (uint32_t)(use0 >> 32);
            rec[2] = (uint32_t)use1; rec[3] = (uint32_t)(use1 >> 32);
            // every step of the record used by both outputs: under one weight the two are equal
            if (use0 != use1 || use0 != (steps >= 64 ? ~0ull : (1ull << steps) - 1)) twins = false;
        }
        plan.pair_twins = twins;
        plan.ell_col.clear();
        plan.rowlen.clear();
        if (N <= kQuadMaxNeurons) build_quad_form(N, rowptr, col, val, plan);
    } else if (force_kernel != SPDNN_KERNEL_GATHER && !(getenv("SPDNN_TILED") && atoi(getenv("SPDNN_TILED")) == 0) &&
               build_tiled_plan(N, rowptr, col, val, plan)) {
        plan.kernel = SPDNN_KERNEL_TILED;
        plan.wmode = exact ? 1 : 2;
        plan.in_pos.resize((size_t)N);
        std::iota(plan.in_pos.begin(), plan.in_pos.end(), 0);
        plan.sel.clear();
        plan.pairs.clear();
        // its GATHER form, for launches too small to fill the chip with tiles, and its ROWTILE form; both over
        // the outputs ordered by length, longest first
        const int kw = (std::max(kmax, 1) + 3) / 4 * 4;   // (the gather kernel takes four entries per trip: rows padded with column 0, weight +0)
        plan.alt_kmax = kw;
        plan.alt_cols.assign((size_t)N * kw, 0);
        plan.alt_wv.assign((size_t)N * kw, 0.0f);
        plan.alt_cnt.resize((size_t)N);
        plan.alt_out_at.resize((size_t)N);
        std::iota(plan.alt_out_at.begin(), plan.alt_out_at.end(), 0);
        std::stable_sort(plan.alt_out_at.begin(), plan.alt_out_at.end(), [&](int32_t x, int32_t y) {
            return rowptr[x + 1] - rowptr[x] > rowptr[y + 1] - rowptr[y];
        });
        const int kpad = (kw + 3) / 4 * 4;   // the kernel requests entries four at a time
        plan.rt_ent.assign((size_t)kpad * N * 2, 0u);
        for (int slot = 0; slot < N; ++slot) {
            const int j = plan.alt_out_at[(size_t)slot];
            const int len = rowptr[j + 1] - rowptr[j];
            plan.alt_cnt[(size_t)slot] = len;
            for (int k = 0; k < len; ++k) {
                const int32_t c = col[rowptr[j] + k];
                const float w = val[rowptr[j] + k];
                plan.alt_cols[(size_t)slot * kw + k] = c;
                plan.alt_wv[(size_t)slot * kw + k] = w;
                uint32_t wb;
                memcpy(&wb, &w, 4);
                plan.rt_ent[((size_t)k * N + slot) * 2] = (uint32_t)c;
                plan.rt_ent[((size_t)k * N + slot) * 2 + 1] = wb;
            }
        }
    } else {
        plan.kernel = SPDNN_KERNEL_GATHER;
        plan.wmode = exact ? 1 : 2;
        plan.in_pos.resize((size_t)N);
        plan.out_at.resize((size_t)N);
        std::iota(plan.in_pos.begin(), plan.in_pos.end(), 0);
        std::iota(plan.out_at.begin(), plan.out_at.end(), 0);
        const int kw = (std::max(kmax, 1) + 3) / 4 * 4;   // (four entries per trip: rows padded with column 0, weight +0)
        plan.ell_col.assign((size_t)N * kw, 0);
        plan.wv.assign((size_t)N * kw, 0.0f);
        plan.rowlen.resize((size_t)N);
        for (int j = 0; j < N; ++j) {
            const int len = rowptr[j + 1] - rowptr[j];
            plan.rowlen[j] = len;
            for (int k = 0; k < len; ++k) {
                plan.ell_col[(size_t)j * kw + k] = col[rowptr[j] + k];
                plan.wv[(size_t)j * kw + k] = val[rowptr[j] + k];
            }
        }
        plan.kmax = kw;
        plan.sel.clear();
        plan.pairs.clear();
    }
    plan.info.kernel = plan.kernel;
    plan.info.block_form = plan.alt_ngroups > 0 ? 1 : (plan.alt_kmax > 0 ? 2 : 0);
    plan.info.plan_bytes = (int64_t)(4 * (plan.ell_col.size() + plan.rowlen.size() + plan.wv.size() +
                                                              plan.blk_cols.size() + plan.blk_cnt.size() + plan.pairs.size() +
                                                              plan.alt_cols.size() + plan.alt_cnt.size() + plan.alt_out_at.size() + plan.alt_wv.size() + plan.rt_ent.size() + plan.quad_col.size() + plan.quad_w.size() +
                                                              plan.out_at.size() + (size_t)N));
    plan.dst.clear();
    plan.failed = false;
    plan.set = true;
}

void plan_adjacency(const LayerPlan& p, int N, std::vector<int32_t>& rowptr, std::vector<int32_t>& col) {
    rowptr.assign((size_t)N + 1, 0);
    col.clear();
    std::vector<std::vector<int32_t>> ins((size_t)N);
    if (p.kernel == SPDNN_KERNEL_BAND) {
        const int K = p.kmax, halo = p.info.band_halo;
        std::vector<int32_t> in_at((size_t)N);
        for (int i = 0; i < N; ++i) in_at[(size_t)p.in_pos[(size_t)i]] = i;
        for (int v = 0; v < N; ++v) {
            // an input of position v lies in [base - halo, base + span): the one position of that
            // range congruent to the selector mod 256
            const int base = halo == K - 1 ? v : v / 16 * 16, lo = base - halo;
            for (int k = 0; k < K; ++k) {
                const int sel = p.sel[(size_t)v * K + k];
                const int q = lo + (((sel - lo) % 256) + 256) % 256;
                ins[(size_t)p.out_at[(size_t)v]].push_back(in_at[(size_t)(((q % N) + N) % N)]);
            }
        }
    } else if (p.kernel == SPDNN_KERNEL_BLOCK) {
        for (int g = 0; g < p.ngroups; ++g)
            for (int o = 0; o < 16; ++o) {
                const int j = p.out_at[(size_t)g * 16 + o];
                if (j < 0) continue;
                for (int k = 0; k < p.blk_cnt[(size_t)g]; ++k) ins[(size_t)j].push_back(p.blk_cols[(size_t)g * 32 + k]);
            }
    } else if (p.kernel == SPDNN_KERNEL_TILED) {
        const int32_t* wave_hdr = p.rowlen.data() + 2 * p.ntiles;
        for (int t = 0; t < p.ntiles; ++t) {
            const int gp0 = p.rowlen[(size_t)2 * t], np = p.rowlen[(size_t)2 * t + 1];
            for (int q = 0; q < np; ++q)
                for (int w = 0; w < kTileOutputs / 64; ++w) {
                    const int rounds = wave_hdr[((size_t)(gp0 + q) * 16 + w) * 2];
                    const size_t blk = (size_t)wave_hdr[((size_t)(gp0 + q) * 16 + w) * 2 + 1];
                    for (int r = 0; r < rounds; ++r)
                        for (int o = 0; o < 64; ++o)
                            for (int k = 0; k < 2; ++k) {
                                const size_t at = ((blk + r) * 128 + (size_t)o * 2 + k) * 2;
                                if (p.wv[at + 1] == 0.0f && std::signbit(p.wv[at + 1])) continue;  // padding
                                uint32_t off;
                                memcpy(&off, &p.wv[at], 4);
                                const int j = p.out_at[(size_t)t * kTileOutputs + w * 64 + o];
                                ins[(size_t)j].push_back(p.ell_col[(size_t)(gp0 + q) * kPanelCols + off / 256]);
                            }
                }
        }
    } else {
        for (int j = 0; j < N; ++j)
            for (int k = 0; k < p.rowlen[(size_t)j]; ++k) ins[(size_t)j].push_back(p.ell_col[(size_t)j * p.kmax + k]);
    }
    for (int j = 0; j < N; ++j) {
        std::sort(ins[(size_t)j].begin(), ins[(size_t)j].end());
        rowptr[(size_t)j + 1] = rowptr[(size_t)j] + (int32_t)ins[(size_t)j].size();
        col.insert(col.end(), ins[(size_t)j].begin(), ins[(size_t)j].end());
    }
}

void receptive_field(const LayerPlan* plans, int N, int n_layers, const int32_t* outs, int n_out,
                     std::vector<int32_t>& inputs) {
    std::vector<uint8_t> need((size_t)N, 0), next((size_t)N, 0);
    for (int t = 0; t < n_out; ++t) need[(size_t)outs[t]] = 1;
    std::vector<int32_t> rowptr, col;
    for (int l = n_layers - 1; l >= 0; --l) {   // from the last layer of the range back to its first
        plan_adjacency(plans[l], N, rowptr, col);
        std::fill(next.begin(), next.end(), 0);
        for (int j = 0; j < N; ++j)
            if (need[(size_t)j])
                for (int e = rowptr[(size_t)j]; e < rowptr[(size_t)j + 1]; ++e) next[(size_t)col[(size_t)e]] = 1;
        need.swap(next);
    }
    inputs.clear();
    for (int i = 0; i < N; ++i) if (need[(size_t)i]) inputs.push_back(i);
}

bool pair_fusable(const LayerPlan& a, const LayerPlan& b, int N) {
    if (a.kernel != SPDNN_KERNEL_BAND || b.kernel != SPDNN_KERNEL_BAND) return false;
    if (a.kmax != 32 || b.kmax != 32 || a.wmode != b.wmode) return false;
    if (a.pair_steps > 36 || b.pair_steps > 36 || a.pair_stride != 16 || b.pair_stride != 16) return false;
    if (a.info.band_halo > 32 || b.info.band_halo > 32 || N < 256 || (N % 256) != 0) return false;
    if ((int)a.dst.size() != N) return false;
    for (int v = 0; v < N; ++v) if (a.dst[(size_t)v] != v) return false;
    return true;
}

void link_layers(LayerPlan& cur, const std::vector<int32_t>* next_in_pos) {
    auto link = [&](const std::vector<int32_t>& out_at, std::vector<int32_t>& dst) {
        const size_t slots = out_at.size();  // N, or 16 per group with -1 padding for BLOCK layers
        dst.resize(slots);
        for (size_t s = 0; s < slots; ++s) {
            const int32_t j = out_at[s];
            dst[s] = j < 0 ? -1 : (next_in_pos ? (*next_in_pos)[(size_t)j] : j);
        }
    };
    link(cur.out_at, cur.dst);
    link(cur.alt_out_at, cur.alt_dst);
}

}  // namespace spdnn
