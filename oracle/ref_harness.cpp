// Command-line harness around the reference's own CPU code.
//
// TEST INFRASTRUCTURE ONLY.  This file contains no reference source: it #includes the
// reference's host headers where they lie (-I<reference>/src, see Makefile) and is built into
// oracle/_ref/ref_check, which exists only in a container that has the reference mounted.
// The tests use it to pin the CPU oracle (spdnn_oracle.c):
//
//   ref_check coo  <weights.tsv>
//       load with ftxj::COOMatrix(file, 1, false) (src/utils/matrix.h:255-282), sort with
//       to_row_first_ordered (matrix.h:245-253) and print "row col val" per element plus the
//       dimensions: the loader's orientation and the accumulation order, bit for bit.
//   ref_check hash <buckets> <domain>
//       print ftxj::HashReorder(buckets, domain).reorder(v) for every v (src/reorder/hash.h:14-31).
//   ref_check spmm <weights.tsv> <neuron> <batch> <input.f32> <output.f32>
//       ftxj::CpuSpmm::run_and_cmp(coo, input, neuron, batch, output, false, true, true)
//       (src/utils/cpu_spmm.h:11-55): prints "[Success]" or aborts on a mismatch > 1e-3.
//   ref_check fuse <neuron> <batch> <int-bias> <input.f32> <output.f32> <w1.tsv> [<w2.tsv> ...]
//       ftxj::CpuSpmmFuse::run_and_cmp(...) (src/utils/cpu_spmm_fuse.h:11-94), same verdict.
//   ref_check transpose_delete <neuron> <old_batch> <new_batch> <input_T.f32> <map.i32> <output.f32>
//       ftxj::CpuTransposeDelete::run_and_cmp (src/utils/cpu_transpose_and_delete.h:11-27).
//   ref_check need_access <block> <w_last.tsv> [<w_before.tsv> ...]
//       ftxj::FuseLayer (src/fuse/fuse.h:8-54) over blocks of <block> consecutive columns of the
//       first file, then fuse() with every further file, then print_need_access().  The files are
//       loaded with COOMatrix(file, 1, true), i.e. row = first number of a line = input neuron and
//       col = second number = output neuron, so that the class's "rows a block of columns needs"
//       reads as "input neurons a block of output neurons needs".
#include <set>
#include "utils/header.h"
#include "reorder/header.h"
#include "fuse/fuse.h"

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

static std::vector<float> read_f32(const char* path, size_t n) {
    std::vector<float> v(n);
    FILE* f = fopen(path, "rb");
    if (!f) { fprintf(stderr, "cannot open %s\n", path); exit(2); }
    if (fread(v.data(), sizeof(float), n, f) != n) { fprintf(stderr, "short read %s\n", path); exit(2); }
    fclose(f);
    return v;
}

static std::vector<int> read_i32(const char* path, size_t n) {
    std::vector<int> v(n);
    FILE* f = fopen(path, "rb");
    if (!f) { fprintf(stderr, "cannot open %s\n", path); exit(2); }
    if (fread(v.data(), sizeof(int), n, f) != n) { fprintf(stderr, "short read %s\n", path); exit(2); }
    fclose(f);
    return v;
}

int main(int argc, char** argv) {
    if (argc < 2) { fprintf(stderr, "usage: ref_check coo|hash|spmm|fuse|transpose_delete|need_access ...\n"); return 2; }
    std::string cmd = argv[1];
    if (cmd == "coo" && argc == 3) {
        ftxj::COOMatrix coo(argv[2], 1, false);
        coo.to_row_first_ordered();
        printf("%d %d %d\n", coo.row_number, coo.col_number, coo.nnzs);
        for (auto it = coo.begin(); it != coo.end(); ++it) {
            auto e = *it;
            printf("%d %d %.9g\n", e.row, e.col, (double)e.val);
        }
        return 0;
    }
    if (cmd == "hash" && argc == 4) {
        int buckets = atoi(argv[2]), domain = atoi(argv[3]);
        ftxj::HashReorder h(buckets, domain);
        for (int v = 0; v < domain; ++v) printf("%d\n", h.reorder(v));
        return 0;
    }
    if (cmd == "spmm" && argc == 7) {
        int neuron = atoi(argv[3]), batch = atoi(argv[4]);
        ftxj::COOMatrix coo(argv[2], 1, false);
        auto in = read_f32(argv[5], (size_t)neuron * batch);
        auto out = read_f32(argv[6], (size_t)neuron * batch);
        ftxj::CpuSpmm::run_and_cmp(coo, in.data(), neuron, batch, out.data(), false, true, true);
        return 0;
    }
    if (cmd == "fuse" && argc >= 8) {
        int neuron = atoi(argv[2]), batch = atoi(argv[3]), bias = atoi(argv[4]);
        auto in = read_f32(argv[5], (size_t)neuron * batch);
        auto out = read_f32(argv[6], (size_t)neuron * batch);
        std::vector<ftxj::COOMatrix> w;
        for (int i = 7; i < argc; ++i) w.push_back(ftxj::COOMatrix(argv[i], 1, false));
        ftxj::CpuSpmmFuse::run_and_cmp(w, in.data(), neuron, batch, bias, out.data(), (int)w.size(),
                                       false, true, true);
        return 0;
    }
    if (cmd == "transpose_delete" && argc == 8) {
        int neuron = atoi(argv[2]), old_batch = atoi(argv[3]), new_batch = atoi(argv[4]);
        auto in = read_f32(argv[5], (size_t)neuron * old_batch);
        auto map = read_i32(argv[6], (size_t)old_batch);
        auto out = read_f32(argv[7], (size_t)neuron * new_batch);
        ftxj::CpuTransposeDelete::run_and_cmp(in.data(), map.data(), old_batch, neuron, new_batch, out.data());
        return 0;
    }
    if (cmd == "need_access" && argc >= 4) {
        const int block = atoi(argv[2]);
        ftxj::COOMatrix last(argv[3], 1, true);
        std::vector<std::vector<int>> block_cols;
        for (int c = 0; c < last.col_number; c += block) {
            block_cols.push_back(std::vector<int>());
            for (int j = c; j < c + block && j < last.col_number; ++j) block_cols.back().push_back(j);
        }
        ftxj::FuseLayer fuse(last, block_cols);
        for (int i = 4; i < argc; ++i) fuse.fuse(ftxj::COOMatrix(argv[i], 1, true));
        fuse.print_need_access();
        return 0;
    }
    fprintf(stderr, "bad arguments\n");
    return 2;
}
