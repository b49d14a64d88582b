// The reference-side binding of the library, written out and built against the reference's own
// host code.
//
// TEST INFRASTRUCTURE ONLY.  This file contains no reference source: it #includes the
// reference's host headers where they lie (-I<reference>/src, see Makefile) and is built into
// oracle/_ref/ref_binding, only in a container that has the reference mounted.  It is what a
// maintainer of the reference would put into src/network.cpp in place of the inspector and the
// call of test_benchmark_graph_challenge (src/network.cpp:87-123): the weights are loaded by the
// reference's ftxj::COOMatrix (src/utils/matrix.h:255-282) and sorted by its
// to_row_first_ordered (matrix.h:245-253), the features are read like its read_input
// (src/network.cpp:33-54) into the same vector<vector<float>>, and everything after that goes
// through the C ABI of include/spdnn.h.
//
//   ref_binding <neuron> <batch> <layer> <data-dir> <bias>
//
// prints "layer l, batch = n" per layer (the reference's line, all_network.cu:508) and
// "category i" for every surviving row (0-based).
#include "utils/header.h"

#include <cstdio>
#include <cstdlib>
#include <fstream>
#include <iostream>
#include <string>
#include <vector>

#include "../include/spdnn.h"

#define CHECK(call)                                                                  \
    do {                                                                             \
        int rc_ = (call);                                                            \
        if (rc_ != SPDNN_OK) {                                                       \
            fprintf(stderr, "%s failed (%d): %s\n", #call, rc_, spdnn_last_error()); \
            return 1;                                                                \
        }                                                                            \
    } while (0)

int main(int argc, char** argv) {
    if (argc != 6) {
        std::cout << "Usage: exe neuron batch layer data-dir bias" << std::endl;
        return 2;
    }
    const int neuron = atoi(argv[1]), batch = atoi(argv[2]), layer = atoi(argv[3]);
    const std::string data = argv[4];
    const float bias = (float)atof(argv[5]);

    spdnn_net* net = nullptr;
    CHECK(spdnn_create(neuron, batch, layer, bias, 32.0f, &net));
    for (int l = 0; l < layer; ++l) {
        char name[4096];
        CHECK(spdnn_weight_file_name(data.c_str(), neuron, l, name, sizeof(name)));
        ftxj::COOMatrix coo(name, 1, false);  // row = output neuron, col = input neuron
        coo.to_row_first_ordered();
        std::vector<int> rowptr(neuron + 1, 0), col;
        std::vector<float> val;
        for (auto it = coo.begin(); it != coo.end(); ++it) {
            rowptr[(*it).row + 1]++;
            col.push_back((*it).col);
            val.push_back((*it).val);
        }
        for (int j = 0; j < neuron; ++j) rowptr[j + 1] += rowptr[j];
        CHECK(spdnn_set_layer_csr(net, l, rowptr.data(), col.data(), val.data()));
    }
    CHECK(spdnn_inspect(net));

    std::vector<std::vector<float>> input(batch, std::vector<float>(neuron, 0.0f));
    {
        std::ifstream f(data + "/sparse-images-" + std::to_string(neuron) + ".tsv");
        if (!f) {
            std::cout << "input file does not exist" << std::endl;
            return 1;
        }
        int b, n;
        float v;
        while (f >> b >> n >> v)
            if (b <= batch) input[b - 1][n - 1] = v;
    }
    std::vector<float> flat((size_t)batch * neuron);
    for (int b = 0; b < batch; ++b) std::copy(input[b].begin(), input[b].end(), flat.begin() + (size_t)b * neuron);
    CHECK(spdnn_set_features_dense(net, flat.data(), batch));

    spdnn_run_options opt;
    CHECK(spdnn_default_run_options(&opt));
    opt.collect_counts = 1;
    spdnn_run_result res;
    CHECK(spdnn_run(net, &opt, &res));
    for (int l = 0; l < layer; ++l) {
        int64_t n = 0;
        CHECK(spdnn_get_active_count(net, l, &n));
        std::cout << "layer " << l << ", batch = " << n << std::endl;
    }
    int64_t cnt = 0;
    CHECK(spdnn_get_categories(net, nullptr, 0, &cnt));
    std::vector<int32_t> ids((size_t)(cnt > 0 ? cnt : 1));
    CHECK(spdnn_get_categories(net, ids.data(), (int64_t)ids.size(), &cnt));
    for (int64_t i = 0; i < cnt; ++i) std::cout << "category " << ids[(size_t)i] << std::endl;
    CHECK(spdnn_destroy(net));
    return 0;
}
