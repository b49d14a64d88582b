// spdnn_network: end-to-end driver with the reference's command line
//
//     spdnn_network neuron batch layer [options]
//
// (reference: src/network.cpp:56-126, "Usage: exe neuron batch layer").  Like the reference it
// takes the bias from the neuron count (network.cpp:73-78), reads the features from
// <data>/sparse-images-<N>.tsv (read_input, network.cpp:33-54) and layer l from
// <data>/neuron<N>/n<N>-l<l+1>.tsv (get_weight_file_name, network.cpp:14-19), then runs all
// layers on the GPU and prints "layer l, batch = n" per layer (all_network.cu:508).  Unlike the
// reference it goes through the C ABI (include/spdnn.h): the inspector runs behind the
// boundary, errors are reported instead of exit()ing inside the library, and the categories
// can be written out.  Where the TSV files are absent but the packed files of the reference's
// library benchmarks exist (<data>/neuron<N>.bin and <data>/sparse-images-<N>.bin,
// benchmark/cusparse/cusparse.cu:318-383) those are read instead.  When no data files are there
// (or with --synthetic) the seeded generator provides weights and features of the same shape.
//
// Options:
//   --data DIR        data directory (default ../data, as in the reference)
//   --synthetic       use the seeded generator even if data files exist
//   --seed S          generator seed (default 0)
//   --density A B     per-row feature density range of the generator (default 0.10 0.25)
//   --no-prune        keep every row through all layers
//   --gather          force the general kernel for every layer
//   --categories F    write the surviving row ids (1-based, one per line) to F
//   --truth F         compare the surviving row ids with the challenge's truth file
//                     (neuron<N>-l<L>-categories.tsv: 1-based ids, one per line); exit status 3
//                     when they differ
//   --quiet           no per-layer lines
#include <sys/stat.h>

#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "../../include/spdnn.h"

static bool file_exists(const std::string& p) {
    struct stat st;
    return stat(p.c_str(), &st) == 0;
}

static double now_s() {
    return std::chrono::duration<double>(std::chrono::steady_clock::now().time_since_epoch()).count();
}

#define CHECK(call)                                                                \
    do {                                                                           \
        int rc_ = (call);                                                          \
        if (rc_ != SPDNN_OK) {                                                     \
            fprintf(stderr, "%s failed (%d): %s\n", #call, rc_, spdnn_last_error()); \
            return 1;                                                              \
        }                                                                          \
    } while (0)

int main(int argc, char** argv) {
    if (argc < 4) {
        printf("Usage: exe neuron batch layer\n");
        return 0;
    }
    const int neuron = atoi(argv[1]);
    const int batch = atoi(argv[2]);
    const int layer = atoi(argv[3]);
    std::string data = "../data", cat_file, truth_file;
    bool synthetic = false, prune = true, quiet = false, gather = false;
    unsigned long long seed = 0;
    float dmin = 0.10f, dmax = 0.25f;
    for (int i = 4; i < argc; ++i) {
        std::string a = argv[i];
        if (a == "--data" && i + 1 < argc) data = argv[++i];
        else if (a == "--synthetic") synthetic = true;
        else if (a == "--seed" && i + 1 < argc) seed = strtoull(argv[++i], nullptr, 10);
        else if (a == "--density" && i + 2 < argc) { dmin = (float)atof(argv[++i]); dmax = (float)atof(argv[++i]); }
        else if (a == "--no-prune") prune = false;
        else if (a == "--gather") gather = true;
        else if (a == "--categories" && i + 1 < argc) cat_file = argv[++i];
        else if (a == "--truth" && i + 1 < argc) truth_file = argv[++i];
        else if (a == "--quiet") quiet = true;
        else { fprintf(stderr, "unknown option %s\n", a.c_str()); return 2; }
    }

    float bias = 0.0f;
    if (spdnn_reference_bias(neuron, &bias) != SPDNN_OK) {
        fprintf(stderr, "neuron must be one of 1024, 4096, 16384, 65536 (got %d)\n", neuron);
        return 2;
    }
    printf("[BEGIN]...\n");
    spdnn_net* net = nullptr;
    CHECK(spdnn_create(neuron, batch, layer, bias, 32.0f, &net));
    if (gather) CHECK(spdnn_set_force_kernel(net, SPDNN_KERNEL_GATHER));

    const std::string feat_file = data + "/sparse-images-" + std::to_string(neuron) + ".tsv";
    char wname[4096];
    CHECK(spdnn_weight_file_name(data.c_str(), neuron, 0, wname, sizeof(wname)));
    const bool from_files = !synthetic && file_exists(feat_file) && file_exists(wname);
    const std::string feat_bin = data + "/sparse-images-" + std::to_string(neuron) + ".bin";
    const std::string weight_bin = data + "/neuron" + std::to_string(neuron) + ".bin";
    const bool from_bin = !synthetic && !from_files && file_exists(feat_bin) && file_exists(weight_bin);

    double t0 = now_s();
    if (from_files) {
        CHECK(spdnn_load_layers_tsv(net, data.c_str(), 0, layer));   // parsed by the inspector's worker threads
        if (!quiet)
            for (int l = 0; l < layer; ++l) {
                CHECK(spdnn_weight_file_name(data.c_str(), neuron, l, wname, sizeof(wname)));
                printf("[%s] to CSR success!\n", wname);
            }
    } else if (from_bin) {
        CHECK(spdnn_load_layers_bin(net, weight_bin.c_str(), 0, layer, 0));
        if (!quiet) printf("[%s] to CSR success!\n", weight_bin.c_str());
    } else {
        printf("data files not used: seeded generator, seed %llu\n", seed);
        CHECK(spdnn_synth_layers(net, seed, 0, layer, 32, 0.0625f));
    }
    CHECK(spdnn_inspect(net));
    int n_band = 0, n_block = 0;
    for (int l = 0; l < layer; ++l) {
        spdnn_layer_plan p;
        CHECK(spdnn_get_layer_plan(net, l, &p));
        if (p.kernel == SPDNN_KERNEL_BAND) ++n_band;
        if (p.kernel == SPDNN_KERNEL_BLOCK) ++n_block;
    }
    printf("Inspector success: %d band layers, %d block layers, %d gather layers (%.2f s)\n", n_band, n_block,
           layer - n_band - n_block, now_s() - t0);

    t0 = now_s();
    if (from_files) CHECK(spdnn_load_features_tsv(net, feat_file.c_str(), batch));
    else if (from_bin) CHECK(spdnn_load_features_bin(net, feat_bin.c_str(), batch));
    else CHECK(spdnn_synth_features(net, seed, batch, dmin, dmax));
    printf("Read Input success! (%.2f s)\n", now_s() - t0);

    spdnn_run_options opt;
    CHECK(spdnn_default_run_options(&opt));
    opt.prune = prune ? 1 : 0;
    opt.collect_counts = 1;
    opt.time_layers = 1;
    spdnn_run_result res;
    CHECK(spdnn_run(net, &opt, &res));

    std::vector<float> ms((size_t)layer);
    CHECK(spdnn_get_layer_times(net, ms.data(), layer));
    double upper_ms = 0.0;
    int64_t entering = batch;
    for (int l = 0; l < layer; ++l) {
        int64_t cnt = 0;
        CHECK(spdnn_get_active_count(net, l, &cnt));
        // the reference's per-layer model: fp32 read + write of the feature block
        // (all_network.cu:335-340), against 8 TB/s here instead of 700 GB/s
        const double min_ms = 8.0 * (double)(prune ? entering : batch) * neuron / 8.0e12 * 1e3;
        upper_ms += min_ms;
        if (!quiet) {
            printf("layer %d, batch = %lld\n", l, (long long)cnt);
            if (ms[(size_t)l] > 0.0f)
                printf("Layer %d exec Time = %f, %fms, Utilization = %f\n", l, ms[(size_t)l], min_ms, min_ms / ms[(size_t)l]);
        }
        entering = cnt;
    }
    const double edges = res.edges;
    printf("Kernel Exec Time = %fms (layers launched %d, compactions %d)\n", res.ms_total, res.layers_run, res.compactions);
    printf("Kernel Exec Upper Time = %fms\n", upper_ms);
    printf("Inference edges/s = %.4e, categories = %lld\n", edges / (res.ms_total * 1e-3), (long long)res.active_rows);
    if (!cat_file.empty()) {
        CHECK(spdnn_write_categories(net, cat_file.c_str()));
        printf("categories written to %s\n", cat_file.c_str());
    }
    int status = 0;
    if (!truth_file.empty()) {
        std::vector<long long> truth;
        FILE* f = fopen(truth_file.c_str(), "r");
        if (!f) {
            fprintf(stderr, "cannot read %s\n", truth_file.c_str());
            return 1;
        }
        long long id;
        while (fscanf(f, "%lld", &id) == 1) truth.push_back(id);
        fclose(f);
        int64_t cnt = 0;
        CHECK(spdnn_get_categories(net, nullptr, 0, &cnt));
        std::vector<int32_t> ids((size_t)(cnt > 0 ? cnt : 1));
        CHECK(spdnn_get_categories(net, ids.data(), (int64_t)ids.size(), &cnt));
        bool same = (int64_t)truth.size() == cnt;
        for (int64_t i = 0; same && i < cnt; ++i) same = truth[(size_t)i] == (long long)ids[(size_t)i] + 1;
        printf("Challenge %s (%lld categories, truth file holds %zu)\n", same ? "PASSED" : "FAILED", (long long)cnt,
               truth.size());
        if (!same) status = 3;
    }
    CHECK(spdnn_destroy(net));
    printf("[END]...\n");
    return status;
}
