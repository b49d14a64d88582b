// C ABI of the library (include/spdnn.h): host orchestration around the kernels.
//
// The layer loop mirrors test_benchmark_graph_challenge (reference
// src/microbenchmark/all_network.cu:207-526) with these differences: weights arrive as CSR and
// go through the inspector behind the boundary; the active-row scan and the repack run on the
// device (the reference copies the flags to the host and scans them there,
// all_network.cu:444-513); the input features are kept untouched so a run can be repeated.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <chrono>
#include <cmath>
#include <condition_variable>
#include <cstdio>
#include <cstring>
#include <deque>
#include <functional>
#include <memory>
#include <mutex>
#include <new>
#include <stdexcept>
#include <string>
#include <thread>
#include <vector>

#include "../../include/spdnn.h"
#include "inspector.hpp"
#include "kernels.hpp"
#include "synth.hpp"
#include "tsv_io.hpp"

using namespace spdnn;

namespace {

thread_local std::string g_err = "";

// device allocations the library has made in this process (spdnn_device_alloc_calls)
std::atomic<int64_t> g_dev_allocs{0};
template <class T> hipError_t dev_malloc(T** p, size_t bytes) {
    g_dev_allocs.fetch_add(1, std::memory_order_relaxed);
    return hipMalloc(reinterpret_cast<void**>(p), bytes);
}

int fail(int code, const std::string& msg) {
    g_err = msg;
    return code;
}

#define HIPCHK(expr)                                                                                 \
    do {                                                                                             \
        hipError_t e_ = (expr);                                                                      \
        if (e_ != hipSuccess)                                                                        \
            return fail(SPDNN_E_DEVICE, std::string(#expr) + ": " + hipGetErrorString(e_));         \
    } while (0)

// Scratch memory of spdnn_get_activations_noalloc, the one entry point that allocates nothing: a
// row table (global id -> physical row), the ids and physical rows of one pass, and the row-major
// staging rows of one pass.  Each GPU holds its own copy of the array until the process ends.  In
// host code the array's name is only a stand-in for the symbol: the device address is looked up
// once per device (scratch_base) and everything on the host side uses that pointer.
constexpr size_t kScratchTableRows = (size_t)1 << 20;              // rows (batch) the row table holds
constexpr size_t kScratchPassRows = 16384;                         // requested rows per pass at most
constexpr size_t kScratchStageBytes = (size_t)8 << 20;             // staging rows of one pass
constexpr size_t kScratchTableOff = 0;
constexpr size_t kScratchIdsOff = kScratchTableRows * 4;
constexpr size_t kScratchPhysOff = kScratchIdsOff + kScratchPassRows * 4;
constexpr size_t kScratchStageOff = kScratchPhysOff + kScratchPassRows * 4;
constexpr size_t kScratchBytes = kScratchStageOff + kScratchStageBytes;  // 12.1 MiB
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

constexpr int kMaxDevices = 16;
unsigned char* g_scratch_ptr[kMaxDevices] = {};
std::mutex g_scratch_mutex;

// Device address of `scratch` on the current device, looked up on the first call per device.
hipError_t scratch_base(unsigned char** out) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= kMaxDevices) return hipErrorInvalidDevice;
    std::lock_guard<std::mutex> lk(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return e;
        if (!p) return hipErrorInvalidSymbol;
        g_scratch_ptr[dev] = static_cast<unsigned char*>(p);
    }
    *out = g_scratch_ptr[dev];
    return hipSuccess;
}

// Temporary device allocation / event that is released on every return path.
struct DevTmp {
    void* p = nullptr;
    ~DevTmp() { if (p) hipFree(p); }
    hipError_t alloc(size_t bytes) { return dev_malloc(&p, bytes); }
    template <class T> T* as() const { return static_cast<T*>(p); }
};
struct EventTmp {
    hipEvent_t e = nullptr;
    ~EventTmp() { if (e) hipEventDestroy(e); }
    hipError_t create() { return hipEventCreate(&e); }
};

// Small worker pool for the per-layer inspector jobs (bounded queue so that pending CSR copies
// stay small).
class JobPool {
  public:
    explicit JobPool(int nthreads) {
        for (int i = 0; i < nthreads; ++i) workers_.emplace_back([this] { loop(); });
    }
    ~JobPool() {
        {
            std::unique_lock<std::mutex> lk(m_);
            stop_ = true;
        }
        cv_job_.notify_all();
        for (auto& t : workers_) t.join();
    }
    void submit(std::function<void()> f) {
        std::unique_lock<std::mutex> lk(m_);
        cv_room_.wait(lk, [this] { return q_.size() < 2 * workers_.size() + 2; });
        q_.push_back(std::move(f));
        ++pending_;
        cv_job_.notify_one();
    }
    void wait_all() {
        std::unique_lock<std::mutex> lk(m_);
        cv_done_.wait(lk, [this] { return pending_ == 0; });
    }

  private:
    void loop() {
        for (;;) {
            std::function<void()> f;
            {
                std::unique_lock<std::mutex> lk(m_);
                cv_job_.wait(lk, [this] { return stop_ || !q_.empty(); });
                if (q_.empty()) return;
                f = std::move(q_.front());
                q_.pop_front();
                cv_room_.notify_one();
            }
            try { f(); } catch (...) {}  // jobs report through their own state; nothing may escape a worker
            {
                std::unique_lock<std::mutex> lk(m_);
                if (--pending_ == 0) cv_done_.notify_all();
            }
        }
    }
    std::vector<std::thread> workers_;
    std::deque<std::function<void()>> q_;
    std::mutex m_;
    std::condition_variable cv_job_, cv_room_, cv_done_;
    size_t pending_ = 0;
    bool stop_ = false;
};

int host_threads() {
    const char* e = getenv("SPDNN_HOST_THREADS");
    int n = e ? atoi(e) : 0;
    if (n <= 0) {
        n = (int)std::thread::hardware_concurrency();
        const char* omp = getenv("OMP_NUM_THREADS");
        if (omp && atoi(omp) > 0) n = std::min(n > 0 ? n : 16, atoi(omp));
    }
    return std::max(1, std::min(n, 32));
}

struct DevLayer {
    uint32_t* pairs = nullptr;
    int32_t* ell = nullptr;
    int32_t* rowlen = nullptr;
    float* wv = nullptr;
    int32_t* dst = nullptr;
    int32_t* blk_cols = nullptr;
    int32_t* blk_cnt = nullptr;
    int32_t* alt_cols = nullptr;   // the BLOCK form of a run-chain BAND layer (see LayerPlan)
    int32_t* alt_cnt = nullptr;
    int32_t* alt_dst = nullptr;
    float* alt_wv = nullptr;       // (with alt_cols / alt_cnt / alt_dst: the GATHER form of a TILED layer)
    uint32_t* rt_ent = nullptr;    // (with alt_cnt / alt_dst: its ROWTILE form)
    uint32_t* quad_col = nullptr;  // the QUAD form of a BAND layer (with dst)
    float* quad_w = nullptr;
};

// Where the arrays of one layer's plan lie inside its block of device memory (and inside the
// pinned host copy of that block when plans are streamed): pairs, ell, rowlen, wv, dst, blk_cols,
// blk_cnt, alt_cols, alt_cnt, alt_dst, alt_wv, rt_ent, quad_col, quad_w, each aligned to 256 bytes.
constexpr int kPlanArrays = 14;
struct PlanLayout {
    size_t off[kPlanArrays] = {};
    size_t len[kPlanArrays] = {};
    size_t bytes = 0;
};

}  // namespace

struct spdnn_net {
    int N = 0, max_batch = 0, L = 0;
    float bias = 0.0f, clampv = 32.0f;
    int rl = 4, RB = 256;
    int rows_cap = 0;
    int force_kernel = SPDNN_KERNEL_AUTO;
    // With |bias| >= 2^-40 a nonzero output fl(acc + bias) is at least an ulp of the bias, far
    // above the denormal range, so products with power-of-two weights (|w| <= 2^24 down to 2^-24)
    // are exact.  With a zero or tiny bias activations can decay into the denormal range, where
    // the fused multiply-add would round differently from the reference's multiply-then-add.
    bool fma_ok = true;
    std::vector<LayerPlan> layers;
    std::unique_ptr<JobPool> pool;
    bool inspected = false;

    // device
    bool dev_ready = false, uploaded = false;
    int n_cu = 256;
    hipStream_t stream = nullptr;
    void* arena = nullptr;
    std::vector<DevLayer> dl;
    std::vector<PlanLayout> lay;
    // Streamed plans (plan_window >= 2): the device holds `plan_window` slots of the largest
    // plan's size; layer l uses slot l % plan_window.  A second stream copies the plan of layer
    // l + plan_window from pinned host memory into the slot as soon as layer l has finished,
    // so the copy runs under the layers in between.
    int plan_window = 0;
    size_t slot_bytes = 0;
    char* h_plans = nullptr;          // pinned: all plans, back to back
    std::vector<size_t> h_plan_off;
    std::vector<int> slot_layer;      // layer whose plan the slot holds (or is being filled with)
    std::vector<char> slot_busy;      // a kernel that reads the slot has been launched since it was filled
    std::vector<hipEvent_t> ev_slot_ready, ev_slot_free;
    hipStream_t copy_stream = nullptr;
    // input labellings: layer 0's stays on the device, another layer's is sent when asked for
    int32_t* d_lab = nullptr;
    int lab_layer = -1;
    Feat F, A, C;             // features as handed over, and the two work buffers the layers ping-pong between
    std::vector<float*> feat_allocs;  // the allocations behind them
    int feat_paired = 0, feat_candidates = 0;
    int32_t* d_active_mid = nullptr;  // row stamps of the first layer of a fused pair (see PairLaunch)
    int32_t *d_active = nullptr, *d_gid = nullptr, *d_gid_tmp = nullptr, *d_count = nullptr;
    int32_t* d_count_partial = nullptr;   // see launch_count_stamp_range
    int32_t *d_alive_src = nullptr, *d_alive_gid = nullptr, *d_nonfinite = nullptr;
    int32_t* h_count = nullptr;  // pinned
    int32_t* d_counts = nullptr; // per-layer active-row counters (device)
    int32_t* h_counts = nullptr; // pinned mirror
    hipEvent_t ev_start = nullptr, ev_stop = nullptr;
    std::vector<hipEvent_t> ev_layer;

    // state
    int batch = 0;
    bool have_features = false;
    Feat cur;
    int cur_layer = 0;
    int carried = 0;
    int stamp = 0;
    int64_t alive = 0;        // rows active after the last layer run
    bool alive_list_valid = false;
    bool gid_dirty = false;   // a repack permuted d_gid since it was last initialised
    int last_stamp = 0;       // stamp of the newest layer, valid for the current row slots (0 = none)
    // A launch that skips row blocks without an active row leaves those blocks of its output buffer
    // unwritten (they hold an older layer's values).  Consumers that look at the stamps never read
    // them; a later launch that does not look (pruning off) would.  Set by launches that may skip,
    // cleared when every carried block has been written again (new run, repack).
    bool blocks_skipped = false;
    // Persistent launches (several layers per launch, see PersistLaunch).  SPDNN_PERSIST: 0 = never unless the
    // caller asks (fuse_layers >= 2), 1 = where a layer's launch moves at most persist_max_bytes (default).
    int persist_mode = 1;
    int persist_layers = 64;          // layers per persistent launch at most (SPDNN_PERSIST_LAYERS)
    // By default a launch is persistent where one layer reads + writes between these many bytes (SPDNN_PERSIST_MIN_BYTES,
    // SPDNN_PERSIST_MAX_BYTES).  Measured, batch 60000, sustained, per layer: N=1024 102.7 -> 99.1 us, N=4096 344 -> 325 us,
    // N=16384 1285 -> 1280 us (beyond the upper bound: left alone); N=1024 with batch 6000 15.9 -> 18.2 us (below the lower).
    long long persist_min_bytes = (long long)1 << 28, persist_max_bytes = (long long)1 << 31;
    int persist_min_blocks = 64;      // fewest row blocks a persistent launch is made for by default (SPDNN_PERSIST_MIN_BLOCKS)
    int persist_xcd = -1;             // one unit queue per XCD: -1 = from 8 row blocks up, 0 / 1 (SPDNN_PERSIST_XCD)
    int persist_light = 1;            // SPDNN_PERSIST_LIGHT_SYNC=0: the writer's L2 write-back also with XCD queues
    int persist_seglen = 0;           // band positions / groups per unit, 0 = heuristic (SPDNN_PERSIST_SEGLEN)
    int resident_mode = 1;            // 1: layers with a BLOCK form of one exact weight run as resident launches where the
                                      // shape fits (rows kept in LDS through the layers; SPDNN_RESIDENT=0: never)
    long long persist_wait_us = 2000000;   // longest wait of a unit for its row block (SPDNN_PERSIST_WAIT_US)
    int band_seglen = 0;              // SPDNN_BAND_SEGLEN: band positions per workgroup of the per-layer walk (0 = run-time selection)
    int band_direct_lds = 1;          // SPDNN_BAND_DIRECT_LDS=0: the per-layer walk never loads straight into LDS
    int32_t* d_done = nullptr;        // [L][done_stride] units finished per layer and row block
    int done_stride = 0;
    PersistCtl* d_ctl = nullptr;      // [L] control words, one per persistent launch of a run
    int32_t* d_abort = nullptr;
    int32_t* d_frontier = nullptr;    // [done_stride]
    int32_t* h_pwords = nullptr;      // pinned [L]: completion word of every persistent launch of a run
    size_t search_peak_bytes = 0;     // device memory the placement search held at its peak
    bool run_verbose = false;         // SPDNN_RUN_VERBOSE=1: spdnn_run reports its persistent launches on stderr
    int add_only = 1;         // band layers with one power-of-two weight add their inputs and scale the sum once
                              // (SPDNN_BAND_SUM_THEN_SCALE=0: a multiply-add per input)
    bool fuse_pairs = true;   // fused pairs where the inspector found them (SPDNN_FUSE_PAIRS=0: never)
    int pair_seglen = 0;      // band positions per workgroup of a fused pair, 0 = heuristic (SPDNN_PAIR_SEGLEN)
    // rows x neurons below which a pair runs as two launches (SPDNN_PAIR_MIN_ELEMS).  Measured, layers over one
    // neuron order, N = 1024 ... 65536: from 2^23 elements up the fused pair takes 0.83 - 0.95 of the time of two
    // launches (0.98 at N=4096, batch 60000), at 2^22 and below up to 2.6 times as long (a 16-wave workgroup
    // per CU, few segments).
    int64_t pair_min_elems = (int64_t)1 << 23;
    int64_t block_form_max_elems = (int64_t)1 << 26;  // see use_block_form
    int64_t tiled_min_rows = 8192;                    // see use_gather_form (SPDNN_TILED_MIN_ROWS)
    bool tiled_min_rows_given = false;                // ... set in the environment: also layers with a ROWTILE form follow it
    int rowtile_mode = 1;                             // TILED layers up to 8192 neurons wide run their ROWTILE form (SPDNN_ROWTILE=0: the tiles)
    int band_resident_mode = 1;                       // BAND layers up to 1024 neurons wide join resident launches (SPDNN_BAND_RESIDENT=0: never)
    int band_resident_min_layers = 0;                 // ... of at least this many layers (SPDNN_BAND_RESIDENT_MIN_LAYERS; 0: 6, from 16384 rows up 16)
    long long stream_min_bytes = 96ll << 20;          // see BandLaunch (SPDNN_STREAM_MIN_BYTES, read at creation)
    long long count_timeout_ms = 60000;               // longest wait for one layer's counts (SPDNN_COUNT_TIMEOUT_MS)
    LayerDesc* d_table = nullptr;   // one entry per layer (resident plans only)
    std::vector<char> pending; // layer has an inspection job in flight
    std::vector<int64_t> counts;
    std::vector<float> layer_ms;

    // measured band-walk configuration per (row blocks, entries per row)
    struct Tuned { int nblk, K, shape, seglen; };
    std::vector<Tuned> tuned;
    bool autotune = true;
    // exploration in progress: real layers are launched with the candidates in turn and timed
    struct Cand { int shape, seglen; float best_ms; int samples; };
    struct Explore { int nblk, K, issued; std::vector<Cand> cands; };
    struct Trial { int nblk, K, cand; hipEvent_t e0, e1; };
    std::vector<Explore> exploring;
    std::deque<Trial> trials;           // launched, not yet read back
    std::vector<hipEvent_t> ev_free;    // timing events for trials
};

namespace {

void release_device_base(spdnn_net* n) {
    hipFree(n->d_active_mid); n->d_active_mid = nullptr;
    hipFree(n->d_active); hipFree(n->d_gid); hipFree(n->d_gid_tmp);
    hipFree(n->d_alive_src); hipFree(n->d_alive_gid); hipFree(n->d_count); hipFree(n->d_count_partial); hipFree(n->d_nonfinite);
    hipFree(n->d_counts);
    hipFree(n->d_done); hipFree(n->d_ctl); hipFree(n->d_abort); hipFree(n->d_frontier);
    n->d_done = n->d_abort = n->d_frontier = nullptr;
    n->d_ctl = nullptr;
    if (n->h_pwords) hipHostFree(n->h_pwords);
    n->h_pwords = nullptr;
    if (n->h_count) hipHostFree(n->h_count);
    if (n->h_counts) hipHostFree(n->h_counts);
    n->d_active = n->d_gid = n->d_gid_tmp = n->d_alive_src = n->d_alive_gid = nullptr;
    n->d_count_partial = nullptr;
    n->d_count = n->d_nonfinite = n->d_counts = n->h_count = n->h_counts = nullptr;
    for (hipEvent_t e : n->ev_layer) hipEventDestroy(e);
    for (const spdnn_net::Trial& t : n->trials) { hipEventDestroy(t.e0); hipEventDestroy(t.e1); }
    for (hipEvent_t e : n->ev_free) hipEventDestroy(e);
    n->trials.clear();
    n->ev_free.clear();
    n->exploring.clear();
    n->ev_layer.clear();
    if (n->ev_start) hipEventDestroy(n->ev_start);
    if (n->ev_stop) hipEventDestroy(n->ev_stop);
    if (n->stream) hipStreamDestroy(n->stream);
    n->ev_start = n->ev_stop = nullptr;
    n->stream = nullptr;
    n->dev_ready = false;
}

int init_device(spdnn_net* n) {
    int cnt = 0;
    hipError_t e = hipGetDeviceCount(&cnt);
    if (e != hipSuccess || cnt < 1) return fail(SPDNN_E_DEVICE, "no HIP device available");
    HIPCHK(hipSetDevice(0));
    hipDeviceProp_t p;
    HIPCHK(hipGetDeviceProperties(&p, 0));
    if (strncmp(p.gcnArchName, "gfx950", 6) != 0)
        return fail(SPDNN_E_DEVICE, std::string("kernels are built for gfx950, device is ") + p.gcnArchName);
    n->n_cu = p.multiProcessorCount;
    unsigned char* scratch_ptr = nullptr;
    HIPCHK(scratch_base(&scratch_ptr));  // set-up, with the device current: later calls only read the pointer
    HIPCHK(hipStreamCreate(&n->stream));
    HIPCHK(hipEventCreate(&n->ev_start));
    HIPCHK(hipEventCreate(&n->ev_stop));
    const size_t rows = (size_t)n->rows_cap;
    HIPCHK(dev_malloc(&n->d_active, rows * 4));
    HIPCHK(dev_malloc(&n->d_active_mid, rows * 4));
    HIPCHK(hipMemset(n->d_active_mid, 0, rows * 4));
    HIPCHK(dev_malloc(&n->d_gid, rows * 4));
    HIPCHK(dev_malloc(&n->d_gid_tmp, rows * 4));
    HIPCHK(dev_malloc(&n->d_alive_src, rows * 4));
    HIPCHK(dev_malloc(&n->d_alive_gid, rows * 4));
    HIPCHK(dev_malloc(&n->d_count, 64));
    HIPCHK(dev_malloc(&n->d_count_partial, (size_t)count_stamp_partial_words() * 4));
    HIPCHK(hipMemset(n->d_count_partial, 0, (size_t)count_stamp_partial_words() * 4));
    HIPCHK(dev_malloc(&n->d_nonfinite, 64));
    // coherent: the layer kernels store counts here and the host reads them while kernels still run
    HIPCHK(hipHostMalloc(&n->h_count, 64, hipHostMallocCoherent | hipHostMallocMapped));
    HIPCHK(dev_malloc(&n->d_counts, (size_t)n->L * 4));
    HIPCHK(hipHostMalloc(&n->h_counts, (size_t)n->L * 4, hipHostMallocCoherent | hipHostMallocMapped));
    HIPCHK(hipMemset(n->d_active, 0, rows * 4));
    // persistent launches: units finished per layer and row block, control words per launch, completion words
    n->done_stride = n->rows_cap / n->RB;
    HIPCHK(dev_malloc(&n->d_done, (size_t)n->L * (size_t)n->done_stride * 4));
    HIPCHK(dev_malloc(&n->d_ctl, (size_t)n->L * sizeof(PersistCtl)));
    HIPCHK(dev_malloc(&n->d_abort, 64));
    HIPCHK(hipMemset(n->d_abort, 0, 64));
    HIPCHK(dev_malloc(&n->d_frontier, (size_t)n->done_stride * 4));
    HIPCHK(hipHostMalloc(&n->h_pwords, (size_t)n->L * 4, hipHostMallocCoherent | hipHostMallocMapped));
    n->dev_ready = true;
    return SPDNN_OK;
}

int ensure_device(spdnn_net* n) {
    if (n->dev_ready) return SPDNN_OK;
    const int rc = init_device(n);
    if (rc != SPDNN_OK) release_device_base(n);  // nothing half-built stays behind (g_err is kept)
    return rc;
}

size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }

void free_device(spdnn_net* n);

// The feature buffers: six half-buffers (see Feat).  For large problems the halves of every buffer
// are taken from two different memory regions.  Which allocation lies where only shows in a
// measurement: candidates are allocated one after the other and each is swept by a streaming write
// together with the first one - 6.0 TB/s when the two share a region, 7.2 TB/s when they do not
// (MI355X) - until two candidates of the first one's kind (itself included) and three of the other
// are there; the rest is freed again.  On a fresh
// device the boundary comes after about a third of the memory.  SPDNN_REGION_PAIRING=0 switches
// the search off, SPDNN_ALLOC_VERBOSE=1 prints the measurements.
int alloc_feature_buffers(spdnn_net* n) {
    const size_t half_blocks = ((size_t)n->rows_cap / (size_t)n->RB + 1) / 2;
    const size_t half_bytes = std::max<size_t>(half_blocks, 1) * (size_t)n->N * (size_t)n->RB * 4;
    const bool verbose = getenv("SPDNN_ALLOC_VERBOSE") != nullptr;
    const char* env = getenv("SPDNN_REGION_PAIRING");
    size_t free_b = 0, total_b = 0;
    HIPCHK(hipMemGetInfo(&free_b, &total_b));
    // the search never holds more than this share of the free device memory (candidates + fillers)
    const char* budget_env = getenv("SPDNN_REGION_PAIRING_BUDGET");
    // (0.85 by default: on some boxes the second region only starts behind 180 GB of candidates)
    const double budget_frac = budget_env ? std::min(0.9, std::max(0.05, atof(budget_env))) : 0.85;
    const size_t max_cand = std::min<size_t>(64, (size_t)((double)free_b * budget_frac / (double)half_bytes));
    const char* min_env = getenv("SPDNN_REGION_PAIRING_MIN_GIB");   // smallest half-buffer worth the search
    const double min_gib = min_env ? atof(min_env) : 0.4;
    const bool search = !(env && atoi(env) == 0) && (double)half_bytes >= min_gib * 1073741824.0 && max_cand >= 12;

    std::vector<float*>& c = n->feat_allocs;
    std::vector<double> rate;  // rate[i]: candidate i swept together with candidate 0 (rate[0] unused)
    std::vector<void*> fillers;
    size_t filler_bytes = 0;   // size of one filler
    auto fail_free = [&](int code, const std::string& msg) {
        for (void* f : fillers) hipFree(f);
        for (float* p : c) hipFree(p);
        c.clear();
        return fail(code, msg);
    };
    auto add = [&]() {
        float* p = nullptr;
        if (dev_malloc(&p, half_bytes) != hipSuccess) { (void)hipGetLastError(); return false; }
        c.push_back(p);
        return true;
    };
    for (int i = 0; i < 6; ++i)
        if (!add()) return fail_free(SPDNN_E_NOMEM, "out of device memory for the feature buffers");
    int pick[6] = {0, 1, 2, 3, 4, 5};
    n->feat_paired = 0;
    if (search) {
        EventTmp e0, e1;
        if (e0.create() != hipSuccess || e1.create() != hipSuccess) return fail_free(SPDNN_E_DEVICE, "event creation failed");
        const int64_t nf = (int64_t)(half_bytes / 16) * 4;
        std::vector<int> same, other;
        // streaming-write rate of candidates a and b swept together
        auto probe = [&](size_t a, size_t b, double* gbps) {
            hipError_t e = launch_zero_pair(c[a], c[b], nf, n->stream);  // first touch
            if (e == hipSuccess) e = hipEventRecord(e0.e, n->stream);
            for (int r = 0; r < 2 && e == hipSuccess; ++r) e = launch_zero_pair(c[a], c[b], nf, n->stream);
            if (e == hipSuccess) e = hipEventRecord(e1.e, n->stream);
            if (e == hipSuccess) e = hipEventSynchronize(e1.e);
            float ms = 0.0f;
            if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0.e, e1.e);
            if (e == hipSuccess) *gbps = 4.0 * (double)half_bytes / ((double)ms * 1e-3) / 1e9;
            return e;
        };
        // candidates that share the reference's region (the slow ones) and candidates that do not
        // `strong`: the two best candidates elsewhere reach the rate of two regions (7.2 against 6.0 TB/s);
        // a candidate that straddles a boundary lies in between and makes a poor half (measured: layers of
        // 5.23 - 5.35 ms instead of 5.16 - 5.19 at the cfg4 shape with partners that swept at 6.9 TB/s)
        bool strong = false;
        auto classify = [&](int ref) {
            double lowest = 0.0;
            for (size_t k = 0; k < rate.size(); ++k)
                if ((int)k != ref && (lowest == 0.0 || rate[k] < lowest)) lowest = rate[k];
            same.clear();
            other.clear();
            for (size_t k = 0; k < rate.size(); ++k) {
                if ((int)k == ref) continue;
                if (rate[k] > 1.10 * lowest) other.push_back((int)k);
                else if (rate[k] < 1.05 * lowest) same.push_back((int)k);
            }
            // the clearest cases first: the fastest partners elsewhere, the slowest in the reference's region
            std::sort(other.begin(), other.end(), [&](int a, int b) { return rate[(size_t)a] > rate[(size_t)b]; });
            std::sort(same.begin(), same.end(), [&](int a, int b) { return rate[(size_t)a] < rate[(size_t)b]; });
            same.insert(same.begin(), ref);
            strong = other.size() >= 2 && rate[(size_t)other[1]] >= 1.17 * lowest;
            // The two work buffers, which every layer streams through, need a half of each kind; the
            // feature buffer (read by the first layer only) takes one if there is one.
            return same.size() >= 2 && other.size() >= 3;
        };
        // every step past the first six candidates advances at least 4 GiB through the memory: small
        // half-buffers are spaced out by fillers, which are freed again below
        const size_t filler = half_bytes < ((size_t)4 << 30) ? ((size_t)4 << 30) - half_bytes : 0;
        filler_bytes = filler;
        const size_t budget = (size_t)((double)free_b * budget_frac);
        rate.assign(1, 0.0);
        bool found = false;
        int ref = 0;
        int extra = 0;   // candidates tried beyond the first complete set, looking for clear partners
        for (size_t i = 1; i < max_cand && !(found && (strong || extra >= 6)); ++i) {
            if (i >= c.size()) {
                if ((c.size() + 1) * half_bytes + (fillers.size() + 1) * filler > budget) break;
                if (filler) {
                    void* f = nullptr;
                    if (dev_malloc(&f, filler) != hipSuccess) { (void)hipGetLastError(); break; }
                    fillers.push_back(f);
                }
                if (!add()) break;
            }
            double r = 0.0;
            const hipError_t e = probe(0, i, &r);
            if (e != hipSuccess) return fail_free(SPDNN_E_DEVICE, std::string("region probe: ") + hipGetErrorString(e));
            rate.push_back(r);
            if (found) ++extra;
            found = i >= 5 && classify(0);
        }
        if (!found && rate.size() >= 8) {
            // The first candidate may itself straddle two regions, and then every partner looks fast.
            // Second pass over what is allocated, against the partner that went slowest with it.
            ref = 1;
            for (size_t k = 2; k < rate.size(); ++k) if (rate[k] < rate[(size_t)ref]) ref = (int)k;
            if (verbose) {
                fprintf(stderr, "spdnn: no second region seen from candidate 0 (GB/s:");
                for (size_t k = 1; k < rate.size(); ++k) fprintf(stderr, " %.0f", rate[k]);
                fprintf(stderr, "), second pass against candidate %d\n", ref);
            }
            for (size_t k = 0; k < rate.size(); ++k) {
                if ((int)k == ref) continue;
                const hipError_t e = probe((size_t)ref, k, &rate[k]);
                if (e != hipSuccess) return fail_free(SPDNN_E_DEVICE, std::string("region probe: ") + hipGetErrorString(e));
            }
            found = classify(ref);
        }
        if (verbose) {
            fprintf(stderr, "spdnn: half-buffers of %.1f GB swept together with candidate %d, GB/s:", (double)half_bytes / 1e9, ref);
            for (size_t k = 0; k < rate.size(); ++k) if ((int)k != ref) fprintf(stderr, " %.0f", rate[k]);
            fprintf(stderr, "\nspdnn: %zu in its region, %zu elsewhere%s\n", same.size(), other.size(),
                    found ? ": the work buffers get one half of each" : ": no pairing");
        }
        if (found) {
            for (int b = 0; b < 2; ++b) { pick[2 * b] = same[(size_t)b]; pick[2 * b + 1] = other[(size_t)b]; }
            pick[5] = other[2];
            pick[4] = -1;
            if (same.size() >= 3) pick[4] = same[2];
            for (size_t k = 0; k < c.size() && pick[4] < 0; ++k) {   // else any candidate not taken yet
                bool taken = false;
                for (int q = 0; q < 6; ++q) taken |= q != 4 && pick[q] == (int)k;
                if (!taken) pick[4] = (int)k;
            }
            n->feat_paired = 1;
        }
    }
    n->feat_candidates = (int)c.size();
    Feat* bufs[3] = {&n->A, &n->C, &n->F};
    for (int b = 0; b < 3; ++b) {
        bufs[b]->half[0] = c[(size_t)pick[2 * b]];
        bufs[b]->half[1] = c[(size_t)pick[2 * b + 1]];
    }
    // what the search held at its peak (all candidates and fillers are still allocated here)
    n->search_peak_bytes = c.size() * half_bytes + fillers.size() * filler_bytes;
    // give back what was only a candidate
    for (void* f : fillers) hipFree(f);
    std::vector<float*> keep;
    for (size_t i = 0; i < c.size(); ++i) {
        bool used = false;
        for (int k = 0; k < 6; ++k) used |= pick[k] == (int)i;
        if (used) keep.push_back(c[i]); else hipFree(c[i]);
    }
    c.swap(keep);
    return SPDNN_OK;
}

PlanLayout plan_layout(const LayerPlan& p) {
    PlanLayout y;
    const size_t len[kPlanArrays] = {p.pairs.size() * 4,    p.ell_col.size() * 4,  p.rowlen.size() * 4,   p.wv.size() * 4,
                                     p.dst.size() * 4,      p.blk_cols.size() * 4, p.blk_cnt.size() * 4,  p.alt_cols.size() * 4,
                                     p.alt_cnt.size() * 4,  p.alt_dst.size() * 4,  p.alt_wv.size() * 4,
                                     p.rt_ent.size() * 4,   p.quad_col.size() * 4, p.quad_w.size() * 4};
    for (int k = 0; k < kPlanArrays; ++k) {
        y.off[k] = y.bytes;
        y.len[k] = len[k];
        y.bytes += align256(len[k]);
    }
    return y;
}

void pack_plan(const LayerPlan& p, const PlanLayout& y, char* dst) {
    const void* src[kPlanArrays] = {p.pairs.data(),   p.ell_col.data(),  p.rowlen.data(),  p.wv.data(),      p.dst.data(),
                                    p.blk_cols.data(), p.blk_cnt.data(), p.alt_cols.data(), p.alt_cnt.data(), p.alt_dst.data(),
                                    p.alt_wv.data(),   p.rt_ent.data(),   p.quad_col.data(), p.quad_w.data()};
    for (int k = 0; k < kPlanArrays; ++k)
        if (y.len[k]) memcpy(dst + y.off[k], src[k], y.len[k]);
}

DevLayer plan_at(const PlanLayout& y, char* base) {
    DevLayer d;
    auto at = [&](int k) -> void* { return y.len[k] ? base + y.off[k] : nullptr; };
    d.pairs = (uint32_t*)at(0);
    d.ell = (int32_t*)at(1);
    d.rowlen = (int32_t*)at(2);
    d.wv = (float*)at(3);
    d.dst = (int32_t*)at(4);
    d.blk_cols = (int32_t*)at(5);
    d.blk_cnt = (int32_t*)at(6);
    d.alt_cols = (int32_t*)at(7);
    d.alt_cnt = (int32_t*)at(8);
    d.alt_dst = (int32_t*)at(9);
    d.alt_wv = (float*)at(10);
    d.rt_ent = (uint32_t*)at(11);
    d.quad_col = (uint32_t*)at(12);
    d.quad_w = (float*)at(13);
    return d;
}

int upload_plans(spdnn_net* n) {
    const size_t L = (size_t)n->L;
    n->lay.assign(L, PlanLayout{});
    size_t total = 0, largest = 0;
    for (size_t l = 0; l < L; ++l) {
        n->lay[l] = plan_layout(n->layers[l]);
        total += n->lay[l].bytes;
        largest = std::max(largest, n->lay[l].bytes);
    }
    n->dl.assign(L, DevLayer{});
    const bool streamed = n->plan_window >= 2 && (size_t)n->plan_window < L;
    if (!streamed) {
        HIPCHK(dev_malloc(&n->arena, std::max<size_t>(total, 256)));
        std::vector<char> blob(largest);
        size_t off = 0;
        for (size_t l = 0; l < L; ++l) {
            pack_plan(n->layers[l], n->lay[l], blob.data());
            if (n->lay[l].bytes)
                HIPCHK(hipMemcpy((char*)n->arena + off, blob.data(), n->lay[l].bytes, hipMemcpyHostToDevice));
            n->dl[l] = plan_at(n->lay[l], (char*)n->arena + off);
            off += n->lay[l].bytes;
        }
        std::vector<LayerDesc> table(L);
        for (size_t l = 0; l < L; ++l) {
            const LayerPlan& p = n->layers[l];
            LayerDesc& t = table[l];
            t = LayerDesc{};
            t.wu = p.info.value;
            if (p.kernel == SPDNN_KERNEL_BAND) {
                t.pairs = n->dl[l].pairs;
                t.pw = n->dl[l].wv;
                t.dst = n->dl[l].dst;
                t.steps = p.pair_steps;
                t.halo = p.info.band_halo;
                t.quad_groups = p.quad_groups;   // its QUAD form
                t.quad_col = n->dl[l].quad_col;
                t.quad_w = n->dl[l].quad_w;
                if (p.alt_ngroups > 0) {   // its BLOCK form
                    t.ngroups = p.alt_ngroups;
                    t.blk_cols = n->dl[l].alt_cols;
                    t.blk_cnt = n->dl[l].alt_cnt;
                    t.blk_wv = nullptr;
                    t.blk_dst = n->dl[l].alt_dst;
                }
            } else if (p.kernel == SPDNN_KERNEL_BLOCK) {
                t.ngroups = p.ngroups;
                t.blk_cols = n->dl[l].blk_cols;
                t.blk_cnt = n->dl[l].blk_cnt;
                t.blk_wv = n->dl[l].wv;
                t.blk_dst = n->dl[l].dst;
            } else if (p.kernel == SPDNN_KERNEL_TILED && !p.rt_ent.empty()) {   // its ROWTILE form
                t.rt_ent = n->dl[l].rt_ent;
                t.rt_len = n->dl[l].alt_cnt;
                t.rt_dst = n->dl[l].alt_dst;
                t.rt_kpad = (p.alt_kmax + 3) / 4 * 4;
            }
        }
        HIPCHK(dev_malloc(&n->d_table, table.size() * sizeof(LayerDesc)));
        HIPCHK(hipMemcpy(n->d_table, table.data(), table.size() * sizeof(LayerDesc), hipMemcpyHostToDevice));
        n->slot_bytes = 0;
    } else {
        const size_t S = (size_t)n->plan_window;
        n->slot_bytes = std::max<size_t>(largest, 256);
        HIPCHK(dev_malloc(&n->arena, S * n->slot_bytes));
        HIPCHK(hipHostMalloc((void**)&n->h_plans, std::max<size_t>(total, 256)));
        n->h_plan_off.assign(L, 0);
        size_t off = 0;
        for (size_t l = 0; l < L; ++l) {
            n->h_plan_off[l] = off;
            pack_plan(n->layers[l], n->lay[l], n->h_plans + off);
            off += n->lay[l].bytes;
            n->dl[l] = plan_at(n->lay[l], (char*)n->arena + (l % S) * n->slot_bytes);
        }
        n->slot_layer.assign(S, -1);
        n->slot_busy.assign(S, 0);
        HIPCHK(hipStreamCreateWithFlags(&n->copy_stream, hipStreamNonBlocking));
        for (size_t k = 0; k < S; ++k) {
            hipEvent_t e;
            HIPCHK(hipEventCreateWithFlags(&e, hipEventDisableTiming));
            n->ev_slot_ready.push_back(e);
            HIPCHK(hipEventCreateWithFlags(&e, hipEventDisableTiming));
            n->ev_slot_free.push_back(e);
        }
    }
    HIPCHK(dev_malloc(&n->d_lab, (size_t)n->N * 8));
    HIPCHK(hipMemcpy(n->d_lab, n->layers[0].in_pos.data(), (size_t)n->N * 4, hipMemcpyHostToDevice));
    n->lab_layer = -1;
    int rc = alloc_feature_buffers(n);
    if (rc) return rc;
    n->uploaded = true;
    return SPDNN_OK;
}

int ensure_uploaded(spdnn_net* n) {
    if (n->uploaded) return SPDNN_OK;
    if (!n->inspected) return fail(SPDNN_E_STATE, "spdnn_inspect has not been called");
    int rc = ensure_device(n);
    if (rc) return rc;
    rc = upload_plans(n);
    if (rc != SPDNN_OK) free_device(n);
    return rc;
}

void free_device(spdnn_net* n) {
    if (n->copy_stream) {
        hipStreamSynchronize(n->copy_stream);
        hipStreamDestroy(n->copy_stream);
        n->copy_stream = nullptr;
    }
    for (hipEvent_t e : n->ev_slot_ready) hipEventDestroy(e);
    for (hipEvent_t e : n->ev_slot_free) hipEventDestroy(e);
    n->ev_slot_ready.clear();
    n->ev_slot_free.clear();
    n->slot_layer.clear();
    n->slot_busy.clear();
    if (n->h_plans) hipHostFree(n->h_plans);
    n->h_plans = nullptr;
    if (n->d_lab) hipFree(n->d_lab);
    n->d_lab = nullptr;
    n->lab_layer = -1;
    if (n->arena) hipFree(n->arena);
    if (n->d_table) hipFree(n->d_table);
    n->d_table = nullptr;
    for (float* p : n->feat_allocs) hipFree(p);
    n->feat_allocs.clear();
    n->arena = nullptr;
    n->F = n->A = n->C = Feat();
    n->uploaded = false;
    n->have_features = false;
}

bool plans_streamed(const spdnn_net* n) { return n->copy_stream != nullptr; }

// Streamed plans: starts the copy of layer l's plan into its slot (unless the slot holds it or is
// being filled with it already).  The copy waits for the last kernel that read the slot.
hipError_t plan_fetch(spdnn_net* n, int l) {
    const size_t slot = (size_t)l % (size_t)n->plan_window;
    if (n->slot_layer[slot] == l) return hipSuccess;
    hipError_t e;
    if (n->slot_busy[slot]) {
        if ((e = hipStreamWaitEvent(n->copy_stream, n->ev_slot_free[slot], 0)) != hipSuccess) return e;
    }
    const PlanLayout& y = n->lay[(size_t)l];
    if (y.bytes) {
        e = hipMemcpyAsync((char*)n->arena + slot * n->slot_bytes, n->h_plans + n->h_plan_off[(size_t)l], y.bytes,
                           hipMemcpyHostToDevice, n->copy_stream);
        if (e != hipSuccess) return e;
    }
    if ((e = hipEventRecord(n->ev_slot_ready[slot], n->copy_stream)) != hipSuccess) return e;
    n->slot_layer[slot] = l;
    n->slot_busy[slot] = 0;
    return hipSuccess;
}

// Before the launch of layer l: its plan is in its slot (the compute stream waits for the copy).
hipError_t plan_acquire(spdnn_net* n, int l) {
    if (!plans_streamed(n)) return hipSuccess;
    hipError_t e = plan_fetch(n, l);
    if (e != hipSuccess) return e;
    return hipStreamWaitEvent(n->stream, n->ev_slot_ready[(size_t)l % (size_t)n->plan_window], 0);
}

// After the launch of layer l: the slot is handed to the layer that uses it next.
hipError_t plan_release(spdnn_net* n, int l) {
    if (!plans_streamed(n)) return hipSuccess;
    const size_t slot = (size_t)l % (size_t)n->plan_window;
    hipError_t e = hipEventRecord(n->ev_slot_free[slot], n->stream);
    if (e != hipSuccess) return e;
    n->slot_busy[slot] = 1;
    const int next = l + n->plan_window;
    return next < n->L ? plan_fetch(n, next) : hipSuccess;
}

// physical-column labelling of the buffer that holds the state after `layers_done` layers
// (nullptr = identity, after the last layer); *out is device memory
hipError_t labelling_dev(spdnn_net* n, int layers_done, const int32_t** out) {
    if (layers_done >= n->L) { *out = nullptr; return hipSuccess; }
    if (layers_done == 0) { *out = n->d_lab; return hipSuccess; }
    int32_t* second = n->d_lab + n->N;
    if (n->lab_layer != layers_done) {
        hipError_t e = hipMemcpy(second, n->layers[(size_t)layers_done].in_pos.data(), (size_t)n->N * 4,
                                 hipMemcpyHostToDevice);
        if (e != hipSuccess) return e;
        n->lab_layer = layers_done;
    }
    *out = second;
    return hipSuccess;
}

void reset_state(spdnn_net* n) {
    if (n->stamp > 0x60000000) {  // row stamps are launch numbers: start over long before they wrap
        hipMemsetAsync(n->d_active, 0, (size_t)n->rows_cap * 4, n->stream);
        hipMemsetAsync(n->d_active_mid, 0, (size_t)n->rows_cap * 4, n->stream);
        n->stamp = 0;
    }
    if (n->gid_dirty) {
        launch_iota_gid(n->d_gid, n->rows_cap, n->batch, n->stream);
        n->gid_dirty = false;
    }
    n->cur = n->F;
    n->last_stamp = 0;
    n->blocks_skipped = false;
    n->cur_layer = 0;
    n->carried = ((n->batch + n->RB - 1) / n->RB) * n->RB;
    n->alive = n->batch;
    n->alive_list_valid = false;
}

// inspect_layer for a worker thread: a worker must not let an exception escape (std::terminate); the
// layer stays unset and spdnn_inspect reports what happened
void inspect_on_worker(int N, const std::vector<int32_t>& rp, const std::vector<int32_t>& col, const std::vector<float>& val,
                       int force, bool fma_ok, LayerPlan* plan, const std::vector<int32_t>* common_pos = nullptr) {
    try {
        inspect_layer(N, rp, col, val, force, fma_ok, *plan, common_pos);
    } catch (const std::bad_alloc&) {
        plan->set = false;
        plan->failed = plan->failed_nomem = true;
    } catch (const std::exception& e) {
        plan->set = false;
        plan->failed = true;
        plan->failed_nomem = false;
        plan->fail_text = e.what();
    } catch (...) {
        plan->set = false;
        plan->failed = true;
        plan->failed_nomem = false;
        plan->fail_text = "unknown exception";
    }
}

int submit_layer(spdnn_net* n, int layer, std::shared_ptr<std::vector<int32_t>> rp,
                 std::shared_ptr<std::vector<int32_t>> col, std::shared_ptr<std::vector<float>> val) {
    n->inspected = false;
    const int force = n->force_kernel;
    const int N = n->N;
    LayerPlan* plan = &n->layers[(size_t)layer];
    const bool fma_ok = n->fma_ok;
    n->pool->submit([=] { inspect_on_worker(N, *rp, *col, *val, force, fma_ok, plan); });
    return SPDNN_OK;
}

}  // namespace

// Exception barrier of the C ABI: status codes, never an exception across the boundary and never
// std::terminate (a failed allocation inside a loader or the inspector ends here).
template <class F> int guarded(F&& f) {
    try {
        return f();
    } catch (const std::bad_alloc&) {
        return fail(SPDNN_E_NOMEM, "out of host memory");
    } catch (const std::length_error&) {
        return fail(SPDNN_E_NOMEM, "out of host memory (size beyond what a container can hold)");
    } catch (const std::exception& e) {
        return fail(SPDNN_E_ARG, std::string("unexpected failure: ") + e.what());
    } catch (...) {
        return fail(SPDNN_E_ARG, "unexpected failure");
    }
}

extern "C" {

int spdnn_version(void) { return 200; }

const char* spdnn_last_error(void) { return g_err.c_str(); }

static int spdnn_create_impl(int neuron, int max_batch, int layers, float bias, float clamp, spdnn_net** out) {
    if (!out) return fail(SPDNN_E_ARG, "out is NULL");
    *out = nullptr;
    if (neuron < 1 || neuron > (1 << 24)) return fail(SPDNN_E_ARG, "neuron must be in [1, 2^24]");
    if (max_batch < 1) return fail(SPDNN_E_ARG, "max_batch must be positive");
    if (layers < 1) return fail(SPDNN_E_ARG, "layers must be positive");
    if (!std::isfinite(bias) || !(clamp > 0.0f) || !(clamp <= 1.2676506e30f) || !(std::fabs(bias) <= 1.2676506e30f))
        return fail(SPDNN_E_ARG, "bias must be finite and clamp positive, both at most 2^100 in magnitude");
    spdnn_net* n = new (std::nothrow) spdnn_net();
    if (!n) return fail(SPDNN_E_NOMEM, "out of host memory");
    n->N = neuron; n->max_batch = max_batch; n->L = layers; n->bias = bias; n->clampv = clamp;
    n->fma_ok = std::fabs(bias) >= 9.094947e-13f && clamp >= 9.094947e-13f;  // 2^-40
    int rl = 4;
    if (const char* e = getenv("SPDNN_ROWS_PER_LANE")) rl = atoi(e);
    if (rl != 1 && rl != 2 && rl != 4) { delete n; return fail(SPDNN_E_ARG, "SPDNN_ROWS_PER_LANE must be 1, 2 or 4"); }
    n->rl = rl; n->RB = 64 * rl;
    n->rows_cap = ((max_batch + n->RB - 1) / n->RB) * n->RB;
    n->layers.resize((size_t)layers);
    n->pending.assign((size_t)layers, 0);
    n->counts.assign((size_t)layers, -1);
    n->layer_ms.assign((size_t)layers, 0.0f);
    n->pool.reset(new JobPool(host_threads()));
    if (const char* e = getenv("SPDNN_AUTOTUNE")) n->autotune = atoi(e) != 0;
    if (const char* e = getenv("SPDNN_RUN_VERBOSE")) n->run_verbose = atoi(e) != 0;
    if (const char* e = getenv("SPDNN_PERSIST")) n->persist_mode = atoi(e) != 0 ? 1 : 0;
    if (const char* e = getenv("SPDNN_PERSIST_LAYERS")) n->persist_layers = std::max(2, atoi(e));
    if (const char* e = getenv("SPDNN_PERSIST_MAX_BYTES")) n->persist_max_bytes = atoll(e);
    if (const char* e = getenv("SPDNN_PERSIST_MIN_BYTES")) n->persist_min_bytes = atoll(e);
    if (const char* e = getenv("SPDNN_PERSIST_XCD")) n->persist_xcd = atoi(e);
    if (const char* e = getenv("SPDNN_PERSIST_MIN_BLOCKS")) n->persist_min_blocks = std::max(1, atoi(e));
    if (const char* e = getenv("SPDNN_PERSIST_LIGHT_SYNC")) n->persist_light = atoi(e) != 0 ? 1 : 0;
    if (const char* e = getenv("SPDNN_PERSIST_SEGLEN")) n->persist_seglen = std::max(0, atoi(e));
    if (const char* e = getenv("SPDNN_RESIDENT")) n->resident_mode = atoi(e) != 0 ? 1 : 0;
    if (const char* e = getenv("SPDNN_PERSIST_WAIT_US")) n->persist_wait_us = std::max(0ll, atoll(e));
    if (const char* e = getenv("SPDNN_BAND_SEGLEN")) n->band_seglen = std::max(0, atoi(e));
    if (const char* e = getenv("SPDNN_BAND_DIRECT_LDS")) n->band_direct_lds = atoi(e) != 0 ? 1 : 0;
    if (const char* e = getenv("SPDNN_FUSE_PAIRS")) n->fuse_pairs = atoi(e) != 0;
    if (const char* e = getenv("SPDNN_BAND_SUM_THEN_SCALE")) n->add_only = atoi(e) != 0 ? 1 : 0;
    if (const char* e = getenv("SPDNN_PAIR_SEGLEN")) n->pair_seglen = atoi(e);
    if (const char* e = getenv("SPDNN_PAIR_MIN_ELEMS")) n->pair_min_elems = atoll(e);
    if (const char* e = getenv("SPDNN_BLOCK_FORM_MAX_ELEMS")) n->block_form_max_elems = atoll(e);
    if (const char* e = getenv("SPDNN_TILED_MIN_ROWS")) { n->tiled_min_rows = atoll(e); n->tiled_min_rows_given = true; }
    if (const char* e = getenv("SPDNN_ROWTILE")) n->rowtile_mode = atoi(e) != 0 ? 1 : 0;
    if (const char* e = getenv("SPDNN_BAND_RESIDENT")) n->band_resident_mode = atoi(e) != 0 ? 1 : 0;
    if (const char* e = getenv("SPDNN_BAND_RESIDENT_MIN_LAYERS")) n->band_resident_min_layers = std::max(0, atoi(e));
    if (const char* e = getenv("SPDNN_STREAM_MIN_BYTES")) n->stream_min_bytes = atoll(e);
    if (const char* e = getenv("SPDNN_COUNT_TIMEOUT_MS")) n->count_timeout_ms = std::max(1ll, atoll(e));
    if (const char* e = getenv("SPDNN_PLAN_WINDOW")) {
        const int w = atoi(e);
        if (w == 0 || (w >= 2 && w <= 64)) n->plan_window = w;
    }
    *out = n;
    return SPDNN_OK;
}

static int spdnn_destroy_impl(spdnn_net* n) {
    if (!n) return SPDNN_OK;
    n->pool->wait_all();
    n->pool.reset();
    if (n->dev_ready) {
        hipStreamSynchronize(n->stream);
        free_device(n);
        release_device_base(n);
    }
    delete n;
    return SPDNN_OK;
}

static int spdnn_reference_bias_impl(int neuron, float* bias) {
    if (!bias) return fail(SPDNN_E_ARG, "bias is NULL");
    switch (neuron) {
        case 1024: *bias = -0.3f; return SPDNN_OK;
        case 4096: *bias = -0.35f; return SPDNN_OK;
        case 16384: *bias = -0.4f; return SPDNN_OK;
        case 65536: *bias = -0.45f; return SPDNN_OK;
        default: return fail(SPDNN_E_ARG, "no reference bias for this neuron count");
    }
}

static int spdnn_set_force_kernel_impl(spdnn_net* n, int kernel) {
    if (!n) return fail(SPDNN_E_ARG, "net is NULL");
    if (kernel != SPDNN_KERNEL_AUTO && kernel != SPDNN_KERNEL_GATHER)
        return fail(SPDNN_E_ARG, "only AUTO or GATHER can be forced");
    for (const LayerPlan& p : n->layers)
        if (p.set) return fail(SPDNN_E_STATE, "set the forced kernel before any layer");
    n->force_kernel = kernel;
    return SPDNN_OK;
}

static int spdnn_set_layer_csr_impl(spdnn_net* n, int layer, const int32_t* rowptr, const int32_t* col, const float* val) {
    if (!n) return fail(SPDNN_E_ARG, "net is NULL");
    if (layer < 0 || layer >= n->L) return fail(SPDNN_E_ARG, "layer out of range");
    auto rp = std::make_shared<std::vector<int32_t>>();
    auto cc = std::make_shared<std::vector<int32_t>>();
    auto vv = std::make_shared<std::vector<float>>();
    const std::string err = normalize_csr(n->N, rowptr, col, val, *rp, *cc, *vv);
    if (!err.empty()) return fail(SPDNN_E_ARG, err);
    if (n->pending[(size_t)layer]) {  // the layer is being replaced: never race with its earlier job
        n->pool->wait_all();
        std::fill(n->pending.begin(), n->pending.end(), 0);
    }
    n->pending[(size_t)layer] = 1;
    return submit_layer(n, layer, rp, cc, vv);
}

static int spdnn_load_layer_tsv_impl(spdnn_net* n, int layer, const char* path) {
    if (!n || !path) return fail(SPDNN_E_ARG, "NULL argument");
    if (layer < 0 || layer >= n->L) return fail(SPDNN_E_ARG, "layer out of range");
    std::vector<int32_t> rp, cc;
    std::vector<float> vv;
    std::string err;
    if (!read_weight_tsv_csr(path, n->N, rp, cc, vv, err)) return fail(SPDNN_E_IO, err);
    return spdnn_set_layer_csr(n, layer, rp.data(), cc.data(), vv.data());
}

static int spdnn_load_layers_tsv_impl(spdnn_net* n, const char* data_dir, int first, int count) {
    if (!n || !data_dir) return fail(SPDNN_E_ARG, "NULL argument");
    if (first < 0 || count < 0 || first + count > n->L) return fail(SPDNN_E_ARG, "layer range out of bounds");
    n->pool->wait_all();
    std::fill(n->pending.begin(), n->pending.end(), 0);
    n->inspected = false;
    const int N = n->N, force = n->force_kernel;
    const bool fma_ok = n->fma_ok;
    const std::string dir = data_dir;
    // every worker parses, validates and inspects whole layers; the first failure by layer number is reported
    auto errs = std::make_shared<std::vector<std::string>>((size_t)count);
    auto codes = std::make_shared<std::vector<int>>((size_t)count, SPDNN_OK);
    for (int l = first; l < first + count; ++l) {
        LayerPlan* plan = &n->layers[(size_t)l];
        const size_t k = (size_t)(l - first);
        n->pool->submit([=] {
            plan->set = false;   // until the inspection has succeeded (whatever fails on the way)
            const std::string path = dir + "/neuron" + std::to_string(N) + "/n" + std::to_string(N) + "-l" +
                                     std::to_string(l + 1) + ".tsv";
            std::vector<int32_t> rp, cc, rp2, cc2;
            std::vector<float> vv, vv2;
            std::string err;
            if (!read_weight_tsv_csr(path, N, rp, cc, vv, err)) {
                (*errs)[k] = err;
                (*codes)[k] = SPDNN_E_IO;
                plan->set = false;
                return;
            }
            err = normalize_csr(N, rp.data(), cc.data(), vv.data(), rp2, cc2, vv2);
            if (!err.empty()) {
                (*errs)[k] = path + ": " + err;
                (*codes)[k] = SPDNN_E_ARG;
                plan->set = false;
                return;
            }
            inspect_on_worker(N, rp2, cc2, vv2, force, fma_ok, plan);
        });
    }
    n->pool->wait_all();
    for (size_t k = 0; k < (size_t)count; ++k)
        if ((*codes)[k] != SPDNN_OK) return fail((*codes)[k], (*errs)[k]);
    return SPDNN_OK;
}

static int spdnn_load_layers_bin_impl(spdnn_net* n, const char* path, int first, int count, int64_t nnz_per_layer) {
    if (!n || !path) return fail(SPDNN_E_ARG, "NULL argument");
    if (first < 0 || count < 0 || first + count > n->L) return fail(SPDNN_E_ARG, "layer range out of bounds");
    const int64_t nnz = nnz_per_layer > 0 ? nnz_per_layer : (int64_t)32 * n->N;
    if (nnz > (int64_t)INT32_MAX) return fail(SPDNN_E_ARG, "nnz_per_layer too large");
    std::vector<int32_t> rp, cc;
    std::vector<float> vv;
    std::string err;
    for (int l = first; l < first + count; ++l) {
        if (!read_weight_bin_csr(path, n->N, l, nnz, rp, cc, vv, err)) return fail(SPDNN_E_IO, err);
        const int rc = spdnn_set_layer_csr(n, l, rp.data(), cc.data(), vv.data());
        if (rc) return rc;
    }
    return SPDNN_OK;
}

static int spdnn_weight_file_name_impl(const char* data_dir, int neuron, int layer, char* out, int cap) {
    if (!data_dir || !out || cap < 1) return fail(SPDNN_E_ARG, "NULL argument");
    const int w = snprintf(out, (size_t)cap, "%s/neuron%d/n%d-l%d.tsv", data_dir, neuron, neuron, layer + 1);
    if (w < 0 || w >= cap) return fail(SPDNN_E_ARG, "buffer too small");
    return SPDNN_OK;
}

static int spdnn_synth_layer_csr_impl(uint64_t seed, int layer, int neuron, int nnz_per_row, float value,
                          int32_t* rowptr, int32_t* col, float* val) {
    if (!rowptr || !col || !val) return fail(SPDNN_E_ARG, "NULL argument");
    std::vector<int32_t> rp, cc;
    std::vector<float> vv;
    if (!synth_layer_csr(seed, layer, neuron, nnz_per_row, value, rp, cc, vv))
        return fail(SPDNN_E_ARG, "bad generator arguments");
    std::copy(rp.begin(), rp.end(), rowptr);
    std::copy(cc.begin(), cc.end(), col);
    std::copy(vv.begin(), vv.end(), val);
    return SPDNN_OK;
}

static int spdnn_synth_layers_impl(spdnn_net* n, uint64_t seed, int first, int count, int nnz_per_row, float value) {
    if (!n) return fail(SPDNN_E_ARG, "net is NULL");
    if (first < 0 || count < 0 || first + count > n->L) return fail(SPDNN_E_ARG, "layer range out of bounds");
    if (nnz_per_row < 1 || nnz_per_row > n->N || !std::isfinite(value))
        return fail(SPDNN_E_ARG, "bad nnz_per_row or value");
    n->pool->wait_all();
    std::fill(n->pending.begin(), n->pending.end(), 0);
    n->inspected = false;
    const int N = n->N, force = n->force_kernel;
    const bool fma_ok = n->fma_ok;
    for (int l = first; l < first + count; ++l) {
        n->pending[(size_t)l] = 1;
        LayerPlan* plan = &n->layers[(size_t)l];
        n->pool->submit([=] {
            plan->set = false;   // until the inspection has succeeded (whatever fails on the way)
            std::vector<int32_t> rp, cc;
            std::vector<float> vv;
            synth_layer_csr(seed, l, N, nnz_per_row, value, rp, cc, vv);
            inspect_on_worker(N, rp, cc, vv, force, fma_ok, plan);
        });
    }
    return SPDNN_OK;
}

// Every layer inspected?  Otherwise the status that says what happened to the first one that is not.
static int layers_all_set(spdnn_net* n) {
    for (int l = 0; l < n->L; ++l)
        if (!n->layers[(size_t)l].set) {
            const LayerPlan& p = n->layers[(size_t)l];
            if (p.failed && p.failed_nomem)
                return fail(SPDNN_E_NOMEM, "the inspection of layer " + std::to_string(l) + " ran out of host memory; hand it over again");
            if (p.failed)
                return fail(SPDNN_E_UNSUPPORTED, "the inspection of layer " + std::to_string(l) + " failed: " + p.fail_text);
            return fail(SPDNN_E_STATE, "layer " + std::to_string(l) + " has not been set");
        }
    return SPDNN_OK;
}

// Second pass over the run-chain layers with one exact weight.  Each of them chose a labelling of its
// own, so no two agree on where a neuron sits and none can hand its outputs to the next one in LDS.
// When the network's files share one neuron numbering there is an order that serves several of them at
// once (common_run_order, taken from the first such layer whose groups form a single cycle): every
// layer it fits (common_order_offset: the stride of that layer and twice it) is laid out again in that
// order, and neighbours among them then pass pair_fusable.
static void adopt_common_order(spdnn_net* n) {
    if (getenv("SPDNN_COMMON_ORDER") && atoi(getenv("SPDNN_COMMON_ORDER")) == 0) return;
    const int N = n->N;
    auto pos = std::make_shared<std::vector<int32_t>>();
    std::vector<int32_t> rp, cc;
    int tried = 0;
    for (int l = 0; l < n->L && pos->empty() && tried < 4; ++l) {
        const LayerPlan& p = n->layers[(size_t)l];
        if (p.kernel != SPDNN_KERNEL_BAND || p.alt_ngroups == 0 || p.rc_cycles != 1) continue;
        ++tried;
        plan_adjacency(p, N, rp, cc);
        if (!common_run_order(N, rp, cc, *pos)) pos->clear();
    }
    if (pos->empty()) return;
    const int force = n->force_kernel;
    const bool fma_ok = n->fma_ok;
    for (int l = 0; l < n->L; ++l) {
        LayerPlan* p = &n->layers[(size_t)l];
        if (p->kernel != SPDNN_KERNEL_BAND || p->alt_ngroups == 0 || p->rc_cycles > 2) continue;
        if (p->info.common_order > 0 && p->in_pos == *pos) continue;   // laid out that way by an earlier call
        n->pool->submit([=] {
            try {
                std::vector<int32_t> rowptr, col;
                plan_adjacency(*p, N, rowptr, col);
                if (common_order_offset(N, rowptr, col, *pos) == 0) return;
                const std::vector<float> val(col.size(), p->info.value);
                inspect_on_worker(N, rowptr, col, val, force, fma_ok, p, pos.get());
            } catch (...) {
                // out of memory before the layer was touched: it keeps the labelling it has
            }
        });
    }
    n->pool->wait_all();
}

static int spdnn_inspect_impl(spdnn_net* n) {
    if (!n) return fail(SPDNN_E_ARG, "net is NULL");
    n->pool->wait_all();
    std::fill(n->pending.begin(), n->pending.end(), 0);
    if (int rc = layers_all_set(n)) return rc;
    adopt_common_order(n);
    if (int rc = layers_all_set(n)) return rc;
    for (int l = 0; l < n->L; ++l) {
        LayerPlan* cur = &n->layers[(size_t)l];
        const std::vector<int32_t>* nxt = l + 1 < n->L ? &n->layers[(size_t)l + 1].in_pos : nullptr;
        n->pool->submit([=] { link_layers(*cur, nxt); });
    }
    n->pool->wait_all();
    for (int l = 0; l < n->L; ++l) {
        LayerPlan& p = n->layers[(size_t)l];
        p.fuse_next = l + 1 < n->L && n->rl == 4 && pair_fusable(p, n->layers[(size_t)l + 1], n->N);
        p.info.fuse_next = p.fuse_next ? 1 : 0;
    }
    if (n->uploaded) free_device(n);  // plans changed: upload again on next use
    n->tuned.clear();
    n->exploring.clear();
    for (const spdnn_net::Trial& t : n->trials) { n->ev_free.push_back(t.e0); n->ev_free.push_back(t.e1); }
    n->trials.clear();
    n->inspected = true;
    return SPDNN_OK;
}

static int spdnn_set_plan_window_impl(spdnn_net* n, int slots) {
    if (!n) return fail(SPDNN_E_ARG, "net is NULL");
    if (slots != 0 && (slots < 2 || slots > 64)) return fail(SPDNN_E_ARG, "plan window is 0 (all plans resident) or 2..64 slots");
    if (n->uploaded) return fail(SPDNN_E_STATE, "plans are on the device already: set the window before the features");
    n->plan_window = slots;
    return SPDNN_OK;
}

static int spdnn_get_plan_memory_impl(const spdnn_net* n, int* window, int64_t* device_bytes, int64_t* pinned_bytes) {
    if (!n) return fail(SPDNN_E_ARG, "net is NULL");
    if (!n->uploaded) return fail(SPDNN_E_STATE, "plans are not on the device yet");
    int64_t total = 0;
    for (const PlanLayout& y : n->lay) total += (int64_t)y.bytes;
    const bool st = plans_streamed(n);
    if (window) *window = st ? n->plan_window : 0;
    if (device_bytes) *device_bytes = st ? (int64_t)n->plan_window * (int64_t)n->slot_bytes : total;
    if (pinned_bytes) *pinned_bytes = st ? total : 0;
    return SPDNN_OK;
}

static int spdnn_get_layer_plan_impl(const spdnn_net* n, int layer, spdnn_layer_plan* out) {
    if (!n || !out) return fail(SPDNN_E_ARG, "NULL argument");
    if (layer < 0 || layer >= n->L) return fail(SPDNN_E_ARG, "layer out of range");
    const_cast<spdnn_net*>(n)->pool->wait_all();
    if (!n->layers[(size_t)layer].set) return fail(SPDNN_E_STATE, "layer has not been set");
    *out = n->layers[(size_t)layer].info;
    return SPDNN_OK;
}

static int spdnn_get_band_plan_impl(const spdnn_net* n, int layer, int32_t* in_pos, int32_t* out_at, uint8_t* sel) {
    if (!n) return fail(SPDNN_E_ARG, "net is NULL");
    if (layer < 0 || layer >= n->L) return fail(SPDNN_E_ARG, "layer out of range");
    const_cast<spdnn_net*>(n)->pool->wait_all();
    const LayerPlan& p = n->layers[(size_t)layer];
    if (!p.set || p.kernel != SPDNN_KERNEL_BAND) return fail(SPDNN_E_STATE, "not a BAND layer");
    if (in_pos) std::copy(p.in_pos.begin(), p.in_pos.end(), in_pos);
    if (out_at) std::copy(p.out_at.begin(), p.out_at.end(), out_at);
    if (sel) std::copy(p.sel.begin(), p.sel.end(), sel);
    return SPDNN_OK;
}

static int spdnn_get_band_pairs_impl(const spdnn_net* n, int layer, int* steps, int* stride, int* padded_steps,
                         int* has_weights, uint32_t* records, float* weights) {
    if (!n) return fail(SPDNN_E_ARG, "net is NULL");
    if (layer < 0 || layer >= n->L) return fail(SPDNN_E_ARG, "layer out of range");
    const_cast<spdnn_net*>(n)->pool->wait_all();
    const LayerPlan& p = n->layers[(size_t)layer];
    if (!p.set || p.kernel != SPDNN_KERNEL_BAND) return fail(SPDNN_E_STATE, "not a BAND layer");
    if (steps) *steps = p.pair_steps;
    if (stride) *stride = p.pair_stride;
    if (padded_steps) *padded_steps = p.pair_padded;
    if (has_weights) *has_weights = p.wmode != 0 ? 1 : 0;
    if (records) std::copy(p.pairs.begin(), p.pairs.end(), records);
    if (weights) std::copy(p.wv.begin(), p.wv.end(), weights);
    return SPDNN_OK;
}

static int spdnn_get_band_quads_impl(const spdnn_net* n, int layer, int* groups, uint32_t* columns, float* weights) {
    if (!n) return fail(SPDNN_E_ARG, "net is NULL");
    if (layer < 0 || layer >= n->L) return fail(SPDNN_E_ARG, "layer out of range");
    const_cast<spdnn_net*>(n)->pool->wait_all();
    const LayerPlan& p = n->layers[(size_t)layer];
    if (!p.set || p.kernel != SPDNN_KERNEL_BAND) return fail(SPDNN_E_STATE, "not a BAND layer");
    if (groups) *groups = p.quad_groups;
    if (columns) std::copy(p.quad_col.begin(), p.quad_col.end(), columns);
    if (weights) std::copy(p.quad_w.begin(), p.quad_w.end(), weights);
    return SPDNN_OK;
}

static int spdnn_get_layer_dst_impl(const spdnn_net* n, int layer, int32_t* dst) {
    if (!n || !dst) return fail(SPDNN_E_ARG, "NULL argument");
    if (layer < 0 || layer >= n->L) return fail(SPDNN_E_ARG, "layer out of range");
    if (!n->inspected) return fail(SPDNN_E_STATE, "spdnn_inspect has not been called");
    const LayerPlan& p = n->layers[(size_t)layer];
    std::copy(p.dst.begin(), p.dst.end(), dst);
    return SPDNN_OK;
}

static int spdnn_receptive_field_impl(spdnn_net* n, int first_layer, int n_layers, const int32_t* out_neurons, int n_out,
                          int32_t* in_neurons, int64_t cap, int64_t* count) {
    if (!n || !count || (n_out > 0 && !out_neurons)) return fail(SPDNN_E_ARG, "NULL argument");
    if (first_layer < 0 || n_layers < 1 || first_layer + n_layers > n->L) return fail(SPDNN_E_ARG, "layer range out of bounds");
    if (n_out < 0 || cap < 0) return fail(SPDNN_E_ARG, "negative size");
    for (int t = 0; t < n_out; ++t)
        if (out_neurons[t] < 0 || out_neurons[t] >= n->N) return fail(SPDNN_E_ARG, "neuron out of range");
    n->pool->wait_all();
    for (int l = first_layer; l < first_layer + n_layers; ++l)
        if (!n->layers[(size_t)l].set) return fail(SPDNN_E_STATE, "layer " + std::to_string(l) + " has not been set");
    std::vector<int32_t> in;
    receptive_field(&n->layers[(size_t)first_layer], n->N, n_layers, out_neurons, n_out, in);
    *count = (int64_t)in.size();
    if (in_neurons) std::copy(in.begin(), in.begin() + (size_t)std::min<int64_t>(cap, (int64_t)in.size()), in_neurons);
    return SPDNN_OK;
}

static int spdnn_get_layer_slots_impl(const spdnn_net* n, int layer, int* slots) {
    if (!n || !slots) return fail(SPDNN_E_ARG, "NULL argument");
    if (layer < 0 || layer >= n->L) return fail(SPDNN_E_ARG, "layer out of range");
    const_cast<spdnn_net*>(n)->pool->wait_all();
    if (!n->layers[(size_t)layer].set) return fail(SPDNN_E_STATE, "layer has not been set");
    *slots = (int)n->layers[(size_t)layer].out_at.size();
    return SPDNN_OK;
}

static int spdnn_get_input_labelling_impl(const spdnn_net* n, int layer, int32_t* phys_col) {
    if (!n || !phys_col) return fail(SPDNN_E_ARG, "NULL argument");
    if (layer < 0 || layer > n->L) return fail(SPDNN_E_ARG, "layer out of range");
    const_cast<spdnn_net*>(n)->pool->wait_all();
    if (layer == n->L) {
        for (int i = 0; i < n->N; ++i) phys_col[i] = i;
        return SPDNN_OK;
    }
    const LayerPlan& p = n->layers[(size_t)layer];
    if (!p.set) return fail(SPDNN_E_STATE, "layer has not been set");
    std::copy(p.in_pos.begin(), p.in_pos.end(), phys_col);
    return SPDNN_OK;
}

static int spdnn_hash_reorder_impl(int v, int buckets, int domain, int* out) {
    if (!out) return fail(SPDNN_E_ARG, "out is NULL");
    if (buckets <= 0 || domain <= 0 || v < 0 || v >= domain) return fail(SPDNN_E_ARG, "ERROR: Hasing Function error!");
    const int width = domain / buckets;
    *out = v / buckets + (v % buckets) * width;
    return SPDNN_OK;
}

// ---- features ----------------------------------------------------------------------------

static int begin_features(spdnn_net* n, int batch) {
    if (!n) return fail(SPDNN_E_ARG, "net is NULL");
    if (batch < 1 || batch > n->max_batch) return fail(SPDNN_E_ARG, "batch must be in [1, max_batch]");
    if (!n->inspected) return fail(SPDNN_E_STATE, "spdnn_inspect has not been called (or a layer changed since)");
    int rc = ensure_uploaded(n);
    if (rc) return rc;
    n->batch = batch;
    n->have_features = false;
    return SPDNN_OK;
}

static int spdnn_set_features_dense_impl(spdnn_net* n, const float* rowmajor, int batch) {
    if (!rowmajor) return fail(SPDNN_E_ARG, "rowmajor is NULL");
    int rc = begin_features(n, batch);
    if (rc) return rc;
    const int RB = n->RB, N = n->N;
    // staging chunk: a whole number of row blocks, about 256 MiB
    int64_t chunk_rows = std::max<int64_t>(RB, ((int64_t)(256 << 20) / ((int64_t)N * 4)) / RB * RB);
    chunk_rows = std::min<int64_t>(chunk_rows, n->rows_cap);
    DevTmp stage_buf;
    HIPCHK(stage_buf.alloc((size_t)chunk_rows * N * 4));
    float* stage = stage_buf.as<float>();
    HIPCHK(hipMemsetAsync(n->d_nonfinite, 0, 8, n->stream));
    const int padded = ((batch + RB - 1) / RB) * RB;
    for (int64_t r0 = 0; r0 < padded; r0 += chunk_rows) {
        const int64_t rows_here = std::min<int64_t>(chunk_rows, padded - r0);
        const int64_t real = std::max<int64_t>(0, std::min<int64_t>(rows_here, batch - r0));
        if (real > 0)
            HIPCHK(hipMemcpyAsync(stage, rowmajor + (size_t)r0 * N, (size_t)real * N * 4, hipMemcpyHostToDevice,
                                  n->stream));
        // rows >= real inside the chunk are written as zero by the kernel (nrows = real)
        HIPCHK(launch_pack_rows(stage, n->F, n->d_lab, N, r0, (int)std::max<int64_t>(real, 1), n->rl,
                                n->d_nonfinite, n->stream));
        HIPCHK(hipStreamSynchronize(n->stream));  // the staging buffer is reused by the next chunk
    }
    int32_t bad[2] = {0, 0};
    HIPCHK(hipMemcpy(bad, n->d_nonfinite, 8, hipMemcpyDeviceToHost));
    if (bad[0]) return fail(SPDNN_E_ARG, "features contain NaN, infinity or values above 2^100 in magnitude");
    if (bad[1]) return fail(SPDNN_E_ARG, "features contain nonzero values below 2^-100 in magnitude");
    HIPCHK(launch_iota_gid(n->d_gid, n->rows_cap, batch, n->stream));
    HIPCHK(hipStreamSynchronize(n->stream));
    n->have_features = true;
    reset_state(n);
    return SPDNN_OK;
}

static int spdnn_load_features_tsv_impl(spdnn_net* n, const char* path, int batch) {
    if (!n || !path) return fail(SPDNN_E_ARG, "NULL argument");
    if (batch < 1 || batch > n->max_batch) return fail(SPDNN_E_ARG, "batch must be in [1, max_batch]");
    std::vector<float> dense;
    std::string err;
    int64_t kept = 0;
    if (!read_features_tsv_dense(path, n->N, batch, dense, &kept, err, host_threads())) return fail(SPDNN_E_IO, err);
    return spdnn_set_features_dense(n, dense.data(), batch);
}

static int spdnn_read_features_tsv_impl(const char* path, int neuron, int batch, float* rowmajor, int64_t* kept) {
    if (!path || !rowmajor) return fail(SPDNN_E_ARG, "NULL argument");
    if (neuron < 1 || batch < 1) return fail(SPDNN_E_ARG, "neuron and batch must be positive");
    std::string err;
    int64_t k = 0;
    if (!read_features_tsv_into(path, neuron, batch, rowmajor, &k, err, host_threads())) return fail(SPDNN_E_IO, err);
    if (kept) *kept = k;
    return SPDNN_OK;
}

static int spdnn_load_features_bin_impl(spdnn_net* n, const char* path, int batch) {
    if (!n || !path) return fail(SPDNN_E_ARG, "NULL argument");
    if (batch < 1 || batch > n->max_batch) return fail(SPDNN_E_ARG, "batch must be in [1, max_batch]");
    std::vector<float> dense;
    std::string err;
    int64_t kept = 0;
    if (!read_features_bin_dense(path, n->N, batch, dense, &kept, err)) return fail(SPDNN_E_IO, err);
    return spdnn_set_features_dense(n, dense.data(), batch);
}

static int spdnn_synth_features_impl(spdnn_net* n, uint64_t seed, int batch, float dmin, float dmax) {
    if (!(dmin >= 0.0f) || !(dmax >= dmin) || !(dmax <= 1.0f)) return fail(SPDNN_E_ARG, "need 0 <= dmin <= dmax <= 1");
    int rc = begin_features(n, batch);
    if (rc) return rc;
    // physical column -> neuron (inverse of layer 0's input labelling)
    const std::vector<int32_t>& pos = n->layers[0].in_pos;
    std::vector<int32_t> inv((size_t)n->N);
    for (int i = 0; i < n->N; ++i) inv[(size_t)pos[(size_t)i]] = i;
    DevTmp inv_buf;
    HIPCHK(inv_buf.alloc((size_t)n->N * 4));
    int32_t* d_inv = inv_buf.as<int32_t>();
    HIPCHK(hipMemcpy(d_inv, inv.data(), (size_t)n->N * 4, hipMemcpyHostToDevice));
    const int nblk = (batch + n->RB - 1) / n->RB;
    HIPCHK(launch_synth_features(n->F, d_inv, n->N, batch, nblk, n->rl, seed, dmin, dmax, n->stream));
    HIPCHK(launch_iota_gid(n->d_gid, n->rows_cap, batch, n->stream));
    HIPCHK(hipStreamSynchronize(n->stream));
    n->have_features = true;
    reset_state(n);
    return SPDNN_OK;
}

static int spdnn_synth_features_host_impl(uint64_t seed, int neuron, int64_t row_begin, int64_t nrows, float dmin,
                              float dmax, float* rowmajor) {
    if (!rowmajor || neuron < 1 || nrows < 0) return fail(SPDNN_E_ARG, "bad argument");
    synth_features_host(seed, neuron, row_begin, nrows, dmin, dmax, rowmajor);
    return SPDNN_OK;
}

// ---- inference -----------------------------------------------------------------------------

static int spdnn_default_run_options_impl(spdnn_run_options* o) {
    if (!o) return fail(SPDNN_E_ARG, "opt is NULL");
    memset(o, 0, sizeof(*o));
    o->prune = 1;
    o->first_layer = 0;
    o->n_layers = -1;
    o->compact_threshold = 0.75f;
    o->fuse_layers = 0;
    return SPDNN_OK;
}

static BandLaunch band_args(spdnn_net* n, int l, const Feat& in, const Feat& out, int nblk, int stamp) {
    const LayerPlan& p = n->layers[(size_t)l];
    const DevLayer& d = n->dl[(size_t)l];
    BandLaunch a{};
    a.yin = in; a.yout = out; a.pairs = d.pairs; a.pw = d.wv; a.dst = d.dst; a.active = n->d_active;
    a.steps = p.pair_steps; a.stride = p.pair_stride; a.twins = p.pair_twins ? 1 : 0; a.add_only = n->add_only;
    a.N = n->N; a.K = p.kmax; a.nblk = nblk; a.stamp = stamp; a.rl = n->rl; a.wmode = p.wmode;
    a.halo = p.info.band_halo;
    a.wu = p.info.value; a.bias = n->bias; a.clampv = n->clampv; a.n_cu = n->n_cu;
    a.shape = -1; a.seglen = 0; a.count_prev = nullptr; a.prev_stamp = 0; a.check_dead = 0;
    a.direct_lds = n->band_direct_lds;
    a.stream_min_bytes = n->stream_min_bytes;
    return a;
}

static const spdnn_net::Tuned* find_tuned(const spdnn_net* n, int nblk, int K) {
    for (const auto& t : n->tuned)
        if (t.K == K && nblk * 8 >= t.nblk * 7 && nblk * 8 <= t.nblk * 9) return &t;
    return nullptr;
}

static bool same_bucket(int nblk, int ref) { return nblk * 8 >= ref * 7 && nblk * 8 <= ref * 9; }

// Run-time kernel selection for band layers (the measured half of the inspector's choice), at no
// extra launches: until a configuration is known for this row-block count, the real layers are
// launched with the candidate tile shapes and segment lengths in turn (every candidate gives the
// same result), each launch bracketed by two events; the times are read back a few launches later
// and after two samples of every candidate the fastest becomes the record for this row-block count.
static spdnn_net::Explore* explore_for(spdnn_net* n, int nblk, int K, int layers_left) {
    for (auto& e : n->exploring)
        if (e.K == K && same_bucket(nblk, e.nblk)) return &e;
    spdnn_net::Explore e{nblk, K, 0, {}};
    std::vector<std::pair<double, spdnn_net::Cand>> scored;
    for (int shape = 0; shape < band_shape_count(n->rl, n->band_direct_lds); ++shape) {
        int lens[20];
        const int nc = band_seglen_candidates(n->N, K, nblk, n->rl, shape, n->n_cu, lens, 20);
        for (int c = 0; c < nc; ++c)
            scored.push_back({band_seglen_score(n->N, K, nblk, n->rl, shape, n->n_cu, lens[c]),
                              spdnn_net::Cand{shape, lens[c], 0.0f, 0}});
    }
    // most promising first, so that a run too short
    // to finish the exploration still spends its layers on good candidates
    std::stable_sort(scored.begin(), scored.end(), [](const auto& a, const auto& b) { return a.first > b.first; });
    for (const auto& sc : scored) e.cands.push_back(sc.second);
    // a new exploration needs at least one full round of candidates ahead of it
    if (e.cands.empty() || layers_left < (int)e.cands.size()) return nullptr;
    n->exploring.push_back(std::move(e));
    return &n->exploring.back();
}

static const int kTrialSamples = 2;

// Reads back finished trials, all of them or all but the newest `keep`.
static int resolve_trials(spdnn_net* n, size_t keep) {
    while (n->trials.size() > keep) {
        const spdnn_net::Trial t = n->trials.front();
        n->trials.pop_front();
        float ms = 0.0f;
        hipError_t err = hipEventSynchronize(t.e1);
        if (err == hipSuccess) err = hipEventElapsedTime(&ms, t.e0, t.e1);
        n->ev_free.push_back(t.e0);
        n->ev_free.push_back(t.e1);
        if (err != hipSuccess) return fail(SPDNN_E_DEVICE, std::string("band tuning: ") + hipGetErrorString(err));
        for (size_t i = 0; i < n->exploring.size(); ++i) {
            spdnn_net::Explore& e = n->exploring[i];
            if (e.K != t.K || e.nblk != t.nblk) continue;
            spdnn_net::Cand& c = e.cands[(size_t)t.cand];
            if (c.samples == 0 || ms < c.best_ms) c.best_ms = ms;
            c.samples++;
            bool done = true;
            for (const auto& q : e.cands) done &= q.samples >= kTrialSamples;
            if (done) {
                const spdnn_net::Cand* best = &e.cands[0];
                for (const auto& q : e.cands) if (q.best_ms < best->best_ms) best = &q;
                n->tuned.push_back({e.nblk, e.K, best->shape, best->seglen});
                n->exploring.erase(n->exploring.begin() + (long)i);
            }
            break;
        }
    }
    return SPDNN_OK;
}

// A run-chain BAND layer also has a BLOCK form.  The band walk reads every input column once from
// HBM and wins on large batches; the BLOCK kernel reads every column twice, needs no staging and no
// barriers, and wins while the batch's buffers stay in the on-chip caches (measured cross-over:
// rows x neurons = 2^26, i.e. 256 MiB per buffer - N=4096: 64 row blocks of 256, N=16384: 16).
static bool use_block_form(const spdnn_net* n, const LayerPlan& p, int nblk) {
    return p.kernel == SPDNN_KERNEL_BAND && p.alt_ngroups > 0 &&
           (int64_t)nblk * (int64_t)n->RB * (int64_t)n->N < n->block_form_max_elems;
}

// A TILED layer also carries its GATHER form.  A tile's workgroup takes 64 rows x 1024 outputs with all of a CU's
// LDS, so a launch has rows / 64 x tiles workgroups, each of them tens of microseconds long; where that does not fill
// the chip the gather kernel (8 outputs per wave, no LDS) is the faster one.  Measured cross-over on layers of 1..24
// random inputs per output, per layer: N=1024 4096 rows 46 against 31 us, 16384 rows 55 against 77; N=2048 67 against
// 46 and 162 against 190; N=4096 98 against 79 and 465 against 431 (60000 rows: 1641 against 1900); N <= 512: the
// tiles are never slower.  So: the gather form below 8192 rows on layers of 1024 neurons and more.
// That was measured against the tiles.  The ROWTILE form (whole outputs per thread, up to 8192 neurons) is the faster of
// the two at every size - per layer against the gather form: N=1024 11.5 against 17.5 us at 2048 rows and 71 against 183 at
// 32768, N=2048 19.0 against 19.2 and 176 against 420, N=4096 25.6 against 29.1 and 396 against 923 - so where a layer has
// it the gather form is used only if SPDNN_TILED_MIN_ROWS asks for it.
static bool use_gather_form(const spdnn_net* n, const LayerPlan& p, int nblk) {
    if (p.kernel != SPDNN_KERNEL_TILED || p.alt_kmax <= 0 || n->N < 1024) return false;
    const int rt_rows = rowtile_rows_per_workgroup(n->N);
    const bool has_rowtile = n->rowtile_mode && !p.rt_ent.empty() && rt_rows > 0 && n->RB % rt_rows == 0;
    if (has_rowtile && !n->tiled_min_rows_given) return false;
    return (int64_t)nblk * (int64_t)n->RB < n->tiled_min_rows;
}

static hipError_t launch_layer(spdnn_net* n, int l, const Feat& in, const Feat& out, int nblk, int stamp,
                               int prev_stamp, int check_dead, int32_t* count_prev, int shape, int seglen,
                               const Publish& pub, const int32_t* frontier = nullptr, int frontier_layer = 0) {
    const LayerPlan& p = n->layers[(size_t)l];
    const DevLayer& d = n->dl[(size_t)l];
    if (use_block_form(n, p, nblk)) {
        BlockLaunch b{};
        b.yin = in; b.yout = out; b.cols = d.alt_cols; b.cnt = d.alt_cnt; b.wv = nullptr; b.dst = d.alt_dst;
        b.active = n->d_active; b.count_prev = count_prev; b.check_dead = check_dead; b.N = n->N; b.ngroups = p.alt_ngroups; b.nblk = nblk;
        b.stamp = stamp; b.prev_stamp = prev_stamp; b.rl = n->rl; b.wmode = 0; b.full = p.alt_full ? 1 : 0;
        b.wu = p.info.value; b.bias = n->bias; b.clampv = n->clampv;
        b.publish = pub; b.frontier = frontier; b.frontier_layer = frontier_layer;
        return launch_block(b, n->stream);
    }
    if (p.kernel == SPDNN_KERNEL_BAND) {
        BandLaunch a = band_args(n, l, in, out, nblk, stamp);
        a.count_prev = count_prev;
        a.prev_stamp = prev_stamp;
        a.check_dead = check_dead;
        a.shape = shape;
        a.seglen = seglen > 0 ? seglen : n->band_seglen;
        a.publish = pub; a.frontier = frontier; a.frontier_layer = frontier_layer;
        return launch_band(a, n->stream);
    }
    if (p.kernel == SPDNN_KERNEL_BLOCK) {
        BlockLaunch b{};
        b.yin = in; b.yout = out; b.cols = d.blk_cols; b.cnt = d.blk_cnt; b.wv = d.wv; b.dst = d.dst;
        b.active = n->d_active; b.count_prev = count_prev; b.check_dead = check_dead; b.N = n->N; b.ngroups = p.ngroups; b.nblk = nblk;
        b.stamp = stamp; b.prev_stamp = prev_stamp; b.rl = n->rl; b.wmode = p.wmode; b.full = p.blk_full ? 1 : 0;
        b.wu = p.info.value; b.bias = n->bias; b.clampv = n->clampv;
        b.publish = pub; b.frontier = frontier; b.frontier_layer = frontier_layer;
        return launch_block(b, n->stream);
    }
    if (use_gather_form(n, p, nblk)) {
        GatherLaunch g{};
        g.yin = in; g.yout = out; g.cols = d.alt_cols; g.rowlen = d.alt_cnt; g.wv = d.alt_wv; g.dst = d.alt_dst;
        g.active = n->d_active; g.count_prev = count_prev; g.check_dead = check_dead; g.prev_stamp = prev_stamp; g.N = n->N; g.kmax = p.alt_kmax;
        g.nblk = nblk; g.stamp = stamp; g.rl = n->rl; g.wmode = p.wmode; g.bias = n->bias; g.clampv = n->clampv; g.publish = pub;
        return launch_gather(g, n->stream);
    }
    if (p.kernel == SPDNN_KERNEL_TILED && n->rowtile_mode && !p.rt_ent.empty() && rowtile_rows_per_workgroup(n->N) > 0 &&
        n->RB % rowtile_rows_per_workgroup(n->N) == 0) {
        RowtileLaunch t{};
        t.yin = in; t.yout = out; t.ent = d.rt_ent; t.len = d.alt_cnt; t.dst = d.alt_dst; t.active = n->d_active;
        t.count_prev = count_prev; t.check_dead = check_dead; t.prev_stamp = prev_stamp; t.N = n->N; t.kpad = (p.alt_kmax + 3) / 4 * 4;
        t.rows = nblk * n->RB; t.rl = n->rl; t.wmode = p.wmode; t.stamp = stamp; t.bias = n->bias; t.clampv = n->clampv; t.publish = pub;
        return launch_rowtile(t, n->stream);
    }
    if (p.kernel == SPDNN_KERNEL_TILED) {
        TiledLaunch t{};
        t.yin = in; t.yout = out; t.cols = d.ell; t.hdr = d.rowlen; t.ent = reinterpret_cast<const uint32_t*>(d.wv); t.dst = d.dst;
        t.active = n->d_active; t.count_prev = count_prev; t.check_dead = check_dead; t.prev_stamp = prev_stamp;
        t.N = n->N; t.ntiles = p.ntiles; t.nblk = nblk; t.rl = n->rl; t.wmode = p.wmode; t.stamp = stamp;
        t.bias = n->bias; t.clampv = n->clampv; t.publish = pub;
        return launch_tiled(t, n->stream);
    }
    GatherLaunch g{};
    g.yin = in; g.yout = out; g.cols = d.ell; g.rowlen = d.rowlen; g.wv = d.wv; g.dst = d.dst;
    g.active = n->d_active; g.count_prev = count_prev; g.check_dead = check_dead; g.prev_stamp = prev_stamp; g.N = n->N; g.kmax = p.kmax; g.nblk = nblk; g.stamp = stamp; g.rl = n->rl;
    g.wmode = p.wmode; g.bias = n->bias; g.clampv = n->clampv;
    g.publish = pub;
    return launch_gather(g, n->stream);
}

// Waits until the counts of layers [l0, l0+c) have arrived in pinned host memory (written there
// by the first workgroup of the launch after theirs; -1 = not yet).  Normally they are there or
// arrive within microseconds.  The stream itself is asked only after 100 ms without them, so that
// a failed launch ends the wait: asking puts a marker into the queue, which between two short
// layers costs as much as a layer.  The wait is bounded: after count_timeout_ms without the counts
// of one layer (a kernel that never finishes) the call gives up with SPDNN_E_DEVICE.
static int wait_counts(spdnn_net* n, int l0, int c) {
    volatile int32_t* h = n->h_counts;
    for (int j = l0; j < l0 + c; ++j) {
        if (h[j] >= 0) continue;
        auto t0 = std::chrono::steady_clock::now();
        auto t_start = t0;
        for (unsigned spins = 1; h[j] < 0; ++spins) {
            if ((spins & 255) != 0) continue;
            auto now = std::chrono::steady_clock::now();
            if (now - t_start < std::chrono::microseconds(300)) continue;  // short layers: poll as fast as possible
            // behind a long layer nothing is lost by sleeping between looks: the device has its next launch queued
            std::this_thread::sleep_for(std::chrono::microseconds(50));
            now = std::chrono::steady_clock::now();
            if (now - t0 < std::chrono::milliseconds(100)) continue;
            t0 = now;
            if (now - t_start > std::chrono::milliseconds(n->count_timeout_ms))
                return fail(SPDNN_E_DEVICE, "timed out waiting for the active-row count of layer " + std::to_string(j) +
                                                " (the device did not finish the launch)");
            const hipError_t q = hipStreamQuery(n->stream);
            if (q == hipSuccess) {
                if (h[j] < 0) return fail(SPDNN_E_DEVICE, "layer counts were not handed over");
            } else if (q != hipErrorNotReady) {
                return fail(SPDNN_E_DEVICE, std::string("hipStreamQuery: ") + hipGetErrorString(q));
            }
        }
    }
    return SPDNN_OK;
}

// What layer l runs as in a launch on nblk row blocks, for grouping consecutive layers into one
// persistent launch: layers of one signature share a kernel instantiation and a unit shape.
struct LayerSig {
    int form = -1;   // -1: no persistent form; 0: band walk; 1: BLOCK kernel
    int wmode = 0, unrolled = 0, twins = 0, K = 0, full = 0, ngroups = 0;
    bool operator==(const LayerSig& o) const {
        return form == o.form && wmode == o.wmode && unrolled == o.unrolled && twins == o.twins && K == o.K && full == o.full &&
               ngroups == o.ngroups;
    }
};
static LayerSig layer_sig(const spdnn_net* n, int l, int nblk) {
    const LayerPlan& p = n->layers[(size_t)l];
    LayerSig g;
    if (use_block_form(n, p, nblk)) {
        g.form = 1; g.wmode = 0; g.full = p.alt_full ? 1 : 0; g.ngroups = p.alt_ngroups;
    } else if (p.kernel == SPDNN_KERNEL_BAND) {
        g.form = 0; g.wmode = p.wmode; g.K = p.kmax; g.twins = p.pair_twins ? 1 : 0;
        g.unrolled = band_unrolled(p.kmax, p.pair_steps, p.pair_stride) ? 1 : 0;
    } else if (p.kernel == SPDNN_KERNEL_BLOCK) {
        g.form = 1; g.wmode = p.wmode; g.full = p.blk_full ? 1 : 0; g.ngroups = p.ngroups;
    }
    return g;
}

// Whether layer l can be part of a resident launch (rows kept in LDS through the layers), and in which form: its
// BLOCK form with one exact weight - a BLOCK layer of weight mode 0, or a run-chain BAND layer that carries its
// BLOCK form - or the ROWTILE form of a TILED layer; and a shape the kernel's LDS buffers and numbering hold.
struct ResidentSig {
    int ok = 0;      // 0 no resident form; 1 BLOCK form of one exact weight; 2 ROWTILE form (TILED layers); 3 QUAD form (BAND layers)
    int full = 0, ngroups = 0, wmode = 0;
    int rows = 0;    // rows a workgroup keeps
    bool operator==(const ResidentSig& o) const { return ok == o.ok && full == o.full && ngroups == o.ngroups && wmode == o.wmode; }
};
static ResidentSig resident_sig(const spdnn_net* n, int l) {
    const LayerPlan& p = n->layers[(size_t)l];
    ResidentSig g;
    if (p.kernel == SPDNN_KERNEL_BAND && p.alt_ngroups > 0) { g.ok = 1; g.full = p.alt_full ? 1 : 0; g.ngroups = p.alt_ngroups; }
    else if (p.kernel == SPDNN_KERNEL_BLOCK && p.wmode == 0) { g.ok = 1; g.full = p.blk_full ? 1 : 0; g.ngroups = p.ngroups; }
    else if (p.kernel == SPDNN_KERNEL_TILED && !p.rt_ent.empty() && n->rowtile_mode) { g.ok = 2; g.wmode = p.wmode; }
    else if (p.kernel == SPDNN_KERNEL_BAND && p.quad_groups > 0 && n->band_resident_mode) { g.ok = 3; g.ngroups = p.quad_groups; g.wmode = p.wmode == 2 ? 2 : 1; }
    if (g.ok) {
        g.rows = g.ok == 1 ? resident_rows_per_workgroup(n->N, g.ngroups) : g.ok == 2 ? rowtile_resident_rows(n->N) : band_resident_rows(n->N);
        if (g.rows == 0 || n->RB % g.rows != 0) g.ok = 0;
    }
    return g;
}

// The band resident kernel finds the QUAD form of its j-th layer j strides behind that of its first: whether layer k's
// arrays lie where that rule, set by layers l0 and l0 + 1, puts them.
static bool quad_plans_equidistant(const spdnn_net* n, int l0, int k) {
    const DevLayer& a = n->dl[(size_t)l0];
    const DevLayer& b = n->dl[(size_t)l0 + 1];
    const DevLayer& c = n->dl[(size_t)k];
    const long long stride = (const char*)b.quad_col - (const char*)a.quad_col;
    const long long j = k - l0;
    return (stride % 16) == 0 && (const char*)b.quad_w - (const char*)a.quad_w == stride && (const char*)b.dst - (const char*)a.dst == stride &&
           (const char*)c.quad_col - (const char*)a.quad_col == j * stride && (const char*)c.quad_w - (const char*)a.quad_w == j * stride &&
           (const char*)c.dst - (const char*)a.dst == j * stride;
}

static int spdnn_run_impl(spdnn_net* n, const spdnn_run_options* opt_in, spdnn_run_result* res) {
    if (!n) return fail(SPDNN_E_ARG, "net is NULL");
    spdnn_run_options opt;
    if (opt_in) opt = *opt_in; else spdnn_default_run_options(&opt);
    if (!n->inspected || !n->uploaded) return fail(SPDNN_E_STATE, "inspect the network and set features first");
    if (!n->have_features) return fail(SPDNN_E_STATE, "no features set");
    if (opt.first_layer < 0 || opt.first_layer >= n->L) return fail(SPDNN_E_ARG, "first_layer out of range");
    const int nl = opt.n_layers < 0 ? n->L - opt.first_layer : opt.n_layers;
    if (nl < 1 || opt.first_layer + nl > n->L) return fail(SPDNN_E_ARG, "layer range out of bounds");
    if (opt.prune && n->bias > 0.0f)
        return fail(SPDNN_E_UNSUPPORTED, "pruning needs bias <= 0 (an all-zero row must stay zero)");
    if (opt.fuse_layers < 0) return fail(SPDNN_E_ARG, "fuse_layers negative");
    if (opt.first_layer == 0) reset_state(n);
    else if (opt.first_layer != n->cur_layer) return fail(SPDNN_E_STATE, "first_layer does not continue the current state");
    float thr = opt.compact_threshold > 0.0f ? opt.compact_threshold : 0.75f;
    if (thr > 1.0f) thr = 1.0f;

    if (opt.time_layers) {
        while (n->ev_layer.size() < (size_t)(2 * n->L)) {
            hipEvent_t e;
            HIPCHK(hipEventCreate(&e));
            n->ev_layer.push_back(e);
        }
    }
    const int first = opt.first_layer, last = first + nl - 1;
    for (int l = first; l <= last; ++l) { n->counts[(size_t)l] = -1; n->layer_ms[(size_t)l] = 0.0f; }

    // With bias <= 0 padding rows stay zero, so the layer kernels can count the rows they stamp
    // (one atomic per wave) and no scan is needed for the per-layer counts.  Otherwise the scan,
    // which masks padding rows, counts - only when counts are asked for.
    const bool fused_count = n->bias <= 0.0f;
    const bool scan_count = !fused_count && opt.collect_counts;
    const bool have_counts = fused_count || scan_count;
    if (fused_count) HIPCHK(hipMemsetAsync(n->d_counts + first, 0, (size_t)nl * 4, n->stream));
    // Launches that hold more than one layer need all their plans resident and count on the device:
    // fused pairs (by default and with fused launches asked for, not with fuse_layers = 1) and persistent
    // launches (asked for with fuse_layers >= 2 layers per launch, else by default where a layer moves
    // little enough for the launch boundary to matter).
    const bool no_fusion = scan_count || plans_streamed(n) || opt.fuse_layers == 1;
    const bool pair_mode = n->fuse_pairs && !no_fusion;
    const bool persist_asked = opt.fuse_layers >= 2;
    bool persist_on = !no_fusion && (persist_asked || n->persist_mode == 1);
    const int persist_cmax = persist_asked ? opt.fuse_layers : n->persist_layers;
    const long long persist_wait_us = opt.persist_wait_us < 0 ? 0 : (opt.persist_wait_us > 0 ? opt.persist_wait_us : n->persist_wait_us);
    if (persist_on) {
        HIPCHK(hipMemsetAsync(n->d_done + (size_t)first * n->done_stride, 0, (size_t)nl * n->done_stride * 4, n->stream));
        HIPCHK(hipMemsetAsync(n->d_ctl, 0, (size_t)nl * sizeof(PersistCtl), n->stream));
    }
    if (plans_streamed(n))
        for (int l = first; l <= last && l < first + n->plan_window; ++l) HIPCHK(plan_fetch(n, l));

    // Pruning never waits for the launch it just made: the host looks at the counts of the launch
    // `lookahead` launches back (already finished in steady state).  Counts only go down
    // (bias <= 0), so an older count is a safe upper bound for sizing a repack, and a zero count
    // means every later layer is all zero.
    // The counts reach the host without a copy command between the layers: the first workgroup of
    // every layer launch stores the previous launch's counts into pinned host memory.
    // How far behind depends on how long a layer runs: behind a long layer one launch in the
    // queue keeps the device busy and a compaction should not come late; behind short layers the
    // host needs a lead of a few launches or the device waits for it (measured: leads of 2 to 32
    // launches give the same time per layer; every launch of lead is one more launch made in vain
    // once all rows have died).
    auto lookahead_for = [&](int carried_rows) -> size_t {
        const double us = (double)carried_rows * (double)n->N * 8.0 / 4.0e6 + 6.0;  // at 4 TB/s, plus launch
        return us > 200.0 ? 1 : 3;
    };
    const bool polled = have_counts && opt.prune;
    if (polled) {
        volatile int32_t* h = n->h_counts;
        for (int l = first; l <= last; ++l) h[l] = -1;
    }
    struct Rec { int l0, c, pl; };   // counts of layers [l0, l0+c) on their way to the host; pl: the persistent launch they come from (ordinal), or -1
    struct Timed { int l0, c; };
    std::vector<Rec> recs;
    std::vector<Timed> timed;

    // Everything the layer loop changes, so that it can go back to where a persistent launch started.
    struct State {
        Feat cur; int cur_layer, carried, stamp, last_stamp; bool blocks_skipped;
        int l; bool dead, count_pending; int last_launched; int64_t newest_count; int c_prune;
        Publish pub; size_t nrecs, processed, ntimed; spdnn_run_result r;
    };
    State st{};
    st.l = first; st.dead = n->carried == 0; st.count_pending = false; st.last_launched = -1; st.newest_count = -1;
    st.c_prune = 1; st.pub = Publish{}; st.processed = 0; st.r = spdnn_run_result{};
    auto save = [&]() {
        State s = st;
        s.cur = n->cur; s.cur_layer = n->cur_layer; s.carried = n->carried; s.stamp = n->stamp; s.last_stamp = n->last_stamp;
        s.blocks_skipped = n->blocks_skipped; s.nrecs = recs.size(); s.ntimed = timed.size();
        return s;
    };
    auto restore = [&](const State& s) {
        st = s;
        n->cur = s.cur; n->cur_layer = s.cur_layer; n->carried = s.carried; n->stamp = s.stamp; n->last_stamp = s.last_stamp;
        n->blocks_skipped = s.blocks_skipped;
        recs.resize(s.nrecs);
        timed.resize(s.ntimed);
    };
    // persistent launches whose completion the host has not seen yet, oldest first
    struct PLaunch { State at; int l0, c, nblk, nseg, units, slot; };
    std::deque<PLaunch> pending;
    int next_slot = 0;          // control words of the run's persistent launches, in order
    // a persistent launch that gave up is finished by per-layer launches: layers [fb_l0, fb_l0 + fb_c), each row
    // block from the layer it had reached (d_frontier)
    int fb_l0 = -1, fb_c = 0;
    const int64_t alive_at_start = n->alive;

    // Looks at the completion words of the pending persistent launches, oldest first, up to and including ordinal
    // `upto`.  wait: until each word is there (bounded; the stream is asked after 100 ms as in wait_counts).
    // *failed = index in `pending` of the first launch that did not complete (gave up, or the stream went idle
    // without its word), -1 if none.
    auto settle = [&](bool wait, int upto, int* failed) -> int {
        *failed = -1;
        volatile int32_t* h = n->h_pwords;
        while (!pending.empty() && pending.front().slot <= upto) {
            const PLaunch& pl = pending.front();
            auto t_start = std::chrono::steady_clock::now(), t0 = t_start;
            for (unsigned spins = 1; h[pl.slot] == -1; ++spins) {
                if (!wait) return SPDNN_OK;
                if ((spins & 255) != 0) continue;
                auto now = std::chrono::steady_clock::now();
                if (now - t_start < std::chrono::microseconds(300)) continue;
                std::this_thread::sleep_for(std::chrono::microseconds(50));
                now = std::chrono::steady_clock::now();
                if (now - t0 < std::chrono::milliseconds(100)) continue;
                t0 = now;
                if (now - t_start > std::chrono::milliseconds(n->count_timeout_ms))
                    return fail(SPDNN_E_DEVICE, "timed out waiting for the persistent launch of layers " + std::to_string(pl.l0) +
                                                    ".." + std::to_string(pl.l0 + pl.c - 1) + " (the device did not finish it)");
                const hipError_t q = hipStreamQuery(n->stream);
                if (q == hipSuccess) break;   // everything queued has run: the word is final
                if (q != hipErrorNotReady) return fail(SPDNN_E_DEVICE, std::string("hipStreamQuery: ") + hipGetErrorString(q));
            }
            if (n->run_verbose)
                fprintf(stderr, "spdnn: persistent launch %d (layers %d..%d): word %d of %d units\n", pl.slot, pl.l0,
                        pl.l0 + pl.c - 1, (int)h[pl.slot], pl.units);
            if (h[pl.slot] != pl.units) { *failed = 0; return SPDNN_OK; }
            pending.pop_front();
        }
        return SPDNN_OK;
    };
    // Goes back to the start of pending[idx], which did not complete: waits for the device, reads how far every row
    // block got, and has the layer loop run that launch's layers again as per-layer launches; persistent launches
    // are off for the rest of the run.
    auto fall_back = [&](int idx) -> int {
        const PLaunch pl = pending[(size_t)idx];
        HIPCHK(hipStreamSynchronize(n->stream));
        std::vector<int32_t> done((size_t)pl.c * (size_t)n->done_stride);
        HIPCHK(hipMemcpy(done.data(), n->d_done + (size_t)pl.l0 * n->done_stride, done.size() * 4, hipMemcpyDeviceToHost));
        std::vector<int32_t> frontier((size_t)n->done_stride, 0);
        for (int rb = 0; rb < pl.nblk; ++rb) {
            int j = 0;
            while (j < pl.c && done[(size_t)j * n->done_stride + rb] >= pl.nseg) ++j;
            frontier[(size_t)rb] = j;
        }
        HIPCHK(hipMemcpy(n->d_frontier, frontier.data(), frontier.size() * 4, hipMemcpyHostToDevice));
        HIPCHK(hipMemset(n->d_abort, 0, 4));
        if (n->run_verbose) {
            fprintf(stderr, "spdnn: persistent launch %d (layers %d..%d) did not complete; layers done per row block:", pl.slot,
                    pl.l0, pl.l0 + pl.c - 1);
            for (int rb = 0; rb < pl.nblk; ++rb) fprintf(stderr, " %d", frontier[(size_t)rb]);
            fprintf(stderr, "\n");
        }
        const int lo = pl.at.count_pending ? std::max(first, pl.l0 - 1) : pl.l0;   // counts from here on are taken again
        if (fused_count) HIPCHK(hipMemset(n->d_counts + lo, 0, (size_t)(last - lo + 1) * 4));
        if (polled) {
            volatile int32_t* h = n->h_counts;
            for (int l = lo; l <= last; ++l) h[l] = -1;
        }
        const int fallbacks = st.r.persistent_fallbacks + 1;
        restore(pl.at);
        st.r.persistent_fallbacks = fallbacks;
        pending.clear();
        fb_l0 = pl.l0;
        fb_c = pl.c;
        persist_on = false;
        return SPDNN_OK;
    };

    HIPCHK(hipEventRecord(n->ev_start, n->stream));
    for (;;) {   // once; again from its start after a persistent launch that did not complete
        int failed = -1;
        while (st.l <= last && failed < 0) {
            const int l = st.l;
            const LayerPlan& p = n->layers[(size_t)l];
            if (st.dead) {  // every row died earlier: the remaining outputs are all zero
                st.r.edges += (double)n->batch * (double)p.info.nnz;
                n->cur_layer = ++st.l;
                continue;
            }
            const int nblk = n->carried / n->RB;
            const bool fb = l == fb_l0;   // the layers of a launch that gave up, now one by one
            // a fused pair (intermediate tile in LDS) where the inspector found one; not while the band
            // walk's BLOCK form would run the layers (small batches of run-chain layers)
            // (the size threshold belongs to the default; a caller that asks for fused launches gets them)
            auto is_pair = [&](int k) {
                const LayerPlan& pk = n->layers[(size_t)k];
                return pair_mode && pk.fuse_next && k + 1 <= last && !use_block_form(n, pk, nblk) &&
                       (opt.fuse_layers >= 2 || (int64_t)nblk * (int64_t)n->RB * (int64_t)n->N >= n->pair_min_elems);
            };
            // a resident launch (rows kept in LDS through the layers) where consecutive layers have the structure for it:
            // no launch, fused or not, that goes through memory between the layers comes near it
            int c = 1;
            bool resident = false, persist = false;
            ResidentSig rsig;
            int cmax = std::min(persist_cmax, last - l + 1);
            if (opt.prune && !persist_asked) cmax = std::min(cmax, st.c_prune);   // short launches while the counts still move
            // (with at most 16 rows known alive - the rows of one workgroup of a resident launch - the run is about to end:
            // layer by layer, so that the host sees the end when it comes instead of queueing launches of many layers)
            if (opt.prune && !persist_asked && st.newest_count >= 0 && st.newest_count <= 16) cmax = 1;
            if (!fb && persist_on && n->resident_mode && n->d_table && (rsig = resident_sig(n, l)).ok) {
                // Bringing the rows in and out costs such a launch as much as two layers save it with 16 rows per workgroup
                // (64-byte pieces of a column) and as much as eight save it with 4 rows (16-byte pieces): measured
                // at 2048 and at 60000 rows.  So left to the library: from 2 layers (even while the counts still move -
                // workgroups whose rows have all died leave early) and from 8; a caller that asks for launches of a
                // given length gets them.
                const bool wide_rows = rsig.rows >= 16 && rsig.ok != 3;
                // (band quads: a layer inside the launch takes 0.88 of its time alone at 60000 rows, 0.76 at 6000, and rows in
                // and out cost the launch what 1.5 layers take at either size: worth it from 16 and from 6 layers)
                const int band_rmin = n->band_resident_min_layers >= 2 ? n->band_resident_min_layers : (n->carried >= 16384 ? 16 : 6);
                const int rmin = (persist_asked || wide_rows) ? 2 : rsig.ok == 3 ? band_rmin : 8;
                const int rmax = std::min(wide_rows ? std::max(cmax, 2) : cmax, last - l + 1);
                int k = 1;
                while (k < rmax && resident_sig(n, l + k) == rsig && (rsig.ok != 3 || quad_plans_equidistant(n, l, l + k))) ++k;
                // (entry lists for 8 or 4 rows at a time: on large launches the per-layer kernel, which reads them for 16, is the
                // faster one - measured per layer at batch 60000: N=2048 376 against 337 us, N=4096 1232 against 948; at 2048
                // rows 13 against 38 and 42 against 57)
                const bool too_large = !persist_asked && rsig.ok == 2 && !wide_rows && n->carried >= n->tiled_min_rows;
                if (k >= rmin && !too_large) { c = k; resident = true; }
            }
            const bool pair = !fb && !resident && is_pair(l);
            if (pair) c = 2;
            // a persistent launch: consecutive layers of one kernel form and variant
            LayerSig sig;
            if (fb) {
                c = fb_c;
            } else if (!pair && !resident && persist_on) {
                sig = layer_sig(n, l, nblk);
                const long long layer_bytes = 8ll * (long long)n->carried * (long long)n->N;
                const bool small = layer_bytes >= n->persist_min_bytes && layer_bytes <= n->persist_max_bytes && nblk >= n->persist_min_blocks;
                if (sig.form >= 0 && (persist_asked || small) && cmax >= 2 && next_slot < n->L) {
                    int k = 1;
                    while (k < cmax && !is_pair(l + k) && layer_sig(n, l + k, nblk) == sig) ++k;   // (a fused pair stays a pair)
                    if (k >= 2) { c = k; persist = true; }
                }
            }
            // launches of other kinds must not run on the ruins of a persistent launch: see it complete first
            if (!persist && !pending.empty()) {
                const int rc = settle(true, INT_MAX, &failed);
                if (rc) return rc;
                if (failed >= 0) break;
            }
            for (int j = 0; j < c; ++j) st.r.edges += (double)n->batch * (double)n->layers[(size_t)(l + j)].info.nnz;
            // the layer before this launch, if the row slots still carry its stamps: its rows are
            // counted by this launch (unless a scan has counted them already), and with
            // pruning the row blocks it left without an active row are skipped
            const int prev_stamp = n->last_stamp;
            // (a run without pruning that continues a pruned one keeps skipping: the blocks skipped
            // so far hold stale values, and with bias <= 0 a dead row stays dead, so skipping is exact)
            const int check_dead = (opt.prune || n->blocks_skipped) ? 1 : 0;
            State at_start{};
            if (persist) at_start = save();
            if (check_dead && (prev_stamp != 0 || c > 1)) n->blocks_skipped = true;
            const bool group = persist || fb || resident;   // c layers whose rows are counted behind them, from the stamps
            int32_t* const count_prev = (fused_count && st.count_pending && prev_stamp != 0 && !group) ? n->d_counts + (l - 1) : nullptr;
            const Feat in = n->cur;
            Feat out = (n->cur == n->A) ? n->C : n->A;
            // band tile shape and segment length: the record for this row-block count, else the next
            // candidate of the exploration (timed), else the launcher's own heuristic
            int shape = -1, seglen = 0;
            bool trial = false;
            spdnn_net::Trial tr{};
            if (c == 1 && p.kernel == SPDNN_KERNEL_BAND && !use_block_form(n, p, nblk)) {
                if (const spdnn_net::Tuned* t = find_tuned(n, nblk, p.kmax)) {
                    shape = t->shape;
                    seglen = t->seglen;
                } else if (n->autotune && n->band_seglen == 0) {
                    spdnn_net::Explore* e = explore_for(n, nblk, p.kmax, last - l + 1);
                    if (e && e->issued < kTrialSamples * (int)e->cands.size()) {
                        const int ci = e->issued++ % (int)e->cands.size();
                        shape = e->cands[(size_t)ci].shape;
                        seglen = e->cands[(size_t)ci].seglen;
                        while (n->ev_free.size() < 2) {
                            hipEvent_t ev;
                            HIPCHK(hipEventCreate(&ev));
                            n->ev_free.push_back(ev);
                        }
                        tr = {e->nblk, e->K, ci, n->ev_free[n->ev_free.size() - 1], n->ev_free[n->ev_free.size() - 2]};
                        n->ev_free.resize(n->ev_free.size() - 2);
                        trial = true;
                    }
                }
            }
            const int stamp0 = n->stamp + 1;
            n->stamp += c;
            if (opt.time_layers) HIPCHK(hipEventRecord(n->ev_layer[(size_t)(2 * l)], n->stream));
            if (persist) {
                PersistLaunch pl{};
                pl.table = n->d_table + l; pl.nlayers = c; pl.block_form = sig.form; pl.first_in = in; pl.buf_a = n->A; pl.buf_c = n->C;
                pl.active = n->d_active; pl.done = n->d_done + (size_t)l * n->done_stride; pl.done_stride = n->done_stride;
                pl.ngroups = sig.ngroups; pl.ctl = n->d_ctl + next_slot;
                pl.prev_ctl = pending.empty() ? nullptr : n->d_ctl + pending.back().slot;
                pl.prev_units = pending.empty() ? 0 : pending.back().units;
                pl.abort = n->d_abort; pl.host_word = n->h_pwords + next_slot;
                pl.N = n->N; pl.K = sig.K; pl.nblk = nblk; pl.rl = n->rl; pl.wmode = sig.wmode; pl.stamp0 = stamp0;
                pl.prev_stamp = prev_stamp; pl.check_dead = check_dead; pl.unrolled = sig.unrolled; pl.add_only = n->add_only;
                pl.twins = sig.twins; pl.full = sig.full; pl.seglen = n->persist_seglen; pl.direct_lds = n->band_direct_lds;
                // one queue per XCD where every XCD gets a row block: what the layers of a row block hand to each other
                // then stays in one XCD's L2 and the writer need not write that L2 back (measured at N=1024, batch 6000, per
                // layer: the write-back 12 us of a 17 us layer)
                pl.xcd_queues = n->persist_xcd >= 0 ? (n->persist_xcd ? 1 : 0) : (nblk >= 8 ? 1 : 0);
                pl.light_sync = n->persist_light;
                pl.wait_limit = persist_wait_us * 100;
                pl.n_cu = n->n_cu; pl.stream_min_bytes = n->stream_min_bytes; pl.bias = n->bias; pl.clampv = n->clampv;
                pl.publish = st.pub;
                volatile int32_t* hw = n->h_pwords;
                hw[next_slot] = -1;
                HIPCHK(launch_persist(pl, n->stream));
                PLaunch rec{};
                rec.at = at_start; rec.l0 = l; rec.c = c; rec.nblk = nblk; rec.units = persist_units(pl);
                rec.nseg = rec.units / (nblk * c); rec.slot = next_slot++;
                pending.push_back(rec);
                if (n->run_verbose)
                    fprintf(stderr, "spdnn: persistent launch %d: layers %d..%d, %d row blocks, form %d, %d units/row block, %d units, "
                                    "xcd queues %d, light %d\n", rec.slot, l, l + c - 1, nblk, sig.form, rec.nseg, rec.units,
                            pl.xcd_queues, pl.light_sync);
                for (int j = 1; j < c; ++j) out = (out == n->A) ? n->C : n->A;  // where the last layer wrote
                st.r.persistent_launches += 1;
            } else if (resident) {
                ResidentLaunch rl{};
                rl.table = n->d_table + l; rl.nlayers = c; rl.first_in = in; rl.buf_a = n->A; rl.buf_c = n->C; rl.active = n->d_active;
                rl.N = n->N; rl.ngroups = rsig.ngroups; rl.rows = n->carried; rl.rl = n->rl; rl.full = rsig.full;
                rl.stamp0 = stamp0; rl.prev_stamp = prev_stamp; rl.check_dead = check_dead; rl.bias = n->bias; rl.clampv = n->clampv;
                rl.publish = st.pub;
                if (rsig.ok == 3) {
                    const DevLayer& d0 = n->dl[(size_t)l];
                    rl.quad_col = d0.quad_col; rl.quad_w = d0.quad_w; rl.quad_dst = d0.dst;
                    rl.quad_stride = c > 1 ? (long long)((const char*)n->dl[(size_t)l + 1].quad_col - (const char*)d0.quad_col) : 0;
                }
                HIPCHK(rsig.ok == 1 ? launch_block_resident(rl, n->stream)
                       : rsig.ok == 2 ? launch_rowtile_resident(rl, rsig.wmode, n->stream) : launch_band_resident(rl, rsig.wmode, n->stream));
                if (n->run_verbose)
                    fprintf(stderr, "spdnn: resident launch (%s): layers %d..%d, %d rows, %d rows per workgroup\n",
                            rsig.ok == 1 ? "groups" : rsig.ok == 2 ? "entry lists" : "band quads", l, l + c - 1, n->carried, rsig.rows);
                for (int j = 1; j < c; ++j) out = (out == n->A) ? n->C : n->A;  // where the last layer wrote
                st.r.resident_launches += 1;
            } else if (fb) {
                Feat fin = in, fout = out;
                for (int j = 0; j < c; ++j) {
                    int sh = -1, sl = 0;
                    const LayerPlan& pj = n->layers[(size_t)(l + j)];
                    if (const spdnn_net::Tuned* t = find_tuned(n, nblk, pj.kmax)) { sh = t->shape; sl = t->seglen; }
                    HIPCHK(launch_layer(n, l + j, fin, fout, nblk, stamp0 + j, j == 0 ? prev_stamp : stamp0 + j - 1, check_dead,
                                        nullptr, sh, sl, j == 0 ? st.pub : Publish{}, n->d_frontier, j));
                    out = fout;
                    fin = fout;
                    fout = (fout == n->A) ? n->C : n->A;
                }
                fb_l0 = -1;
            } else if (c == 1) {
                HIPCHK(plan_acquire(n, l));
                if (trial) HIPCHK(hipEventRecord(tr.e0, n->stream));
                HIPCHK(launch_layer(n, l, in, out, nblk, stamp0, prev_stamp, check_dead, count_prev, shape, seglen, st.pub));
                if (trial) {
                    HIPCHK(hipEventRecord(tr.e1, n->stream));
                    n->trials.push_back(tr);
                    int rc = resolve_trials(n, 3);
                    if (rc) return rc;
                }
                HIPCHK(plan_release(n, l));
            } else {
                const LayerPlan& q = n->layers[(size_t)l + 1];
                const DevLayer &da = n->dl[(size_t)l], &db = n->dl[(size_t)l + 1];
                PairLaunch pl{};
                pl.yin = in; pl.yout = out; pl.pairs_a = da.pairs; pl.pw_a = da.wv; pl.pairs_b = db.pairs; pl.pw_b = db.wv;
                pl.dst = db.dst; pl.active = n->d_active; pl.active_mid = n->d_active_mid; pl.count_prev = count_prev;
                pl.N = n->N; pl.nblk = nblk; pl.rl = n->rl; pl.wmode = p.wmode; pl.add_only = n->add_only;
                pl.halo_a = p.info.band_halo; pl.steps_a = p.pair_steps; pl.halo_b = q.info.band_halo; pl.steps_b = q.pair_steps;
                pl.stamp_a = stamp0; pl.stamp_b = stamp0 + 1; pl.prev_stamp = prev_stamp; pl.check_dead = check_dead;
                pl.seglen = n->pair_seglen; pl.n_cu = n->n_cu; pl.stream_min_bytes = n->stream_min_bytes;
                pl.wu_a = p.info.value; pl.wu_b = q.info.value; pl.bias = n->bias; pl.clampv = n->clampv;
                pl.publish = st.pub;
                HIPCHK(launch_band_pair(pl, n->stream));
                // the first layer's rows: nobody looks at active_mid again, so they are counted here
                if (fused_count) HIPCHK(launch_count_stamped(n->d_active_mid, n->carried, stamp0, n->d_counts + l, n->stream));
            }
            if (opt.time_layers) { HIPCHK(hipEventRecord(n->ev_layer[(size_t)(2 * l + 1)], n->stream)); timed.push_back({l, c}); }
            st.r.layers_run += c;
            st.r.launches += (fb ? c : 1);
            if (pair) st.r.fused_pairs += 1;
            st.last_launched = l + c - 1;
            n->last_stamp = stamp0 + c - 1;
            n->cur = out;
            n->cur_layer = l + c;
            if (scan_count) {
                HIPCHK(launch_scan_active(n->d_active, n->d_gid, n->carried, n->last_stamp, n->d_count, n->d_alive_src,
                                          n->d_alive_gid, n->stream));
                HIPCHK(hipMemcpyAsync(n->d_counts + l, n->d_count, 4, hipMemcpyDeviceToDevice, n->stream));
            }
            if (fused_count && group) {
                // The rows the layers of the launch left active, from the stamps behind it: a row that carries the
                // stamp of layer j or of a later one was active after layer j (bias <= 0: a zero row stays zero).
                // The layer before the launch is counted the same way if nobody has counted it yet.  The kernel
                // hands its counts to the host itself.
                const bool with_prev = st.count_pending && prev_stamp != 0 && prev_stamp == stamp0 - 1;
                const int lo = with_prev ? l - 1 : l, cnt = c + (with_prev ? 1 : 0);
                HIPCHK(launch_count_stamp_range(n->d_active, n->carried, with_prev ? prev_stamp : stamp0, cnt, n->d_counts + lo,
                                                polled ? n->h_counts + lo : nullptr, n->d_count_partial, n->stream));
                if (polled) {
                    if (st.pub.n > 0) recs.push_back({(int)(st.pub.src - n->d_counts), st.pub.n, -1});
                    recs.push_back({lo, cnt, persist ? next_slot - 1 : -1});
                }
                st.pub = Publish{};
                st.count_pending = false;
            } else if (fused_count) {
                // Counts that are final once this launch has finished: the previous layer's (counted at
                // this launch's start) and, of a fused pair, its first layer's.  The next launch hands
                // them to the host; this launch handed over the ones before (pub).
                if (polled && st.pub.n > 0) recs.push_back({(int)(st.pub.src - n->d_counts), st.pub.n, -1});
                // (of a pair the first layer is counted behind the launch and the second, like a single
                // layer, by whatever comes next)
                const int lo = count_prev ? l - 1 : l, hi = pair ? l + 1 : l;
                st.pub = Publish{};
                if (polled && hi > lo) { st.pub.src = n->d_counts + lo; st.pub.dst = n->h_counts + lo; st.pub.n = hi - lo; }
                st.count_pending = true;
            }
            st.l = l + c;
            if (!opt.prune) continue;

            // a record is pushed when the launch that hands it over is queued, i.e. one launch late
            // (while the counts are unknown or still moving the host waits for each launch's counts: a launch made on rows
            // that have died since costs more than the round trip)
            const size_t lookahead = st.c_prune <= 1 ? 0 : lookahead_for(n->carried) - 1;
            while (recs.size() - st.processed > lookahead && !st.dead && failed < 0) {
                const Rec rc = recs[st.processed++];
                const int wrc = wait_counts(n, rc.l0, rc.c);
                if (wrc) return wrc;
                if (rc.pl >= 0) {   // counts taken behind a persistent launch mean something only if it completed
                    const int src = settle(true, rc.pl, &failed);
                    if (src) return src;
                    if (failed >= 0) break;
                }
                const int64_t before = st.newest_count;
                int64_t layer_before = before;
                for (int j = rc.l0; j < rc.l0 + rc.c && !st.dead; ++j) {
                    layer_before = st.newest_count;
                    st.newest_count = n->h_counts[j];
                    if (st.newest_count == 0) st.dead = true;
                }
                // layers per multi-layer launch while pruning: all that are allowed once a layer has left the count as it
                // was, doubled while the counts hold still (within 3 % from one record to the next), one layer per
                // launch again when they move
                if (layer_before > 0 && st.newest_count == layer_before) st.c_prune = std::max(2, persist_cmax);
                else if (before > 0 && st.newest_count * 100 >= before * 97) st.c_prune = std::min(persist_cmax, std::max(2, st.c_prune * 2));
                else st.c_prune = 1;
            }
            if (failed >= 0) break;
            if (st.dead) { n->carried = 0; continue; }
            if (st.newest_count > 0 && (double)st.newest_count <= (double)thr * (double)n->carried && st.l < n->L) {
                const int nb = (int)((st.newest_count + n->RB - 1) / n->RB);  // upper bound of what is alive now
                if (nb * n->RB < n->carried) {
                    if (!pending.empty()) {   // the repack overwrites a work buffer: not on the ruins of a persistent launch
                        const int rc = settle(true, INT_MAX, &failed);
                        if (rc) return rc;
                        if (failed >= 0) break;
                    }
                    const Feat dstbuf = (n->cur == n->A) ? n->C : n->A;
                    HIPCHK(launch_scan_active(n->d_active, n->d_gid, n->carried, n->last_stamp, n->d_count,
                                              n->d_alive_src, n->d_alive_gid, n->stream));
                    if (st.count_pending) {  // the scan has just counted the newest layer's rows
                        HIPCHK(hipMemcpyAsync(n->d_counts + (st.l - 1), n->d_count, 4, hipMemcpyDeviceToDevice, n->stream));
                        st.count_pending = false;
                    }
                    HIPCHK(launch_repack(n->cur, dstbuf, n->d_count, n->d_alive_src, n->d_alive_gid, n->d_gid_tmp,
                                         n->N, n->rl, nb, n->stream));
                    std::swap(n->d_gid, n->d_gid_tmp);
                    n->gid_dirty = true;
                    n->cur = dstbuf;
                    n->carried = nb * n->RB;
                    n->last_stamp = 0;  // the row slots moved: the stamps no longer describe them
                    n->blocks_skipped = false;  // every carried block has just been written
                    st.r.compactions++;
                }
            }
        }
        if (failed < 0) {
            // categories of the last layer: survivor list by the scan.  After a final repack the list
            // produced for the repack is that list already.
            n->alive_list_valid = false;
            if (!st.dead && st.last_launched == last) {
                if (n->last_stamp != 0) {
                    HIPCHK(launch_scan_active(n->d_active, n->d_gid, n->carried, n->last_stamp, n->d_count, n->d_alive_src,
                                              n->d_alive_gid, n->stream));
                }
                HIPCHK(hipMemcpyAsync(n->h_count, n->d_count, 4, hipMemcpyDeviceToHost, n->stream));
                if (st.count_pending)  // no launch follows the last layer: the scan's count is its count
                    HIPCHK(hipMemcpyAsync(n->d_counts + last, n->d_count, 4, hipMemcpyDeviceToDevice, n->stream));
                n->alive_list_valid = true;
            }
            HIPCHK(hipEventRecord(n->ev_stop, n->stream));
            if (have_counts && st.last_launched >= first)   // all of them once more (the last launch's have no launch after it)
                HIPCHK(hipMemcpyAsync(n->h_counts + first, n->d_counts + first, (size_t)(st.last_launched - first + 1) * 4,
                                      hipMemcpyDeviceToHost, n->stream));
            HIPCHK(hipStreamSynchronize(n->stream));
            if (plans_streamed(n)) HIPCHK(hipStreamSynchronize(n->copy_stream));
            // everything has run: the completion words are final
            const int rc = settle(false, INT_MAX, &failed);
            if (rc) return rc;
            if (failed < 0 && !pending.empty()) failed = 0;   // a word still missing: that launch never finished its units
            if (failed < 0) break;
        }
        const int rc = fall_back(failed);
        if (rc) return rc;
    }
    {
        int rc = resolve_trials(n, 0);
        if (rc) return rc;
    }
    spdnn_run_result& r = st.r;
    HIPCHK(hipEventElapsedTime(&r.ms_total, n->ev_start, n->ev_stop));
    for (const Timed& t : timed) {
        float ms = 0.0f;
        HIPCHK(hipEventElapsedTime(&ms, n->ev_layer[(size_t)(2 * t.l0)], n->ev_layer[(size_t)(2 * t.l0 + 1)]));
        for (int j = 0; j < t.c; ++j) n->layer_ms[(size_t)(t.l0 + j)] = ms / (float)t.c;
        r.ms_kernels += ms;
    }
    // per-layer counts: everything that was launched has finished now
    const int last_launched = st.last_launched;
    bool zero_seen = false;
    for (int l = first; l <= last; ++l) {
        if (zero_seen) { n->counts[(size_t)l] = 0; continue; }
        if (l <= last_launched && have_counts) n->counts[(size_t)l] = n->h_counts[l];
        else if (l > last_launched) n->counts[(size_t)l] = (last_launched >= first || n->carried == 0) ? 0 : -1;
        if (n->counts[(size_t)l] == 0) zero_seen = true;
    }
    if (st.dead || zero_seen) { if (opt.prune) n->carried = 0; n->alive = 0; }
    else if (n->alive_list_valid) n->alive = n->h_count[0];
    if (n->alive == 0) n->alive_list_valid = true;  // the empty list
    // byte model: rows entering each launched layer
    int64_t entering = alive_at_start;
    for (int l = first; l <= last_launched; ++l) {
        const LayerPlan& p = n->layers[(size_t)l];
        r.alg_bytes += 8.0 * (double)((opt.prune && have_counts) ? entering : n->batch) * (double)n->N +
                       8.0 * (double)p.info.nnz + 4.0 * (double)(n->N + 1);
        if (n->counts[(size_t)l] >= 0) entering = n->counts[(size_t)l];
    }
    r.active_rows = n->alive;
    r.carried_rows = n->carried;
    if (res) *res = r;
    return SPDNN_OK;
}

static int spdnn_get_active_count_impl(const spdnn_net* n, int layer, int64_t* count) {
    if (!n || !count) return fail(SPDNN_E_ARG, "NULL argument");
    if (layer < 0 || layer >= n->L) return fail(SPDNN_E_ARG, "layer out of range");
    if (n->counts[(size_t)layer] < 0) return fail(SPDNN_E_STATE, "no count recorded for this layer");
    *count = n->counts[(size_t)layer];
    return SPDNN_OK;
}

static int spdnn_get_categories_impl(spdnn_net* n, int32_t* ids, int64_t cap, int64_t* cnt) {
    if (!n || !cnt) return fail(SPDNN_E_ARG, "NULL argument");
    if (!n->have_features) return fail(SPDNN_E_STATE, "no features set");
    if (n->cur_layer == 0) {  // nothing run yet: every row counts
        *cnt = n->batch;
        if (ids) {
            if (cap < n->batch) return fail(SPDNN_E_ARG, "ids buffer too small");
            for (int i = 0; i < n->batch; ++i) ids[i] = i;
        }
        return SPDNN_OK;
    }
    *cnt = n->alive;
    if (!ids || n->alive == 0) return SPDNN_OK;
    if (cap < n->alive) return fail(SPDNN_E_ARG, "ids buffer too small");
    if (!n->alive_list_valid) return fail(SPDNN_E_STATE, "no active list available");
    HIPCHK(hipMemcpy(ids, n->d_alive_gid, (size_t)n->alive * 4, hipMemcpyDeviceToHost));
    return SPDNN_OK;
}

static int spdnn_get_activations_impl(spdnn_net* n, const int32_t* rows, int nrows, float* rowmajor) {
    if (!n || !rows || !rowmajor) return fail(SPDNN_E_ARG, "NULL argument");
    if (!n->have_features) return fail(SPDNN_E_STATE, "no features set");
    if (nrows < 0) return fail(SPDNN_E_ARG, "nrows negative");
    if (nrows == 0) return SPDNN_OK;
    // global id -> physical row of the current buffer
    std::vector<int32_t> gid((size_t)std::max(n->carried, 1));
    if (n->carried > 0) HIPCHK(hipMemcpy(gid.data(), n->d_gid, (size_t)n->carried * 4, hipMemcpyDeviceToHost));
    std::vector<int32_t> where((size_t)n->batch, -1);
    for (int r = 0; r < n->carried; ++r)
        if (gid[(size_t)r] >= 0 && gid[(size_t)r] < n->batch) where[(size_t)gid[(size_t)r]] = r;
    std::vector<int32_t> phys((size_t)nrows);
    for (int i = 0; i < nrows; ++i) {
        if (rows[i] < 0 || rows[i] >= n->batch) return fail(SPDNN_E_ARG, "row id out of range");
        phys[(size_t)i] = where[(size_t)rows[i]];
    }
    const int chunk = 4096;
    DevTmp phys_buf, out_buf;
    HIPCHK(phys_buf.alloc((size_t)chunk * 4));
    if (out_buf.alloc((size_t)chunk * (size_t)n->N * 4) != hipSuccess) return fail(SPDNN_E_NOMEM, "out of device memory");
    int32_t* d_phys = phys_buf.as<int32_t>();
    float* d_out = out_buf.as<float>();
    const int32_t* lab = nullptr;
    HIPCHK(labelling_dev(n, n->cur_layer, &lab));
    for (int i0 = 0; i0 < nrows; i0 += chunk) {
        const int m = std::min(chunk, nrows - i0);
        HIPCHK(hipMemcpyAsync(d_phys, phys.data() + i0, (size_t)m * 4, hipMemcpyHostToDevice, n->stream));
        HIPCHK(launch_unpack_rows(n->cur, lab, d_phys, m, n->N, n->rl, n->d_active, n->last_stamp, d_out, n->stream));
        HIPCHK(hipMemcpyAsync(rowmajor + (size_t)i0 * n->N, d_out, (size_t)m * n->N * 4, hipMemcpyDeviceToHost, n->stream));
        HIPCHK(hipStreamSynchronize(n->stream));
    }
    return SPDNN_OK;
}

static int spdnn_get_activations_noalloc_impl(spdnn_net* n, const int32_t* rows, int nrows, float* rowmajor) {
    if (!n || !rows || !rowmajor) return fail(SPDNN_E_ARG, "NULL argument");
    if (!n->have_features) return fail(SPDNN_E_STATE, "no features set");
    if (nrows < 0) return fail(SPDNN_E_ARG, "nrows negative");
    if (nrows == 0) return SPDNN_OK;
    if ((size_t)n->batch > kScratchTableRows)
        return fail(SPDNN_E_UNSUPPORTED, "spdnn_get_activations_noalloc serves batches of at most " +
                                             std::to_string(kScratchTableRows) + " rows (this one has " +
                                             std::to_string(n->batch) + "); use spdnn_get_activations");
    const size_t row_bytes = (size_t)n->N * 4;
    if (row_bytes > kScratchStageBytes)
        return fail(SPDNN_E_UNSUPPORTED, "spdnn_get_activations_noalloc serves rows of at most " +
                                             std::to_string(kScratchStageBytes / 4) + " neurons (this network has " +
                                             std::to_string(n->N) + "); use spdnn_get_activations");
    for (int i = 0; i < nrows; ++i)
        if (rows[i] < 0 || rows[i] >= n->batch) return fail(SPDNN_E_ARG, "row id out of range");
    unsigned char* base = nullptr;
    HIPCHK(scratch_base(&base));
    int32_t* const d_where = reinterpret_cast<int32_t*>(base + kScratchTableOff);
    int32_t* const d_ids = reinterpret_cast<int32_t*>(base + kScratchIdsOff);
    int32_t* const d_phys = reinterpret_cast<int32_t*>(base + kScratchPhysOff);
    float* const d_out = reinterpret_cast<float*>(base + kScratchStageOff);
    // the table keeps the last call's contents: written anew (every entry, then the carried rows)
    HIPCHK(launch_row_table(n->d_gid, n->carried, n->batch, d_where, n->stream));
    const int32_t* lab = nullptr;
    HIPCHK(labelling_dev(n, n->cur_layer, &lab));
    const int chunk = (int)std::min<size_t>(kScratchPassRows, kScratchStageBytes / row_bytes);
    for (int i0 = 0; i0 < nrows; i0 += chunk) {
        const int m = std::min(chunk, nrows - i0);
        HIPCHK(hipMemcpyAsync(d_ids, rows + i0, (size_t)m * 4, hipMemcpyHostToDevice, n->stream));
        HIPCHK(launch_lookup_rows(d_ids, m, d_where, d_phys, n->stream));
        HIPCHK(launch_unpack_rows(n->cur, lab, d_phys, m, n->N, n->rl, n->d_active, n->last_stamp, d_out, n->stream));
        HIPCHK(hipMemcpyAsync(rowmajor + (size_t)i0 * n->N, d_out, (size_t)m * row_bytes, hipMemcpyDeviceToHost, n->stream));
        HIPCHK(hipStreamSynchronize(n->stream));  // the staging rows are reused by the next pass
    }
    return SPDNN_OK;
}

static int spdnn_get_band_tuning_impl(const spdnn_net* n, int index, int* row_blocks, int* shape, int* seglen) {
    if (!n) return fail(SPDNN_E_ARG, "net is NULL");
    if (index < 0 || index >= (int)n->tuned.size()) return fail(SPDNN_E_ARG, "no such tuning record");
    const spdnn_net::Tuned& t = n->tuned[(size_t)index];
    if (row_blocks) *row_blocks = t.nblk;
    if (shape) *shape = t.shape;
    if (seglen) *seglen = t.seglen;
    return SPDNN_OK;
}

static int spdnn_get_layer_times_impl(const spdnn_net* n, float* ms, int cnt) {
    if (!n || !ms) return fail(SPDNN_E_ARG, "NULL argument");
    if (cnt < 0 || cnt > n->L) return fail(SPDNN_E_ARG, "n out of range");
    std::copy(n->layer_ms.begin(), n->layer_ms.begin() + cnt, ms);
    return SPDNN_OK;
}

static int spdnn_write_categories_impl(spdnn_net* n, const char* path) {
    if (!n || !path) return fail(SPDNN_E_ARG, "NULL argument");
    int64_t cnt = 0;
    int rc = spdnn_get_categories(n, nullptr, 0, &cnt);
    if (rc) return rc;
    std::vector<int32_t> ids((size_t)std::max<int64_t>(cnt, 1));
    rc = spdnn_get_categories(n, ids.data(), (int64_t)ids.size(), &cnt);
    if (rc) return rc;
    FILE* f = fopen(path, "w");
    if (!f) return fail(SPDNN_E_IO, std::string("cannot write ") + path);
    for (int64_t i = 0; i < cnt; ++i) fprintf(f, "%d\n", ids[(size_t)i] + 1);
    fclose(f);
    return SPDNN_OK;
}

// ---- device utilities ------------------------------------------------------------------------

static int spdnn_measure_copy_bandwidth_impl(int64_t bytes, int reps, double* gbps) {
    if (!gbps || bytes < 1024 || reps < 1) return fail(SPDNN_E_ARG, "bad argument");
    bytes &= ~(int64_t)1023;
    DevTmp abuf, bbuf;
    EventTmp ev0, ev1;
    if (abuf.alloc((size_t)bytes) != hipSuccess || bbuf.alloc((size_t)bytes) != hipSuccess)
        return fail(SPDNN_E_NOMEM, "out of device memory");
    float *a = abuf.as<float>(), *b = bbuf.as<float>();
    HIPCHK(hipMemset(a, 0, (size_t)bytes));
    HIPCHK(ev0.create());
    HIPCHK(ev1.create());
    HIPCHK(launch_copy_f4(a, b, bytes / 4, nullptr));
    HIPCHK(hipEventRecord(ev0.e, nullptr));
    for (int i = 0; i < reps; ++i) HIPCHK(launch_copy_f4(a, b, bytes / 4, nullptr));
    HIPCHK(hipEventRecord(ev1.e, nullptr));
    HIPCHK(hipEventSynchronize(ev1.e));
    float ms = 0.0f;
    HIPCHK(hipEventElapsedTime(&ms, ev0.e, ev1.e));
    if (ms <= 0.0f) return fail(SPDNN_E_DEVICE, "copy benchmark failed");
    *gbps = 2.0 * (double)bytes * reps / (ms * 1e-3) / 1e9;
    return SPDNN_OK;
}

static int spdnn_measure_buffer_copy_bandwidth_impl(spdnn_net* n, int reps, double* gbps) {
    if (!n || !gbps || reps < 1) return fail(SPDNN_E_ARG, "bad argument");
    if (!n->uploaded || !n->have_features) return fail(SPDNN_E_STATE, "no feature buffers yet: set features first");
    const int nblk = (n->batch + n->RB - 1) / n->RB;
    const int64_t half_floats = (int64_t)((nblk + 1) / 2) * n->N * n->RB;
    EventTmp ev0, ev1;
    HIPCHK(ev0.create());
    HIPCHK(ev1.create());
    // the work buffers hold nothing a caller can still ask for once the state is reset
    reset_state(n);
    HIPCHK(launch_copy_pair(n->A, n->C, half_floats, n->stream));
    HIPCHK(hipEventRecord(ev0.e, n->stream));
    for (int i = 0; i < reps; ++i) HIPCHK(launch_copy_pair(n->A, n->C, half_floats, n->stream));
    HIPCHK(hipEventRecord(ev1.e, n->stream));
    HIPCHK(hipEventSynchronize(ev1.e));
    float ms = 0.0f;
    HIPCHK(hipEventElapsedTime(&ms, ev0.e, ev1.e));
    if (ms <= 0.0f) return fail(SPDNN_E_DEVICE, "copy benchmark failed");
    *gbps = 4.0 * (double)half_floats * 4.0 * reps / (ms * 1e-3) / 1e9;
    return SPDNN_OK;
}

static int spdnn_device_info_impl(char* name, int cap, int* compute_units, int64_t* hbm_bytes) {
    int cnt = 0;
    if (hipGetDeviceCount(&cnt) != hipSuccess || cnt < 1) return fail(SPDNN_E_DEVICE, "no HIP device available");
    hipDeviceProp_t p;
    HIPCHK(hipGetDeviceProperties(&p, 0));
    if (name && cap > 0) snprintf(name, (size_t)cap, "%s (%s)", p.name, p.gcnArchName);
    if (compute_units) *compute_units = p.multiProcessorCount;
    if (hbm_bytes) *hbm_bytes = (int64_t)p.totalGlobalMem;
    return SPDNN_OK;
}

static int spdnn_get_feature_placement_impl(const spdnn_net* n, int* paired, int* candidates, int64_t* search_peak_bytes) {
    if (!n) return fail(SPDNN_E_ARG, "net is NULL");
    if (!n->uploaded) return fail(SPDNN_E_STATE, "no feature buffers yet");
    if (paired) *paired = n->feat_paired;
    if (candidates) *candidates = n->feat_candidates;
    if (search_peak_bytes) *search_peak_bytes = (int64_t)n->search_peak_bytes;
    return SPDNN_OK;
}

static int spdnn_device_alloc_calls_impl(int64_t* calls) {
    if (!calls) return fail(SPDNN_E_ARG, "calls is NULL");
    *calls = g_dev_allocs.load(std::memory_order_relaxed);
    return SPDNN_OK;
}

static int spdnn_device_memory_impl(int64_t* free_bytes, int64_t* total_bytes) {
    size_t f = 0, t = 0;
    HIPCHK(hipMemGetInfo(&f, &t));
    if (free_bytes) *free_bytes = (int64_t)f;
    if (total_bytes) *total_bytes = (int64_t)t;
    return SPDNN_OK;
}

static int spdnn_device_synchronize_impl(void) {
    HIPCHK(hipDeviceSynchronize());
    return SPDNN_OK;
}


// ---- the entry points proper: every one behind the exception barrier ----
int spdnn_create(int neuron, int max_batch, int layers, float bias, float clamp, spdnn_net** out) {
    return guarded([&] { return spdnn_create_impl(neuron, max_batch, layers, bias, clamp, out); });
}
int spdnn_destroy(spdnn_net* n) {
    return guarded([&] { return spdnn_destroy_impl(n); });
}
int spdnn_reference_bias(int neuron, float* bias) {
    return guarded([&] { return spdnn_reference_bias_impl(neuron, bias); });
}
int spdnn_set_force_kernel(spdnn_net* n, int kernel) {
    return guarded([&] { return spdnn_set_force_kernel_impl(n, kernel); });
}
int spdnn_set_layer_csr(spdnn_net* n, int layer, const int32_t* rowptr, const int32_t* col, const float* val) {
    return guarded([&] { return spdnn_set_layer_csr_impl(n, layer, rowptr, col, val); });
}
int spdnn_load_layer_tsv(spdnn_net* n, int layer, const char* path) {
    return guarded([&] { return spdnn_load_layer_tsv_impl(n, layer, path); });
}
int spdnn_load_layers_tsv(spdnn_net* n, const char* data_dir, int first, int count) {
    return guarded([&] { return spdnn_load_layers_tsv_impl(n, data_dir, first, count); });
}
int spdnn_load_layers_bin(spdnn_net* n, const char* path, int first, int count, int64_t nnz_per_layer) {
    return guarded([&] { return spdnn_load_layers_bin_impl(n, path, first, count, nnz_per_layer); });
}
int spdnn_weight_file_name(const char* data_dir, int neuron, int layer, char* out, int cap) {
    return guarded([&] { return spdnn_weight_file_name_impl(data_dir, neuron, layer, out, cap); });
}
int spdnn_synth_layer_csr(uint64_t seed, int layer, int neuron, int nnz_per_row, float value, int32_t* rowptr, int32_t* col, float* val) {
    return guarded([&] { return spdnn_synth_layer_csr_impl(seed, layer, neuron, nnz_per_row, value, rowptr, col, val); });
}
int spdnn_synth_layers(spdnn_net* n, uint64_t seed, int first, int count, int nnz_per_row, float value) {
    return guarded([&] { return spdnn_synth_layers_impl(n, seed, first, count, nnz_per_row, value); });
}
int spdnn_inspect(spdnn_net* n) {
    return guarded([&] { return spdnn_inspect_impl(n); });
}
int spdnn_set_plan_window(spdnn_net* n, int slots) {
    return guarded([&] { return spdnn_set_plan_window_impl(n, slots); });
}
int spdnn_get_plan_memory(const spdnn_net* n, int* window, int64_t* device_bytes, int64_t* pinned_bytes) {
    return guarded([&] { return spdnn_get_plan_memory_impl(n, window, device_bytes, pinned_bytes); });
}
int spdnn_get_layer_plan(const spdnn_net* n, int layer, spdnn_layer_plan* out) {
    return guarded([&] { return spdnn_get_layer_plan_impl(n, layer, out); });
}
int spdnn_get_band_plan(const spdnn_net* n, int layer, int32_t* in_pos, int32_t* out_at, uint8_t* sel) {
    return guarded([&] { return spdnn_get_band_plan_impl(n, layer, in_pos, out_at, sel); });
}
int spdnn_get_band_pairs(const spdnn_net* n, int layer, int* steps, int* stride, int* padded_steps, int* has_weights, uint32_t* records, float* weights) {
    return guarded([&] { return spdnn_get_band_pairs_impl(n, layer, steps, stride, padded_steps, has_weights, records, weights); });
}
int spdnn_get_band_quads(const spdnn_net* n, int layer, int* groups, uint32_t* columns, float* weights) {
    return guarded([&] { return spdnn_get_band_quads_impl(n, layer, groups, columns, weights); });
}
int spdnn_get_layer_dst(const spdnn_net* n, int layer, int32_t* dst) {
    return guarded([&] { return spdnn_get_layer_dst_impl(n, layer, dst); });
}
int spdnn_receptive_field(spdnn_net* n, int first_layer, int n_layers, const int32_t* out_neurons, int n_out, int32_t* in_neurons, int64_t cap, int64_t* count) {
    return guarded([&] { return spdnn_receptive_field_impl(n, first_layer, n_layers, out_neurons, n_out, in_neurons, cap, count); });
}
int spdnn_get_layer_slots(const spdnn_net* n, int layer, int* slots) {
    return guarded([&] { return spdnn_get_layer_slots_impl(n, layer, slots); });
}
int spdnn_get_input_labelling(const spdnn_net* n, int layer, int32_t* phys_col) {
    return guarded([&] { return spdnn_get_input_labelling_impl(n, layer, phys_col); });
}
int spdnn_hash_reorder(int v, int buckets, int domain, int* out) {
    return guarded([&] { return spdnn_hash_reorder_impl(v, buckets, domain, out); });
}
int spdnn_set_features_dense(spdnn_net* n, const float* rowmajor, int batch) {
    return guarded([&] { return spdnn_set_features_dense_impl(n, rowmajor, batch); });
}
int spdnn_load_features_tsv(spdnn_net* n, const char* path, int batch) {
    return guarded([&] { return spdnn_load_features_tsv_impl(n, path, batch); });
}
int spdnn_read_features_tsv(const char* path, int neuron, int batch, float* rowmajor, int64_t* kept) {
    return guarded([&] { return spdnn_read_features_tsv_impl(path, neuron, batch, rowmajor, kept); });
}
int spdnn_load_features_bin(spdnn_net* n, const char* path, int batch) {
    return guarded([&] { return spdnn_load_features_bin_impl(n, path, batch); });
}
int spdnn_synth_features(spdnn_net* n, uint64_t seed, int batch, float dmin, float dmax) {
    return guarded([&] { return spdnn_synth_features_impl(n, seed, batch, dmin, dmax); });
}
int spdnn_synth_features_host(uint64_t seed, int neuron, int64_t row_begin, int64_t nrows, float dmin, float dmax, float* rowmajor) {
    return guarded([&] { return spdnn_synth_features_host_impl(seed, neuron, row_begin, nrows, dmin, dmax, rowmajor); });
}
int spdnn_default_run_options(spdnn_run_options* o) {
    return guarded([&] { return spdnn_default_run_options_impl(o); });
}
int spdnn_run(spdnn_net* n, const spdnn_run_options* opt_in, spdnn_run_result* res) {
    return guarded([&] { return spdnn_run_impl(n, opt_in, res); });
}
int spdnn_get_active_count(const spdnn_net* n, int layer, int64_t* count) {
    return guarded([&] { return spdnn_get_active_count_impl(n, layer, count); });
}
int spdnn_get_categories(spdnn_net* n, int32_t* ids, int64_t cap, int64_t* cnt) {
    return guarded([&] { return spdnn_get_categories_impl(n, ids, cap, cnt); });
}
int spdnn_get_activations(spdnn_net* n, const int32_t* rows, int nrows, float* rowmajor) {
    return guarded([&] { return spdnn_get_activations_impl(n, rows, nrows, rowmajor); });
}
int spdnn_get_activations_noalloc(spdnn_net* n, const int32_t* rows, int nrows, float* rowmajor) {
    return guarded([&] { return spdnn_get_activations_noalloc_impl(n, rows, nrows, rowmajor); });
}
int spdnn_get_band_tuning(const spdnn_net* n, int index, int* row_blocks, int* shape, int* seglen) {
    return guarded([&] { return spdnn_get_band_tuning_impl(n, index, row_blocks, shape, seglen); });
}
int spdnn_get_layer_times(const spdnn_net* n, float* ms, int cnt) {
    return guarded([&] { return spdnn_get_layer_times_impl(n, ms, cnt); });
}
int spdnn_write_categories(spdnn_net* n, const char* path) {
    return guarded([&] { return spdnn_write_categories_impl(n, path); });
}
int spdnn_measure_copy_bandwidth(int64_t bytes, int reps, double* gbps) {
    return guarded([&] { return spdnn_measure_copy_bandwidth_impl(bytes, reps, gbps); });
}
int spdnn_measure_buffer_copy_bandwidth(spdnn_net* n, int reps, double* gbps) {
    return guarded([&] { return spdnn_measure_buffer_copy_bandwidth_impl(n, reps, gbps); });
}
int spdnn_device_info(char* name, int cap, int* compute_units, int64_t* hbm_bytes) {
    return guarded([&] { return spdnn_device_info_impl(name, cap, compute_units, hbm_bytes); });
}
int spdnn_get_feature_placement(const spdnn_net* n, int* paired, int* candidates, int64_t* search_peak_bytes) {
    return guarded([&] { return spdnn_get_feature_placement_impl(n, paired, candidates, search_peak_bytes); });
}
int spdnn_device_alloc_calls(int64_t* calls) {
    return guarded([&] { return spdnn_device_alloc_calls_impl(calls); });
}
int spdnn_device_memory(int64_t* free_bytes, int64_t* total_bytes) {
    return guarded([&] { return spdnn_device_memory_impl(free_bytes, total_bytes); });
}
int spdnn_device_synchronize(void) {
    return guarded([&] { return spdnn_device_synchronize_impl(); });
}
}  // extern "C"
