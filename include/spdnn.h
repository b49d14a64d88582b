/*
 * spdnn.h - C ABI of the MI355X (gfx950) Sparse DNN Graph Challenge inference library.
 *
 * The library computes the layer chain  Y_{l+1} = min(ReLU(Y_l * W_l + bias), 32)  on one GPU
 * with hand-written HIP kernels.  It is the drop-in for the reference's single-GPU executor
 *
 *     void ftxj::test_benchmark_graph_challenge(input, weight, row_access, batch, neuron, bias, env)
 *     (reference: src/microbenchmark/header.h:16-19, defined at
 *      src/microbenchmark/all_network.cu:207-526, sole caller src/network.cpp:123)
 *
 * and for the host pieces that executor depends on (TSV loaders, reorder, inspector).  Where
 * the reference passes STL containers holding inspector-specific streams, this ABI takes plain
 * CSR per layer (row = OUTPUT neuron, col = INPUT neuron: the reference's in-memory convention,
 * src/utils/matrix.h:272-278) and dense or generated features; reorder, layout and kernel
 * selection happen behind the boundary.
 *
 * Conventions
 *   - every function returns an int status (SPDNN_OK = 0); none of them calls exit().  The
 *     reference's Safe_Call (src/gpu_lib/gpu_runtime.h:6-17) and launch checks
 *     (all_network.cu:362-366) terminate the process instead.
 *   - all pointers are HOST pointers unless a name ends in _dev; the library copies what it
 *     needs before returning, the caller may free its buffers immediately.
 *   - a handle is used by one host thread at a time.
 *   - row ids ("global ids", categories) are 0-based positions in the feature matrix that was
 *     handed over.
 *   - value ranges, checked at the boundary (SPDNN_E_ARG): weights finite with |w| <= 2^21;
 *     features finite with |x| <= 2^100 and, when nonzero, |x| >= 2^-100; bias finite, clamp
 *     positive, both at most 2^100.  Inside these no sum of products overflows and none
 *     underflows where that could change a rounding, so no infinity or NaN arises in the chain
 *     and the results equal the reference's CPU arithmetic bit for bit.  (The reference's
 *     ternary clamp would pass a NaN through, all_network.cu:8-10.)
 */
#ifndef SPDNN_H
#define SPDNN_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct spdnn_net spdnn_net;

enum spdnn_status {
    SPDNN_OK = 0,
    SPDNN_E_ARG = 1,         /* invalid argument (bad size, index out of range, non-finite value) */
    SPDNN_E_STATE = 2,       /* call made in the wrong order (e.g. run before inspect)           */
    SPDNN_E_IO = 3,          /* file missing or malformed                                         */
    SPDNN_E_DEVICE = 4,      /* HIP runtime error or no gfx950 device                             */
    SPDNN_E_NOMEM = 5,       /* host or device allocation failed                                  */
    SPDNN_E_UNSUPPORTED = 6  /* valid request the library cannot serve                            */
};

/* Kernel classes the inspector chooses from (per layer). */
enum spdnn_kernel {
    SPDNN_KERNEL_AUTO = 0,
    SPDNN_KERNEL_GATHER = 1, /* general CSR/ELL gather, any sparsity pattern                      */
    SPDNN_KERNEL_BAND = 2,   /* row-succ / tiled: relabelled circulant band walked through an LDS ring */
    SPDNN_KERNEL_BLOCK = 3,  /* groups of outputs that read the same inputs (RadiX-Net style): the shared
                                input columns are held in registers and reused by every output of the group */
    SPDNN_KERNEL_TILED = 4   /* any sparsity pattern, staged through LDS: up to 8192 neurons a workgroup keeps 16, 8 or 4
                                feature rows (all columns) and every thread computes whole outputs for them; beyond,
                                tiles of 1024 outputs whose input columns are staged panel by panel                */
};

typedef struct spdnn_layer_plan {
    int32_t kernel;          /* spdnn_kernel chosen for the layer                                 */
    int32_t max_row_nnz;     /* longest row                                                       */
    int32_t regular;         /* 1: every row and every column holds exactly max_row_nnz entries   */
    int32_t uniform_value;   /* 1: all values equal `value`                                       */
    float   value;
    int32_t exact_products;  /* 1: every value is 0 or +-2^e, so x*w is exact and fma == mul+add  */
    int32_t band_halo;       /* BAND: input columns a segment needs before its first position
                                (max_row_nnz-1 for a circulant band, 32 for run chains); else -1  */
    int64_t nnz;
    int64_t plan_bytes;      /* device bytes held for this layer                                  */
    int32_t block_form;      /* second form the layer holds for small launches: 1 = a run-chain BAND layer with its
                                BLOCK form, 2 = a TILED layer with its GATHER form (used below 8192 rows on layers of
                                1024 neurons and more that have no ROWTILE form - wider than 8192 neurons or
                                SPDNN_ROWTILE=0 - or where SPDNN_TILED_MIN_ROWS asks for it); 0 = none */
    int32_t fuse_next;       /* 1 (after spdnn_inspect): this layer and the next can run as one fused launch, the
                                activations between them kept in LDS (see spdnn_run_options.fuse_layers)  */
    int32_t common_order;    /* run chains, after spdnn_inspect: 0 = the layer has a labelling of its own; 1 or 2 = it is
                                laid out in the neuron order its network's RadiX-Net layers share, the second run of
                                every group that many 16-neuron slots behind the group (what lets neighbours fuse)  */
} spdnn_layer_plan;

typedef struct spdnn_run_options {
    int32_t prune;             /* 1: drop rows that are all zero between layers (requires bias <= 0) */
    int32_t first_layer;       /* 0 starts from the features; >0 continues from the current state  */
    int32_t n_layers;          /* number of layers to run, -1 = through the last                   */
    int32_t collect_counts;    /* 1: record the active-row count after every layer                 */
    int32_t time_layers;       /* 1: bracket every layer with HIP events                           */
    float   compact_threshold; /* prune: repack when active <= threshold * carried (0 = default .75) */
    int32_t fuse_layers;       /* launches that hold more than one layer.  1 = every layer its own launch.  0 = default:
                                  - resident launches where consecutive layers have a BLOCK form with one exact weight
                                    (RadiX-Net layers) or are TILED layers, at most 4096 neurons wide, or are BAND layers
                                    at most 1024 neurons wide (from 6 layers on, from 16 at 16384 rows and more): a workgroup
                                    keeps 16, 8 or 4 rows in LDS through up to 64 layers (SPDNN_RESIDENT=0: never;
                                    SPDNN_BAND_RESIDENT=0: not the BAND layers);
                                  - pairs of layers the inspector marked fuse_next as one launch with the intermediate tile
                                    in LDS, on launches of 2^23 rows x neurons and more (SPDNN_PAIR_MIN_ELEMS);
                                  - persistent launches (up to 64 layers of one kernel form, a dependency per row block
                                    between the layers) where a layer moves 256 MiB - 2 GiB on 64 row blocks or more
                                    (SPDNN_PERSIST=0: never);
                                  - every other layer as its own launch.
                                  n >= 2: the pairs, and elsewhere resident or persistent launches of up to n layers
                                  whatever the size.  Results are the same bit for bit in every mode. */
    int32_t persist_wait_us;   /* persistent launches: longest wait of a unit for its row block in microseconds; 0 = default
                                  (2 s, SPDNN_PERSIST_WAIT_US), negative = give up at the first look that finds the row
                                  block not ready (exercises the fall-back to per-layer launches)                     */
    int32_t reserved[2];
} spdnn_run_options;

typedef struct spdnn_run_result {
    int32_t layers_run;      /* layers actually launched (fewer when every row died)              */
    int32_t compactions;     /* number of row repacks                                             */
    int64_t active_rows;     /* rows active after the last requested layer                        */
    int64_t carried_rows;    /* rows physically carried at the end                                */
    float   ms_total;        /* HIP-event time, first launch to last completion                   */
    float   ms_kernels;      /* sum of per-layer kernel times (time_layers only, else 0)          */
    double  alg_bytes;       /* sum over layers of 8*B_l*N + nnz_l*8 + 4*(N+1)                     */
    double  edges;           /* batch * nnz summed over the layers requested                      */
    int32_t launches;        /* layer-kernel launches made (a fused launch counts once)           */
    int32_t fused_pairs;     /* of them, fused pairs of layers (intermediate tile in LDS)         */
    int32_t persistent_launches;   /* of them, persistent launches (several layers, a dependency per row block)   */
    int32_t persistent_fallbacks;  /* persistent launches that gave up and were finished by per-layer launches     */
    int32_t resident_launches;     /* of the launches, resident ones (several layers, the rows kept in LDS throughout) */
    int32_t reserved;
} spdnn_run_result;

/* ---- life cycle ------------------------------------------------------------------------- */

/* Library version (major*10000 + minor*100 + patch). */
int spdnn_version(void);

/* Text of the most recent error on this thread (never NULL). */
const char* spdnn_last_error(void);

/* Creates a network of `layers` square layers of width `neuron`, for at most `max_batch`
 * feature rows.  bias and clamp are the epilogue constants (reference: bias by neuron count,
 * src/network.cpp:73-78; clamp 32, all_network.cu:8-10).  Touches no device. */
int spdnn_create(int neuron, int max_batch, int layers, float bias, float clamp, spdnn_net** out);

/* Releases host and device memory (the reference never frees, all_network.cu:240-303). */
int spdnn_destroy(spdnn_net* net);

/* Bias the reference driver selects for a neuron count (src/network.cpp:73-78): -0.3, -0.35,
 * -0.4, -0.45 for 1024, 4096, 16384, 65536; returns SPDNN_E_ARG for other widths (the
 * reference silently uses 0 there). */
int spdnn_reference_bias(int neuron, float* bias);

/* ---- weights ---------------------------------------------------------------------------- */

/* Hands over layer `layer` as CSR with row = output neuron, col = input neuron, what
 * COOMatrix(file,1,false) + CSRCSCMatrix hold in the reference (src/utils/matrix.h:255-282,
 * :329-343).  Columns inside a row may come in any order; accumulation is always in ascending
 * input index, the order of the reference's CPU checker (src/utils/cpu_spmm.h:14-35). */
int spdnn_set_layer_csr(spdnn_net* net, int layer, const int32_t* rowptr, const int32_t* col, const float* val);

/* Reads a weight TSV in the challenge format ("in out value", 1-based), the file format of
 * COOMatrix(file, 1, false) (src/utils/matrix.h:255-282), and sets the layer. */
int spdnn_load_layer_tsv(spdnn_net* net, int layer, const char* path);

/* Reads layers [first, first+count) from <data_dir>/neuron<N>/n<N>-l<layer+1>.tsv (the names of
 * get_weight_file_name, src/network.cpp:14-19) - the loop of src/network.cpp:96-120, with the
 * files parsed, checked and inspected side by side on the library's worker threads (one layer of
 * N=65536 is 39 MB of text, the 1920 of them 75 GB).  Returns when every layer is done; the first
 * failing layer by number is reported (SPDNN_E_IO names the file) and stays unset. */
int spdnn_load_layers_tsv(spdnn_net* net, const char* data_dir, int first, int count);

/* Reads layers [first, first+count) from a packed binary weight file "neuron<N>.bin" as the
 * reference's library benchmarks consume it (readweights, benchmark/cusparse/cusparse.cu:318-358):
 * one record per layer of int32 row[nnz], int32 col[nnz], float32 val[nnz], 1-based, with
 * row = OUTPUT neuron (the CSR row there) and col = input neuron.  nnz_per_layer = 0 means
 * 32 * neuron, the only size the reference reads. */
int spdnn_load_layers_bin(spdnn_net* net, const char* path, int first, int count, int64_t nnz_per_layer);

/* File name the reference driver uses for a layer: <dir>/neuron<N>/n<N>-l<layer+1>.tsv
 * (get_weight_file_name, src/network.cpp:14-19). */
int spdnn_weight_file_name(const char* data_dir, int neuron, int layer, char* out, int cap);

/* Generates `count` synthetic layers [first, first+count) with the seeded permuted-stride
 * generator: W_l[i, (pi_l(i) + o_l + k*s_l) mod N] = value for k = 0..nnz_per_row-1.  Runs on
 * host threads and feeds the same path as spdnn_set_layer_csr. */
int spdnn_synth_layers(spdnn_net* net, uint64_t seed, int first, int count, int nnz_per_row, float value);

/* Host copy of one synthetic layer in CSR form (rowptr[N+1], col/val[N*nnz_per_row]). */
int spdnn_synth_layer_csr(uint64_t seed, int layer, int neuron, int nnz_per_row, float value,
                          int32_t* rowptr, int32_t* col, float* val);

/* ---- inspector -------------------------------------------------------------------------- */

/* The per-layer inspector (classification, relabelling, kernel choice, plan emission; the role
 * of BlockContainer + MaxInReuseBSchedule in src/network.cpp:105-120) runs on host worker
 * threads as layers are handed over.  spdnn_inspect waits for it, checks that every layer is
 * set and links consecutive layers (each layer stores its outputs in the column order the next
 * one reads).  Host only; plans are uploaded on first device use. */
int spdnn_inspect(spdnn_net* net);

/* SPDNN_KERNEL_AUTO (default) lets the inspector choose per layer; SPDNN_KERNEL_GATHER makes it
 * emit the general kernel for every layer.  Must be called before the first layer is set. */
int spdnn_set_force_kernel(spdnn_net* net, int kernel);

/* Streamed plans, for networks whose plans should not (or do not) all stay in device memory: the
 * device holds `slots` plan-sized slots (2..64; 0 = every plan resident, the default), all plans
 * stay in pinned host memory, and a second stream copies the plan of layer l + slots into the slot
 * of layer l as soon as layer l has finished, under the layers in between.  This is the double
 * buffer of src/microbenchmark/out_memory.cu:318-327 (two weight/index buffers) and :367-386 (copy
 * of layer l+1 on a memory stream while layer l runs), with events between the two streams instead
 * of that loop's host synchronisation per layer.  Results are the same as with resident plans;
 * launches that fuse several layers are not used.  Call before the features are handed over
 * (SPDNN_E_STATE afterwards; spdnn_inspect after a layer change opens the choice again).  A window
 * that is not smaller than the layer count leaves the plans resident.  Environment default:
 * SPDNN_PLAN_WINDOW. */
int spdnn_set_plan_window(spdnn_net* net, int slots);

/* Where the plans are once they are uploaded: window (0 = resident), bytes of device memory they
 * occupy, bytes of pinned host memory behind them (0 when resident). */
int spdnn_get_plan_memory(const spdnn_net* net, int* window, int64_t* device_bytes, int64_t* pinned_bytes);

int spdnn_get_layer_plan(const spdnn_net* net, int layer, spdnn_layer_plan* out);

/* Host view of a BAND plan, for verification: position of every input neuron along the band
 * (in_pos[N]), the output neuron computed at every band position (out_at[N]), and per position
 * the ring selectors of its inputs in accumulation order (sel[N*max_row_nnz], position mod 256).
 * Any pointer may be NULL.  SPDNN_E_STATE if the layer is not a BAND layer. */
int spdnn_get_band_plan(const spdnn_net* net, int layer, int32_t* in_pos, int32_t* out_at, uint8_t* sel);

/* Number of schedule slots of a layer: neuron for BAND and GATHER layers, 16 per group for BLOCK
 * layers (unused slots carry -1 in dst). */
int spdnn_get_layer_slots(const spdnn_net* net, int layer, int* slots);

/* Physical output column of every schedule slot of a layer (dst[slots]); needs spdnn_inspect. */
/* What the band kernel streams for a BAND layer: one record per pair of neighbouring band positions
 * (2u, 2u+1).  The two outputs add their inputs in ascending input index, so their lists merge into
 * one list of *steps steps in which a shared input appears once.  A record is *stride dwords: the
 * 64-bit use mask of output 2u (low dword first), the use mask of output 2u+1, then one byte per
 * step = band position of the step's input mod 256 (padded with repeats of the last step).
 * *has_weights tells whether the kernel streams weights (0: the layer has one exact value and the
 * arithmetic takes it from the use masks).  `records` (neuron/2 * *stride dwords) and `weights`
 * (neuron/2 * *padded_steps * 2 floats when *has_weights: per step the weight for output 2u and for
 * output 2u+1, 0 where unused) may be NULL, like every out-parameter. */
int spdnn_get_band_pairs(const spdnn_net* net, int layer, int* steps, int* stride, int* padded_steps,
                         int* has_weights, uint32_t* records, float* weights);

/* The QUAD form a BAND layer of up to 1024 neurons also carries, for resident launches (16 rows of a workgroup kept in
 * LDS through the layers): the four outputs at band positions 4c .. 4c+3 share one merged list of steps, in *groups
 * groups of four.  columns (neuron/4 * *groups * 4 words): the input column of every step as its byte offset in a buffer
 * of 16 rows per column (column * 64); weights (neuron/4 * *groups * 4 * 4 floats: [quad][group][step][output]): the
 * step's weight in each of the four outputs, 0 where the output does not use it.  *groups = 0: the layer has no such
 * form.  No counterpart in the reference (its kernels keep a layer's outputs in shared memory for one layer only);
 * inspection interface like spdnn_get_band_pairs. */
int spdnn_get_band_quads(const spdnn_net* net, int layer, int* groups, uint32_t* columns, float* weights);

int spdnn_get_layer_dst(const spdnn_net* net, int layer, int32_t* dst);

/* Receptive field of a block of output neurons through consecutive layers: the input neurons of layer
 * first_layer that the neurons out_neurons[0..n_out) of layer first_layer + n_layers - 1 depend on -
 * the analysis of the reference's FuseLayer (src/fuse/fuse.h:13-53: the constructor gathers the inputs
 * of a block of output columns of one layer, every fuse() call carries the set one layer further
 * back), on which its fused kernel sizes the tile of the layer before (src/microbenchmark/fuse.cu:226-248).
 * *count receives the size of the set; in_neurons (may be NULL) its first min(*count, cap) members,
 * ascending.  A pair of layers can keep its intermediate tile on chip only where this set stays a
 * small multiple of the block for every block of a tiling; spdnn_inspect marks the pairs it fuses
 * (spdnn_layer_plan.fuse_next).  Host only; needs the layers set (their inspection is waited for). */
int spdnn_receptive_field(spdnn_net* net, int first_layer, int n_layers, const int32_t* out_neurons, int n_out,
                          int32_t* in_neurons, int64_t cap, int64_t* count);

/* Physical column of every neuron in the buffer layer `layer` reads (layer == layers: the
 * final output, always the identity). */
int spdnn_get_input_labelling(const spdnn_net* net, int layer, int32_t* phys_col);

/* HashReorder::reorder (src/reorder/hash.h:14-31): v -> v / buckets + (v % buckets) * (domain / buckets).
 * Returns SPDNN_E_ARG where the reference prints an error and exits. */
int spdnn_hash_reorder(int v, int buckets, int domain, int* out);

/* ---- features --------------------------------------------------------------------------- */

/* Dense row-major fp32 features, batch x neuron (what read_input + the flatten at
 * all_network.cu:240-247 produce).  Requires spdnn_inspect. */
int spdnn_set_features_dense(spdnn_net* net, const float* rowmajor, int batch);

/* Sparse feature TSV in the challenge format ("row neuron value", 1-based; rows beyond batch
 * are skipped): read_input, src/network.cpp:33-54. */
int spdnn_load_features_tsv(spdnn_net* net, const char* path, int batch);

/* The same file into host memory: read_input of src/network.cpp:33-54 itself (dense batch x neuron,
 * row-major, zero where the file says nothing; of an entry that occurs twice the last line counts,
 * network.cpp:47).  *kept (may be NULL) receives the number of lines stored.  The file is parsed in
 * parts by the library's host threads.  Host only: needs no device and no handle.  After a failure
 * the contents of rowmajor are unspecified. */
int spdnn_read_features_tsv(const char* path, int neuron, int batch, float* rowmajor, int64_t* kept);

/* Packed binary features "sparse-images-<N>.bin" (readinput, benchmark/cusparse/cusparse.cu:361-383):
 * int32 row[] = neuron, int32 col[] = image, float32 val[], 1-based, the entry count being the file
 * size / 12; images beyond batch are skipped. */
int spdnn_load_features_bin(spdnn_net* net, const char* path, int batch);

/* Seeded Bernoulli rows generated on the device: row r has density uniform in [dmin, dmax],
 * entries are 0.0f / 1.0f.  spdnn_synth_features_host produces the same values on the host. */
int spdnn_synth_features(spdnn_net* net, uint64_t seed, int batch, float dmin, float dmax);
int spdnn_synth_features_host(uint64_t seed, int neuron, int64_t row_begin, int64_t nrows,
                              float dmin, float dmax, float* rowmajor);

/* ---- inference -------------------------------------------------------------------------- */

int spdnn_default_run_options(spdnn_run_options* opt);

/* Runs layers [first_layer, first_layer + n_layers): the layer loop of
 * test_benchmark_graph_challenge (all_network.cu:333-519).  Every layer kernel counts the rows
 * the layer before it left active; with prune the host reads the count of a layer a few launches
 * back (never of the one just launched; a following launch stores it into pinned host memory),
 * stops launching once it is zero, and queues the on-device scan + repack when few enough rows
 * are left.  One host synchronisation, at the end. */
int spdnn_run(spdnn_net* net, const spdnn_run_options* opt, spdnn_run_result* result);

/* Active-row count recorded after layer `layer` of the last run (collect_counts or prune),
 * the number the reference prints as "layer l, batch = n" (all_network.cu:508). */
int spdnn_get_active_count(const spdnn_net* net, int layer, int64_t* count);

/* Global ids (ascending) of the rows that are nonzero after the last layer run: the challenge's
 * categories.  *n receives the count; ids may be NULL to query it. */
int spdnn_get_categories(spdnn_net* net, int32_t* ids, int64_t cap, int64_t* n);

/* Current activations of the given global rows, row-major nrows x neuron in natural neuron
 * order (rows that were pruned are zero).  The reference copies the whole buffer back
 * (all_network.cu:521). */
int spdnn_get_activations(spdnn_net* net, const int32_t* rows, int nrows, float* rowmajor);

/* spdnn_get_activations for callers that cannot allocate device memory (tight serving loops,
 * harnesses that forbid hipMalloc).  No counterpart in the reference.  It allocates nothing, but it
 * is not a call for inside a HIP graph capture: it synchronises its stream once per pass and copies
 * to and from pageable host memory.  Same arguments and results as spdnn_get_activations, but where that call allocates
 * its row list and its row-major staging rows for every call, this one calls no hipMalloc / hipFree:
 * it works in a 12.1 MiB scratch array that is part of the library's device code (one copy per GPU,
 * held until the process ends): a row table (global id -> physical row, filled by two small
 * kernels at every call), the ids of one pass and 8 MiB of staging rows.
 * Limits: batch <= 1048576 rows and neuron <= 2097152 (one row must fit the staging rows);
 * beyond them SPDNN_E_UNSUPPORTED.  All handles of a process share one GPU's scratch array: calls
 * that overlap in time on one GPU (from several host threads or handles) race and must be
 * serialised by the caller. */
int spdnn_get_activations_noalloc(spdnn_net* net, const int32_t* rows, int nrows, float* rowmajor);

/* Band-walk configuration measured at run time (record `index` = 0, 1, ...; SPDNN_E_ARG past the
 * last): row blocks it was measured for, kernel variant (256-row blocks: 0 = the next chunk's columns
 * go from HBM straight into the LDS ring, 1 = through registers; one variant for smaller row blocks;
 * the tile is 8 waves x one output pair and a 64-slot LDS ring in every case) and band positions per
 * workgroup. */
int spdnn_get_band_tuning(const spdnn_net* net, int index, int* row_blocks, int* shape, int* seglen);

/* Per-layer kernel milliseconds of the last run made with time_layers. */
int spdnn_get_layer_times(const spdnn_net* net, float* ms, int n);

/* Writes the categories as the challenge's truth-file format: one 1-based row id per line. */
int spdnn_write_categories(spdnn_net* net, const char* path);

/* ---- device utilities ------------------------------------------------------------------- */

/* Measured device-to-device copy bandwidth (GB/s, read + write bytes over HIP-event time) of a
 * plain float4 copy kernel over `bytes` bytes: the box's practical HBM peak. */
int spdnn_measure_copy_bandwidth(int64_t bytes, int reps, double* gbps);

/* The same measurement over the network's own work buffers (one copied to the other, the rows of
 * the current batch): the copy rate a layer kernel could reach at best with these buffers where
 * they lie (their halves may sit in two memory regions, see spdnn_get_feature_placement).
 * Needs features; the state of the network is reset as at the start of a run from layer 0. */
int spdnn_measure_buffer_copy_bandwidth(spdnn_net* net, int reps, double* gbps);

/* Name and compute-unit count of device 0. */
int spdnn_device_info(char* name, int cap, int* compute_units, int64_t* hbm_bytes);

/* How the feature buffers were placed (after features were set): *paired = 1 if the two halves of
 * every buffer lie in different memory regions (searched for half-buffers of 0.4 GiB and more, see
 * SPDNN_REGION_PAIRING), *candidates = half-buffers allocated during the search (6 = no search),
 * *search_peak_bytes = device memory the search held at its peak (candidates and the fillers between
 * them; everything beyond the six half-buffers kept was freed again before the call returned).  Any
 * pointer may be NULL. */
int spdnn_get_feature_placement(const spdnn_net* net, int* paired, int* candidates, int64_t* search_peak_bytes);

/* Free and total device memory of device 0 in bytes (what hipMemGetInfo reports); either pointer
 * may be NULL.  Sizing aid: a network holds three feature buffers of rows*neuron*4 bytes plus the
 * layer plans. */
int spdnn_device_memory(int64_t* free_bytes, int64_t* total_bytes);

int spdnn_device_synchronize(void);

/* Number of device allocations (hipMalloc) the library has made in this process so far: a diagnostic for
 * callers that must know that a call allocates nothing (spdnn_get_activations_noalloc leaves it unchanged). */
int spdnn_device_alloc_calls(int64_t* calls);

#ifdef __cplusplus
}
#endif
#endif /* SPDNN_H */
