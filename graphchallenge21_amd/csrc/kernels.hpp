// Launch wrappers of the gfx950 kernels (kernels.hip).  Everything here takes device pointers.
//
// Feature layout in HBM ("row-block layout"): rows are grouped in blocks of RB = 64*RL rows
// (RL = rows per lane, 1, 2 or 4); inside a block the matrix is column-major:
//
//     Y[(block * N + column) * RB + row_in_block]        (fp32)
//
// so one neuron column of one row block is RB*4 contiguous bytes (256 B .. 1 KiB), the unit
// every kernel loads, stores, gathers and scatters.  A wavefront owns one row block; lane i
// holds rows i*RL .. i*RL+RL-1, indices and weights are wave-uniform scalars.
#pragma once
#include <hip/hip_runtime.h>
#include <cstdint>

namespace spdnn {

// A feature buffer lives in TWO allocations: row block rb is block rb >> 1 of half[rb & 1].  Device
// memory falls into a few large regions (a third of the memory each on MI355X), and a kernel that
// streams through buffers whose row blocks alternate between two regions runs a fifth faster than one
// whose buffers lie in a single region (measured: 6.1 against 5.1 TB/s for the memory skeleton of the
// band walk); the host puts the two halves into different regions where it can.
struct Feat {
    float* half[2] = {nullptr, nullptr};
    bool operator==(const Feat& o) const { return half[0] == o.half[0] && half[1] == o.half[1]; }
    explicit operator bool() const { return half[0] != nullptr; }
};

// Counts of an earlier launch handed to the host: the first workgroup of a layer kernel copies
// src[0..n) (device counters, final because that launch has finished) to dst (pinned host memory,
// where the host polls them).  A copy command between two layer launches would cost more than
// a small layer itself.
struct Publish {
    const int32_t* src = nullptr;
    int32_t* dst = nullptr;
    int n = 0;
};

struct BandLaunch {
    Feat yin;                // input buffer (row-block layout, labelled by the layer's band order)
    Feat yout;               // output buffer (labelled for the next layer through dst)
    const uint32_t* pairs;   // [N/2][stride] per pair of neighbouring outputs: 2 x 64-bit use masks, then one
                             // ring selector byte per merged step, in accumulation order
    const float* pw;         // [N/2][4*ceil(steps/4)][2] weights per step and output (0 where unused), or
                             // nullptr (uniform exact value)
    const int32_t* dst;      // [N] physical output column per band position
    int32_t* active;         // [rows] row stamp: active[row] = stamp if the row has a nonzero output
    int32_t* count_prev;     // device counter of the layer that stamped prev_stamp: this launch adds the rows that layer left active (may be nullptr)
    int N, K, nblk, stamp, rl;
    int steps, stride;       // merged steps per pair (K .. 36); dwords per pair record (16)
    int halo;                // input columns a segment needs before its first position: K-1 .. 32
    int prev_stamp = 0;      // stamp of the previous layer if the row slots still carry it (0 = none)
    int check_dead = 0;      // 1: row blocks the previous layer left without an active row are skipped
    int wmode;               // 0 uniform exact value, 1 per-entry fma (exact products), 2 mul then add
    int add_only = 1;        // wmode 0: add the inputs and scale the sum once (0: a multiply-add per input)
    int twins = 0;           // 1 (wmode 0): the two outputs of every pair use the same inputs (groups of identical rows,
                             // as in a run chain), so they are equal: one accumulator per pair, stored twice
    float wu, bias, clampv;
    int n_cu;
    int shape = -1;          // variant (see band_shape_count): 256-row blocks 0 = direct-to-LDS loads, 1 = through registers; < 0 = default
    int seglen = 0;          // band positions per workgroup; 0 = heuristic
    long long stream_min_bytes = 96ll << 20;  // launches that read + write at least this much hint their
                                              // column loads and stores as touched once
    int direct_lds = 1;      // 256-row blocks: 0 = never load straight into LDS (shape 1 only)
    // finishing a persistent launch that gave up: row blocks with frontier[rb] > frontier_layer have
    // this layer behind them already and are left alone (nullptr = every row block runs)
    const int32_t* frontier = nullptr;
    int frontier_layer = 0;
    Publish publish;
};

struct GatherLaunch {
    Feat yin;
    Feat yout;
    const int32_t* cols;     // [N][kmax] physical input columns in accumulation order
    const int32_t* rowlen;   // [N]
    const float* wv;         // [N][kmax]
    const int32_t* dst;      // [N]
    int32_t* active;
    int32_t* count_prev;     // device counter of the layer that stamped prev_stamp: this launch adds the rows that layer left active (may be nullptr)
    int N, kmax, nblk, stamp, rl;
    int prev_stamp = 0;      // as in BandLaunch
    int check_dead = 0;
    int wmode;               // 1 fma (exact products), 2 mul then add
    float bias, clampv;
    Publish publish;
};

hipError_t launch_band(const BandLaunch& a, hipStream_t s);
// 32 entries per output, at most 36 merged steps per pair, 16-dword records: the unrolled kernel path
bool band_unrolled(int K, int steps, int stride);
// Tuning space of the band walk: number of kernel variants for a row-block size (256-row blocks:
// loads straight into LDS or through registers) and the candidate segment lengths for a variant
// (used by the run-time selection in spdnn_run).
int band_shape_count(int rl, int direct_lds);
int band_seglen_candidates(int N, int K, int nblk, int rl, int shape, int n_cu, int* out, int max_out);
// the occupancy / halo model's score of one candidate (higher is better), for ordering trials
double band_seglen_score(int N, int K, int nblk, int rl, int shape, int n_cu, int seglen);
hipError_t launch_gather(const GatherLaunch& a, hipStream_t s);

// TILED layers: tiles of 1024 outputs, their input columns staged in LDS panel by panel (see LayerPlan).
struct TiledLaunch {
    Feat yin;
    Feat yout;
    const int32_t* cols;     // panels' columns, 512 per panel
    const int32_t* hdr;      // (first panel, panels) per tile, then (rounds, first entry block) per panel and wave
    const uint32_t* ent;     // entry blocks
    const int32_t* dst;      // [ntiles*1024] physical output column, -1 = unused slot
    int32_t* active;
    int32_t* count_prev;     // as in BandLaunch
    int N, ntiles, nblk, rl, wmode, stamp, prev_stamp, check_dead;
    float bias, clampv;
    Publish publish;
};
hipError_t launch_tiled(const TiledLaunch& a, hipStream_t s);

// TILED layers, ROWTILE form: a workgroup stages R feature rows (all N columns) in LDS, laid out [column][row], and
// every thread computes whole outputs for those rows - its own entry list, the rows in registers.  Every lane has its
// own number of entries, so the only padding is the spread of lengths inside a wave (the slots are ordered by
// length), whatever the number of columns.
struct RowtileLaunch {
    Feat yin;
    Feat yout;
    const uint32_t* ent;     // [kpad][N][2] (input column, weight bits) of every slot's k-th entry, zeros behind a list
    const int32_t* len;      // [N] entries per slot
    const int32_t* dst;      // [N] physical output column of the slot
    int32_t* active;
    int32_t* count_prev;     // as in BandLaunch
    int N, kpad, rows, rl, wmode, stamp, prev_stamp, check_dead;   // kpad: rows of `ent`, a multiple of 4; rows: carried rows (whole row blocks)
    float bias, clampv;
    Publish publish;
};
// rows a workgroup stages (16, 8 or 4 by the width), 0 = the width does not fit (more than 8192 neurons)
int rowtile_rows_per_workgroup(int N);
hipError_t launch_rowtile(const RowtileLaunch& a, hipStream_t s);

// BLOCK layers: groups of up to 16 outputs sharing up to 32 input columns.
struct BlockLaunch {
    Feat yin;
    Feat yout;
    const int32_t* cols;     // [ngroups][32] physical input columns, accumulation order
    const int32_t* cnt;      // [ngroups] shared inputs per group
    const float* wv;         // [ngroups*16][32] weights, or nullptr (uniform exact value)
    const int32_t* dst;      // [ngroups*16] physical output column, -1 = unused slot
    int32_t* active;
    int32_t* count_prev;     // as in BandLaunch
    int N, ngroups, nblk, stamp, prev_stamp, check_dead, rl, wmode;
    int full;                // 1: every group has exactly 32 shared inputs
    float wu, bias, clampv;
    const int32_t* frontier = nullptr;   // as in BandLaunch
    int frontier_layer = 0;
    Publish publish;
};
hipError_t launch_block(const BlockLaunch& a, hipStream_t s);

// ------------------------------------------------------------------------------------------
// Several layers per launch ("persistent" launches): the per-layer decomposition - many segments
// per row block - kept, with a dependency per ROW BLOCK where the per-layer launches have a launch
// boundary.  The work of `nlayers` consecutive layers of one kind is cut into units (layer, row
// block, segment) that lie in a queue in layer order; every workgroup claims the next unit with an
// atomic add until the queue is empty.  A unit of layer j waits until all segments of its row block
// have finished layer j-1 (a counter per layer and row block, `done`), then runs exactly what the
// per-layer kernel's workgroup runs.  A unit only ever waits for units claimed BEFORE it by
// workgroups that are running, so the launch cannot deadlock whatever part of its grid is resident.
// Every wait is bounded all the same: after `wait_limit` ticks of the 100 MHz clock the waiting
// workgroup sets `abort`, every workgroup leaves at its next look, and the host finishes the
// layers with per-layer launches (the `frontier` of the per-layer kernels).
//
// With xcd_queues the queue is split in eight, one per XCD: a workgroup reads the number of the
// XCD it runs on from the hardware and serves that queue only; row block rb belongs to queue
// rb % 8.  Everything a row block's layers hand to each other then stays in one XCD's L2, which saves the writer
// the write-back of that L2.
// ------------------------------------------------------------------------------------------
struct LayerDesc {           // one entry of the device-side layer table
    // BAND form
    const uint32_t* pairs;
    const float* pw;
    const int32_t* dst;
    float wu;
    int halo;                // input columns a segment needs before its first position (K-1, or 32 for run chains)
    int steps;               // merged steps per pair (records of 16 dwords: two use masks, 36 one-byte ring selectors)
    // BLOCK form (BLOCK layers; run-chain BAND layers that carry one)
    int ngroups;
    const int32_t* blk_cols;
    const int32_t* blk_cnt;
    const float* blk_wv;
    const int32_t* blk_dst;
    // ROWTILE form (TILED layers up to 8192 neurons wide)
    const uint32_t* rt_ent;
    const int32_t* rt_len;
    const int32_t* rt_dst;
    int rt_kpad;
    // QUAD form (BAND layers up to 1024 neurons wide)
    int quad_groups;
    const uint32_t* quad_col;
    const float* quad_w;
};

struct PersistCtl {          // device words of one persistent launch (zero before the launch)
    int32_t head[8];         // next unit of each queue
    int32_t units_done;      // units finished
    int32_t exited;          // workgroups that have left the kernel
    int32_t pad[6];
};

struct PersistLaunch {
    const LayerDesc* table;       // device pointer to the entry of the launch's first layer
    int nlayers;
    int block_form;               // 0: band walk, 1: BLOCK kernel body
    Feat first_in, buf_a, buf_c;  // layer j reads what layer j-1 wrote; every layer writes the work buffer it did not read
    int32_t* active;
    int32_t* done;                // [nlayers][done_stride] segments finished per layer and row block (zero before the launch)
    int done_stride;              // >= nblk
    int ngroups;                  // BLOCK form: groups per layer (the same for every layer of the launch)
    PersistCtl* ctl;              // this launch's control words
    const PersistCtl* prev_ctl;   // the persistent launch right before this one in the stream (or nullptr) ...
    int prev_units;               // ... and the units it must have finished for this one to start
    int32_t* abort;               // device word: nonzero = a launch gave up; sticky until the host clears it
    int32_t* host_word;           // pinned host word: receives the unit total when the launch is complete, -2 on abort
    int N, K, nblk, rl, wmode, stamp0, prev_stamp, check_dead;
    int unrolled, add_only, twins, full;   // kernel variant, as in BandLaunch / BlockLaunch
    int direct_lds;               // band walk on 256-row blocks: columns straight into the LDS ring (as BandLaunch.direct_lds)
    int seglen;                   // band positions (band walk) or groups (BLOCK) per unit; 0 = heuristic
    int xcd_queues;               // 1: one queue per XCD, row block rb in queue rb % 8
    int light_sync;               // 1 (xcd_queues only): the hand-over between layers stays inside one L2, so the
                                  // writer only waits for its stores (no L2 write-back); the reader invalidates at
                                  // device scope either way
    long long wait_limit;         // ticks of the 100 MHz clock a unit waits for its row block at most
    int n_cu;
    long long stream_min_bytes;
    float bias, clampv;
    Publish publish;
};
// units the launch consists of (what ctl->units_done reaches)
int persist_units(const PersistLaunch& a);
hipError_t launch_persist(const PersistLaunch& a, hipStream_t s);

// Resident launch: `nlayers` consecutive layers that all have a BLOCK form with one exact weight (BLOCK layers of
// weight mode 0, run-chain BAND layers that carry their BLOCK form) and the same group count, run by workgroups
// that keep R rows each in LDS from the first layer to the last (block_resident_kernel); no workgroup waits for
// another, so such a launch cannot give up.  Buffers as in PersistLaunch.  Rows get the stamp of the last layer
// that left them nonzero (stamp0 + j), none if no layer did; count with launch_count_stamp_range.
struct ResidentLaunch {
    const LayerDesc* table;       // device pointer to the entry of the launch's first layer
    int nlayers;
    Feat first_in, buf_a, buf_c;
    int32_t* active;
    int N, ngroups, rows, rl, full;   // rows: carried rows (whole row blocks); full: every group has 32 inputs
    int stamp0, prev_stamp, check_dead;
    float bias, clampv;
    Publish publish;
    // launch_band_resident only: the QUAD form of the launch's first layer (its steps' columns, their weights, the band's
    // dst); the arrays of layer j lie j * quad_stride bytes further on (the plans of consecutive layers of one structure
    // are laid out at equal distances).  It reads no layer table.
    const uint32_t* quad_col;
    const float* quad_w;
    const int32_t* quad_dst;
    long long quad_stride;
};
// The same for TILED layers in their ROWTILE form (any sparsity pattern): `nlayers` consecutive such layers of one
// weight mode, the R rows of a workgroup in LDS from the first layer to the last, every thread computing whole outputs
// from its own entry list (rowtile_resident_kernel).  ngroups and full are not used.
hipError_t launch_rowtile_resident(const ResidentLaunch& a, int wmode, hipStream_t s);
// rows such a workgroup keeps (16, 8 or 4 for up to 1024, 2048, 4096 neurons: two buffers of N x R floats), 0 = too wide
int rowtile_resident_rows(int N);

// The same for BAND layers in their QUAD form (up to 1024 neurons, any weights): 16 rows of a workgroup in LDS, a
// thread computes the four outputs of a quad of band positions for four of the rows (band_resident_kernel).  ngroups:
// groups of four steps per quad, the same for every layer of the launch; full is not used.
hipError_t launch_band_resident(const ResidentLaunch& a, int wmode, hipStream_t s);
// rows such a workgroup keeps (16), 0 = the shape does not fit
int band_resident_rows(int N);

// rows a workgroup keeps (16 or 4), 0 if the shape does not fit: two buffers of (N + 1) x R floats in LDS
// (N <= 1024: 16 rows, N <= 4096: 4) and one (group, row) item per thread of 1024
int resident_rows_per_workgroup(int N, int ngroups);
hipError_t launch_block_resident(const ResidentLaunch& a, hipStream_t s);

// counts[i] = number of rows r < rows with stamps[r] >= stamp_lo + i, for i in [0, n): with bias <= 0 a
// row that is zero stays zero, so the rows that carry the stamp of layer l or a later one are the rows
// layer l left active.  Written to counts_dev and (system scope) to counts_host, either may be nullptr.
// partial: count_stamp_partial_words() words of device memory, zero between the launches that use it (every launch
// leaves it so) - with it the rows are shared out over several workgroups; nullptr: one workgroup counts them all.
hipError_t launch_count_stamp_range(const int32_t* stamps, int rows, int stamp_lo, int n, int32_t* counts_dev,
                                    int32_t* counts_host, int32_t* partial, hipStream_t s);
int count_stamp_partial_words();

// Fused pair: two consecutive BAND layers (32 entries per row, unrolled record form, same weight
// mode, rows per lane 4) of which the first writes its outputs exactly where the second reads them
// (dst = identity) in one launch; the activations between them stay in LDS.  `dst` is the second
// layer's.  Rows the first layer leaves active get stamp_a in active_mid (no other launch looks at
// that array: count them with launch_count_stamped), rows the second leaves active stamp_b in active.
struct PairLaunch {
    Feat yin;
    Feat yout;
    const uint32_t* pairs_a;
    const float* pw_a;
    const uint32_t* pairs_b;
    const float* pw_b;
    const int32_t* dst;
    int32_t* active;
    int32_t* active_mid;
    int32_t* count_prev;     // as in BandLaunch, for the layer before the pair
    int N, nblk, rl, wmode;
    int add_only = 1;             // as in BandLaunch
    int halo_a, steps_a, halo_b, steps_b;
    int stamp_a, stamp_b, prev_stamp, check_dead;
    int seglen;              // band positions of the second layer per workgroup, 0 = heuristic
    int n_cu;
    long long stream_min_bytes;
    float wu_a, wu_b, bias, clampv;
    Publish publish;
};
hipError_t launch_band_pair(const PairLaunch& a, hipStream_t s);
int band_pair_seglen(int N, int nblk, int n_cu);
// count_out += number of rows r < rows with stamps[r] == stamp
hipError_t launch_count_stamped(const int32_t* stamps, int rows, int stamp, int32_t* count_out, hipStream_t s);

// Active-row scan: rows with active[row] == stamp and gid[row] >= 0 survive, in order.
// Writes count[0] = number of survivors, alive_src[k] = physical row of survivor k,
// alive_gid[k] = its global id.
hipError_t launch_scan_active(const int32_t* active, const int32_t* gid, int rows, int stamp,
                              int32_t* count, int32_t* alive_src, int32_t* alive_gid, hipStream_t s);

// Repack: row slot k of the destination takes physical row alive_src[k] of the source for
// k < count[0]; the remaining slots of the last block are zero-filled; gid_out likewise (-1).
hipError_t launch_repack(const Feat& src, const Feat& dst, const int32_t* count, const int32_t* alive_src,
                         const int32_t* alive_gid, int32_t* gid_out, int N, int rl, int dst_blocks,
                         hipStream_t s);

// Seeded Bernoulli features written straight into the row-block layout; col_of_phys maps a
// physical column to its neuron.
hipError_t launch_synth_features(const Feat& y, const int32_t* col_of_phys, int N, int batch, int nblk, int rl,
                                 uint64_t seed, float dmin, float dmax, hipStream_t s);

// Row-major chunk [nrows][N] (nrows rows starting at row0, row0 a multiple of RB) into the
// row-block layout with column labelling phys_of_col; rows >= batch are zero.  nonfinite[0] is
// set to 1 if a value is NaN or infinite.
hipError_t launch_pack_rows(const float* rowmajor, const Feat& y, const int32_t* phys_of_col, int N,
                            int64_t row0, int nrows, int rl, int32_t* nonfinite, hipStream_t s);

// Row-block layout to row-major for a list of physical rows (-1 gives a zero row).
// `active`/`stamp`: rows whose stamp differs read back as zero rows (stamp 0 = no check).
hipError_t launch_unpack_rows(const Feat& y, const int32_t* phys_of_col, const int32_t* phys_rows,
                              int nreq, int N, int rl, const int32_t* active, int stamp, float* rowmajor,
                              hipStream_t s);

hipError_t launch_iota_gid(int32_t* gid, int rows, int batch, hipStream_t s);
// where[g] = physical row (< carried) whose global id is g, -1 if none, for g in [0, batch)
hipError_t launch_row_table(const int32_t* gid, int carried, int batch, int32_t* where, hipStream_t s);
// phys[i] = where[ids[i]] (ids already checked against the batch on the host)
hipError_t launch_lookup_rows(const int32_t* ids, int n, const int32_t* where, int32_t* phys, hipStream_t s);
hipError_t launch_copy_f4(const float* src, float* dst, int64_t n_floats, hipStream_t s);
// copies both halves of src to the halves of dst concurrently (even / odd workgroups), n floats each
hipError_t launch_copy_pair(const Feat& src, const Feat& dst, int64_t n_floats_each, hipStream_t s);
// zero-fills p[0..n) and q[0..n) concurrently (even / odd workgroups): a probe of whether two
// buffers lie in the same memory region
hipError_t launch_zero_pair(float* p, float* q, int64_t n_floats_each, hipStream_t s);

}  // namespace spdnn
