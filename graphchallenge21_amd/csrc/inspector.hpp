// Host inspector: turns one layer's CSR into the arrays the kernels stream.
//
// Plays the role of the reference's src/inspector (BlockContainer + MaxInReuseBSchedule,
// called from src/network.cpp:105-120), re-designed: instead of searching for dense rectangles
// in a hash-reordered matrix it classifies the layer, looks for a relabelling of inputs and
// outputs under which the layer is a circulant band, and emits either a BAND plan (ring
// selectors in accumulation order) or a general GATHER plan.
#pragma once
#include <cstdint>
#include <string>
#include <vector>

#include "../../include/spdnn.h"

namespace spdnn {

constexpr int kTileOutputs = 1024;  // TILED: outputs per tile (16 waves x 64)
constexpr int kPanelCols = 512;     // TILED: input columns staged in LDS at a time
constexpr int kQuadMaxNeurons = 1024;  // BAND: widest layer that carries its QUAD form (two buffers of N x 16 rows in LDS)
constexpr int kQuadColumnBytes = 64;   // ... whose columns are 16 rows of 4 bytes: the form holds byte offsets

struct LayerPlan {
    bool set = false;
    bool failed = false;            // the inspection job ended in an exception
    bool failed_nomem = false;      // ... which was a failed host allocation
    std::string fail_text;          // ... what the exception said
    spdnn_layer_plan info{};
    int kernel = SPDNN_KERNEL_GATHER;
    int wmode = 2;                  // 0 uniform exact value, 1 exact products, 2 multiply then add
    int kmax = 0;
    // physical column of every input neuron in the buffer this layer reads
    std::vector<int32_t> in_pos;
    // neuron computed at every schedule slot (BAND: band position; GATHER: the neuron itself)
    std::vector<int32_t> out_at;
    std::vector<uint8_t> sel;       // BAND: [N][K] input position mod 256, accumulation order (host view only)
    // BAND, what the kernel streams: per pair of neighbouring band positions pair_stride dwords - two
    // 64-bit use masks (output 2u, output 2u+1), then one selector byte per merged step (pair_steps
    // of them, padded to whole dwords)
    std::vector<uint32_t> pairs;
    int pair_steps = 0, pair_stride = 0, pair_padded = 0;  // padded: steps a record and the weights are laid out for
    std::vector<int32_t> ell_col;   // GATHER: [N][kmax] physical input column, accumulation order
    std::vector<int32_t> rowlen;    // GATHER: [N]
    // BLOCK: groups of up to 16 outputs that read the same (up to 32) inputs
    int ngroups = 0;
    bool blk_full = false;          // every group has exactly 32 shared inputs
    std::vector<int32_t> blk_cols;  // [ngroups][32] physical input columns, accumulation order (padded)
    std::vector<int32_t> blk_cnt;   // [ngroups] number of shared inputs
    std::vector<float> wv;          // weights in accumulation order: BAND [N/2][padded steps][2], GATHER [N][kmax],
                                    // BLOCK [ngroups*16][32] (empty when wmode 0)
    std::vector<int32_t> dst;       // [N] physical column of slot's output in the next buffer
    // A run-chain BAND layer with one exact weight value also carries its BLOCK form (same input
    // labelling, so either kernel can run the layer): for batches whose buffers fit the on-chip
    // caches the BLOCK kernel is the faster of the two.
    int alt_ngroups = 0;
    bool alt_full = false;
    std::vector<int32_t> alt_cols;   // [alt_ngroups][32] physical input columns, accumulation order
    std::vector<int32_t> alt_cnt;    // [alt_ngroups]
    std::vector<int32_t> alt_out_at; // [alt_ngroups*16] output neuron of the slot, -1 = unused
    std::vector<int32_t> alt_dst;    // [alt_ngroups*16] physical column in the next buffer
    // A TILED layer carries its GATHER form in the same arrays (alt_ngroups stays 0): alt_cols [N][alt_kmax] input
    // columns in accumulation order, alt_cnt [N] row lengths, alt_wv [N][alt_kmax] weights, alt_out_at [N] = the output
    // neuron of every slot, alt_dst [N].  A tile's workgroup needs 64 rows x 1024 outputs to itself: on small batches of wide
    // layers that leaves most of the chip idle, and the gather kernel, which spreads over 8 outputs per wave, is faster.
    std::vector<float> alt_wv;
    int alt_kmax = 0;
    // ... and its ROWTILE form over the same slots (outputs ordered by length, longest first, so that the 64 lanes of a
    // wave have about the same number of entries): rt_ent [alt_kmax rounded up to 4][N][2] = (input column, weight bits)
    // of the slot's k-th entry, zeros behind a list, entry-major so that the lanes of a wave read neighbouring words.
    std::vector<uint32_t> rt_ent;
    // A BAND layer of up to 1024 neurons also carries its QUAD form, for launches that keep 16 rows of a workgroup in
    // LDS through the layers: the four outputs at band positions 4c .. 4c+3 add their inputs in ascending input index,
    // so their lists merge into one list of steps (K + 3 for a circulant band), padded to quad_groups groups of four.
    // quad_col [N/4][quad_groups][4] = input column of each step, as the byte offset of the column in a buffer of 16 rows per
    // column; quad_w [N/4][quad_groups][4 steps][4 outputs] = the weight of the step in each output, 0 where the output
    // does not use it (padding steps repeat the last column): the 16 bytes a lane of the quad loads are one step's.
    std::vector<uint32_t> quad_col;
    std::vector<float> quad_w;
    int quad_groups = 0;
    // BAND: neuron j sits at the same band position as an input and as an output (see
    // canonicalize_self_aligned_band); fuse_next: this layer writes its outputs exactly where the
    // next layer's band reads them (dst = identity) and both fit the fused pair kernel
    // TILED: out_at / dst hold ntiles x 1024 slots (-1 = unused); ell_col the panels' columns, 512 per
    // panel (padded); rowlen first (first panel, panels) per tile, then (rounds, first entry block) per
    // panel and wave; wv the entry blocks of 1 KiB: per round 64 outputs x 2 entries x (byte offset of
    // the column's slot in the panel as raw bits, weight)
    int ntiles = 0;
    int rc_cycles = 0;         // run chains: cycles of groups the layer's own labelling found
    bool self_aligned = false;
    bool pair_twins = false;   // BAND, one exact weight: the two outputs of every pair use the same inputs
    bool fuse_next = false;
};

// Sorts every row of the CSR by input index (stable) and validates it.  Returns an empty
// string on success, an error text otherwise.
std::string normalize_csr(int N, const int32_t* rowptr, const int32_t* col, const float* val,
                          std::vector<int32_t>& out_rowptr, std::vector<int32_t>& out_col,
                          std::vector<float>& out_val);

// Looks for a relabelling under which output v reads inputs v-K+1..v (mod N).  rowptr/col must
// be normalized, every row and column holding exactly K entries.  On success in_pos[i] is the
// band position of input i and out_at[v] the output neuron at position v.
bool discover_band(int N, int K, const std::vector<int32_t>& rowptr, const std::vector<int32_t>& col,
                   std::vector<int32_t>& in_pos, std::vector<int32_t>& out_at);

// Groups outputs whose input lists are identical (at most 16 per group, lists of at most 32).
// Returns false when the layer has too few duplicates to be worth it.
bool discover_blocks(int N, const std::vector<int32_t>& rowptr, const std::vector<int32_t>& col,
                     std::vector<std::vector<int32_t>>& groups);

// For a layer of 32 entries per row whose groups (from discover_blocks) hold exactly 16 outputs each:
// looks for the chain structure of a RadiX-Net layer - every group reads two runs of 16 inputs and
// every run is read by two groups, so groups and runs form cycles - and lays the cycles out so
// that the group at band positions [16t, 16t+16) reads only positions in [16t-32, 16t+16) (mod N).
// The result is a BAND labelling (in_pos, out_at) for a halo of 32.
bool discover_run_chains(int N, const std::vector<int32_t>& rowptr, const std::vector<int32_t>& col,
                         const std::vector<std::vector<int32_t>>& groups, std::vector<int32_t>& in_pos,
                         std::vector<int32_t>& out_at, int* cycles = nullptr);

// One neuron order for the RadiX-Net layers of a network whose files share a (hidden) neuron
// numbering - layer l's output j and layer l+1's input j are the same neuron, and under the hidden
// numbering group g of every such layer reads neuron blocks g and g + m_l (mod N/16).  From a layer
// whose blocks form a single cycle (m coprime to N/16, e.g. stride 16): pos[neuron] = 16 * slot of
// its block along the cycle + rank inside the block, oriented so that the block a slot reads besides
// its own lies one slot back.  False when the layer has no such structure (groups that are not also
// the runs they read, several cycles).
bool common_run_order(int N, const std::vector<int32_t>& rowptr, const std::vector<int32_t>& col,
                      std::vector<int32_t>& pos);

// Whether `pos` is a run-chain labelling of this layer too: every output at slot t reads all of
// slot t and all of slot t - d with the same d for the whole layer.  Returns d (1 or 2: inside the
// band kernel's halo of 32), 0 otherwise.
int common_order_offset(int N, const std::vector<int32_t>& rowptr, const std::vector<int32_t>& col,
                        const std::vector<int32_t>& pos);

// Full per-layer inspection (everything except dst, which needs the next layer's labelling).
// fma_ok: nonzero activations stay far above the denormal range, so that a product with a
// power-of-two weight is exact and a fused multiply-add rounds like multiply-then-add; when false
// every layer uses the unfused pair.  common_pos: the network's common neuron order (common_run_order);
// a run-chain layer with one exact weight that it fits (common_order_offset) takes it for inputs and
// outputs instead of a labelling of its own.
void inspect_layer(int N, const std::vector<int32_t>& rowptr, const std::vector<int32_t>& col,
                   const std::vector<float>& val, int force_kernel, bool fma_ok, LayerPlan& plan,
                   const std::vector<int32_t>* common_pos = nullptr);

// The layer's structure back from its plan: rowptr[N+1] / col[] with row = output neuron and the
// input neurons of every row ascending.
void plan_adjacency(const LayerPlan& plan, int N, std::vector<int32_t>& rowptr, std::vector<int32_t>& col);

// Receptive field of a block of output neurons through n_layers consecutive layers (plans[0] is the
// first of them): the input neurons of plans[0] that the outputs `outs` of plans[n_layers-1] depend
// on, ascending.  The analysis of the reference's FuseLayer (src/fuse/fuse.h:13-53: the constructor
// collects the entries of the last layer that lead into the block, every fuse() call carries the
// set one layer further back).
void receptive_field(const LayerPlan* plans, int N, int n_layers, const int32_t* outs, int n_out,
                     std::vector<int32_t>& inputs);

// Whether layers a and b (consecutive, a already linked to b) can run as one fused launch: both
// circulant or run-chain bands of 32 entries per row in the unrolled record form with the same
// weight mode, a's outputs landing exactly on b's band (dst = identity).
bool pair_fusable(const LayerPlan& a, const LayerPlan& b, int N);

// dst[slot] = physical column (in the next buffer) of the neuron computed at `slot`.
void link_layers(LayerPlan& cur, const std::vector<int32_t>* next_in_pos);

}  // namespace spdnn
