// Internal declarations shared by the host API, the repacker and the kernel launchers.
#pragma once

#include <cstddef>
#include <cstdint>
#include <string>
#include <vector>

#include "ovfcc.h"

struct ovfcc_gnode;
struct ovfcc_fold;
struct ovfcc_gather_fold;

namespace ovfcc {

// ---- tiled layout ------------------------------------------------------------------------
// The unit every fast kernel streams is a 1 KiB tile read by one wave64 with one 128-bit load
// per lane.  A tile covers 16 output channels; lane l serves channel (l & 15) and k-quarter
// (l >> 4).  A "k-block" is 128 consecutive input channels: one tile for 4-bit weights, two
// consecutive tiles (64 inputs each) for 8-bit weights.
//
// 4-bit tile, lane l, dword j (0..3), element e (0..7):
//     k_local = 32*j + 8*(l >> 4) + e          nibble position in the dword = (e >> 1) + 4*(e & 1)
//   so that masking with 0x000F000F / 0x00F000F0 (and once more after >> 8) yields the element
//   pairs (0,1) (2,3) (4,5) (6,7) as packed halves, the order one MFMA operand register holds.
// 8-bit tile, lane l, dword d (0..3), byte b (0..3):
//     k_local = 32*(d >> 1) + 8*(l >> 4) + 4*(d & 1) + b      (within the tile's 64 inputs)
// Weights are stored unsigned: i4 xor 8, i8 xor 0x80, with the zero-point raised to match.
// Tiles are ordered [N/16][K/k_per_tile]; scales f16 and zero-points u8 as [N/16][groups][16].
// Groups of 32 or 64 inputs (4-bit weights only) divide a k-block in four or two: their parameters are
// stored [N/16][K/128][16][groups per k-block], so that a lane finds the scales of its channel for one
// k-block in one 4- or 8-byte load; group i of a k-block scales the inputs of dwords 4 i / gpb .. of a tile.
constexpr int kTileRows = 16;
constexpr int kTileBytes = 1024;
constexpr int kBlockK = 128;

struct Layout {
    bool tiled = false;
    int bits = 4;
    int64_t n_tiles = 0;        // N / 16
    int64_t k_blocks = 0;       // K / 128
    int64_t tiles_per_kblock = 1;
    int64_t groups = 0;         // K / G
    int64_t kblocks_per_group = 0;
    int groups_per_kblock = 1;  // 2 or 4 when G is 64 or 32
    bool zp_table = false;      // per-(n, group) zero-points stored as a table
    int zp_const = 0;           // zero-point used when there is no table (includes the unsigned offset)
    int zp_offset = 0;          // 8 for i4, 128 for i8, else 0
    size_t w_bytes = 0, scale_bytes = 0, zp_bytes = 0;
    // Gated-linear-unit epilogue (OVFCC_GLU_*, 0 = none).  In the tiled layout the 16-channel tiles of gate and up
    // projection alternate (tile 2 j = gate channels 16 j .., tile 2 j + 1 = up channels 16 j ..; bias likewise),
    // so that the wave that finishes a gate tile also holds the matching up tile.
    int glu = 0;
    bool glu_gate_second = false;
    int gemv_c = 0;         // k-blocks per wave of the matrix-vector kernel, fixed when the node's channel-major
                            // parameter tables are written (0: the node has none)
    bool dynquant = false;  // the node allows int8 activations (OVFCC_DYNQUANT_I8) where a kernel exists
    bool dynquant_grouped = false;  // ... quantised per group of 128 inputs rather than per token (4-bit nodes)
    bool dynquant_asym = false;     // ... as unsigned bytes with a zero-point per token (8-bit per-channel nodes)
    // element index of the scale / zero-point of channel r of tile nt for group g
    size_t param_index(int64_t nt, int64_t g, int r) const {
        if (groups_per_kblock == 1)
            return (size_t)(nt * groups + g) * kTileRows + r;
        const int64_t kb = g / groups_per_kblock, gi = g % groups_per_kblock;
        return ((size_t)(nt * k_blocks + kb) * kTileRows + r) * groups_per_kblock + gi;
    }
    // 16-channel block of the OpenVINO-order channel axis that tile nt holds
    int64_t source_tile(int64_t nt) const {
        if (!glu)
            return nt;
        const bool is_gate = (nt & 1) == 0;
        return (is_gate != glu_gate_second ? 0 : n_tiles / 2) + (nt >> 1);
    }
};

// The constants of one matched node (include/ovfcc_graph.h) in the form ovfcc_weights_create takes them.
struct FoldConstants {
    ovfcc_fc_desc desc{};
    const void* weights = nullptr;       // the Constant's own bytes, or `packed`
    std::vector<uint8_t> packed;         // a 4-bit expert slice that does not start and end on byte boundaries
    std::vector<uint16_t> scales;        // f16 bits, [N, K/G] ([K/G, N] for input-major constants)
    std::vector<uint8_t> zero_points;    // packed u4 / u8, or one element
    std::vector<uint16_t> bias;          // f16 bits, [N]
};
// data[i]: the bytes of node i where it is a Constant the fold names.  Element counts and types are checked
// against the descriptor; real-typed zero-points must hold integers in 0..255 (OVFCC_EUNSUPPORTED otherwise).
int fold_constants(const struct ::ovfcc_gnode* nodes, int n_nodes, const struct ::ovfcc_fold& f, const void* const* data,
                   FoldConstants& out);
int fold_expert_constants(const struct ::ovfcc_gnode* nodes, int n_nodes, const struct ::ovfcc_gather_fold& f, int expert,
                          const void* const* data, FoldConstants& out);

void set_error(const std::string& msg);
int fail(int code, const std::string& msg);

int validate_desc(const ovfcc_fc_desc* d);
// Fills the layout for a validated descriptor (tiled == false when the fallback applies).
Layout make_layout(const ovfcc_fc_desc& d);
int scalar_zero_point(const ovfcc_fc_desc& d, const void* zp);

// Input-major constants (OVFCC_W_INPUT_MAJOR) brought to the node's own order: W [K, N] -> [N, K], scales and
// zero-point tables [K/G, N] -> [N, K/G], each packed over its flattened index.  A scalar zero-point (one element)
// is copied.  Vectors that the descriptor does not use stay empty.
struct OutputMajorCopy {
    std::vector<uint8_t> w, zp;
    std::vector<uint16_t> scales;
};
void transpose_input_major(const ovfcc_fc_desc& d, const void* w, const void* scales, const void* zp,
                           OutputMajorCopy* out);

void repack_weights(const ovfcc_fc_desc& d, const Layout& L, const void* w, void* w_tiled);
void repack_params(const ovfcc_fc_desc& d, const Layout& L, const void* scales, const void* zp, void* scale_tiled,
                   void* zp_tiled);
void unrepack_weights(const ovfcc_fc_desc& d, const Layout& L, const void* w_tiled, void* w);
void unrepack_params(const ovfcc_fc_desc& d, const Layout& L, const void* scale_tiled, const void* zp_tiled,
                     void* scales, void* zp);

// ---- kernel launch parameters ------------------------------------------------------------------
struct FcDeviceArgs {
    const void* w;       // tiled or OpenVINO layout
    const void* scale;
    const void* zp;      // table, raw zp, or null
    const void* bias;    // f16 [N] or null
    const void* scale_cm = nullptr;  // channel-major copies [N/16][16][wave][slot] of scales and zero-point table,
    const void* zp_cm = nullptr;     // where the node has them (tiled 4-bit weights, groups of 128 inputs)
    const void* x;       // f16 [M,K]
    void* y;             // f16 or f32 [M,N]
    float* workspace;    // split-K partials
    unsigned* counters;  // split-K arrival counters, one per 16-channel tile, zero between launches
    int64_t M, N, K, group_size;
    int w_type, zp_type, zp_scalar;
    int out_f32;         // output_type f32 instead of f16
    int64_t N_out;       // row length of y: N, or N / 2 with a gated-linear-unit epilogue
    int gate_offset, up_offset;  // untiled layout with such an epilogue: first gate / up channel
    int tile_rows = 0;   // async prefill kernel: 64 or 128 (grouped runs: also 80, 96) forces the tile height, 0 leaves it to the planner
    // grouped prefill launch whose slices gather their rows themselves: row_map[item.reserved + r] is the row of item.x
    // that slice row r reads (negative: none); x_rows = rows of that matrix.  Null: slices read contiguous rows.
    const int* row_map = nullptr;
    int64_t x_rows = 0;
    bool want_async = false;  // take the all-asynchronous prefill kernel wherever it can run the node, also where
                              // smaller tiles would spread a small node further (a slice table in device memory
                              // has no other reader)
    Layout layout;
};

struct LaunchPlan {
    int kernel = OVFCC_KERNEL_AUTO;
    int split_k = 1;
    int kblocks_per_split = 0;
    int tile_m = 0, tile_n = 0;
    int tiles_per_group = 1;    // decode kernel: 16-channel tiles per workgroup
    bool x_in_lds = false;      // decode kernel: activations staged in LDS
    bool direct = false;        // prefill family: the kernels that feed weights from registers
    bool async_dma = false;     // ... and of those the one whose operands all travel by direct-to-LDS loads
    bool big = false;           // prefill family: the 4-bit kernel with 256 x 256 tiles (whole tiles, no split-K)
    bool batch = false;         // decode family: the small-batch kernel (waves own channel tiles)
    bool gemv = false;          // decode family: the matrix-vector kernel for M <= 4 (4-bit weights, G = 128)
    int gemv_c = 0;             // ... and its k-blocks per wave (2, 4 or 8)
    bool gemv16 = false;        // decode family: its 16-row sibling with stationary activations (5 <= M <= 48)
    bool gemv16_stream = false; // decode family: the 16-row kernel that streams its activations (long K, 5 <= M <= 16)
    int tiles_x = 0, tiles_y = 0;  // async prefill kernel: the tile grid; its launch is 1-D
    int full_tiles = 0;         // ... of which this many run unsplit (the rest in split_k parts each)
    unsigned grid[3] = {1, 1, 1};
    unsigned block = 256;
    unsigned dynamic_lds = 0;   // bytes of dynamic LDS (decode kernel: the cross-wave reduction buffer)
    size_t workspace_bytes = 0;
    size_t counter_count = 0;
    int n_cus = 0;  // routed grouped launches: the compute-unit count that the cut along K is chosen for on the device
    const char* name = "";
};

// Chooses kernel family and decomposition (force_kernel / force_split 0 = policy).
int plan_launch(const FcDeviceArgs& a, int force_kernel, int force_split, int n_cus, LaunchPlan* plan);
// OVFCC_* overrides of the process environment: cached at the first use, re-read by env_reload only.
// env_generation changes with every (re)read; plans cached under an older generation are stale.
int env_int(const char* name, int fallback);
void env_reload();
unsigned env_generation();
// Enqueues on `stream` (a hipStream_t passed as void*); returns a HIP error code (0 = success).
int launch_fc(const FcDeviceArgs& a, const LaunchPlan& plan, void* stream);
int launch_plain(const FcDeviceArgs& a, const LaunchPlan& plan, void* stream);
int launch_decode(const FcDeviceArgs& a, const LaunchPlan& plan, void* stream);
int launch_batch(const FcDeviceArgs& a, const LaunchPlan& plan, void* stream);
int launch_gemv(const FcDeviceArgs& a, const LaunchPlan& plan, void* stream);
int launch_gemv16(const FcDeviceArgs& a, const LaunchPlan& plan, void* stream);
int launch_gemv16_stream(const FcDeviceArgs& a, const LaunchPlan& plan, void* stream);
// dynamic LDS of the 16-row kernel with streamed activations
size_t gemv16s_lds_bytes(int waves, int tiles);
// dynamic LDS of the 16-row kernel: c k-blocks per wave, `waves` waves, one or two buffers of partial sums
size_t gemv16_lds_bytes(int c, int waves, int red_bufs);
// k-blocks per wave that the 16-row kernel runs a node with, given those of the node's channel-major tables and the
// number of parts K is cut in
int gemv16_kblocks_per_wave(int c_table, int split_k = 1);
// dynamic LDS of the matrix-vector kernel: c k-blocks per wave, m rows, `waves` waves per workgroup
size_t gemv_lds_bytes(int c, int m, int waves);
// [N/16][groups][16] scales f16 (and zero-points u8, or null) -> channel-major [N/16][16][groups]
int launch_gemv_params(const void* scale_tiled, const void* zp_tiled, void* scale_cm, void* zp_cm, int64_t n_tiles,
                       int64_t groups, int c_slots, void* stream);
// k-blocks per wave of the matrix-vector kernel for a node (0: the kernel does not fit it)
int gemv_kblocks_per_wave(const Layout& L, int n_cus);

// Problems of one grouped launch (passed in the kernel arguments: at most 4 KiB)
constexpr int kMaxGroupItems = 64;
struct BatchGroupItem {
    const void* w;
    const void* scale;
    const void* zp;
    const void* bias;
    const void* x;
    void* y;
    int M;  // rows of this problem (0 = skip), at most kDecodeMaxRows (decode) or kPrefillGroupRows (prefill)
    int reserved;  // with a row map (FcDeviceArgs::row_map): the map entry of the slice's first row; else 0
};
struct BatchGroupTable {
    BatchGroupItem item[kMaxGroupItems];
};
int launch_batch_grouped(const BatchGroupTable& tab, int n_items, const FcDeviceArgs& a, const LaunchPlan& plan,
                         void* stream);
// Same table, items of at most tile_m rows, 4-bit async prefill kernel; plan is that of one node of tile_m * n_items rows.
#ifdef __HIPCC__
#define OVFCC_HOST_DEVICE __host__ __device__
#else
#define OVFCC_HOST_DEVICE
#endif
// What a grouped launch whose slice count is known only on the device reads there: the routing kernel counts the
// slices and cuts K by the rule below, the host sizes grid, workspace and counters for the worst slice count.
struct RoutedHeader {
    int tiles_y;       // slices in use
    int split_k;       // parts along K of the tiles that are split (1: whole tiles only)
    int kb_per_split;  // k-blocks per part
    int grid;          // workgroups with work: full_tiles + (tiles_x * tiles_y - full_tiles) * split_k
    int full_tiles;    // tiles that one workgroup each computes whole; the rest are split
    int pad[3];        // the slice table follows the header: keeps it 8-byte aligned
};
// K is split while the tiles alone leave compute units idle and every part keeps at least eight k-blocks (the
// planner's rule for the register-fed prefill kernels).  With more tiles than compute units, the tiles of a last
// round that would fill at most half of them are split instead, so that the launch ends with a full round of shorter
// workgroups rather than a half-empty round of whole tiles (tile_work, device_common.h).
OVFCC_HOST_DEVICE inline RoutedHeader routed_header(int tiles_x, int slices, int kb_total, int n_cus) {
    const long long tiles = (long long)tiles_x * slices;
    int split = 1;
    while (split < 8 && tiles * split * 2 <= n_cus && kb_total / (split * 2) >= 8)
        split *= 2;
    long long full = split == 1 ? tiles : 0;
    const long long rest = tiles % n_cus;
    if (split == 1 && tiles > n_cus && rest != 0) {
        while (split < 8 && rest * split * 2 <= n_cus && kb_total / (split * 2) >= 8)
            split *= 2;
        if (split > 1)
            full = tiles - rest;
    }
    const int per = (kb_total + split - 1) / split;
    split = (kb_total + per - 1) / per;
    RoutedHeader h;
    h.tiles_y = slices, h.split_k = split, h.kb_per_split = per, h.full_tiles = (int)full;
    h.grid = (int)(full + (tiles - full) * split);
    h.pad[0] = h.pad[1] = h.pad[2] = 0;
    return h;
}
// f32 tiles that the split parts of such a launch park in the workspace
OVFCC_HOST_DEVICE inline long long routed_parked_tiles(const RoutedHeader& h, int tiles_x) {
    return h.split_k > 1 ? ((long long)tiles_x * h.tiles_y - h.full_tiles) * h.split_k : 0;
}
// Slice height (64, 80, 96 or 128 rows) of a grouped prefill launch over items of these row counts (plan.cpp).
int rows_cap_for(const int64_t* rows, int n, bool mid_ok);
int launch_prefill_async_grouped(const BatchGroupTable& tab, int n_items, const FcDeviceArgs& a, const LaunchPlan& plan,
                                 void* stream, const BatchGroupItem* dev_tab = nullptr,
                                 const RoutedHeader* dev_hdr = nullptr);
// Routing of a mixture-of-experts layer on the device: buckets the R = M * top_k (row, selection) pairs of
// indices [M, top_k] (device memory) by expert, ascending inside a bucket, and writes the row maps and the slice
// table that the gather kernel and the grouped launch read -- first[slot] = row of A that bucket slot `slot`
// reads (m, or i * M + m with one batch of A per selection); second[slot] = i * M + m (inverse == 0) or
// second[m * top_k + i] = slot, -1 for an index outside [0, n_experts) (inverse != 0); table[.] = the experts' rows
// cut into equal slices of at most `cap` rows, n_slices_max = ceil(R / cap) + n_experts entries, unused ones with
// M = 0; *header = routed_header(tiles_x, slices in use, kb_total, n_cus).  x_base / y_base: where bucket slot 0's
// gathered row and result row lie.
struct ExpertPointers {
    const void* w[kMaxGroupItems];
    const void* scale[kMaxGroupItems];
    const void* zp[kMaxGroupItems];
    const void* bias[kMaxGroupItems];
};
// A second slice table from the same buckets, written by the same launch (the down projection of an expert block,
// whose rows are the bucket slots themselves): its own expert pointers, buffers, strides and header.  table == null:
// none.  At most kMaxSecondTableItems experts, so that both pointer sets fit the kernel arguments.
constexpr int kMaxSecondTableItems = 32;
struct SecondTable {
    const void* w[kMaxSecondTableItems];
    const void* scale[kMaxSecondTableItems];
    const void* zp[kMaxSecondTableItems];
    const void* bias[kMaxSecondTableItems];
    const void* x_base;
    size_t x_row_bytes;
    void* y_base;
    size_t y_row_bytes;
    BatchGroupItem* table;
    RoutedHeader* header;
    int tiles_x, kb_total;
};
// unrouted_y: the final result [top_k, M, row] of a GatherMatmul; the rows of pairs whose index names no expert are
// zeroed there (no bucket owns them, so nothing else writes them).
// x_mapped != 0: the slices leave the gather to the grouped launch -- every entry gets x = x_base and reserved = its
// first bucket slot, and the launch reads its rows through `first`.
int launch_moe_route(const int* indices_dev, int64_t M, int top_k, int n_experts, int a_batches, int inverse, int cap,
                     int x_mapped, const ExpertPointers& experts, const void* x_base, size_t x_row_bytes, void* y_base,
                     size_t y_row_bytes, int* first, int* second, BatchGroupItem* table, int n_slices_max,
                     RoutedHeader* header, int tiles_x, int kb_total, int n_cus, void* stream,
                     const SecondTable* second_table = nullptr, void* unrouted_y = nullptr, size_t unrouted_row_bytes = 0);
// GroupedMatMul with offsets in device memory: table[0 .. n_slices_max) and *header as for launch_moe_route, from
// cumulative row ends over rows that are already contiguous per group; rows of y from the last offset on are
// zeroed; tail: one int of scratch.
int launch_offsets_table(const int* offsets_dev, int n_groups, int64_t rows, int cap, const ExpertPointers& groups,
                         const void* x_base, size_t x_row_bytes, void* y_base, size_t y_row_bytes,
                         BatchGroupItem* table, int n_slices_max, RoutedHeader* header, int* tail, int tiles_x,
                         int kb_total, int n_cus, void* stream);
// The gated MLP as one launch (kernel_mlp.hip): gate / up node g with its gated linear unit, down node d, M <= 4.
// mid: [M, d.K] f16 scratch; sync: mlp_sync_bytes(grid) bytes that are zero between launches; error: a host-visible
// word the kernel sets when its wait for the other workgroups ran out after spin_limit polls.
size_t mlp_sync_bytes(int grid);
bool mlp_fused_applies(const Layout& g, const Layout& d, int64_t M, int grid);
int launch_mlp(const FcDeviceArgs& g, const FcDeviceArgs& d, void* mid, unsigned* sync, unsigned* error, int grid,
               int n_cus, unsigned spin_limit, void* stream);
int launch_prefill(const FcDeviceArgs& a, const LaunchPlan& plan, void* stream);
int launch_prefill_wide(const FcDeviceArgs& a, const LaunchPlan& plan, void* stream);
int launch_prefill_direct(const FcDeviceArgs& a, const LaunchPlan& plan, void* stream);
int launch_prefill_async(const FcDeviceArgs& a, const LaunchPlan& plan, void* stream);
int launch_prefill_big(const FcDeviceArgs& a, const LaunchPlan& plan, void* stream);
// Per-row int8 quantisation of x [M, K] f16 (K % 128 == 0): xq [M, K] in the weight tiles' input order, one
// inverse scale and one sum of quantised values per row.
int launch_dynquant(const void* x, void* xq, float* inv_scale, int* qsum, int64_t M, int64_t K, void* stream);
// The same for tiled 4-bit weights with one group per 128 inputs (W4A8): activations quantised per token
// (inv [M]) or per row and k-block (grouped; inv holds dynquant_w4_scale_floats floats), the integer kernel over
// them, and whether that kernel can run a node.
size_t dynquant_w4_scale_floats(int64_t M, int64_t K, bool grouped);
int launch_dynquant_w4(const void* x, void* xq, float* inv, int64_t M, int64_t K, bool grouped, void* stream);
bool prefill_i8w4_applies(const Layout& L, int64_t N, int zp_type);
int launch_prefill_i8w4(const FcDeviceArgs& a, const void* xq, const float* inv, bool grouped, void* stream);
// The asymmetric form: unsigned bytes with a zero-point per row, stored minus 128 (xq, za) for the integer kernel's
// signed operands; and the per-channel sums cw[n] = sum_k (w[n, k] - zp[n]) that form needs, from a node's tiled
// 8-bit weights (channels in tiled order).  sum_k (q - za)(w - zp) has to fit 32 bits: K <= kI8AsymMaxK.
constexpr int64_t kI8AsymMaxK = 32768;
int launch_dynquant_asym(const void* x, void* xq, float* inv_scale, int* qsum, int* za, int64_t M, int64_t K,
                         void* stream);
int launch_i8_colsum(const void* w_tiled, const void* zp_tiled, int zp_const, int* cw, int64_t n_tiles, int64_t k_blocks,
                     void* stream);
// Integer prefill kernel over launch_dynquant's outputs (za and cw null) or launch_dynquant_asym's: tiled 8-bit
// weights, one group per channel, N % 256 == 0.
int launch_prefill_i8(const FcDeviceArgs& a, const void* xq, const float* inv_scale, const int* qsum, const int* za,
                      const int* cw, void* stream);
// dst[r] = src[src_row[r]] (dst_row null) or dst[dst_row[r]] = src[r] (src_row null), rows of row_bytes % 16 == 0 bytes;
// the caller guarantees that every index is a row of the buffer it addresses
int launch_rows(void* dst, const void* src, const int* src_row, const int* dst_row, int rows, int row_bytes,
                void* stream);
// y[m, :] = sum_j routing[m, j] * d[pos[m * top_k + j], :], rows of H (a multiple of 4) channels; d f16 or f32
int launch_moe_combine(void* y, const void* d, const void* routing, const int* pos, int rows, int top_k, int H,
                       int d_f32, int out_f32, void* stream);

// Scratch array of the entry point that allocates nothing: arrival counters, then split-K partial tiles
constexpr size_t kStaticCounterBytes = (size_t)64 << 10;
constexpr size_t kStaticWorkspaceBytes = (size_t)32 << 20;
int static_scratch_setup(int device);
void* static_scratch_ptr(int device);
int launch_zero_u32(unsigned* p, size_t n, void* stream);

constexpr int kDecodeMaxRows = 48;                       // rows one decode-family launch covers
constexpr int kPrefillGroupRows = 128;                   // rows per slice of a grouped prefill launch (one tile)
constexpr int kChunkedMinPrefillRows = 48;                // ... unless, above this, the async prefill kernel fills the chip
constexpr int kChunkedMaxRows = 128;                     // up to here M is cut into decode launches
constexpr int kPrefillTileM = 128, kPrefillTileN = 128;  // square prefill kernel
constexpr int kPrefillWideN = 256;                         // wide prefill kernel: 128 x 256

}  // namespace ovfcc
