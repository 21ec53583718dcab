// Internal declarations shared by the HIP translation units of libatenia_moe_hip.so.
// gfx950 (MI355X, wave64) only.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "select_wave.h"

namespace atenia_moe {

// ---- limits ------------------------------------------------------------------------------
constexpr int kMaxRouterRows = 256;  // E (+1 for the shared-expert gate row) handled per block
constexpr int kPermuteBlock = 1024;  // pairs per permute block
constexpr int kTileM = 256;          // token rows per tile of the tiled expert kernels

// ---- weight storage in HBM ---------------------------------------------------------------
// bf16 and int8 expert matrices W[N, K] ("[out, in]", K contiguous in the reference layout)
// are stored as 1 KiB "B blocks": block (nb, kb) covers rows 16*nb .. 16*nb+15 and KB
// consecutive k (KB = 32 for bf16, 64 for int8).  Inside a block, lane l of a wavefront
// owns 16 bytes: row 16*nb + (l & 15), k = KB*kb + (KB/4)*(l >> 4) .. + KB/4 - 1.  That is
// the register layout of the B operand of v_mfma_f32_16x16x32_bf16, so a wave streams a row
// strip with one fully contiguous 1 KiB load per block.  Blocks are ordered [nb][kb].
// N is padded to a multiple of 16 and K to a multiple of KB with zeros.
constexpr int kBlockBytes = 1024;
constexpr int kKbBf16 = 32;
constexpr int kKbInt8 = 64;
// f32 expert matrices use the same blocks with KB = 16: a lane slot is 4 consecutive k of one row
// (the chunk a lane of v_mfma_f64_16x16x4_f64 feeds one instruction at a time from).
constexpr int kKbF32 = 16;

static inline int round_up(int v, int m) { return (v + m - 1) / m * m; }

// A set of row groups (one group per expert) for the expert kernels.  All device pointers.
struct GroupDesc {
  const int32_t* offsets;   // [G+1] first row of each group in grouped order
  const int32_t* active;    // [<=G] ids of the groups that have rows, ascending
  const int32_t* n_active;  // [1]
  const int32_t* perm;      // [rows] pair id (token*pair_div + slot) of each grouped row
  int pair_div;             // token = pair id / pair_div
  // One-token launches whose router also wrote the grouping: the token's experts in ascending
  // order, [pair_div] entries; group j is then expert idx1[j] with the single row j = pair j.
  // A kernel that sees it reads one value where the lists above cost three dependent loads.
  // Null otherwise.
  const int32_t* idx1;
};

// One expert projection family as stored on the device.
struct WeightSet {
  const void* w;            // blocks (see above)
  const float* scale;       // int8: per output row, [G, N] (unpadded N stride = n_rows);
                            // per-group int8: [G][n_kgroups][n_pad] (see group_blocks)
  int group_blocks;         // per-group int8: 64-k blocks per scale group (0 = one scale per row)
  int n_kgroups;            // per-group int8: scale groups along K
  int64_t expert_stride;    // elements (f32) or bytes (blocked) between experts
  int n_rows;               // N (unpadded)
  int n_pad;                // padded N
  int k_cols;               // K (unpadded)
  int k_pad;                // padded K
};

// ---- stage launchers (each returns a hipError_t from the launch) --------------------------
struct PermuteArgs;
struct RouterArgs {
  const void* x;        // [T, d] f32 or bf16
  int x_is_bf16;
  int T, d, E, k, renorm;
  const float* w_router;     // [E, d]
  int w_fits_bf16;           // every value of w_router and shared_gate is exactly a bf16 value
  const int32_t* w_lsb_min;  // [E + 1] lowest last-bit exponent of each router row / the gate (or null)
  // bf16 copy of [w_router ; shared_gate] in chunk-major order [ceil(d / 32) * 4][w_rows_pad][8]
  // (rows past the last one and columns past d are zeros) and the squared norm of each of its
  // rows; both null unless w_fits_bf16 and d % 8 == 0.  What the matrix-core router reads.
  const uint16_t* w_t8;
  int w_rows_pad;         // multiple of 16
  const double* w_norm2;  // [w_rows_pad]
  const float* router_bias;  // [E] or null
  const float* shared_gate;  // [d] or null
  int32_t* idx;              // [T, k]
  float* w;                  // [T, k]
  float* sgate;              // [T] (written when shared_gate != null)
  uint16_t* xb;              // [T, d_pad] bf16 copy of x (null = do not write)
  int d_pad;
  int32_t* status;           // [2]: code, (token << 10 | expert)
  int token_kernel_max_tokens;  // batches up to this size use the one-workgroup-per-token kernel
  // When T == 1 and the per-token kernel runs, it also writes the expert grouping (the
  // result of kernel 2 for a single token is known as soon as the top-k is), saving a launch.
  const struct PermuteArgs* fuse_permute;  // null = do not fuse
  // non-null: write the raw logits [T, E] here and leave idx / w alone (another kernel routes)
  float* logits_out;
  // scratch [T, E] the launcher may use to split the work of few tokens over more workgroups
  // (null = none)
  float* logits_tmp;
  // T == 1 only: when the launcher spreads the rows over workgroups (logits to logits_tmp), it
  // may leave the selection and the grouping to the caller's next launch instead of a small
  // launch of its own; *fused_permute is then 2.
  int defer_select;
};
// *fused_permute is set to 1 when the launch also produced the expert grouping, to 2 when the
// logits are in logits_tmp and the caller's next launch has to route the token (defer_select).
hipError_t launch_router(const RouterArgs& a, hipStream_t s, int* fused_permute);

// DeepSeek-V3 routing from raw logits (src/moe/v3_router.rs:206-309).
struct V3RouteArgs {
  const float* logits;  // [T, E]
  const float* bias;    // [E] e_score_correction_bias (selection only)
  int T, E, k, n_group, topk_group, norm_topk_prob;
  double routed_scaling_factor;
  int32_t* idx;         // [T, k] ascending
  float* w;             // [T, k]
  int32_t* status;      // [2]: code, (token << 10 | expert)
};
hipError_t launch_v3_route(const V3RouteArgs& a, hipStream_t s);

struct PermuteArgs {
  const int32_t* idx;  // [P] expert of each pair, P = T*k
  int T, k, E;
  int32_t* counts;     // [E]
  int32_t* offsets;    // [E+1]
  int32_t* perm;       // [P]
  int32_t* inv;        // [P] position of each pair in grouped order
  int32_t* active;     // [E]
  int32_t* n_active;   // [1]
  int32_t* blk_counts; // [nblk, E] scratch (multi-block path)
  int32_t* shared_offsets;  // [2] = {0, T} (may be null)
  // Row tiles of kTileM rows for the tiled expert kernels: expert and first row (relative to
  // the expert's group) of each tile, experts ascending; may be null.
  int32_t* tile_group;      // [<= ceil(P / kTileM) + E]
  int32_t* tile_m0;
  int32_t* n_tiles;         // [1]
  int32_t* shared_n_tiles;  // [1] = ceil(T / kTileM) (may be null)
  // Tiles of uneven height (max_tile_groups == 9, see permute.hip): rows of each tile and its
  // index inside its expert | (tiles of the expert << 16); may be null when max_tile_groups <= 8.
  int32_t* tile_rows;
  int32_t* tile_li;
  int max_tile_groups;      // 0 / 8: 256-row tiles; 9: tiles of up to 288 rows
};
hipError_t launch_permute(const PermuteArgs& a, hipStream_t s, int* n_launches);

struct FfnArgs {
  int wdtype;          // ATENIA_MOE_WEIGHT_*
  int f32_accumulate;  // f32 weights only: the projections accumulate in f32 (Strict / Fast)
  GroupDesc g;
  int n_groups_max;    // upper bound of *n_active (grid sizing)
  int rows_max;        // upper bound of rows in any one group (grid sizing)
  // gate/up phase: x -> h
  WeightSet gate, up;
  const void* x;       // bf16 [T, x_stride] (blocked weights) or f32 [T, x_stride]
  int x_stride;
  void* h;             // bf16 [rows, h_stride] or f32
  int h_stride;
  // down phase: h -> y
  WeightSet down;
  float* y;            // f32 [rows, y_stride] indexed by PAIR id (token*pair_div+slot)
  int y_stride;
  // bf16 pipelined / two-workgroup tiled down kernels only: y (and its partial buffers) holds
  // bf16 values, rounded to nearest even, in the first half of the same allocation -- half the
  // bytes written here and read back by the combine.  Element strides stay as they are.
  int y_bf16;
  // Tiled down phase only: the tiles of a partly filled last round may be cut into up to
  // y_parts k ranges, range i writing its partial sums to y + i * y_part_stride; part_flags
  // [pairs, ceil(d / 256)] receives the number of buffers written per (pair, column tile) and
  // the combine adds those up in order.  y_parts <= 1 or part_flags == null: never split.
  int y_parts;
  size_t y_part_stride;  // elements
  uint8_t* part_flags;
  int n_cus;             // compute units of the device
  // Streaming family only: the mid-batch kernel (token rows shared through LDS, up to 128 rows
  // of an expert per pass) instead of the register-resident one; needs ffn_mid_supported().
  int use_mid;
  // tiled kernels only
  int use_tiled;
  // Tiled bf16 kernels: the form that runs two workgroups per compute unit (128-row slices of
  // the 256-row tiles; for short K).  Needs tiles of at most 256 rows: tile_rows / tile_li null.
  int use_duo;
  // The row-tile list holds tiles of up to nine 32-row groups (PermuteArgs::max_tile_groups == 9);
  // only the bf16 pipelined kernel reads such a list.
  int tall_tiles;
  const int32_t* tile_group;
  const int32_t* tile_m0;
  const int32_t* n_tiles;
  const int32_t* tile_rows;  // null: every tile is min(kTileM, rows left) high
  const int32_t* tile_li;    // null: tile i of an expert starts at row i * kTileM
  int max_row_tiles;   // upper bound of *n_tiles (grid sizing)
  // Single-token decode (see launch_ffn_down_decode1): routing weights [k], layer output [d]
  // and optional residual [d] of the one token; the down launch then also does the combine.
  const float* fuse_w;
  float* fuse_out;
  const float* fuse_residual;
  const float* fuse_sgate;  // [1] sigmoid gate of the shared expert, or null (weight 1)
  int fuse_k;
  // Single token whose routing the router launch left undone (RouterArgs::defer_select): the
  // gate/up launch routes it from the logits; sel.logits == null otherwise.
  InlineSelect sel;
};
bool tiled_supported(const WeightSet& w, int wdtype);
// Whether these weights (one projection family) can go through the mid-batch streaming kernel.
bool ffn_mid_supported(const WeightSet& w, int wdtype);
// True when the tiled down launch for these weights can split the k range of tail tiles.
bool tiled_down_splits_tail(const WeightSet& down, int wdtype);
hipError_t launch_ffn_up_tiled(const FfnArgs& a, hipStream_t s);
// Gate/up of the routed experts and of a shared expert as one launch of the bf16 pipelined kernel
// (routed tiles first): both argument sets must ask for that kernel (tiled_up_pair_supported).
bool tiled_up_pair_supported(const FfnArgs& a, const FfnArgs& shared);
hipError_t launch_ffn_up_tiled_pair(const FfnArgs& a, const FfnArgs& shared, hipStream_t s);
// The same for the down phase, `first`'s tiles in front (the caller puts the longer K there);
// both sets must store y in the same element type.
bool tiled_down_pair_supported(const FfnArgs& first, const FfnArgs& second);
hipError_t launch_ffn_down_tiled_pair(const FfnArgs& first, const FfnArgs& second, hipStream_t s);
hipError_t launch_ffn_down_tiled(const FfnArgs& a, hipStream_t s);
// `shared` (may be null): the shared expert's arguments; when ffn_stream_fuses_shared(a, *shared,
// phase) holds, its work is done by the same launch and the caller must not launch it again.
hipError_t launch_ffn_up(const FfnArgs& a, hipStream_t s, const FfnArgs* shared = nullptr);
hipError_t launch_ffn_down(const FfnArgs& a, hipStream_t s, const FfnArgs* shared = nullptr);
bool ffn_stream_fuses_shared(const FfnArgs& a, const FfnArgs& shared, bool down_phase);
// One token, at most two experts per token, blocked (bf16 / int8) weights: the down projection
// of all the token's experts and the weighted combine in one launch.
bool ffn_down_decode1_supported(int T, const FfnArgs& a, int k, bool tiled, const FfnArgs* shared);
hipError_t launch_ffn_down_decode1(const FfnArgs& a, hipStream_t s, const FfnArgs* shared);

struct CombineArgs {
  int T, k, d;
  const float* w;        // [T, k]
  const float* y;        // [T*k, y_stride] pair order
  int y_stride;
  // partial buffers (see FfnArgs): part_flags[pair * flag_cols + c / 256] of them are added up
  // in order before weighting; null = one buffer everywhere
  const uint8_t* part_flags;
  int flag_cols;
  size_t y_part_stride;  // elements
  int y_bf16;            // y and its partial buffers hold bf16 (see FfnArgs::y_bf16)
  const float* y_shared; // [T, y_stride] or null
  int ys_bf16;           // the same for y_shared
  const float* sgate;    // [T] or null (scale 1)
  const float* residual; // [T, d] or null: out = residual + combine (one more f32 add); may be `out`
  float* out;            // [T, d]
};
hipError_t launch_combine(const CombineArgs& a, hipStream_t s);

struct NormArgs {
  const float* x;      // [T, d]
  const float* gamma;  // [d]
  float eps;
  int policy;          // ATENIA_MOE_NORM_*
  int T, d;
  float* y;            // [T, d]
};
hipError_t launch_rmsnorm_gamma(const NormArgs& a, hipStream_t s);

// Rewrites a row-major [n_rows, k_cols] matrix (bf16 bits or int8) into B blocks.
hipError_t launch_repack_blocks(const void* src, void* dst, int n_rows, int k_cols, int n_pad,
                                int k_pad, int elem_bytes, hipStream_t s);
hipError_t launch_fill_i32(int32_t* p, int n, int32_t v, int32_t step, hipStream_t s);
// Per-group int8 blocks + scales [G][n_kgroups][n_pad] -> bf16 blocks of the same matrix:
// value = bf16_rne((float)q * scale[row, k group]).
hipError_t launch_dequant_group_blocks(const void* q_blocks, const float* scales, void* bf16_blocks,
                                       int G, int n_pad, int k_pad, int group_blocks, int n_kgroups,
                                       hipStream_t s);

}  // namespace atenia_moe
