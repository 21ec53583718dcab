// Shared by the MFMA-tiled expert kernels (ffn_tiled.hip, ffn_tiled_duo.hip): operand types,
// the launch parameters, which tile a workgroup computes, and the global -> LDS load helper.
// gfx950 only.  Everything here sits in an unnamed namespace: each translation unit gets its own copy.
#pragma once

#include <type_traits>

#include "moe_internal.h"

namespace atenia_moe {

struct TiledParams {
  const uint4* wa;      // gate (up phase) or down blocks
  const uint4* wb;      // up blocks
  const float* sa;      // int8 row scales [G, n_rows]
  const float* sb;
  int64_t w_stride_u4;
  int n_rows;           // unpadded N
  int n_blocks;         // n_pad / 16
  int nkb;              // K blocks per strip (32 k each for bf16, 64 k for int8)
  int k_pad;
  const uint16_t* a;    // bf16 rows
  int a_stride;
  void* out;
  int out_stride;
  int out_bf16;         // down phase: y is stored as bf16 (nearest even) instead of f32
  GroupDesc g;
  const int32_t* tile_group;  // [n_tiles] expert of each row tile
  const int32_t* tile_m0;     // [n_tiles] first row (relative to the group) of each row tile
  const int32_t* n_tiles;     // [1]
  const int32_t* tile_rows;   // [n_tiles] rows of each tile, or null: min(TM, rows left)
  const int32_t* tile_li;     // [n_tiles] index inside the expert | (its tiles << 16), or null
  int n_col_tiles;
  // k split of the tail tiles (pipelined down kernels; max_parts <= 1: off).  Workgroup ids
  // below wg_upper are the tiles themselves, ids from wg_upper on the extra k ranges of the
  // tiles in the last, partly filled round over the n_cus compute units.
  int max_parts;
  int wg_upper;
  int n_cus;
  size_t out_part_stride;     // elements between the partial output buffers
  uint8_t* part_flags;        // [pairs, n_col_tiles] partial buffers written per (row, column tile)
};

// The form of the bf16 tiled kernels that runs two workgroups per compute unit (ffn_tiled_duo.hip).
bool tiled_duo_supported(const TiledParams& p);
hipError_t launch_tiled_duo_up(const TiledParams& p, int max_row_tiles, hipStream_t s);
hipError_t launch_tiled_duo_down(const TiledParams& p, int max_row_tiles, hipStream_t s);

namespace {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;

constexpr int kThreads = 256;
constexpr int TM = kTileM;   // 256 token rows
constexpr int TNB = 256;     // B rows per tile (gate/up: 128 + 128)
constexpr int TK = 64;       // k per LDS stage
constexpr int kChunk = 1024; // bytes
constexpr int kAStage = (TM / 16) * (TK / 32) * kChunk;   // 32 KiB
constexpr int kBStage = (TNB / 16) * (TK / 32) * kChunk;  // 32 KiB
constexpr int kStage = kAStage + kBStage;
constexpr int kLdsBytes = 2 * kStage;                     // 128 KiB


__device__ inline uint16_t bf16_rne(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

// Two f32 -> two bf16 (round to nearest even) in one v_cvt_pk_bf16_f32; low half = a.
typedef __attribute__((ext_vector_type(2))) float f32x2_t;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
__device__ inline uint32_t bf16_rne_pair(float a, float b) {
  f32x2_t v = {a, b};
  bf16x2_t h = __builtin_convertvector(v, bf16x2_t);
  return *(uint32_t*)&h;
}

// silu(g) * u with the hardware exp2 / rcp (1 ulp each; the result is rounded to bf16 next).
__device__ inline float swiglu_fast(float g, float u) {
  const float t = __builtin_amdgcn_exp2f(g * -1.4426950408889634f);
  return g * __builtin_amdgcn_rcpf(1.f + t) * u;
}

__device__ inline uint32_t pack_i8_pair(uint32_t w, int sh) {
  float f0 = (float)(int8_t)((w >> sh) & 0xff);
  float f1 = (float)(int8_t)((w >> (sh + 8)) & 0xff);
  // |q| <= 128 is exact in bf16, so dropping the low 16 bits loses nothing: one byte permute
  // takes the high halves of both floats (bytes 2, 3 of f0 below bytes 2, 3 of f1).
  return __builtin_amdgcn_perm(__float_as_uint(f1), __float_as_uint(f0), 0x07060302u);
}
__device__ inline void widen_i8x16(uint4 q, uint4& lo, uint4& hi) {
  lo.x = pack_i8_pair(q.x, 0);
  lo.y = pack_i8_pair(q.x, 16);
  lo.z = pack_i8_pair(q.y, 0);
  lo.w = pack_i8_pair(q.y, 16);
  hi.x = pack_i8_pair(q.z, 0);
  hi.y = pack_i8_pair(q.z, 16);
  hi.z = pack_i8_pair(q.w, 0);
  hi.w = pack_i8_pair(q.w, 16);
}

__device__ inline f32x4 mfma(uint4 a, uint4 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(*(bf16x8*)&a, *(bf16x8*)&b, c, 0, 0, 0);
}

// Which (row tile, column tile) a workgroup computes.
//
// XCD-aware order: hardware deals consecutive workgroup ids round-robin to the 8 XCDs, each
// with its own L2, so XCD x is given the contiguous run [x*per_xcd, (x+1)*per_xcd) of the
// logical tile order.  In that order an expert's tiles are contiguous and walked in patches of
// (all row tiles of the expert) x (8 column tiles): the ~32 workgroups an XCD runs at a time
// share ~4 activation tiles and 8 weight tiles instead of streaming 64 different ones.
constexpr int kColGroup = 8;
__device__ inline bool tile_of_workgroup(const TiledParams& p, int wid, int& rt, int& ct) {
  const int n_row_tiles = *p.n_tiles;
  const int nct = p.n_col_tiles;
  const int total = n_row_tiles * nct;
  const int per_xcd = (total + 7) / 8;
  const int slot = wid / 8;
  const int logical = (wid % 8) * per_xcd + slot;
  if (slot >= per_xcd || logical >= total) return false;
  // Row tiles are sorted by expert, so the expert owning this logical id is the expert of
  // row tile logical / nct; that tile's m0 tells where the expert's tiles start.
  const int rt_any = logical / nct;
  int first, nt;
  if (p.tile_li) {  // tiles of uneven height: the list says where the expert's tiles start
    const int li = p.tile_li[rt_any];
    first = rt_any - (li & 0xffff);
    nt = li >> 16;
  } else {
    const int e = p.tile_group[rt_any];
    const int cnt = p.g.offsets[e + 1] - p.g.offsets[e];
    first = rt_any - p.tile_m0[rt_any] / TM;
    nt = (cnt + TM - 1) / TM;
  }
  int local = logical - first * nct;
  const int full = nct / kColGroup;
  const int patch = nt * kColGroup;
  int cg, gw;
  if (local < full * patch) {
    cg = local / patch;
    local -= cg * patch;
    gw = kColGroup;
  } else {
    local -= full * patch;
    cg = full;
    gw = nct - full * kColGroup;
  }
  const int rl = local / gw;
  rt = first + rl;
  ct = cg * kColGroup + (local - rl * gw);
  return true;
}

// The same order for kernels whose workgroups take a slice of NS-th of a row tile's height (rows
// sub * TM / NS ..): every row tile counts as NS consecutive ones, so the slices of a tile and the
// column tiles of a patch stay neighbours in an XCD's run.
template <int NS>
__device__ inline bool tile_of_workgroup_sub(const TiledParams& p, int wid, int& rt, int& sub, int& ct) {
  const int n_row_tiles = *p.n_tiles * NS;
  const int nct = p.n_col_tiles;
  const int total = n_row_tiles * nct;
  const int per_xcd = (total + 7) / 8;
  const int slot = wid / 8;
  const int logical = (wid % 8) * per_xcd + slot;
  if (slot >= per_xcd || logical >= total) return false;
  const int rt_any = logical / nct / NS;
  int first, nt;
  if (p.tile_li) {
    const int li = p.tile_li[rt_any];
    first = rt_any - (li & 0xffff);
    nt = li >> 16;
  } else {
    const int e = p.tile_group[rt_any];
    const int cnt = p.g.offsets[e + 1] - p.g.offsets[e];
    first = rt_any - p.tile_m0[rt_any] / TM;
    nt = (cnt + TM - 1) / TM;
  }
  first *= NS;
  nt *= NS;
  int local = logical - first * nct;
  const int full = nct / kColGroup;
  const int patch = nt * kColGroup;
  int cg, gw;
  if (local < full * patch) {
    cg = local / patch;
    local -= cg * patch;
    gw = kColGroup;
  } else {
    local -= full * patch;
    cg = full;
    gw = nct - full * kColGroup;
  }
  const int rl = local / gw;
  const int v = first + rl;
  rt = v / NS;
  sub = v - rt * NS;
  ct = cg * kColGroup + (local - rl * gw);
  return true;
}

// Tail split of the down phase.  With one workgroup per CU at a time, tiles run in rounds of
// n_cus; when the last round is at most half full, each of its tiles is cut into S k ranges
// (S <= max_parts) so that the round fills the chip and lasts 1/S as long.  Range 0 is
// computed by the tile's own workgroup, ranges 1..S-1 by workgroups with ids from wg_upper on;
// range i writes its partial sums to buffer i, and range 0 records S per (row, column tile) so
// that the combine adds up exactly the buffers that were written.  Sets wid (the tile's
// workgroup id for tile_of_workgroup), S and part; false = nothing to do.
// bid: the workgroup's id within its launch (blockIdx.x, or the id inside its own part of a launch
// that carries two parameter sets).
__device__ inline bool split_of_workgroup(const TiledParams& p, int bid, int n_stages, int& wid, int& S,
                                          int& part) {
  wid = bid;
  S = 1;
  part = 0;
  if (p.max_parts <= 1) return true;
  const int total = *p.n_tiles * p.n_col_tiles;
  const int per_xcd = (total + 7) / 8;
  const int full_slots = (total / p.n_cus) * (p.n_cus / 8);  // slots per XCD in the full rounds
  const int tail = 8 * (per_xcd - full_slots);               // tile slots of the last round
  int s_tail = 1;
  if (tail > 0 && 2 * tail <= p.n_cus) s_tail = min(min(p.max_parts, p.n_cus / tail), n_stages / 2);
  if (s_tail < 1) s_tail = 1;
  if (bid >= p.wg_upper) {
    const int x = bid - p.wg_upper;
    if (s_tail == 1 || x >= tail * (s_tail - 1)) return false;
    part = 1 + x / tail;
    const int j = x - (part - 1) * tail;
    wid = (full_slots + j / 8) * 8 + (j & 7);
    S = s_tail;
    return true;
  }
  if (wid / 8 >= full_slots) S = s_tail;
  return true;
}

typedef __attribute__((address_space(3))) void* lptr_t;

// One wave-wide 16-byte-per-lane load from global memory straight into LDS: lane l's bytes
// land at lds_addr + 16*l.  Written as inline assembly so that the compiler's wait-count
// insertion does not tie later LDS reads to these loads (it would drain all stages); the
// kernel waits for exactly the stage it needs with an explicit s_waitcnt before its barrier.
__device__ inline void dma16(const void* gaddr, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off"
               :
               : "v"(gaddr), "s"(lds_addr)
               : "memory", "m0");
}

typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16;

// v_mfma_f32_32x32x16_bf16 operand layout: A lane l holds row l%32, k = 8*(l/32)..+7 of a
// 32 x 16 fragment; B the same with columns; D register r of lane l is element
// (row 8*(r/4) + 4*(l/32) + r%4, column l%32).  Measured on MI355X the 32x32x16 form sustains
// about 1.35x the rate of 16x16x32 in this kind of loop, so the tiled kernel uses it: an LDS
// chunk (1 KiB) is one 32 x 16 fragment.
__device__ inline f32x16 mfma32(uint4 a, uint4 b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(*(bf16x8*)&a, *(bf16x8*)&b, c, 0, 0, 0);
}

// s_waitcnt vmcnt(N) lgkmcnt(0): vmcnt[3:0] in bits 3:0, vmcnt[5:4] in bits 15:14, expcnt
// (bits 6:4) left at "no wait".  lgkmcnt(0) makes sure the wave's own LDS reads have returned
// before it passes the barrier behind which other waves refill the buffers it read.
template <int N>
__device__ inline void wait_vm_lgkm0() {
  __builtin_amdgcn_s_waitcnt(0x0070 | (N & 15) | ((N >> 4) << 14));
}

}  // namespace

}  // namespace atenia_moe
