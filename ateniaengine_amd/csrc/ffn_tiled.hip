// Kernel 3, tiled form: grouped SwiGLU expert GEMMs for large row counts (prefill).
//
//   gate/up : H[rows of e, f] = silu(X_e W_g^T) * (X_e W_u^T)     (src/moe/dense.rs:253-266)
//   down    : Y[rows of e, d] = H_e W_d^T                         (src/moe/dense.rs:267-269)
// on v_mfma_f32_16x16x32_bf16 with f32 accumulation.  The bound is the matrix pipeline.
//
// A workgroup (4 waves, one per SIMD) owns a 256 x 256 output tile of one expert: 256
// grouped token rows by 256 weight rows (gate/up phase: 128 gate rows plus the SAME 128 up
// rows, so silu(g)*u is formed in registers).  Each wave owns 128 x 128 of it as 8 x 8 MFMA
// tiles (256 accumulator registers); per 32-wide k step it reads 8 A and 8 B fragments from
// LDS for 64 MFMAs, which keeps LDS at half its bandwidth.
//
// LDS holds both operands as 1 KiB chunks already in MFMA register order (lane l owns bytes
// 16*l), so every fragment read is one conflict-free ds_read_b128.  Weights are stored in HBM
// in that same chunk layout (moe_internal.h), so a B chunk is a straight 1 KiB copy; token
// rows are gathered through the permutation while they are loaded (no permuted copy of X is
// ever written).  INT8 W8A16 weights are widened to bf16 on their way into LDS and the
// per-row scale is applied to the accumulator.
//
// Two LDS stages of 64 k each: global loads of stage i+1 are issued into registers before
// the MFMAs of stage i and stored to the other LDS buffer after them.
#include <type_traits>

#include "moe_internal.h"

#include "../../include/atenia_moe_hip.h"

namespace atenia_moe {

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
  GroupDesc g;
  const int32_t* tile_group;  // [n_tiles] expert of each row tile
  const int32_t* tile_m0;     // [n_tiles] first row (relative to the group) of each row tile
  const int32_t* n_tiles;     // [1]
  int n_col_tiles;
};

__device__ inline uint16_t bf16_rne(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

__device__ inline uint32_t pack_i8_pair(uint32_t w, int sh) {
  float f0 = (float)(int8_t)((w >> sh) & 0xff);
  float f1 = (float)(int8_t)((w >> (sh + 8)) & 0xff);
  return (__float_as_uint(f0) >> 16) | (__float_as_uint(f1) & 0xffff0000u);
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
__device__ inline bool tile_of_workgroup(const TiledParams& p, int& rt, int& ct) {
  const int n_row_tiles = *p.n_tiles;
  const int nct = p.n_col_tiles;
  const int total = n_row_tiles * nct;
  const int per_xcd = (total + 7) / 8;
  const int slot = blockIdx.x / 8;
  const int logical = (blockIdx.x % 8) * per_xcd + slot;
  if (slot >= per_xcd || logical >= total) return false;
  // Row tiles are sorted by expert, so the expert owning this logical id is the expert of
  // row tile logical / nct; that tile's m0 tells where the expert's tiles start.
  const int rt_any = logical / nct;
  const int e = p.tile_group[rt_any];
  const int first = rt_any - p.tile_m0[rt_any] / TM;
  const int cnt = p.g.offsets[e + 1] - p.g.offsets[e];
  const int nt = (cnt + TM - 1) / TM;
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

template <bool INT8, bool UP>
__global__ __launch_bounds__(kThreads) void ffn_tiled_kernel(TiledParams p) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  int rt, ct;
  if (!tile_of_workgroup(p, rt, ct)) return;

  const int e = p.tile_group[rt];
  const int tm0 = p.tile_m0[rt];
  const int base = p.g.offsets[e];
  const int cnt = p.g.offsets[e + 1] - base;
  const int rows_here = min(TM, cnt - tm0);

  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int kq = lane >> 4, mm = lane & 15;
  const int wm = wave >> 1, wn = wave & 1;
  constexpr int BROWS = UP ? 128 : 256;  // distinct weight rows per tile
  const int nb0 = ct * (BROWS / 16);     // first 16-row weight block of the tile

  // ---- what this thread loads each stage -------------------------------------------------
  // A: chunks c = wave*8 + j  ->  (msub = c >> 1, k32 = c & 1); 4 distinct rows per thread.
  const uint16_t* arow[4];
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    int m = (wave * 4 + q) * 16 + mm;
    if (m >= rows_here) m = 0;  // clamp: such rows are computed but never stored
    int src;
    if (UP) src = p.g.perm[base + tm0 + m] / p.g.pair_div;
    else src = base + tm0 + m;
    arow[q] = p.a + (size_t)src * p.a_stride + (INT8 ? 16 * kq : 8 * kq);
  }
  // B (bf16): chunks c = wave*8 + j -> (nsub = c >> 1, k32 = c & 1), a straight block copy.
  // B (int8): blocks nsub = wave*4 + j, one 64-k block each, widened into two chunks.
  constexpr int NBL = INT8 ? 4 : 8;  // B loads per thread per stage
  const uint4* bptr[INT8 ? 4 : 4];
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    int nsub = wave * 4 + q;
    int nb;
    const uint4* wbase;
    if (UP) {
      wbase = nsub < 8 ? p.wa : p.wb;
      nb = nb0 + (nsub & 7);
    } else {
      wbase = p.wa;
      nb = nb0 + nsub;
    }
    if (nb >= p.n_blocks) nb = p.n_blocks - 1;  // clamp: columns past N are never stored
    bptr[q] = wbase + (size_t)e * p.w_stride_u4 + (size_t)nb * p.nkb * 64 + lane;
  }

  uint4 ra[8], rb[NBL];
  auto load_stage = [&](int ks) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int q = j >> 1, k32 = j & 1;
      const int koff = ks * TK + (INT8 ? 8 * k32 : 32 * k32);
      ra[j] = *(const uint4*)(arow[q] + koff);
    }
    if (INT8) {
#pragma unroll
      for (int q = 0; q < 4; ++q) rb[q] = bptr[q][(size_t)ks * 64];
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) rb[j] = bptr[j >> 1][(size_t)(ks * 2 + (j & 1)) * 64];
    }
  };
  auto store_stage = [&](int buf) {
    uint8_t* sA = lds + buf * kStage;
    uint8_t* sB = sA + kAStage;
#pragma unroll
    for (int j = 0; j < 8; ++j)
      *(uint4*)(sA + (wave * 8 + j) * kChunk + lane * 16) = ra[j];
    if (INT8) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        uint4 lo, hi;
        widen_i8x16(rb[q], lo, hi);
        *(uint4*)(sB + ((wave * 4 + q) * 2 + 0) * kChunk + lane * 16) = lo;
        *(uint4*)(sB + ((wave * 4 + q) * 2 + 1) * kChunk + lane * 16) = hi;
      }
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j)
        *(uint4*)(sB + (wave * 8 + j) * kChunk + lane * 16) = rb[j];
    }
  };

  f32x4 acc[8][8];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

  // Row sub-tiles of this wave that hold real rows (uniform per wave).
  const int my_rows = rows_here - wm * 128;
  const int mt = my_rows <= 0 ? 0 : min(8, (my_rows + 15) >> 4);

  const int nks = p.k_pad / TK;
  load_stage(0);
  store_stage(0);
  __syncthreads();
  for (int ks = 0; ks < nks; ++ks) {
    const bool more = ks + 1 < nks;
    if (more) load_stage(ks + 1);
    const uint8_t* sA = lds + (ks & 1) * kStage;
    const uint8_t* sB = sA + kAStage;
#pragma unroll
    for (int k32 = 0; k32 < 2; ++k32) {
      uint4 bf[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        // gate/up: j < 4 gate sub-tiles 4*wn+j, j >= 4 the matching up sub-tiles
        int nsub = UP ? ((j < 4 ? 0 : 8) + 4 * wn + (j & 3)) : (8 * wn + j);
        bf[j] = *(const uint4*)(sB + (nsub * 2 + k32) * kChunk + lane * 16);
      }
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        if (i < mt) {
          uint4 af = *(const uint4*)(sA + ((wm * 8 + i) * 2 + k32) * kChunk + lane * 16);
#pragma unroll
          for (int j = 0; j < 8; ++j) acc[i][j] = mfma(af, bf[j], acc[i][j]);
        }
      }
    }
    if (more) store_stage((ks + 1) & 1);
    __syncthreads();
  }

  // ---- epilogue ----------------------------------------------------------------------------
  // D layout: lane holds rows 4*kq + r (r = 0..3) of column mm of each 16 x 16 tile.
  if (UP) {
    uint16_t* h = (uint16_t*)p.out;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = (nb0 + 4 * wn + j) * 16 + mm;
      const bool n_ok = n < p.n_blocks * 16;
      float sa = 1.f, sb = 1.f;
      if (INT8) {
        sa = n < p.n_rows ? p.sa[(size_t)e * p.n_rows + n] : 0.f;
        sb = n < p.n_rows ? p.sb[(size_t)e * p.n_rows + n] : 0.f;
      }
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        if (i >= mt) continue;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int m = wm * 128 + i * 16 + 4 * kq + r;
          if (m < rows_here && n_ok) {
            float g = acc[i][j][r] * sa;
            float u = acc[i][j + 4][r] * sb;
            float hv = (g / (1.f + __expf(-g))) * u;
            h[(size_t)(base + tm0 + m) * p.out_stride + n] = bf16_rne(hv);
          }
        }
      }
    }
  } else {
    float* y = (float*)p.out;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      if (i >= mt) continue;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int m = wm * 128 + i * 16 + 4 * kq + r;
        if (m >= rows_here) continue;
        const int pair = p.g.perm[base + tm0 + m];
        float* yr = y + (size_t)pair * p.out_stride;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int n = (nb0 + 8 * wn + j) * 16 + mm;
          if (n < p.n_rows) {
            float s = INT8 ? p.sa[(size_t)e * p.n_rows + n] : 1.f;
            yr[n] = acc[i][j][r] * s;
          }
        }
      }
    }
  }
}

// ---- bf16 form with direct global->LDS loads and a four-stage ring -------------------------
// Same tiling.  Each stage holds 32 k of both operands (16 KiB + 16 KiB); a wave fills a
// 1 KiB chunk with one global_load_lds_dwordx4 (lane l's 16 bytes land at chunk + 16*l), so
// no operand passes through registers on its way to LDS and three stages (about 3 * 64 MFMAs
// of work) are always in flight behind the one being multiplied.  The four stage buffers are
// separate arrays and the k loop is unrolled by four, so each fragment read names its buffer
// statically.
typedef __attribute__((address_space(1))) const void* gptr_t;
typedef __attribute__((address_space(3))) void* lptr_t;
constexpr int kDmaStageU4 = 2 * 16 * 64;  // uint4 per stage: 16 A chunks + 16 B chunks

__device__ inline void wait_vmcnt(int n) {
  // s_waitcnt vmcnt(n) lgkmcnt(0): vmcnt[3:0] in bits 3:0, vmcnt[5:4] in bits 15:14, expcnt
  // (bits 6:4) left at "no wait", lgkmcnt (bits 11:8) = 0.  lgkmcnt(0) makes sure this wave's
  // own LDS reads of the previous step have returned before it passes the barrier after
  // which other waves refill that buffer.
  if (n >= 16) __builtin_amdgcn_s_waitcnt(0x4070);
  else if (n >= 8) __builtin_amdgcn_s_waitcnt(0x0078);
  else if (n >= 4) __builtin_amdgcn_s_waitcnt(0x0074);
  else __builtin_amdgcn_s_waitcnt(0x0070);
}

// One wave-wide 16-byte-per-lane load from global memory straight into LDS: lane l's bytes
// land at lds_addr + 16*l.  Written as inline assembly so that the compiler's wait-count
// insertion does not tie later LDS reads to these loads (it would drain all stages); the
// kernel waits for exactly the stage it needs with wait_vmcnt() before its barrier.
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

template <bool UP>
__global__ __launch_bounds__(kThreads) void ffn_tiled_dma_kernel(TiledParams p) {
  // B ring: four stages of 32 k, chunk c = (32-row group ng = c/2, k half c%2), 16 KiB each.
  // A ring: two stages of 64 k (32 KiB each).  An A chunk is 8 rows x 64 k: one load
  // instruction reads eight full 128-byte lines (a 32-row x 16-k fragment would touch 32
  // lines for 32 bytes each and starve the load path).  Inside a chunk the 16-byte segment
  // s of row r is stored at slot r*8 + (s ^ r ^ (chunk & 1)), which makes the 32-row
  // fragment reads below free of LDS bank conflicts.
  __shared__ uint4 A0[2048], A1[2048];
  __shared__ uint4 B0[1024], B1[1024], B2[1024], B3[1024];
  int rt, ct;
  if (!tile_of_workgroup(p, rt, ct)) return;

  const int e = p.tile_group[rt];
  const int tm0 = p.tile_m0[rt];
  const int base = p.g.offsets[e];
  const int cnt = p.g.offsets[e + 1] - base;
  const int rows_here = min(TM, cnt - tm0);

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform, kept scalar
  const int kh = lane >> 5, l32 = lane & 31;
  const int wm = wave >> 1, wn = wave & 1;
  constexpr int BROWS = UP ? 128 : 256;
  const int nb0 = ct * (BROWS / 16);

  // ---- loads issued by this thread --------------------------------------------------------
  // A: per 64-k stage this wave fills chunks 8*wave .. 8*wave+7 (rows 64*wave .. +63); lane l
  // fetches row l/8 of the chunk, segment (l%8) ^ (l/8) ^ (chunk&1).
  const uint16_t* arow[8];
  {
    const int r8 = lane >> 3, pslot = lane & 7;
#pragma unroll
    for (int q = 0; q < 8; ++q) {
      int m = (wave * 8 + q) * 8 + r8;
      if (m >= rows_here) m = 0;  // clamp: such rows are computed but never stored
      int src;
      if (UP) src = p.g.perm[base + tm0 + m] / p.g.pair_div;
      else src = base + tm0 + m;
      const int seg = pslot ^ r8 ^ (q & 1);
      arow[q] = p.a + (size_t)src * p.a_stride + seg * 8;
    }
  }
  // B: per 32-k stage this wave fills chunks 4*wave .. 4*wave+3 (row groups 2*wave, 2*wave+1,
  // both k halves).  Inside a stored 16-row x 32-k block the lane slot is (k quarter)*16 +
  // row%16 with k quarter = 2*half + kh.
  const uint4* bptr[2];
#pragma unroll
  for (int q = 0; q < 2; ++q) {
    int ng = wave * 2 + q;
    int brow;
    const uint4* wbase;
    if (UP) {
      wbase = ng < 4 ? p.wa : p.wb;
      brow = (ng & 3) * 32 + l32;
    } else {
      wbase = p.wa;
      brow = ng * 32 + l32;
    }
    int nb = nb0 + (brow >> 4);
    if (nb >= p.n_blocks) nb = p.n_blocks - 1;  // clamp: columns past N are never stored
    bptr[q] = wbase + (size_t)e * p.w_stride_u4 + (size_t)nb * p.nkb * 64 + kh * 16 + (brow & 15);
  }
  // ---- fragment read offsets (uint4 units) ------------------------------------------------
  // A fragment (row group mg = 4*wm + i, k16 index u of the stage): row m32 of the group is
  // chunk mg*4 + m32/8, row m32%8; segment 2u + kh.
  int aoff[4];
  {
    const int r8 = l32 & 7, cpar = (l32 >> 3) & 1;
    const int rowbase = (wm * 16 + (l32 >> 3)) * 64 + r8 * 8;
#pragma unroll
    for (int u = 0; u < 4; ++u) aoff[u] = rowbase + ((2 * u + kh) ^ r8 ^ cpar);
  }

  f32x16 acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
  const int my_rows = rows_here - wm * 128;
  const int nks = p.k_pad / 32;

  auto issue_a = [&](uint4* A, int t) {  // 64-k stage t
    const uint32_t sbase = (uint32_t)(uintptr_t)(lptr_t)A + wave * 8 * kChunk;
#pragma unroll
    for (int q = 0; q < 8; ++q) dma16(arow[q] + (size_t)t * 64, sbase + q * kChunk);
  };
  auto issue_b = [&](uint4* B, int ks) {  // 32-k stage ks
    const uint32_t sbase = (uint32_t)(uintptr_t)(lptr_t)B + wave * 4 * kChunk;
#pragma unroll
    for (int q = 0; q < 2; ++q)
#pragma unroll
      for (int h = 0; h < 2; ++h)
        dma16(bptr[q] + (size_t)ks * 64 + 32 * h, sbase + (q * 2 + h) * kChunk);
  };
  // One 32-k step.  Per wave the loads are issued in the order
  //   A(0) B(0) B(1) B(2) | step 0: A(1) B(3) | step 1: B(4) | step 2: A(2) B(5) | ...
  // (8 instructions per A stage, 4 per B stage) and complete in order, so before the
  // barrier of an even step at most 8 younger loads may be pending and before an odd step
  // 16; WAIT carries that count (smaller at the very end).  A bare s_barrier is used:
  // __syncthreads() would also drain every outstanding load, and the later stages must stay
  // in flight.  ODD / ISSUE_A / ISSUE_B / MUL are compile-time: a step is straight-line code.
  auto step = [&](auto odd_c, auto wait_c, auto issue_a_c, auto issue_b_c, auto mul_c,
                  const uint4* Acur, uint4* Anext, const uint4* Bcur, uint4* Brefill, int ks) {
    wait_vmcnt(decltype(wait_c)::value);
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    uint4 fa[2][4], fb[2][4];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        // gate/up: j < 2 gate groups 2*wn+j, j >= 2 the matching up groups
        int ng = UP ? ((j < 2 ? 0 : 4) + 2 * wn + (j & 1)) : (4 * wn + j);
        fb[h][j] = Bcur[(ng * 2 + h) * 64 + lane];
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
        fa[h][i] = Acur[i * 256 + aoff[2 * decltype(odd_c)::value + h]];
    }
    if (decltype(issue_a_c)::value) issue_a(Anext, ks / 2 + 1);
    if (decltype(issue_b_c)::value) issue_b(Brefill, ks + 3);
    // Rows past the end of a partial tile were clamped to a real row when loading; their
    // products are computed and dropped, which keeps this loop free of per-row branches.
    if (decltype(mul_c)::value == 2) {
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int j = 0; j < 4; ++j) acc[i][j] = mfma32(fa[h][i], fb[h][j], acc[i][j]);
    } else if (decltype(mul_c)::value == 1) {
      // partial tile: only the 32-row groups that hold rows (wave-uniform branches)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if (i * 32 < my_rows) {
#pragma unroll
          for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[i][j] = mfma32(fa[h][i], fb[h][j], acc[i][j]);
        }
      }
    }
  };
  using std::integral_constant;
  typedef integral_constant<bool, true> yes;
  typedef integral_constant<bool, false> no;
  typedef integral_constant<int, 2> mul_all;
  typedef integral_constant<int, 1> mul_some;
  typedef integral_constant<int, 0> mul_none;
  typedef integral_constant<int, 16> w16;
  typedef integral_constant<int, 8> w8;
  typedef integral_constant<int, 4> w4;
  typedef integral_constant<int, 0> w0;
  auto run = [&](auto mul_c) {
    issue_a(A0, 0);
    issue_b(B0, 0);
    issue_b(B1, 1);
    issue_b(B2, 2);
    int ks = 0;
    for (; ks + 4 < nks; ks += 4) {
      step(no{}, w8{}, yes{}, yes{}, mul_c, A0, A1, B0, B3, ks);
      step(yes{}, w16{}, no{}, yes{}, mul_c, A0, A1, B1, B0, ks + 1);
      step(no{}, w8{}, yes{}, yes{}, mul_c, A1, A0, B2, B1, ks + 2);
      step(yes{}, w16{}, no{}, yes{}, mul_c, A1, A0, B3, B2, ks + 3);
    }
    step(no{}, w8{}, yes{}, yes{}, mul_c, A0, A1, B0, B3, ks);
    step(yes{}, w16{}, no{}, no{}, mul_c, A0, A1, B1, B0, ks + 1);
    step(no{}, w4{}, no{}, no{}, mul_c, A1, A0, B2, B1, ks + 2);
    step(yes{}, w0{}, no{}, no{}, mul_c, A1, A0, B3, B2, ks + 3);
  };
  // nks is a multiple of 4 and at least 8 (checked by the launcher).  A wave whose half of
  // a partial tile holds no rows still feeds LDS and meets the barriers, without MFMAs; one
  // with fewer than four 32-row groups multiplies only those.
  if (my_rows >= 97) run(mul_all{});
  else if (my_rows > 0) run(mul_some{});
  else run(mul_none{});

  if (UP) {
    uint16_t* h = (uint16_t*)p.out;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int n = nb0 * 16 + (2 * wn + j) * 32 + l32;
      const bool n_ok = n < p.n_blocks * 16;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int m = wm * 128 + i * 32 + 8 * (r >> 2) + 4 * kh + (r & 3);
          if (m < rows_here && n_ok) {
            float g = acc[i][j][r];
            float u = acc[i][j + 2][r];
            float hv = (g / (1.f + __expf(-g))) * u;
            h[(size_t)(base + tm0 + m) * p.out_stride + n] = bf16_rne(hv);
          }
        }
      }
    }
  } else {
    float* y = (float*)p.out;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = wm * 128 + i * 32 + 8 * (r >> 2) + 4 * kh + (r & 3);
        if (m >= rows_here) continue;
        const int pair = p.g.perm[base + tm0 + m];
        float* yr = y + (size_t)pair * p.out_stride;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int n = nb0 * 16 + (4 * wn + j) * 32 + l32;
          if (n < p.n_rows) yr[n] = acc[i][j][r];
        }
      }
    }
  }
}

template <bool UP>
hipError_t launch_tiled_dma(const TiledParams& p, int max_row_tiles, hipStream_t s) {
  int n_wg = max_row_tiles * p.n_col_tiles;
  n_wg = (n_wg + 7) / 8 * 8;
  ffn_tiled_dma_kernel<UP><<<n_wg, kThreads, 0, s>>>(p);
  return hipGetLastError();
}

template <bool INT8, bool UP>
hipError_t launch_tiled(const TiledParams& p, int max_row_tiles, hipStream_t s) {
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute((const void*)ffn_tiled_kernel<INT8, UP>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
    if (e != hipSuccess) return e;
    attr_set = true;
  }
  // Upper bound of the grid; workgroups past the real tile count return at once.
  int n_wg = max_row_tiles * p.n_col_tiles;
  n_wg = (n_wg + 7) / 8 * 8;
  ffn_tiled_kernel<INT8, UP><<<n_wg, kThreads, kLdsBytes, s>>>(p);
  return hipGetLastError();
}

}  // namespace

bool tiled_supported(const WeightSet& w, int wdtype) {
  if (wdtype == ATENIA_MOE_WEIGHT_F32) return false;
  return w.k_pad % TK == 0;
}

hipError_t launch_ffn_up_tiled(const FfnArgs& a, hipStream_t s) {
  const bool int8 = a.wdtype == ATENIA_MOE_WEIGHT_INT8_W8A16;
  TiledParams p{};
  p.wa = (const uint4*)a.gate.w;
  p.wb = (const uint4*)a.up.w;
  p.sa = a.gate.scale;
  p.sb = a.up.scale;
  p.w_stride_u4 = a.gate.expert_stride / 16;
  p.n_rows = a.gate.n_rows;
  p.n_blocks = a.gate.n_pad / 16;
  p.nkb = a.gate.k_pad / (int8 ? kKbInt8 : kKbBf16);
  p.k_pad = a.gate.k_pad;
  p.a = (const uint16_t*)a.x;
  p.a_stride = a.x_stride;
  p.out = a.h;
  p.out_stride = a.h_stride;
  p.g = a.g;
  p.tile_group = a.tile_group;
  p.tile_m0 = a.tile_m0;
  p.n_tiles = a.n_tiles;
  p.n_col_tiles = (a.gate.n_pad + 127) / 128;
  if (!int8 && p.k_pad % 128 == 0 && p.k_pad >= 256) return launch_tiled_dma<true>(p, a.max_row_tiles, s);
  return int8 ? launch_tiled<true, true>(p, a.max_row_tiles, s)
              : launch_tiled<false, true>(p, a.max_row_tiles, s);
}

hipError_t launch_ffn_down_tiled(const FfnArgs& a, hipStream_t s) {
  const bool int8 = a.wdtype == ATENIA_MOE_WEIGHT_INT8_W8A16;
  TiledParams p{};
  p.wa = (const uint4*)a.down.w;
  p.wb = nullptr;
  p.sa = a.down.scale;
  p.sb = nullptr;
  p.w_stride_u4 = a.down.expert_stride / 16;
  p.n_rows = a.down.n_rows;
  p.n_blocks = a.down.n_pad / 16;
  p.nkb = a.down.k_pad / (int8 ? kKbInt8 : kKbBf16);
  p.k_pad = a.down.k_pad;
  p.a = (const uint16_t*)a.h;
  p.a_stride = a.h_stride;
  p.out = a.y;
  p.out_stride = a.y_stride;
  p.g = a.g;
  p.tile_group = a.tile_group;
  p.tile_m0 = a.tile_m0;
  p.n_tiles = a.n_tiles;
  p.n_col_tiles = (a.down.n_pad + 255) / 256;
  if (!int8 && p.k_pad % 128 == 0 && p.k_pad >= 256) return launch_tiled_dma<false>(p, a.max_row_tiles, s);
  return int8 ? launch_tiled<true, false>(p, a.max_row_tiles, s)
              : launch_tiled<false, false>(p, a.max_row_tiles, s);
}

}  // namespace atenia_moe
