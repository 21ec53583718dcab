// Kernel 3, tiled form: grouped SwiGLU expert GEMMs for large row counts (prefill).
//
//   gate/up : H[rows of e, f] = silu(X_e W_g^T) * (X_e W_u^T)     (src/moe/dense.rs:253-266)
//   down    : Y[rows of e, d] = H_e W_d^T                         (src/moe/dense.rs:267-269)
// on bf16 MFMA with f32 accumulation.  The bound is the matrix pipeline.
//
// A workgroup (4 waves, one per SIMD) owns a 256 x 256 output tile of one expert: 256 grouped
// token rows by 256 weight rows (gate/up phase: 128 gate rows plus the SAME 128 up rows, so
// silu(g)*u is formed in registers); each wave owns 128 x 128 of it.  Token rows are gathered
// through the permutation while they are loaded (no permuted copy of X is ever written).
//
// Three kernels share this tiling:
//   ffn_tiled_pipe_kernel     bf16 weights, K a multiple of 64 and >= 128: 4 x 4 tiles of
//                             v_mfma_f32_32x32x16_bf16 per wave, operands go global -> LDS
//                             directly (global_load_lds_dwordx4) into a ring of three 64-k A
//                             stages and three 32-k B stages, software-pipelined in units of 16
//                             MFMAs with one barrier per 32-k step; row tiles of up to nine
//                             32-row groups (the ninth in a ring and registers of its own)
//   ffn_tiled_pipe_i8_kernel  INT8 W8A16, K >= 128: same pipeline, weights stay int8 into LDS and
//                             are widened to bf16 in registers, row scale applied to the
//                             accumulator
//   ffn_tiled_kernel          fallback for other K: 8 x 8 tiles of v_mfma_f32_16x16x32_bf16 per
//                             wave, two 64-k LDS stages filled through registers (int8 widened on
//                             the way into LDS)
// Weights are stored in HBM as 1 KiB blocks already in MFMA register order (moe_internal.h), so
// a B chunk is a straight 1 KiB copy and every B fragment read is one ds_read_b128.
#include "ffn_tiled_common.h"

#include "../../include/atenia_moe_hip.h"

namespace atenia_moe {

namespace {

// (types, TiledParams, the tile order and the LDS-DMA helpers live in ffn_tiled_common.h)
template <bool INT8, bool UP>
__global__ __launch_bounds__(kThreads) void ffn_tiled_kernel(TiledParams p) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  int rt, ct;
  if (!tile_of_workgroup(p, blockIdx.x, rt, ct)) return;

  const int e = p.tile_group[rt];
  const int tm0 = p.tile_m0[rt];
  const int base = p.g.offsets[e];
  const int cnt = p.g.offsets[e + 1] - base;
  const int rows_here = min(TM, cnt - tm0);

  const int tid = threadIdx.x, lane = tid & 63;
  // scalar wave id: guards around MFMAs must be scalar branches (MFMA does not obey EXEC)
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
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

// ---- bf16 form: direct global->LDS loads, multi-stage rings, software-pipelined k loop ------
// Same 256 x 256 tiling on v_mfma_f32_32x32x16_bf16 (each wave 128 x 128 = 4 x 4 MFMA tiles).
// LDS holds a ring of three 64-k A stages (32 KiB each), a ring of three 32-k B stages
// (16 KiB each) and a ring of three 4 KiB stages for the ninth row group of a tall tile.  A
// wave fills a 1 KiB chunk with one global_load_lds_dwordx4 (lane l's 16 bytes land at
// chunk + 16*l), so no operand passes through registers on its way to LDS.
// The k loop works in k16 units of 16 MFMAs: while one unit multiplies, the 8 fragment reads
// of the next unit and 4 loads of a stage several steps ahead are issued between its MFMAs
// (pinned with sched_barrier), and the single barrier per 32-k step sits between the two
// units of the step so that no wave waits for LDS right after it.
constexpr int kRingA = 3;  // A stages of 64 k (32 KiB each)
constexpr int kRingB = 3;  // B stages of 32 k (16 KiB each); a fourth measured no faster
// Rows 256..287 of a nine-group tile: their own ring of 64-k stages (4 KiB each = four chunks of
// 8 rows x 128 bytes, swizzled like the A chunks), one stage per A stage.
constexpr int kXaStage = 256;  // uint4 per stage

// YB (down phase only): y leaves as bf16 (TiledParams::out_bf16), staged through LDS.
// The tile of workgroup `bid` of a launch described by p.
// SC: the weights are the int8 values of a W8A16 layer widened to bf16 (exactly), and the f32
// accumulators are multiplied by the per-row scales p.sa / p.sb [E, n_rows] on their way out.
template <bool UP, bool YB, bool SC = false>
__device__ __forceinline__ void pipe_tile(const TiledParams& p, int bid) {
  static_assert(!(SC && YB), "scaled outputs are stored as f32");
  constexpr int NA = kRingA, NB = kRingB;
  constexpr int XA0 = NA * 2048 + NB * 1024;            // first uint4 of the extra-rows ring
  __shared__ uint4 S[XA0 + NA * kXaStage];              // A ring, B ring, extra-rows ring
  int wid, n_parts, part;  // k range `part` of `n_parts` (1 unless this is a split tail tile)
  if (!split_of_workgroup(p, bid, p.k_pad / 64, wid, n_parts, part)) return;
  int rt, ct;
  if (!tile_of_workgroup(p, wid, rt, ct)) return;

  const int e = p.tile_group[rt];
  const int tm0 = p.tile_m0[rt];
  const int base = p.g.offsets[e];
  const int cnt = p.g.offsets[e + 1] - base;
  const int rows_here = p.tile_rows ? p.tile_rows[rt] : min(TM, cnt - tm0);
  // A tile of nine 32-row groups: rows 256.. ride along as a ninth group whose 32 x 256 results
  // are shared out over the four waves (two 32 x 32 blocks each).
  const bool tall = rows_here > TM;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int kh = lane >> 5, l32 = lane & 31;
  const int wm = wave >> 1, wn = wave & 1;
  constexpr int BROWS = UP ? 128 : 256;
  const int nb0 = ct * (BROWS / 16);

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
    if (nb >= p.n_blocks) nb = p.n_blocks - 1;
    bptr[q] = wbase + (size_t)e * p.w_stride_u4 + (size_t)nb * p.nkb * 64 + kh * 16 + (brow & 15);
  }
  // The first B stages are requested before anything that depends on the row list:
  // weight tiles come from HBM (the longest latency of the prologue) and need nothing but
  // the tile coordinates, so they fly while the pair ids of the A rows are looked up.
  const int st_lo = (p.k_pad / 64) * part / n_parts, st_hi = (p.k_pad / 64) * (part + 1) / n_parts;
  const int nks = 2 * (st_hi - st_lo);  // 32-k steps of this workgroup's k range
  const int ks0 = 2 * st_lo;
  const uint32_t sb_fill = (uint32_t)(uintptr_t)(lptr_t)S + NA * 32768 + wave * 4 * kChunk;
  auto dma_b = [&](int buf, int q, int ks) {  // q = 2 * row group + k half
    dma16(bptr[q >> 1] + (size_t)(ks0 + ks) * 64 + 32 * (q & 1), sb_fill + buf * 16384 + q * kChunk);
  };
#pragma unroll
  for (int t = 0; t < NB; ++t)
#pragma unroll
    for (int q = 0; q < 4; ++q) dma_b(t, q, min(t, nks - 1));

  // A stage: 256 rows x 64 k as 32 chunks of 8 rows x 128 bytes, so that one load instruction
  // reads eight full 128-byte lines.  Row r, 16-byte segment s of chunk c is stored at slot
  // 8r + (s ^ r ^ (c & 1)); lane l of the filling load fetches row l/8, segment
  // (l%8) ^ (l/8) ^ (c&1).  Wave w fills chunks 8w .. 8w+7, four per step.
  const uint16_t* arow[8];
  {
    const int r8 = lane >> 3, pslot = lane & 7;
#pragma unroll
    for (int q = 0; q < 8; ++q) {
      int m = (wave * 8 + q) * 8 + r8;
      if (m >= rows_here) m = 0;
      int src;
      if (UP) src = p.g.perm[base + tm0 + m] / p.g.pair_div;
      else src = base + tm0 + m;
      arow[q] = p.a + (size_t)src * p.a_stride + (pslot ^ r8 ^ (q & 1)) * 8;
    }
  }
  // extra rows (tall tiles): wave w fills chunk w of a stage, rows 256 + 8 w ..
  const uint16_t* xrow = nullptr;
  if (tall) {
    const int r8 = lane >> 3, pslot = lane & 7;
    int m = TM + wave * 8 + r8;
    if (m >= rows_here) m = 0;
    int src;
    if (UP) src = p.g.perm[base + tm0 + m] / p.g.pair_div;
    else src = base + tm0 + m;
    xrow = p.a + (size_t)src * p.a_stride + (pslot ^ r8 ^ (wave & 1)) * 8;
  }
  // fragment read offsets (uint4 units inside a stage): A row group i adds 256, k16 unit u of
  // the 64-k stage selects the swizzled segment; B row group j of this wave, unit u adds 64.
  int aoff[4];
  {
    const int r8 = l32 & 7, cpar = (l32 >> 3) & 1;
    const int rowbase = (wm * 16 + (l32 >> 3)) * 64 + r8 * 8;
#pragma unroll
    for (int u = 0; u < 4; ++u) aoff[u] = rowbase + ((2 * u + kh) ^ r8 ^ cpar);
  }
  // the ninth group's fragment of unit u sits at aoff[u] of row group 0 in its own ring
  const int xoff0 = XA0 - wm * 16 * 64;
  const int boff0 = NA * 2048 + (UP ? 2 * wn : 4 * wn) * 128 + lane;
  constexpr int kBJ1 = 128, kBJ2 = UP ? 512 : 256, kBJ3 = UP ? 640 : 384;

  f32x16 acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
  const int my_rows = rows_here - wm * 128;

  const uint32_t sa_fill = (uint32_t)(uintptr_t)(lptr_t)S + wave * 8 * kChunk;
  auto dma_a = [&](int buf, int q, int t) {  // chunk q of this wave, 64-k stage t
    dma16(arow[q] + (size_t)(ks0 / 2 + t) * 64, sa_fill + buf * 32768 + q * kChunk);
  };
  const uint32_t xa_fill = (uint32_t)(uintptr_t)(lptr_t)S + XA0 * 16 + wave * kChunk;
  auto dma_xa = [&](int buf, int t) {  // this wave's chunk of the extra rows, 64-k stage t
    dma16(xrow + (size_t)(ks0 / 2 + t) * 64, xa_fill + buf * (kXaStage * 16));
  };

  // the 8 fragment reads of one k16 unit, in the order the MFMAs consume them
  auto read_frag = [&](int n, uint4 (&FA)[4], uint4 (&FB)[4], int a0, int b0) {
    switch (n) {
      case 0: FA[0] = S[a0]; break;
      case 1: FB[0] = S[b0]; break;
      case 2: FB[1] = S[b0 + kBJ1]; break;
      case 3: FB[2] = S[b0 + kBJ2]; break;
      case 4: FB[3] = S[b0 + kBJ3]; break;
      case 5: FA[1] = S[a0 + 256]; break;
      case 6: FA[2] = S[a0 + 512]; break;
      default: FA[3] = S[a0 + 768]; break;
    }
  };
  // One k16 unit: 16 MFMAs on (FA, FB).  Behind MFMA m < 8 goes read m of the next unit;
  // behind MFMAs 8, 10, 12, 14 one load each of the stage being refilled, so LDS and the load
  // path see an even stream instead of bursts.
  auto half = [&](auto mul_c, auto dma_c, auto dma_is_a_c, uint4 (&FA)[4], uint4 (&FB)[4],
                  uint4 (&NA_)[4], uint4 (&NB_)[4], int a0, int b0, int dbuf, int dks, auto aq0_c) {
    constexpr int MUL = decltype(mul_c)::value;
#pragma unroll
    for (int m = 0; m < 16; ++m) {
      const int i = m >> 2, j = m & 3;
      if (MUL == 2 || (MUL == 1 && i * 32 < my_rows)) acc[i][j] = mfma32(FA[i], FB[j], acc[i][j]);
      if (m < 8) read_frag(m, NA_, NB_, a0, b0);
      if (decltype(dma_c)::value && m >= 8 && (m & 1) == 0) {
        if (decltype(dma_is_a_c)::value) dma_a(dbuf, decltype(aq0_c)::value + ((m - 8) >> 1), dks);
        else dma_b(dbuf, (m - 8) >> 1, dks);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  using std::integral_constant;
  typedef integral_constant<bool, true> yes;
  typedef integral_constant<bool, false> no;

  // Step s (32 k) = unit 0 on (fa0, fb0), then unit 1 on (fa1, fb1).
  //   first half : reads unit 1 of stage s; issues A(s + NA - 1) into the A buffer freed by
  //                the previous step's barrier
  //   middle     : waits until this wave's loads of stage s + 1 have landed, barrier
  //   second half: reads unit 0 of stage s + 1; issues B(s + NB) into the B buffer of stage s
  // Loads complete in issue order ... A(s+1) | B(s+NB-2) A(s+2) B(s+NB-1) A(s+3) at the middle
  // of step s, so 4 * (NA - 2) groups of 4 loads may stay in flight behind the wait (half of
  // that in a wave that loads no A rows).  Stages past the end of k are clamped to the last
  // one: they land in buffers nobody reads and keep the wait counts uniform.
  auto run = [&](auto mul_c, auto la_c) {
    constexpr bool LA = decltype(la_c)::value;
    typedef integral_constant<int, 0> q0;
    typedef integral_constant<int, 4> q4;
    uint4 fa0[4], fb0[4], fa1[4], fb1[4];
    const int nst = nks / 2;  // 64-k stages
    auto fill_a = [&](int t) {
      if (LA) {
#pragma unroll
        for (int q = 0; q < 8; ++q) dma_a(t, q, min(t, nst - 1));
      }
    };
    // issued so far: B0 .. B(NB-1); now A0 A1, then per step: half of A(s/2 + 2), B(s + NB).
    // A wave that loads A rows waits for everything (A1 lands right behind A0), one that
    // does not only for B0.
    // In the middle of step s the wave needs its loads of B(s + 1); issued after them are
    // (NB - 1) halves of A stages and (NB - 2) B stages, of which the A half of step s - 2 must
    // have landed as well (the next A stage's first rows): at most 4 groups of 4 may stay out.
    constexpr int kMidWait = LA ? (4 * (2 * NB - 3) < 16 ? 4 * (2 * NB - 3) : 16) : 4 * (NB - 2);
    fill_a(0); fill_a(1);
    wait_vm_lgkm0<LA ? 0 : 4 * (NB - 1)>();
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
#pragma unroll
    for (int n = 0; n < 8; ++n) read_frag(n, fa0, fb0, aoff[0], boff0);
    int abuf = 0, bbuf = 0;  // buffers of the stages step s reads
    for (int s = 0; s < nks; s += 2) {
      const int abuf_n = abuf + 1 == NA ? 0 : abuf + 1;
      const int abuf_i = abuf == 0 ? NA - 1 : abuf - 1;  // freed by the previous stage
      const int ta = min(s / 2 + NA - 1, nst - 1);
      // even step: k16 units 0, 1 of the A stage
      {
        const int bbuf_n = bbuf + 1 == NB ? 0 : bbuf + 1;
        half(mul_c, la_c, yes{}, fa0, fb0, fa1, fb1, aoff[1] + abuf * 2048, boff0 + bbuf * 1024 + 64,
             abuf_i, ta, q0{});
        wait_vm_lgkm0<kMidWait>();
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        half(mul_c, yes{}, no{}, fa1, fb1, fa0, fb0, aoff[2] + abuf * 2048, boff0 + bbuf_n * 1024,
             bbuf, min(s + NB, nks - 1), q0{});
        bbuf = bbuf_n;
      }
      // odd step: units 2, 3; its second half reads unit 0 of the next A stage
      {
        const int bbuf_n = bbuf + 1 == NB ? 0 : bbuf + 1;
        half(mul_c, la_c, yes{}, fa0, fb0, fa1, fb1, aoff[3] + abuf * 2048, boff0 + bbuf * 1024 + 64,
             abuf_i, ta, q4{});
        wait_vm_lgkm0<kMidWait>();
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        half(mul_c, yes{}, no{}, fa1, fb1, fa0, fb0, aoff[0] + abuf_n * 2048, boff0 + bbuf_n * 1024,
             bbuf, min(s + 1 + NB, nks - 1), q0{});
        bbuf = bbuf_n;
      }
      abuf = abuf_n;
    }
    wait_vm_lgkm0<0>();
  };
  // ---- tiles of nine groups ------------------------------------------------------------------
  // The same pipeline with 18 MFMAs per unit: behind the 16 of the main 256 rows come two on the
  // ninth group's fragment FX and two of the B fragments the wave holds anyway (gate / up group
  // wm of its half in the gate/up phase, groups 2 wm, 2 wm + 1 in the down phase).  FX of the
  // next unit is read behind the first of them; the wave's one load per 64-k stage of the extra
  // rows goes behind MFMA 9 of the step half that issues A chunks 0..3.  Every wave of such a
  // tile loads A rows and all main row groups are full, so there is one form only.
  auto half_tall = [&](f32x16 (&accx)[2], auto dma_is_a_c, auto xa_c, uint4 (&FA)[4], uint4 (&FB)[4], uint4 (&NA_)[4],
                       uint4 (&NB_)[4], uint4& FX, uint4& NX, int a0, int b0, int x0, int dbuf,
                       int dks, auto aq0_c) {
#pragma unroll
    for (int m = 0; m < 18; ++m) {
      if (m < 16) {
        const int i = m >> 2, j = m & 3;
        acc[i][j] = mfma32(FA[i], FB[j], acc[i][j]);
      } else {
        const int jj = m - 16;
        const uint4 b_lo = UP ? FB[jj == 0 ? 0 : 2] : FB[jj];       // wm == 0
        const uint4 b_hi = UP ? FB[jj == 0 ? 1 : 3] : FB[2 + jj];   // wm == 1
        uint4 bsel;
        bsel.x = wm ? b_hi.x : b_lo.x;
        bsel.y = wm ? b_hi.y : b_lo.y;
        bsel.z = wm ? b_hi.z : b_lo.z;
        bsel.w = wm ? b_hi.w : b_lo.w;
        // The ninth group's accumulators live in ordinary VGPRs (the 256 accumulation registers
        // are taken): the instruction is spelled out so that the allocator cannot move them.
        // Nothing reads these registers before the same instruction of the next unit, sixteen
        // matrix instructions later, so no wait states are owed there; the two owed between the
        // selects that write the B operand and the instruction reading it are spelled out too
        // (the compiler counts them for the matrix instructions it emits itself, not for this).
        const bf16x8 fxv = *(const bf16x8*)&FX, bv = *(const bf16x8*)&bsel;
        asm volatile("s_nop 1\n\tv_mfma_f32_32x32x16_bf16 %0, %1, %2, %0"
                     : "+v"(accx[jj])
                     : "v"(fxv), "v"(bv));
      }
      if (m < 8) read_frag(m, NA_, NB_, a0, b0);
      if (m == 16) NX = S[x0];
      if (m >= 8 && m < 16 && (m & 1) == 0) {
        if (decltype(dma_is_a_c)::value) dma_a(dbuf, decltype(aq0_c)::value + ((m - 8) >> 1), dks);
        else dma_b(dbuf, (m - 8) >> 1, dks);
      }
      if (decltype(xa_c)::value && m == 9) dma_xa(dbuf, dks);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  auto run_tall = [&](f32x16 (&accx)[2]) {
    typedef integral_constant<int, 0> q0;
    typedef integral_constant<int, 4> q4;
    uint4 fa0[4], fb0[4], fa1[4], fb1[4], fx0, fx1;
#pragma unroll
    for (int r = 0; r < 16; ++r) accx[0][r] = accx[1][r] = 0.f;
    const int nst = nks / 2;  // 64-k stages
    // issued so far: B0 .. B(NB-1); now A0 X0 A1 X1.  Per pair of steps a wave then issues
    // A-half, X, B | A-half, B; in the middle of step s it needs B(s + 1), behind which went
    // (NB - 1) A halves, (NB - 2) B stages and (NB - 1) / 2 rounded either way X loads.  With
    // NB = 3: two A halves, one B stage and exactly one X load (one of steps s - 1, s is even).
    static_assert(NB == 3, "the wait count below is worked out for a B ring of three stages");
#pragma unroll
    for (int t = 0; t < 2; ++t) {
#pragma unroll
      for (int q = 0; q < 8; ++q) dma_a(t, q, min(t, nst - 1));
      dma_xa(t, min(t, nst - 1));
    }
    wait_vm_lgkm0<0>();
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
#pragma unroll
    for (int n = 0; n < 8; ++n) read_frag(n, fa0, fb0, aoff[0], boff0);
    fx0 = S[xoff0 + aoff[0]];
    int abuf = 0, bbuf = 0;
    for (int s = 0; s < nks; s += 2) {
      const int abuf_n = abuf + 1 == NA ? 0 : abuf + 1;
      const int abuf_i = abuf == 0 ? NA - 1 : abuf - 1;
      const int ta = min(s / 2 + NA - 1, nst - 1);
      const int xcur = xoff0 + abuf * kXaStage, xnext = xoff0 + abuf_n * kXaStage;
      {
        const int bbuf_n = bbuf + 1 == NB ? 0 : bbuf + 1;
        half_tall(accx, yes{}, yes{}, fa0, fb0, fa1, fb1, fx0, fx1, aoff[1] + abuf * 2048,
                  boff0 + bbuf * 1024 + 64, xcur + aoff[1], abuf_i, ta, q0{});
        wait_vm_lgkm0<13>();
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        half_tall(accx, no{}, no{}, fa1, fb1, fa0, fb0, fx1, fx0, aoff[2] + abuf * 2048,
                  boff0 + bbuf_n * 1024, xcur + aoff[2], bbuf, min(s + NB, nks - 1), q0{});
        bbuf = bbuf_n;
      }
      {
        const int bbuf_n = bbuf + 1 == NB ? 0 : bbuf + 1;
        half_tall(accx, yes{}, no{}, fa0, fb0, fa1, fb1, fx0, fx1, aoff[3] + abuf * 2048,
                  boff0 + bbuf * 1024 + 64, xcur + aoff[3], abuf_i, ta, q4{});
        wait_vm_lgkm0<13>();
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        half_tall(accx, no{}, no{}, fa1, fb1, fa0, fb0, fx1, fx0, aoff[0] + abuf_n * 2048,
                  boff0 + bbuf_n * 1024, xnext + aoff[0], bbuf, min(s + 1 + NB, nks - 1), q0{});
        bbuf = bbuf_n;
      }
      abuf = abuf_n;
    }
    wait_vm_lgkm0<0>();
  };
  const bool loads_a = wave * 64 < rows_here;
  if (tall) {
    f32x16 accx[2];  // rows 256.. x this wave's two column groups
    run_tall(accx);
    // a matrix instruction's results may be read by other instructions 18 passes-of-4 later
    asm volatile("s_nop 15\n\ts_nop 15" : "+v"(accx[0]), "+v"(accx[1])::"memory");
    if (UP) {  // gate in accx[0], up in accx[1], this wave's 32 x 32 block
      uint16_t* h = (uint16_t*)p.out;
      const int n = nb0 * 16 + (2 * wn + wm) * 32 + l32;
      float sg = 1.f, su = 1.f;
      if (SC) {
        const size_t at = (size_t)e * p.n_rows + min(n, p.n_rows - 1);
        sg = p.sa[at];
        su = p.sb[at];
      }
      if (n < p.n_blocks * 16) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int mrow = TM + 8 * (r >> 2) + 4 * kh + (r & 3);
          if (mrow < rows_here)
            h[(size_t)(base + tm0 + mrow) * p.out_stride + n] = (uint16_t)bf16_rne_pair(
                SC ? swiglu_fast(accx[0][r] * sg, accx[1][r] * su) : swiglu_fast(accx[0][r], accx[1][r]), 0.f);
        }
      }
    } else {  // column groups 4 wn + 2 wm, + 1 of this wave
      float* y = (float*)p.out + (size_t)part * p.out_part_stride;
      uint16_t* yb = (uint16_t*)p.out + (size_t)part * p.out_part_stride;
      float sx[2] = {1.f, 1.f};
      if (SC) {
#pragma unroll
        for (int jj = 0; jj < 2; ++jj)
          sx[jj] = p.sa[(size_t)e * p.n_rows +
                        min(nb0 * 16 + (4 * wn + 2 * wm + jj) * 32 + l32, p.n_rows - 1)];
      }
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = TM + 8 * (r >> 2) + 4 * kh + (r & 3);
        if (m >= rows_here) continue;
        const int pair = p.g.perm[base + tm0 + m];
        if (p.part_flags && part == 0 && wn == 0 && wm == 0 && l32 == 0)
          p.part_flags[(size_t)pair * p.n_col_tiles + ct] = (uint8_t)n_parts;
        float* yr = y + (size_t)pair * p.out_stride;
        uint16_t* ybr = yb + (size_t)pair * p.out_stride;
#pragma unroll
        for (int jj = 0; jj < 2; ++jj) {
          const int n = nb0 * 16 + (4 * wn + 2 * wm + jj) * 32 + l32;
          if (n < p.n_rows) {
            if (YB) ybr[n] = (uint16_t)bf16_rne_pair(accx[jj][r], 0.f);
            else yr[n] = SC ? accx[jj][r] * sx[jj] : accx[jj][r];
          }
        }
      }
    }
  } else if (my_rows >= 97) run(integral_constant<int, 2>{}, yes{});
  else if (my_rows > 0) {
    if (loads_a) run(integral_constant<int, 1>{}, yes{});
    else run(integral_constant<int, 1>{}, no{});
  } else {
    if (loads_a) run(integral_constant<int, 0>{}, yes{});
    else run(integral_constant<int, 0>{}, no{});
  }

  if (UP) {
    // silu(g) * u, rounded to bf16, staged through LDS so that every global store is a full
    // 128-byte line: the wave's 128 x 64 block goes to its own region with a row pitch of
    // 144 bytes and is read back 16 bytes per lane, 8 lanes per row.
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();  // every wave's loads have landed and its reads are done
    asm volatile("" ::: "memory");
    constexpr int kPitch = 144;
    char* stage = (char*)S + wave * (128 * kPitch);
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      float sg = 1.f, su = 1.f;
      if (SC) {
        const size_t at = (size_t)e * p.n_rows + min(nb0 * 16 + (2 * wn + j) * 32 + l32, p.n_rows - 1);
        sg = p.sa[at];
        su = p.sb[at];
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
#pragma unroll
        for (int r = 0; r < 16; r += 2) {  // rows m and m + 1
          const int m = i * 32 + 8 * (r >> 2) + 4 * kh + (r & 3);
          const uint32_t hh =
              SC ? bf16_rne_pair(swiglu_fast(acc[i][j][r] * sg, acc[i][j + 2][r] * su),
                                 swiglu_fast(acc[i][j][r + 1] * sg, acc[i][j + 2][r + 1] * su))
                 : bf16_rne_pair(swiglu_fast(acc[i][j][r], acc[i][j + 2][r]),
                                 swiglu_fast(acc[i][j][r + 1], acc[i][j + 2][r + 1]));
          char* dst = stage + m * kPitch + (j * 32 + l32) * 2;
          *(uint16_t*)dst = (uint16_t)hh;
          *(uint16_t*)(dst + kPitch) = (uint16_t)(hh >> 16);
        }
      }
    }
    // the region is private to the wave: no barrier, the compiler orders the LDS accesses
    uint16_t* h = (uint16_t*)p.out;
    const int n0 = nb0 * 16 + wn * 64;  // first column of the wave's block
    const int c8 = lane & 7, r8 = lane >> 3;
#pragma unroll
    for (int it = 0; it < 16; ++it) {
      const int m = it * 8 + r8;
      const uint4 v = *(const uint4*)(stage + m * kPitch + c8 * 16);
      const int mrow = wm * 128 + m;
      const int n = n0 + c8 * 8;
      if (mrow < rows_here && n < p.n_blocks * 16)
        *(uint4*)(h + (size_t)(base + tm0 + mrow) * p.out_stride + n) = v;
    }
  } else if (YB) {
    // y as bf16, staged through LDS like h above so that every global store is 16 bytes per lane
    // and a row's 256 bytes leave as two full lines: the wave's 128 x 128 block goes to its own
    // region with a row pitch of 272 bytes and is read back 16 lanes per row, 4 rows at a time.
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();  // every wave's loads have landed and its reads are done
    asm volatile("" ::: "memory");
    constexpr int kPitch = 272;
    char* stage = (char*)S + wave * (128 * kPitch);
    const int r4 = lane >> 4, c16 = lane & 15;
    int pair_of[32];  // pair id of the rows this lane stores
#pragma unroll
    for (int it = 0; it < 32; ++it) {
      const int m = wm * 128 + it * 4 + r4;
      pair_of[it] = p.g.perm[base + tm0 + min(m, rows_here - 1)];
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
#pragma unroll
        for (int r = 0; r < 16; r += 2) {  // rows m and m + 1
          const int m = i * 32 + 8 * (r >> 2) + 4 * kh + (r & 3);
          const uint32_t hh = bf16_rne_pair(acc[i][j][r], acc[i][j][r + 1]);
          char* dst = stage + m * kPitch + (j * 32 + l32) * 2;
          *(uint16_t*)dst = (uint16_t)hh;
          *(uint16_t*)(dst + kPitch) = (uint16_t)(hh >> 16);
        }
      }
    }
    uint16_t* yb = (uint16_t*)p.out + (size_t)part * p.out_part_stride;
    const int n = nb0 * 16 + wn * 128 + c16 * 8;
#pragma unroll
    for (int it = 0; it < 32; ++it) {
      const int m = it * 4 + r4;
      const uint4 v = *(const uint4*)(stage + m * kPitch + c16 * 16);
      const int mrow = wm * 128 + m;
      if (mrow >= rows_here) continue;
      const int pair = pair_of[it];
      if (p.part_flags && part == 0 && wn == 0 && c16 == 0)
        p.part_flags[(size_t)pair * p.n_col_tiles + ct] = (uint8_t)n_parts;
      if (n < p.n_rows) *(uint4*)(yb + (size_t)pair * p.out_stride + n) = v;
    }
  } else {
    float* y = (float*)p.out + (size_t)part * p.out_part_stride;
    // The pair id of every row first, in one batch of loads: fetched next to the stores they
    // address, each would wait out its own L2 round trip (the compiler cannot move a load of
    // perm above a store to y).
    float sd[4] = {1.f, 1.f, 1.f, 1.f};
    if (SC) {
#pragma unroll
      for (int j = 0; j < 4; ++j)
        sd[j] = p.sa[(size_t)e * p.n_rows + min(nb0 * 16 + (4 * wn + j) * 32 + l32, p.n_rows - 1)];
    }
    int pair_of[4][16];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = wm * 128 + i * 32 + 8 * (r >> 2) + 4 * kh + (r & 3);
        pair_of[i][r] = p.g.perm[base + tm0 + min(m, rows_here - 1)];
      }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = wm * 128 + i * 32 + 8 * (r >> 2) + 4 * kh + (r & 3);
        if (m >= rows_here) continue;
        const int pair = pair_of[i][r];
        if (p.part_flags && part == 0 && wn == 0 && l32 == 0)
          p.part_flags[(size_t)pair * p.n_col_tiles + ct] = (uint8_t)n_parts;
        float* yr = y + (size_t)pair * p.out_stride;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int n = nb0 * 16 + (4 * wn + j) * 32 + l32;
          if (n < p.n_rows) yr[n] = SC ? acc[i][j][r] * sd[j] : acc[i][j][r];
        }
      }
    }
  }
}

template <bool UP, bool YB = false, bool SC = false>
__global__ __launch_bounds__(kThreads) void ffn_tiled_pipe_kernel(TiledParams p) {
  pipe_tile<UP, YB, SC>(p, (int)blockIdx.x);
}

// Gate/up launch of the routed experts and of a shared expert in one grid: workgroups below
// n_first take the routed experts' tiles (p), the others the shared expert's (ps), in that order,
// so the compute units that the last routed tiles leave idle start on the shared expert instead
// of waiting for a second launch (each launch by itself ends on a partly filled round of tiles).
// The parameter set is picked field by field with the workgroup-uniform condition: selecting a
// reference to one of two by-value kernel arguments makes the compiler copy the struct to the stack.
__device__ __forceinline__ TiledParams pick_params(const TiledParams& a, const TiledParams& b, bool second) {
  TiledParams q;
#define ATENIA_PICK(f) q.f = second ? b.f : a.f
  ATENIA_PICK(wa); ATENIA_PICK(wb); ATENIA_PICK(sa); ATENIA_PICK(sb); ATENIA_PICK(w_stride_u4);
  ATENIA_PICK(n_rows); ATENIA_PICK(n_blocks); ATENIA_PICK(nkb); ATENIA_PICK(k_pad); ATENIA_PICK(a);
  ATENIA_PICK(a_stride); ATENIA_PICK(out); ATENIA_PICK(out_stride); ATENIA_PICK(out_bf16);
  ATENIA_PICK(g.offsets); ATENIA_PICK(g.active); ATENIA_PICK(g.n_active); ATENIA_PICK(g.perm);
  ATENIA_PICK(g.pair_div); ATENIA_PICK(g.idx1);
  ATENIA_PICK(tile_group); ATENIA_PICK(tile_m0); ATENIA_PICK(n_tiles); ATENIA_PICK(tile_rows);
  ATENIA_PICK(tile_li); ATENIA_PICK(n_col_tiles); ATENIA_PICK(max_parts); ATENIA_PICK(wg_upper);
  ATENIA_PICK(n_cus); ATENIA_PICK(out_part_stride); ATENIA_PICK(part_flags);
#undef ATENIA_PICK
  return q;
}
__global__ __launch_bounds__(kThreads) void ffn_tiled_pipe_up2_kernel(TiledParams p, TiledParams ps,
                                                                      int n_first) {
  const bool second = (int)blockIdx.x >= n_first;
  const TiledParams q = pick_params(p, ps, second);
  pipe_tile<true, false>(q, second ? (int)blockIdx.x - n_first : (int)blockIdx.x);
}
// The same for the down phase (the caller puts the parameter set with the longer K first).
template <bool YB>
__global__ __launch_bounds__(kThreads) void ffn_tiled_pipe_down2_kernel(TiledParams p, TiledParams ps,
                                                                        int n_first) {
  const bool second = (int)blockIdx.x >= n_first;
  const TiledParams q = pick_params(p, ps, second);
  pipe_tile<false, YB>(q, second ? (int)blockIdx.x - n_first : (int)blockIdx.x);
}

// ---- INT8 W8A16 form of the pipelined kernel -----------------------------------------------
// Same tiling, A ring and k16-unit pipeline.  Weights stay int8 all the way into LDS: a B stage
// is 64 k = 16 stored blocks (16 KiB, one load instruction per block), so there is one barrier
// per 64 k.  A lane reads its 8 int8 of a fragment with one ds_read_b64 and widens them to
// bf16 in registers (exact: |q| <= 127) between the MFMAs of the unit before; the per-row scale
// multiplies the f32 accumulator in the epilogue.
__device__ inline void widen_i8x4(uint32_t w, uint32_t& lo, uint32_t& hi) {
  const float f0 = (float)(int8_t)(w & 0xff), f1 = (float)(int8_t)((w >> 8) & 0xff);
  const float f2 = (float)(int8_t)((w >> 16) & 0xff), f3 = (float)(int8_t)(w >> 24);
  // bf16 pair = high halves of two f32
  lo = __builtin_amdgcn_perm(__float_as_uint(f1), __float_as_uint(f0), 0x07060302u);
  hi = __builtin_amdgcn_perm(__float_as_uint(f3), __float_as_uint(f2), 0x07060302u);
}

template <bool UP>
__global__ __launch_bounds__(kThreads) void ffn_tiled_pipe_i8_kernel(TiledParams p) {
  constexpr int NA = kRingA, NB = 4;          // 64-k stages: A 32 KiB, B 16 KiB
  __shared__ uint4 S[NA * 2048 + NB * 1024];  // A ring, then B ring
  int wid, n_parts, part;  // k range `part` of `n_parts` (1 unless this is a split tail tile)
  if (!split_of_workgroup(p, (int)blockIdx.x, p.k_pad / 64, wid, n_parts, part)) return;
  int rt, ct;
  if (!tile_of_workgroup(p, wid, rt, ct)) return;

  const int e = p.tile_group[rt];
  const int tm0 = p.tile_m0[rt];
  const int base = p.g.offsets[e];
  const int cnt = p.g.offsets[e + 1] - base;
  const int rows_here = min(TM, cnt - tm0);

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int kh = lane >> 5, l32 = lane & 31;
  const int wm = wave >> 1, wn = wave & 1;
  constexpr int BROWS = UP ? 128 : 256;
  const int nb0 = ct * (BROWS / 16);

  // B: LDS chunk c of a stage holds the stored block of strip c (gate/up: chunks 0-7 gate
  // strips, 8-15 the matching up strips); wave w fills chunks 4w .. 4w+3.
  const uint4* bptr[4];
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const int c = wave * 4 + q;
    const uint4* wbase = (UP && c >= 8) ? p.wb : p.wa;
    int nb = nb0 + (UP ? (c & 7) : c);
    if (nb >= p.n_blocks) nb = p.n_blocks - 1;  // clamp: columns past N are never stored
    bptr[q] = wbase + (size_t)e * p.w_stride_u4 + (size_t)nb * p.nkb * 64 + lane;
  }
  // The first three B stages are requested before the row list is looked up (see the bf16
  // kernel).
  const int st0 = (p.k_pad / 64) * part / n_parts;
  const int nst = (p.k_pad / 64) * (part + 1) / n_parts - st0;  // 64-k stages of this k range
  const uint32_t sb_fill = (uint32_t)(uintptr_t)(lptr_t)S + NA * 32768 + wave * 4 * kChunk;
  auto dma_b = [&](int buf, int q, int t) {
    dma16(bptr[q] + (size_t)(st0 + t) * 64, sb_fill + buf * 16384 + q * kChunk);
  };
#pragma unroll
  for (int t = 0; t < 3; ++t)
#pragma unroll
    for (int q = 0; q < 4; ++q) dma_b(t, q, min(t, nst - 1));

  const uint16_t* arow[8];  // as in the bf16 kernel
  {
    const int r8 = lane >> 3, pslot = lane & 7;
#pragma unroll
    for (int q = 0; q < 8; ++q) {
      int m = (wave * 8 + q) * 8 + r8;
      if (m >= rows_here) m = 0;
      int src;
      if (UP) src = p.g.perm[base + tm0 + m] / p.g.pair_div;
      else src = base + tm0 + m;
      arow[q] = p.a + (size_t)src * p.a_stride + (pslot ^ r8 ^ (q & 1)) * 8;
    }
  }
  int aoff[4];
  {
    const int r8 = l32 & 7, cpar = (l32 >> 3) & 1;
    const int rowbase = (wm * 16 + (l32 >> 3)) * 64 + r8 * 8;
#pragma unroll
    for (int u = 0; u < 4; ++u) aoff[u] = rowbase + ((2 * u + kh) ^ r8 ^ cpar);
  }
  // B fragment j, k16 unit u, in 8-byte units: strip (2 * group + l32/16), slot 16u + l32%16 of
  // the block, half kh of the slot.
  const uint2* S2 = (const uint2*)S;
  const int boff0 = NA * 4096 + ((UP ? 2 * wn : 4 * wn) * 2 + (l32 >> 4)) * 128 + (l32 & 15) * 2 + kh;
  constexpr int kBJ1 = 256, kBJ2 = UP ? 1024 : 512, kBJ3 = UP ? 1280 : 768;

  f32x16 acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
  const int my_rows = rows_here - wm * 128;

  const uint32_t sa_fill = (uint32_t)(uintptr_t)(lptr_t)S + wave * 8 * kChunk;
  auto dma_a = [&](int buf, int q, int t) {
    dma16(arow[q] + (size_t)(st0 + t) * 64, sa_fill + buf * 32768 + q * kChunk);
  };
  auto read_frag = [&](int n, uint4 (&FA)[4], uint2 (&RB)[4], int a0, int b0) {
    switch (n) {
      case 0: FA[0] = S[a0]; break;
      case 1: RB[0] = S2[b0]; break;
      case 2: RB[1] = S2[b0 + kBJ1]; break;
      case 3: RB[2] = S2[b0 + kBJ2]; break;
      case 4: RB[3] = S2[b0 + kBJ3]; break;
      case 5: FA[1] = S[a0 + 256]; break;
      case 6: FA[2] = S[a0 + 512]; break;
      default: FA[3] = S[a0 + 768]; break;
    }
  };
  auto widen_half = [&](int n, const uint2 (&RB)[4], uint4 (&FB)[4]) {  // n = 2 * fragment + half
    if (n & 1) widen_i8x4(RB[n >> 1].y, FB[n >> 1].z, FB[n >> 1].w);
    else widen_i8x4(RB[n >> 1].x, FB[n >> 1].x, FB[n >> 1].y);
  };
  // One k16 unit: 16 MFMAs on (FA, FB).  Behind MFMA m < 8: read m of the next unit (B raw);
  // behind MFMA m >= 8: half a B fragment of the next unit is widened, and on even m a load
  // of the stage being refilled is issued (A: four per unit, B: two per unit).
  auto half = [&](auto mul_c, auto dma_c, auto dma_is_a_c, uint4 (&FA)[4], uint4 (&FB)[4],
                  uint4 (&NA_)[4], uint4 (&NB_)[4], int a0, int b0, int dbuf, int dt, auto q0_c) {
    constexpr int MUL = decltype(mul_c)::value;
    uint2 raw[4];
#pragma unroll
    for (int m = 0; m < 16; ++m) {
      const int i = m >> 2, j = m & 3;
      if (MUL == 2 || (MUL == 1 && i * 32 < my_rows)) acc[i][j] = mfma32(FA[i], FB[j], acc[i][j]);
      if (m < 8) read_frag(m, NA_, raw, a0, b0);
      else widen_half(m - 8, raw, NB_);
      if (decltype(dma_c)::value && m >= 8 && (m & 1) == 0) {
        if (decltype(dma_is_a_c)::value) dma_a(dbuf, decltype(q0_c)::value + ((m - 8) >> 1), dt);
        else if (m < 12) dma_b(dbuf, decltype(q0_c)::value + ((m - 8) >> 1), dt);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  using std::integral_constant;
  typedef integral_constant<bool, true> yes;
  typedef integral_constant<bool, false> no;

  // Iteration t (64 k) = units 0..3 of stage t.  Loads issued: unit 0: first half of A(t+2),
  // unit 1: first half of B(t+3), unit 2: second half of A(t+2), unit 3 (behind the barrier):
  // second half of B(t+3).  The barrier sits between units 2 and 3: by then this wave has
  // read all of stage t except unit 3 (already in registers), and waits for its loads of
  // stage t+1; younger loads then in flight: A(t+2) (8) and half of B(t+2), B(t+3) (2 + 2).
  auto run = [&](auto mul_c, auto la_c) {
    constexpr bool LA = decltype(la_c)::value;
    typedef integral_constant<int, 0> q0;
    typedef integral_constant<int, 2> q2;
    typedef integral_constant<int, 4> q4;
    uint4 fa0[4], fb0[4], fa1[4], fb1[4];
    auto fill_a = [&](int t) {
      if (LA) {
#pragma unroll
        for (int q = 0; q < 8; ++q) dma_a(t, q, min(t, nst - 1));
      }
    };
    // issued so far: B0 B1 B2; now A0 A1 (a wave that loads A rows then waits for all of it)
    fill_a(0); fill_a(1);
    wait_vm_lgkm0<LA ? 0 : 8>();
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    {
      uint2 raw[4];
#pragma unroll
      for (int n = 0; n < 8; ++n) read_frag(n, fa0, raw, aoff[0], boff0);
#pragma unroll
      for (int n = 0; n < 8; ++n) widen_half(n, raw, fb0);
    }
    int abuf = 0, bbuf = 0;
    for (int t = 0; t < nst; ++t) {
      const int abuf_n = abuf + 1 == NA ? 0 : abuf + 1;
      const int abuf_i = abuf == 0 ? NA - 1 : abuf - 1;
      const int bbuf_n = bbuf + 1 == NB ? 0 : bbuf + 1;
      const int bbuf_i = bbuf == 0 ? NB - 1 : bbuf - 1;
      const int ta = min(t + NA - 1, nst - 1), tb = min(t + NB - 1, nst - 1);
      const int a_cur = abuf * 2048, b_cur = boff0 + bbuf * 2048;
      half(mul_c, la_c, yes{}, fa0, fb0, fa1, fb1, aoff[1] + a_cur, b_cur + 32, abuf_i, ta, q0{});
      half(mul_c, yes{}, no{}, fa1, fb1, fa0, fb0, aoff[2] + a_cur, b_cur + 64, bbuf_i, tb, q0{});
      half(mul_c, la_c, yes{}, fa0, fb0, fa1, fb1, aoff[3] + a_cur, b_cur + 96, abuf_i, ta, q4{});
      wait_vm_lgkm0<LA ? 12 : 6>();
      asm volatile("" ::: "memory");
      __builtin_amdgcn_s_barrier();
      asm volatile("" ::: "memory");
      half(mul_c, yes{}, no{}, fa1, fb1, fa0, fb0, aoff[0] + abuf_n * 2048, boff0 + bbuf_n * 2048,
           bbuf_i, tb, q2{});
      abuf = abuf_n;
      bbuf = bbuf_n;
    }
    wait_vm_lgkm0<0>();
  };
  const bool loads_a = wave * 64 < rows_here;
  if (my_rows >= 97) run(integral_constant<int, 2>{}, yes{});
  else if (my_rows > 0) {
    if (loads_a) run(integral_constant<int, 1>{}, yes{});
    else run(integral_constant<int, 1>{}, no{});
  } else {
    if (loads_a) run(integral_constant<int, 0>{}, yes{});
    else run(integral_constant<int, 0>{}, no{});
  }

  if (UP) {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();  // every wave's loads have landed and its reads are done
    asm volatile("" ::: "memory");
    constexpr int kPitch = 144;
    char* stage = (char*)S + wave * (128 * kPitch);
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int n = min(nb0 * 16 + (2 * wn + j) * 32 + l32, p.n_rows - 1);
      const float sg = p.sa[(size_t)e * p.n_rows + n], su = p.sb[(size_t)e * p.n_rows + n];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
#pragma unroll
        for (int r = 0; r < 16; r += 2) {  // rows m and m + 1
          const int m = i * 32 + 8 * (r >> 2) + 4 * kh + (r & 3);
          const uint32_t hh =
              bf16_rne_pair(swiglu_fast(acc[i][j][r] * sg, acc[i][j + 2][r] * su),
                            swiglu_fast(acc[i][j][r + 1] * sg, acc[i][j + 2][r + 1] * su));
          char* dst = stage + m * kPitch + (j * 32 + l32) * 2;
          *(uint16_t*)dst = (uint16_t)hh;
          *(uint16_t*)(dst + kPitch) = (uint16_t)(hh >> 16);
        }
      }
    }
    uint16_t* h = (uint16_t*)p.out;
    const int n0 = nb0 * 16 + wn * 64;
    const int c8 = lane & 7, r8 = lane >> 3;
#pragma unroll
    for (int it = 0; it < 16; ++it) {
      const int m = it * 8 + r8;
      const uint4 v = *(const uint4*)(stage + m * kPitch + c8 * 16);
      const int mrow = wm * 128 + m;
      const int n = n0 + c8 * 8;
      if (mrow < rows_here && n < p.n_blocks * 16)
        *(uint4*)(h + (size_t)(base + tm0 + mrow) * p.out_stride + n) = v;
    }
  } else {
    float* y = (float*)p.out + (size_t)part * p.out_part_stride;
    float sd[4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
      sd[j] = p.sa[(size_t)e * p.n_rows + min(nb0 * 16 + (4 * wn + j) * 32 + l32, p.n_rows - 1)];
    int pair_of[4][16];  // all pair ids first, in one batch of loads (see the bf16 kernel)
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = wm * 128 + i * 32 + 8 * (r >> 2) + 4 * kh + (r & 3);
        pair_of[i][r] = p.g.perm[base + tm0 + min(m, rows_here - 1)];
      }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = wm * 128 + i * 32 + 8 * (r >> 2) + 4 * kh + (r & 3);
        if (m >= rows_here) continue;
        const int pair = pair_of[i][r];
        if (p.part_flags && part == 0 && wn == 0 && l32 == 0)
          p.part_flags[(size_t)pair * p.n_col_tiles + ct] = (uint8_t)n_parts;
        float* yr = y + (size_t)pair * p.out_stride;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int n = nb0 * 16 + (4 * wn + j) * 32 + l32;
          if (n < p.n_rows) yr[n] = acc[i][j][r] * sd[j];
        }
      }
    }
  }
}

template <bool UP>
hipError_t launch_tiled_pipe_i8(TiledParams p, int max_row_tiles, hipStream_t s) {
  int n_wg = max_row_tiles * p.n_col_tiles;
  n_wg = (n_wg + 7) / 8 * 8;
  p.wg_upper = n_wg;
  const int extra = p.max_parts > 1 ? p.n_cus : 0;  // room for the extra k ranges of a tail round
  ffn_tiled_pipe_i8_kernel<UP><<<n_wg + extra, kThreads, 0, s>>>(p);
  return hipGetLastError();
}

template <bool UP>
hipError_t launch_tiled_dma(TiledParams p, int max_row_tiles, hipStream_t s) {
  int n_wg = max_row_tiles * p.n_col_tiles;
  n_wg = (n_wg + 7) / 8 * 8;
  p.wg_upper = n_wg;
  const int extra = p.max_parts > 1 ? p.n_cus : 0;  // room for the extra k ranges of a tail round
  if (p.sa) {  // int8 values widened to bf16: scaled f32 results
    if (p.out_bf16 || (UP && !p.sb)) return hipErrorInvalidValue;
    ffn_tiled_pipe_kernel<UP, false, true><<<n_wg + extra, kThreads, 0, s>>>(p);
  } else if (!UP && p.out_bf16) {
    if (p.n_rows % 8) return hipErrorInvalidValue;  // a lane stores 8 columns at once
    ffn_tiled_pipe_kernel<false, true><<<n_wg + extra, kThreads, 0, s>>>(p);
  } else {
    ffn_tiled_pipe_kernel<UP><<<n_wg + extra, kThreads, 0, s>>>(p);
  }
  return hipGetLastError();
}

template <bool INT8, bool UP>
hipError_t launch_tiled(const TiledParams& p, int max_row_tiles, hipStream_t s) {
  static const hipError_t attr_rc =  // set once per instantiation, thread-safe
      hipFuncSetAttribute((const void*)ffn_tiled_kernel<INT8, UP>,
                          hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
  if (attr_rc != hipSuccess) return attr_rc;
  // Upper bound of the grid; workgroups past the real tile count return at once.
  int n_wg = max_row_tiles * p.n_col_tiles;
  n_wg = (n_wg + 7) / 8 * 8;
  ffn_tiled_kernel<INT8, UP><<<n_wg, kThreads, kLdsBytes, s>>>(p);
  return hipGetLastError();
}

}  // namespace

bool tiled_down_splits_tail(const WeightSet& down, int wdtype) {
  if (wdtype == ATENIA_MOE_WEIGHT_F32) return false;
  const bool int8 = wdtype == ATENIA_MOE_WEIGHT_INT8_W8A16;
  return int8 ? down.k_pad >= 128 : (down.k_pad % 64 == 0 && down.k_pad >= 128);
}

bool tiled_supported(const WeightSet& w, int wdtype) {
  if (wdtype == ATENIA_MOE_WEIGHT_F32) return false;
  if (w.group_blocks > 0) return false;  // per-group scales: streaming kernels only
  return w.k_pad % TK == 0;
}

namespace {
TiledParams up_params(const FfnArgs& a) {
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
  p.tile_rows = a.tile_rows;
  p.tile_li = a.tile_li;
  p.n_col_tiles = (a.gate.n_pad + 127) / 128;
  p.max_parts = 1;
  return p;
}
bool up_takes_pipe_bf16(const FfnArgs& a) {
  return a.use_tiled && !a.use_duo && a.wdtype != ATENIA_MOE_WEIGHT_INT8_W8A16 &&
         a.wdtype != ATENIA_MOE_WEIGHT_F32 && a.gate.group_blocks == 0 && a.gate.k_pad % 64 == 0 &&
         a.gate.k_pad >= 128 && (!a.tall_tiles || (a.tile_rows && a.tile_li)) && !a.gate.scale;
}
}  // namespace

// Routed experts and a shared expert in one gate/up launch (ffn_tiled_pipe_up2_kernel): both on
// the bf16 pipelined kernel.
bool tiled_up_pair_supported(const FfnArgs& a, const FfnArgs& shared) {
  return up_takes_pipe_bf16(a) && up_takes_pipe_bf16(shared);
}
hipError_t launch_ffn_up_tiled_pair(const FfnArgs& a, const FfnArgs& shared, hipStream_t s) {
  if (!tiled_up_pair_supported(a, shared)) return hipErrorInvalidValue;
  TiledParams p = up_params(a), ps = up_params(shared);
  int n1 = a.max_row_tiles * p.n_col_tiles, n2 = shared.max_row_tiles * ps.n_col_tiles;
  n1 = (n1 + 7) / 8 * 8;  // whole rounds over the 8 XCDs: the second part starts on XCD 0 again
  n2 = (n2 + 7) / 8 * 8;
  p.wg_upper = n1;
  ps.wg_upper = n2;
  ffn_tiled_pipe_up2_kernel<<<n1 + n2, kThreads, 0, s>>>(p, ps, n1);
  return hipGetLastError();
}

hipError_t launch_ffn_up_tiled(const FfnArgs& a, hipStream_t s) {
  const bool int8 = a.wdtype == ATENIA_MOE_WEIGHT_INT8_W8A16;
  TiledParams p = up_params(a);
  const bool pipe_bf16 = !int8 && p.k_pad % 64 == 0 && p.k_pad >= 128;
  // A list of nine-group tiles in any other kernel would lose the rows past 256 of such a tile.
  if (a.tall_tiles && (!pipe_bf16 || a.use_duo || !p.tile_rows || !p.tile_li)) return hipErrorInvalidValue;
  if (a.use_duo) {
    if (!pipe_bf16 || p.sa) return hipErrorInvalidValue;
    p.tile_rows = nullptr;
    p.tile_li = nullptr;
    p.n_cus = a.n_cus;
    return launch_tiled_duo_up(p, a.max_row_tiles, s);
  }
  if (pipe_bf16) return launch_tiled_dma<true>(p, a.max_row_tiles, s);
  if (!int8 && p.sa) return hipErrorInvalidValue;  // scaled bf16 values: that kernel only
  if (int8 && p.k_pad >= 128) return launch_tiled_pipe_i8<true>(p, a.max_row_tiles, s);
  return int8 ? launch_tiled<true, true>(p, a.max_row_tiles, s)
              : launch_tiled<false, true>(p, a.max_row_tiles, s);
}

namespace {
TiledParams down_params(const FfnArgs& a) {
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
  p.tile_rows = a.tile_rows;
  p.tile_li = a.tile_li;
  p.n_col_tiles = (a.down.n_pad + 255) / 256;
  p.max_parts = 1;
  return p;
}
// k split of the tail round (pipelined kernels; see split_of_workgroup)
void down_split_params(const FfnArgs& a, TiledParams& p) {
  if (a.y_parts > 1 && a.part_flags && a.n_cus >= 8) {
    p.max_parts = a.y_parts;
    p.n_cus = a.n_cus / 8 * 8;
    p.out_part_stride = a.y_part_stride;
    p.part_flags = a.part_flags;
  }
}
bool down_takes_pipe_bf16(const FfnArgs& a) {
  return a.use_tiled && !a.use_duo && a.wdtype != ATENIA_MOE_WEIGHT_INT8_W8A16 &&
         a.wdtype != ATENIA_MOE_WEIGHT_F32 && a.down.group_blocks == 0 && a.down.k_pad % 64 == 0 &&
         a.down.k_pad >= 128 && (!a.tall_tiles || (a.tile_rows && a.tile_li)) &&
         (!a.y_bf16 || a.down.n_rows % 8 == 0) && !a.down.scale;
}
}  // namespace

bool tiled_down_pair_supported(const FfnArgs& first, const FfnArgs& second) {
  return down_takes_pipe_bf16(first) && down_takes_pipe_bf16(second) && !first.y_bf16 == !second.y_bf16;
}
hipError_t launch_ffn_down_tiled_pair(const FfnArgs& first, const FfnArgs& second, hipStream_t s) {
  if (!tiled_down_pair_supported(first, second)) return hipErrorInvalidValue;
  TiledParams p1 = down_params(first), p2 = down_params(second);
  p1.out_bf16 = first.y_bf16;
  p2.out_bf16 = second.y_bf16;
  down_split_params(first, p1);
  down_split_params(second, p2);
  int n1 = first.max_row_tiles * p1.n_col_tiles, n2 = second.max_row_tiles * p2.n_col_tiles;
  n1 = (n1 + 7) / 8 * 8;
  n2 = (n2 + 7) / 8 * 8;
  p1.wg_upper = n1;
  p2.wg_upper = n2;
  const int e1 = p1.max_parts > 1 ? p1.n_cus : 0, e2 = p2.max_parts > 1 ? p2.n_cus : 0;
  if (first.y_bf16) ffn_tiled_pipe_down2_kernel<true><<<n1 + e1 + n2 + e2, kThreads, 0, s>>>(p1, p2, n1 + e1);
  else ffn_tiled_pipe_down2_kernel<false><<<n1 + e1 + n2 + e2, kThreads, 0, s>>>(p1, p2, n1 + e1);
  return hipGetLastError();
}

hipError_t launch_ffn_down_tiled(const FfnArgs& a, hipStream_t s) {
  const bool int8 = a.wdtype == ATENIA_MOE_WEIGHT_INT8_W8A16;
  TiledParams p = down_params(a);
  const bool pipelined = int8 ? p.k_pad >= 128 : (p.k_pad % 64 == 0 && p.k_pad >= 128);
  const bool pipe_bf16 = !int8 && pipelined;
  if (a.tall_tiles && (!pipe_bf16 || a.use_duo || !p.tile_rows || !p.tile_li)) return hipErrorInvalidValue;
  if (a.y_bf16 && !pipe_bf16) return hipErrorInvalidValue;  // only those kernels store bf16
  p.out_bf16 = a.y_bf16;
  if (a.use_duo) {
    // no k split of tail tiles in this form: the caller passes y_parts <= 1
    if (!pipe_bf16 || p.sa || (a.y_parts > 1 && a.part_flags)) return hipErrorInvalidValue;
    p.tile_rows = nullptr;
    p.tile_li = nullptr;
    p.n_cus = a.n_cus;
    return launch_tiled_duo_down(p, a.max_row_tiles, s);
  }
  if (pipelined) down_split_params(a, p);
  if (!int8 && p.k_pad % 64 == 0 && p.k_pad >= 128) return launch_tiled_dma<false>(p, a.max_row_tiles, s);
  if (!int8 && p.sa) return hipErrorInvalidValue;  // scaled bf16 values: that kernel only
  if (int8 && p.k_pad >= 128) return launch_tiled_pipe_i8<false>(p, a.max_row_tiles, s);
  return int8 ? launch_tiled<true, false>(p, a.max_row_tiles, s)
              : launch_tiled<false, false>(p, a.max_row_tiles, s);
}

}  // namespace atenia_moe
