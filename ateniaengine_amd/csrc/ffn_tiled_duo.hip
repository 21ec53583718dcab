// Kernel 3, tiled form for experts with a short K: two workgroups per compute unit.
//
//   gate/up : H[rows of e, f] = silu(X_e W_g^T) * (X_e W_u^T)     (src/moe/dense.rs:253-266)
//   down    : Y[rows of e, d] = H_e W_d^T                         (src/moe/dense.rs:267-269)
// on v_mfma_f32_32x32x16_bf16 with f32 accumulation, bf16 weights, K a multiple of 64.
//
// The pipelined kernel of ffn_tiled.hip gives a wave a 128 x 128 block (256 accumulation
// registers), so one workgroup fills a compute unit and everything a tile does besides its
// matrix instructions -- the look-ups from workgroup id to token rows, the first loads' latency,
// SwiGLU and the stores of the epilogue -- runs with the matrix pipes idle.  That fixed part is a
// fifth of a tile whose K is 4096 and more than a third when K is 1408 or 2048 (and the f32
// stores of a down tile alone take as long as 1400 k of matrix instructions).  Here a workgroup
// owns 128 rows x 256 weight rows, a wave 64 x 128 (128 accumulation registers, 256 registers in
// all) and 80 KiB of LDS, so TWO workgroups share a compute unit and one's prologue, epilogue
// and load stalls run under the other's main loop.  The price is operand traffic: a wave reads
// 6 fragments from LDS per 8 matrix instructions instead of 8 per 16 and a compute unit copies
// every weight tile into LDS twice; with every stall hidden the loop sustains about 0.87 of the
// big tile's rate (measured on this device with the loop alone), which is why the long-K shapes
// keep the big tile.
//
// Row tiles come from the same 256-row tile list: a workgroup takes rows sub * 128 .. of tile rt
// (sub = 0, 1; a workgroup whose half holds no rows returns at once).  LDS: a ring of two 64-k A
// stages (16 KiB each, chunks of 8 rows x 128 bytes, swizzled as in the pipelined kernel) and a
// ring of three 32-k B stages (16 KiB each), filled with global_load_lds_dwordx4.
#include "ffn_tiled_common.h"

#include "../../include/atenia_moe_hip.h"

namespace atenia_moe {

namespace {

constexpr int kDuoRows = 128;   // token rows per workgroup
constexpr int kDuoSub = kTileM / kDuoRows;
constexpr int kDuoNA = 2;       // A stages of 64 k
constexpr int kDuoNB = 3;       // B stages of 32 k
constexpr int kDuoStage = 1024; // uint4 per stage (A and B alike): 16 KiB

// YB (down phase only): y leaves as bf16 (TiledParams::out_bf16), staged through LDS.
template <bool UP, bool YB = false>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(2, 2)))
void ffn_tiled_duo_kernel(TiledParams p) {
  constexpr int NA = kDuoNA, NB = kDuoNB;
  __shared__ uint4 S[(NA + NB) * kDuoStage];  // A ring, then B ring: 80 KiB
  int rt, sub, ct;
  if (!tile_of_workgroup_sub<kDuoSub>(p, blockIdx.x, rt, sub, ct)) return;

  const int e = p.tile_group[rt];
  const int base = p.g.offsets[e];
  const int cnt = p.g.offsets[e + 1] - base;
  const int tile_m0 = p.tile_m0[rt];
  const int tm0 = tile_m0 + sub * kDuoRows;
  const int rows_here = min(kDuoRows, min(TM, cnt - tile_m0) - sub * kDuoRows);
  if (rows_here <= 0) return;

  const int tid = threadIdx.x, lane = tid & 63;
  // scalar wave id: guards around MFMAs must be scalar branches (MFMA does not obey EXEC)
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int kh = lane >> 5, l32 = lane & 31;
  const int wm = wave >> 1, wn = wave & 1;
  constexpr int BROWS = UP ? 128 : 256;
  const int nb0 = ct * (BROWS / 16);

  // B: wave w fills row groups 2w, 2w + 1 (32 weight rows each; gate/up: groups 0-3 gate, 4-7 the
  // matching up rows) of a stage, one chunk per group and k16 half.
  const uint4* bptr[2];
#pragma unroll
  for (int q = 0; q < 2; ++q) {
    const int ng = wave * 2 + q;
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
  const int nks = p.k_pad / 32;  // 32-k steps
  const int nst = nks / 2;       // 64-k stages
  const uint32_t lds0 = (uint32_t)(uintptr_t)(lptr_t)S;
  const uint32_t sb_fill = lds0 + NA * kDuoStage * 16 + wave * 4 * kChunk;
  auto dma_b = [&](int buf, int q, int ks) {  // q = 2 * row group + k half
    dma16(bptr[q >> 1] + (size_t)ks * 64 + 32 * (q & 1), sb_fill + buf * (kDuoStage * 16) + q * kChunk);
  };
  // The first weight stages need nothing but the tile coordinates: they fly while the row list
  // is looked up.
#pragma unroll
  for (int t = 0; t < NB; ++t)
#pragma unroll
    for (int q = 0; q < 4; ++q) dma_b(t, q, min(t, nks - 1));

  // A stage: 128 rows x 64 k as 16 chunks of 8 rows x 128 bytes.  Row r, 16-byte segment s of
  // chunk c sits at slot 8r + (s ^ r ^ (c & 1)); wave w fills chunks 4w .. 4w + 3.  Rows past the
  // end of the tile load row 0 again (computed, never stored), so every wave issues the same loads.
  const uint16_t* arow[4];
  {
    const int r8 = lane >> 3, pslot = lane & 7;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      int m = (wave * 4 + q) * 8 + r8;
      if (m >= rows_here) m = 0;
      int src;
      if (UP) src = p.g.perm[base + tm0 + m] / p.g.pair_div;
      else src = base + tm0 + m;
      arow[q] = p.a + (size_t)src * p.a_stride + (pslot ^ r8 ^ (q & 1)) * 8;
    }
  }
  const uint32_t sa_fill = lds0 + wave * 4 * kChunk;
  auto dma_a = [&](int buf, int q, int t) {  // chunk q of this wave, 64-k stage t
    dma16(arow[q] + (size_t)t * 64, sa_fill + buf * (kDuoStage * 16) + q * kChunk);
  };
  // fragment read offsets (uint4 units inside a stage): row group i adds 256, k16 unit u of the
  // 64-k stage selects the swizzled segment; B row group j of this wave, unit u adds 64.
  int aoff[4];
  {
    const int r8 = l32 & 7, cpar = (l32 >> 3) & 1;
    const int rowbase = (wm * 8 + (l32 >> 3)) * 64 + r8 * 8;
#pragma unroll
    for (int u = 0; u < 4; ++u) aoff[u] = rowbase + ((2 * u + kh) ^ r8 ^ cpar);
  }
  const int boff0 = NA * kDuoStage + (UP ? 2 * wn : 4 * wn) * 128 + lane;
  constexpr int kBJ1 = 128, kBJ2 = UP ? 512 : 256, kBJ3 = UP ? 640 : 384;

  f32x16 acc[2][4];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
  const int my_rows = rows_here - wm * 64;

  // the 6 fragment reads of one k16 unit, in the order the MFMAs consume them
  auto read_frag = [&](int n, uint4 (&FA)[2], uint4 (&FB)[4], int a0, int b0) {
    switch (n) {
      case 0: FA[0] = S[a0]; break;
      case 1: FB[0] = S[b0]; break;
      case 2: FB[1] = S[b0 + kBJ1]; break;
      case 3: FB[2] = S[b0 + kBJ2]; break;
      case 4: FB[3] = S[b0 + kBJ3]; break;
      default: FA[1] = S[a0 + 256]; break;
    }
  };
  using std::integral_constant;
  // One k16 unit: 8 MFMAs on (FA, FB); behind MFMA m < 6 goes read m of the next unit, behind
  // MFMAs 4..7 one load each of the stage being refilled (DMA: 0 none, 1 A chunks, 2 B chunks).
  auto half = [&](auto mul_c, auto dma_c, uint4 (&FA)[2], uint4 (&FB)[4], uint4 (&NA_)[2],
                  uint4 (&NB_)[4], int a0, int b0, int dbuf, int dks) {
    constexpr int MUL = decltype(mul_c)::value;
    constexpr int DMA = decltype(dma_c)::value;
#pragma unroll
    for (int m = 0; m < 8; ++m) {
      const int i = m >> 2, j = m & 3;
      if (MUL == 2 || (MUL == 1 && i == 0)) acc[i][j] = mfma32(FA[i], FB[j], acc[i][j]);
      if (m < 6) read_frag(m, NA_, NB_, a0, b0);
      if (DMA == 1 && m >= 4) dma_a(dbuf, m - 4, dks);
      if (DMA == 2 && m >= 4) dma_b(dbuf, m - 4, dks);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  typedef integral_constant<int, 0> dma_none;
  typedef integral_constant<int, 1> dma_a_c;
  typedef integral_constant<int, 2> dma_b_c;

  // Stage t = steps 2t (k16 units 0, 1 of the A stage) and 2t + 1 (units 2, 3).  Step s:
  //   first half : multiplies the first unit, reads the second; the even step issues A(t + 1)
  //                into the other A buffer (free since the middle of step 2t - 1)
  //   middle     : waits until this wave's loads of B(s + 1) -- and, in an odd step, of A(t + 1)
  //                -- have landed, barrier
  //   second half: multiplies the second unit, reads the first unit of step s + 1; issues
  //                B(s + NB) into the B buffer of step s
  // A wave's loads complete in issue order: ... B(s+1) B(s+2) A(t+1) | middle of even step s,
  // ... B(s+1) A(t+1) B(s+2) | middle of odd step s: two groups of four loads may stay in flight
  // behind the even wait, one behind the odd one.  Stages past the end of k are clamped to the
  // last one (they land in buffers nobody reads) so that the counts stay uniform.
  auto run = [&](auto mul_c) {
    uint4 fa0[2], fb0[4], fa1[2], fb1[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) dma_a(0, q, 0);
#pragma unroll
    for (int q = 0; q < 4; ++q) dma_a(1, q, min(1, nst - 1));
    wait_vm_lgkm0<0>();
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
#pragma unroll
    for (int n = 0; n < 6; ++n) read_frag(n, fa0, fb0, aoff[0], boff0);
    int abuf = 0, bbuf = 0;  // buffers of the stages step s reads
    for (int s = 0; s < nks; s += 2) {
      const int abuf_n = abuf ^ 1;
      const int ta = min(s / 2 + 1, nst - 1);
      {
        const int bbuf_n = bbuf + 1 == NB ? 0 : bbuf + 1;
        half(mul_c, dma_a_c{}, fa0, fb0, fa1, fb1, aoff[1] + abuf * kDuoStage,
             boff0 + bbuf * kDuoStage + 64, abuf_n, ta);
        wait_vm_lgkm0<8>();
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        half(mul_c, dma_b_c{}, fa1, fb1, fa0, fb0, aoff[2] + abuf * kDuoStage,
             boff0 + bbuf_n * kDuoStage, bbuf, min(s + NB, nks - 1));
        bbuf = bbuf_n;
      }
      {
        const int bbuf_n = bbuf + 1 == NB ? 0 : bbuf + 1;
        half(mul_c, dma_none{}, fa0, fb0, fa1, fb1, aoff[3] + abuf * kDuoStage,
             boff0 + bbuf * kDuoStage + 64, 0, 0);
        wait_vm_lgkm0<4>();
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        half(mul_c, dma_b_c{}, fa1, fb1, fa0, fb0, aoff[0] + abuf_n * kDuoStage,
             boff0 + bbuf_n * kDuoStage, bbuf, min(s + 1 + NB, nks - 1));
        bbuf = bbuf_n;
      }
      abuf = abuf_n;
    }
    wait_vm_lgkm0<0>();
  };
  // (Two workgroups that start together on a compute unit do not stay in step: delaying the one
  // in the second wave slot of its SIMDs by 0 to 1.5 main loops in the first round measured the
  // same to 0.5 %, so nothing is staggered.)
  if (my_rows > 32) run(integral_constant<int, 2>{});
  else if (my_rows > 0) run(integral_constant<int, 1>{});
  else run(integral_constant<int, 0>{});

  if (UP) {
    // silu(g) * u, rounded to bf16, staged through LDS so that every global store is a full
    // 128-byte line: the wave's 64 x 64 block goes to its own region with a row pitch of 144
    // bytes and is read back 16 bytes per lane, 8 lanes per row.
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();  // every wave's loads have landed and its reads are done
    asm volatile("" ::: "memory");
    constexpr int kPitch = 144;
    char* stage = (char*)S + wave * (64 * kPitch);
#pragma unroll
    for (int j = 0; j < 2; ++j) {
#pragma unroll
      for (int i = 0; i < 2; ++i) {
#pragma unroll
        for (int r = 0; r < 16; r += 2) {  // rows m and m + 1
          const int m = i * 32 + 8 * (r >> 2) + 4 * kh + (r & 3);
          const uint32_t hh = bf16_rne_pair(swiglu_fast(acc[i][j][r], acc[i][j + 2][r]),
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
    for (int it = 0; it < 8; ++it) {
      const int m = it * 8 + r8;
      const uint4 v = *(const uint4*)(stage + m * kPitch + c8 * 16);
      const int mrow = wm * 64 + m;
      const int n = n0 + c8 * 8;
      if (mrow < rows_here && n < p.n_blocks * 16)
        *(uint4*)(h + (size_t)(base + tm0 + mrow) * p.out_stride + n) = v;
    }
  } else if (YB) {
    // y as bf16, staged through LDS like h above: the wave's 64 x 128 block goes to its own region
    // with a row pitch of 272 bytes and is read back 16 lanes per row, 4 rows at a time, so that
    // a row's 256 bytes leave as two full lines.
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    constexpr int kPitch = 272;
    char* stage = (char*)S + wave * (64 * kPitch);
    const int r4 = lane >> 4, c16 = lane & 15;
    int pair_of[16];  // pair id of the rows this lane stores
#pragma unroll
    for (int it = 0; it < 16; ++it) {
      const int m = wm * 64 + it * 4 + r4;
      pair_of[it] = p.g.perm[base + tm0 + min(m, rows_here - 1)];
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) {
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
    uint16_t* yb = (uint16_t*)p.out;
    const int n = nb0 * 16 + wn * 128 + c16 * 8;
#pragma unroll
    for (int it = 0; it < 16; ++it) {
      const int m = it * 4 + r4;
      const uint4 v = *(const uint4*)(stage + m * kPitch + c16 * 16);
      if (wm * 64 + m < rows_here && n < p.n_rows)
        *(uint4*)(yb + (size_t)pair_of[it] * p.out_stride + n) = v;
    }
  } else {
    float* y = (float*)p.out;
    // The pair id of every row first, in one batch of loads (fetched next to the stores they
    // address, each would wait out its own L2 round trip).
    int pair_of[2][16];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = wm * 64 + i * 32 + 8 * (r >> 2) + 4 * kh + (r & 3);
        pair_of[i][r] = p.g.perm[base + tm0 + min(m, rows_here - 1)];
      }
#pragma unroll
    for (int i = 0; i < 2; ++i) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = wm * 64 + i * 32 + 8 * (r >> 2) + 4 * kh + (r & 3);
        if (m >= rows_here) continue;
        float* yr = y + (size_t)pair_of[i][r] * p.out_stride;
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
hipError_t launch_duo(TiledParams p, int max_row_tiles, hipStream_t s) {
  if (!tiled_duo_supported(p)) return hipErrorInvalidValue;
  int n_wg = max_row_tiles * kDuoSub * p.n_col_tiles;
  n_wg = (n_wg + 7) / 8 * 8;
  if (!UP && p.out_bf16) {
    if (p.n_rows % 8) return hipErrorInvalidValue;  // a lane stores 8 columns at once
    ffn_tiled_duo_kernel<false, true><<<n_wg, kThreads, 0, s>>>(p);
  } else {
    ffn_tiled_duo_kernel<UP><<<n_wg, kThreads, 0, s>>>(p);
  }
  return hipGetLastError();
}

}  // namespace

// bf16 blocks, K in whole 64-k stages (at least two), row tiles of at most 256 rows, no k split.
bool tiled_duo_supported(const TiledParams& p) {
  return p.k_pad % 64 == 0 && p.k_pad >= 128 && p.tile_rows == nullptr && p.tile_li == nullptr &&
         p.max_parts <= 1;
}

hipError_t launch_tiled_duo_up(const TiledParams& p, int max_row_tiles, hipStream_t s) {
  return launch_duo<true>(p, max_row_tiles, s);
}

hipError_t launch_tiled_duo_down(const TiledParams& p, int max_row_tiles, hipStream_t s) {
  return launch_duo<false>(p, max_row_tiles, s);
}

}  // namespace atenia_moe
