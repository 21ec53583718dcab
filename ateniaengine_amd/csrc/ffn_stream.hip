// Kernel 3, weight-streaming form: grouped SwiGLU expert projections for small row counts
// (decode).  Computes, per expert e and per row of tokens routed to it,
//   gate = W_g x, up = W_u x, h = silu(gate) * up        (src/moe/dense.rs:253-266)
//   y    = W_d h                                          (src/moe/dense.rs:267-269)
// with bf16 MFMA (f32 accumulate).  INT8 W8A16 weights (per-output-row scales,
// src/tensor/disk_tier.rs:231-259) are widened to bf16 in registers -- an int8 value is exact
// in bf16 -- and the row scale is applied to the f32 accumulator, which equals
// sum_k (q*scale) x_k of the reference's dequantised weight up to f32 rounding.
//
// The bound here is HBM: every weight byte of an active expert is read exactly once per
// launch, straight from global memory into the MFMA B-operand registers (the weights are
// stored in that register layout, see moe_internal.h), 1 KiB per wave per load, several
// loads in flight.  A workgroup owns one or two adjacent 16-row strips of W_g and W_u (four
// waves) or of W_d (eight waves); its waves split K and reduce through LDS.  Token rows (A
// operand) come from L2.
//
// Kernels: ffn_stream_kernel (any small batch, either phase; its SEL form also routes a single
// token from the router's logits), ffn_mid_kernel (batches whose experts see a few dozen rows
// each: the token rows of a workgroup's eight or four waves go through LDS, up to 128 rows of an
// expert per pass over its weights), ffn_down_decode1_kernel and ffn_down_combine1_kernel (one
// token: the down projections of all its experts, of the shared expert, and the combine in one
// launch), repack_blocks_kernel (load-time repack into the block layout).
#include "moe_internal.h"

#include <type_traits>

#include "../../include/atenia_moe_hip.h"

namespace atenia_moe {

namespace {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;


struct StreamParams {
  const uint4* wa;      // gate (up phase) or down blocks
  const uint4* wb;      // up blocks (up phase only)
  const float* sa;      // int8 row scales of wa, [G, n_rows]; per-group: [G][n_kgroups][n_pad]
  const float* sb;
  int group_blocks;     // per-group int8: 64-k blocks per scale group (0 = per-row scales)
  int n_kgroups;        // per-group int8: scale groups along K
  int64_t w_stride_u4;  // uint4 between experts
  int n_rows;           // unpadded N
  int n_pad;            // N padded to whole 16-row strips
  int nkb;              // K blocks per strip
  const uint16_t* a;    // bf16 rows: x [T, a_stride] (up) or h [rows, a_stride] (down)
  int a_stride;
  void* out;            // up: h bf16 [rows, out_stride]; down: y f32 [pairs, out_stride]
  int out_stride;
  GroupDesc g;
  InlineSelect sel;     // gate/up launch of a single token that routes it itself (logits != null)
  int mid_rot;          // mid-batch kernel: workgroups start their walk over K at different stages
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
  // |q| <= 128 is exact in bf16, so dropping the low 16 bits loses nothing: one byte permute
  // takes the high halves of both floats (bytes 2, 3 of f0 below bytes 2, 3 of f1).
  return __builtin_amdgcn_perm(__float_as_uint(f1), __float_as_uint(f0), 0x07060302u);
}
__device__ inline void widen_i8x16(uint4 q, bf16x8& lo, bf16x8& hi) {
  uint4 l, h;
  l.x = pack_i8_pair(q.x, 0);
  l.y = pack_i8_pair(q.x, 16);
  l.z = pack_i8_pair(q.y, 0);
  l.w = pack_i8_pair(q.y, 16);
  h.x = pack_i8_pair(q.z, 0);
  h.y = pack_i8_pair(q.z, 16);
  h.z = pack_i8_pair(q.w, 0);
  h.w = pack_i8_pair(q.w, 16);
  lo = *(bf16x8*)&l;
  hi = *(bf16x8*)&h;
}

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
// Streaming (non-temporal) 16-byte load: the weights are read once per launch.
__device__ inline uint4 load_stream(const uint4* p) {
  u32x4 v = __builtin_nontemporal_load((const u32x4*)p);
  return make_uint4(v.x, v.y, v.z, v.w);
}

__device__ inline f32x4 mfma(uint4 a, uint4 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(*(bf16x8*)&a, *(bf16x8*)&b, c, 0, 0, 0);
}
__device__ inline f32x4 mfma(bf16x8 a, bf16x8 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}

// MT  : 16-row tiles of tokens held per workgroup (1 or 2)
// INT8: weights are int8 blocks (64 k per block) instead of bf16 blocks (32 k per block)
// UP  : gate/up phase with SwiGLU epilogue, else down phase
// WAVES: waves per workgroup = K slices of the strip
// PG  : int8 with one scale per output row and k group (Q8_0-style): every 64-k block is
//       accumulated on its own and added to the running sum times the scale of its group,
//       sum_g s[n, g] * (sum_{k in g} q[n, k] x[k]), which is the reference's
//       sum_k (q * s) x (src/tensor/quantizer.rs:175-248) up to f32 rounding
// A second parameter set rides along for the shared expert: the workgroups with blockIdx.y ==
// shared_y stream the shared expert's strips (its own weights, width, input and output rows)
// in the same launch as the routed experts', one launch less per phase for layers that have one.
// S  : adjacent 16-row strips per workgroup (1 or 2).  With two, a wave multiplies the token
//      rows it loaded with the blocks of both strips, which halves the activation traffic from
//      L2 per weight byte -- what the streaming rate falls with once an expert has more than 16 rows.
// SEL : single-token gate/up launch that also routes the token (p.sel); a form of its own
//       because the f64 softmax doubles the register count of the whole kernel
template <int MT, bool INT8, bool UP, int WAVES, bool PG, int S = 1, bool SEL = false>
__global__ __launch_bounds__(64 * WAVES) void ffn_stream_kernel(StreamParams p_routed,
                                                                StreamParams p_shared,
                                                                int shared_y) {
  constexpr int kWavesPerWg = WAVES;
  const bool sh = (int)blockIdx.y == shared_y;
  const StreamParams& p = sh ? p_shared : p_routed;
  if ((int)blockIdx.x * 16 * S >= p.n_pad) return;  // the grid spans the wider of the two
  // shared_y == 0: the shared expert comes first in the grid and the routed groups follow
  const int u = sh ? 0 : (int)blockIdx.y - (shared_y == 0 ? 1 : 0);
  int e, base, cnt;
  if (SEL && !sh) {
    // One token whose routing is still open: every wave derives it from the logits (the same
    // bits in all of them), group u is the u-th selected expert, and one wave of the launch
    // writes routing and grouping down for the launches that follow.
    const int ln = threadIdx.x & 63;
    const WaveRouting wr = wave_softmax_topk(p.sel.logits, p.sel.E, p.sel.k, p.sel.renorm, ln);
    if (blockIdx.x == 0 && blockIdx.y == 0 && blockIdx.z == 0 && threadIdx.x < 64)
      wave_write_routing(p.sel, wr, ln);
    e = wave_selected_expert(wr.mask, u);
    if (e < 0 || u >= p.sel.k) return;
    base = u;
    cnt = 1;
  } else if (p.g.idx1) {  // one token: group u is its u-th expert, row u
    if (u >= p.g.pair_div) return;
    e = p.g.idx1[u];
    base = u;
    cnt = 1;
  } else {
    if (u >= *p.g.n_active) return;
    e = p.g.active[u];
    base = p.g.offsets[e];
    cnt = p.g.offsets[e + 1] - base;
  }
  const int m0 = blockIdx.z * 16 * MT;
  if (m0 >= cnt) return;
  // 16-row tiles of this slice that hold rows.  The others are not loaded: their A registers
  // stay zero and their MFMAs run on zeros.  (The MFMAs are deliberately not branched around:
  // with a branch between an MFMA and the VALU instruction that reads its result, hipcc 7.2
  // leaves out the wait states on the taken path and the per-group form read stale sums.)
  const int mt_live = min(MT, (cnt - m0 + 15) >> 4);
  const int nb = blockIdx.x * S;  // first strip; n_pad is a multiple of 16 * S (launcher)
  // The wave id as a scalar: everything derived from it (k range, loop bounds, the guards around
  // the MFMAs) is then a scalar branch.  Left as a vector value the compiler predicates those
  // guards through EXEC, which MFMA instructions do not obey.
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int kq = lane >> 4, mm = lane & 15;
  constexpr int KB = INT8 ? kKbInt8 : kKbBf16;  // k per block
  constexpr int NACC = UP ? 2 : 1;

  const int kb_per = (p.nkb + kWavesPerWg - 1) / kWavesPerWg;
  const int kb0 = wave * kb_per;
  const int kb1 = min(p.nkb, kb0 + kb_per);
  const uint4* pa = p.wa + (size_t)e * p.w_stride_u4 + (size_t)nb * p.nkb * 64 + lane;
  const uint4* pb = UP ? p.wb + (size_t)e * p.w_stride_u4 + (size_t)nb * p.nkb * 64 + lane
                       : nullptr;
  const size_t strip_u4 = (size_t)p.nkb * 64;  // uint4 between adjacent strips

  // Software pipeline over batches of U weight blocks with two register buffers: the loads
  // of batch i+1 are in flight while batch i is multiplied.  The first batch is requested
  // before the dependent look-ups (perm -> token row) below, so the weight stream starts one
  // memory latency after the workgroup does.
  constexpr int U = INT8 ? (MT == 1 && S == 1 && !PG ? 4 : 2) : 4;  // blocks per batch
  constexpr int AV = INT8 ? 2 : 1;       // 16-byte activation pieces per block and row tile
  uint4 wA0[S][U], wB0[S][UP ? U : 1], wA1[S][U], wB1[S][UP ? U : 1];
  uint4 xa0[U][MT][AV], xa1[U][MT][AV];
#pragma unroll
  for (int j = 0; j < U; ++j)
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
      for (int v = 0; v < AV; ++v) xa0[j][i][v] = xa1[j][i][v] = make_uint4(0u, 0u, 0u, 0u);
  // Per-group scales of this lane's output row (column mm of the D layout), one per k group;
  // they are requested together with the weight blocks they belong to.
  const size_t n_pad_s = (size_t)p.n_pad;  // scale rows per k group
  const float* psa = PG ? p.sa + (size_t)e * p.n_kgroups * n_pad_s + nb * 16 + mm : nullptr;
  const float* psb = PG && UP ? p.sb + (size_t)e * p.n_kgroups * n_pad_s + nb * 16 + mm : nullptr;
  constexpr int SP = PG ? S : 1, UA = PG ? U : 1, UB = PG && UP ? U : 1;
  float sA0[SP][UA], sB0[SP][UB], sA1[SP][UA], sB1[SP][UB];
  auto load_w = [&](uint4 (&wa)[S][U], uint4 (&wb)[S][UP ? U : 1], float (&sa)[SP][UA],
                    float (&sb)[SP][UB], int kb) {
#pragma unroll
    for (int j = 0; j < U; ++j) {
      const int kk = min(kb + j, kb1 - 1);  // clamped: a batch past the end is loaded, not used
#pragma unroll
      for (int t = 0; t < S; ++t) {
        wa[t][j] = load_stream(pa + t * strip_u4 + (size_t)kk * 64);
        if (UP) wb[t][j] = load_stream(pb + t * strip_u4 + (size_t)kk * 64);
      }
      if (PG) {
        const int kg = kk / p.group_blocks;
#pragma unroll
        for (int t = 0; t < SP; ++t) {
          sa[t][j] = psa[(size_t)kg * n_pad_s + 16 * t];
          if (UP) sb[t][UB > 1 ? j : 0] = psb[(size_t)kg * n_pad_s + 16 * t];
        }
      }
    }
  };
  if (kb0 < kb1) load_w(wA0, wB0, sA0, sB0, kb0);

  // Token rows of the A operand.  Lanes whose row lies past the end of the group read the
  // group's first row instead: an MFMA output row depends on its own input row only, and
  // rows past the end are never stored.
  const uint16_t* arow[MT];
#pragma unroll
  for (int i = 0; i < MT; ++i) {
    int pos = m0 + 16 * i + mm;
    if (pos >= cnt) pos = m0;
    if (UP) {
      int pair = p.g.idx1 ? base + pos : p.g.perm[base + pos];
      arow[i] = p.a + (size_t)(pair / p.g.pair_div) * p.a_stride + (KB / 4) * kq;
    } else {
      arow[i] = p.a + (size_t)(base + pos) * p.a_stride + (KB / 4) * kq;
    }
  }
  auto load_x = [&](uint4 (&xa)[U][MT][AV], int kb) {
#pragma unroll
    for (int j = 0; j < U; ++j) {
      const int kk = min(kb + j, kb1 - 1);
#pragma unroll
      for (int i = 0; i < MT; ++i)
        if (i < mt_live) {
#pragma unroll
          for (int v = 0; v < AV; ++v)
            xa[j][i][v] = *((const uint4*)(arow[i] + (size_t)kk * KB) + v);
        }
    }
  };

  f32x4 acc[NACC][S][MT];
#pragma unroll
  for (int n = 0; n < NACC; ++n)
#pragma unroll
    for (int t = 0; t < S; ++t)
#pragma unroll
      for (int i = 0; i < MT; ++i) acc[n][t][i] = f32x4{0.f, 0.f, 0.f, 0.f};
  auto multiply = [&](const uint4 (&wa)[S][U], const uint4 (&wb)[S][UP ? U : 1],
                      const float (&sa)[SP][UA], const float (&sb)[SP][UB],
                      const uint4 (&xa)[U][MT][AV], int kb) {
#pragma unroll
    for (int j = 0; j < U; ++j) {
      if (kb + j < kb1) {
        if (INT8 && PG) {
#pragma unroll
          for (int t = 0; t < S; ++t) {
            bf16x8 al, ah, bl, bh;
            widen_i8x16(wa[t][j], al, ah);
            if (UP) widen_i8x16(wb[t][j], bl, bh);
            const float s_a = sa[PG ? t : 0][PG ? j : 0];
            const float s_b = UP ? sb[PG ? t : 0][PG && UP ? j : 0] : 0.f;
#pragma unroll
            for (int i = 0; i < MT; ++i) {
              uint4 x0 = xa[j][i][0], x1 = xa[j][i][AV - 1];
              f32x4 ta = mfma(*(bf16x8*)&x0, al, f32x4{0.f, 0.f, 0.f, 0.f});
              ta = mfma(*(bf16x8*)&x1, ah, ta);
              acc[0][t][i] += ta * s_a;
              if (UP) {
                f32x4 tb = mfma(*(bf16x8*)&x0, bl, f32x4{0.f, 0.f, 0.f, 0.f});
                tb = mfma(*(bf16x8*)&x1, bh, tb);
                acc[NACC - 1][t][i] += tb * s_b;
              }
            }
          }
        } else if (INT8) {
#pragma unroll
          for (int t = 0; t < S; ++t) {
            bf16x8 al, ah, bl, bh;
            widen_i8x16(wa[t][j], al, ah);
            if (UP) widen_i8x16(wb[t][j], bl, bh);
#pragma unroll
            for (int i = 0; i < MT; ++i) {
              uint4 x0 = xa[j][i][0], x1 = xa[j][i][AV - 1];
              acc[0][t][i] = mfma(*(bf16x8*)&x0, al, acc[0][t][i]);
              acc[0][t][i] = mfma(*(bf16x8*)&x1, ah, acc[0][t][i]);
              if (UP) {
                acc[NACC - 1][t][i] = mfma(*(bf16x8*)&x0, bl, acc[NACC - 1][t][i]);
                acc[NACC - 1][t][i] = mfma(*(bf16x8*)&x1, bh, acc[NACC - 1][t][i]);
              }
            }
          }
        } else {
#pragma unroll
          for (int t = 0; t < S; ++t)
#pragma unroll
            for (int i = 0; i < MT; ++i) {
              acc[0][t][i] = mfma(xa[j][i][0], wa[t][j], acc[0][t][i]);
              if (UP) acc[NACC - 1][t][i] = mfma(xa[j][i][0], wb[t][j], acc[NACC - 1][t][i]);
            }
        }
      }
    }
  };

  if (kb0 < kb1) load_x(xa0, kb0);
  for (int kb = kb0; kb < kb1; kb += 2 * U) {
    if (kb + U < kb1) {
      load_w(wA1, wB1, sA1, sB1, kb + U);
      load_x(xa1, kb + U);
    }
    multiply(wA0, wB0, sA0, sB0, xa0, kb);
    if (kb + 2 * U < kb1) {
      load_w(wA0, wB0, sA0, sB0, kb + 2 * U);
      load_x(xa0, kb + 2 * U);
    }
    if (kb + U < kb1) multiply(wA1, wB1, sA1, sB1, xa1, kb + U);
  }

  // Reduce the four K-slices through LDS; wave 0 finishes.
  __shared__ f32x4 red[kWavesPerWg - 1][NACC][S][MT][64];
  if (wave > 0) {
#pragma unroll
    for (int n = 0; n < NACC; ++n)
#pragma unroll
      for (int t = 0; t < S; ++t)
#pragma unroll
        for (int i = 0; i < MT; ++i) red[wave - 1][n][t][i][lane] = acc[n][t][i];
  }
  __syncthreads();
  if (wave != 0) return;
#pragma unroll
  for (int w = 0; w < kWavesPerWg - 1; ++w)
#pragma unroll
    for (int n = 0; n < NACC; ++n)
#pragma unroll
      for (int t = 0; t < S; ++t)
#pragma unroll
        for (int i = 0; i < MT; ++i) acc[n][t][i] += red[w][n][t][i][lane];

  // D layout: lane holds rows 4*kq + r (r = 0..3) of column mm.
#pragma unroll
  for (int t = 0; t < S; ++t) {
    const int n = (nb + t) * 16 + mm;
    float sa = 1.f, sb = 1.f;
    if (INT8 && !PG) {
      sa = n < p.n_rows ? p.sa[(size_t)e * p.n_rows + n] : 0.f;
      if (UP) sb = n < p.n_rows ? p.sb[(size_t)e * p.n_rows + n] : 0.f;
    }
#pragma unroll
    for (int i = 0; i < MT; ++i) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        int pos = m0 + 16 * i + 4 * kq + r;
        if (pos >= cnt) continue;
        if (UP) {
          float g = acc[0][t][i][r] * sa;
          float uu = acc[NACC - 1][t][i][r] * sb;
          float h = (g / (1.f + __expf(-g))) * uu;
          ((uint16_t*)p.out)[(size_t)(base + pos) * p.out_stride + n] = bf16_rne(h);
        } else if (n < p.n_rows) {
          int pair = p.g.idx1 ? base + pos : p.g.perm[base + pos];
          ((float*)p.out)[(size_t)pair * p.out_stride + n] = acc[0][t][i][r] * sa;
        }
      }
    }
  }
}

// Down projection + combine for ONE token with k <= 2 experts, one launch.  A workgroup owns a
// 16-row strip of W_d for every expert of the token: waves [8 j, 8 j + 8) stream the strip of
// expert j, split over K exactly as the eight waves of ffn_stream_kernel<1, INT8, false, 8> do,
// and the partial sums meet in LDS in the same order -- so y is bit-identical to the separate
// down launch -- and lanes 0..15 then finish out[n] = sum_j w_j * y_j[n] (+ residual) with the
// combine kernel's arithmetic (product and sum rounded separately; src/moe/sparse.rs:226-233).
// Saves the combine launch and the bubble in front of it, about 4 % of a batch-1 forward.
template <bool INT8>
__global__ __launch_bounds__(1024) void ffn_down_decode1_kernel(StreamParams p, int k,
                                                               const float* __restrict__ w,
                                                               const float* residual, float* out) {
  constexpr int KS = 8;  // K slices per expert, as in the separate down launch
  const int nb = blockIdx.x;
  // The wave id as a scalar: everything derived from it (k range, loop bounds, the guards around
  // the MFMAs) is then a scalar branch.  Left as a vector value the compiler predicates those
  // guards through EXEC, which MFMA instructions do not obey.
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int kq = lane >> 4, mm = lane & 15;
  const int j = wave / KS, slice = wave - j * KS;
  constexpr int KB = INT8 ? kKbInt8 : kKbBf16;
  __shared__ float red[16][16];
  float partial = 0.f;
  if (j < k && (p.g.idx1 || j < *p.g.n_active)) {  // uniform per wave
    const int e = p.g.idx1 ? p.g.idx1[j] : p.g.active[j];
    const int base = p.g.idx1 ? j : p.g.offsets[e];
    const int kb_per = (p.nkb + KS - 1) / KS;
    const int kb0 = slice * kb_per;
    const int kb1 = min(p.nkb, kb0 + kb_per);
    const uint4* pa = p.wa + (size_t)e * p.w_stride_u4 + (size_t)nb * p.nkb * 64 + lane;
    constexpr int U = 4;
    constexpr int AV = INT8 ? 2 : 1;
    uint4 wA0[U], wA1[U], xa0[U][AV], xa1[U][AV];
    auto load_w = [&](uint4 (&wa)[U], int kb) {
#pragma unroll
      for (int q = 0; q < U; ++q) wa[q] = load_stream(pa + (size_t)min(kb + q, kb1 - 1) * 64);
    };
    if (kb0 < kb1) load_w(wA0, kb0);
    // The expert's single row of h; all 16 MFMA rows read it, only row 0 is kept.
    const uint16_t* arow = p.a + (size_t)base * p.a_stride + (KB / 4) * kq;
    auto load_x = [&](uint4 (&xa)[U][AV], int kb) {
#pragma unroll
      for (int q = 0; q < U; ++q)
#pragma unroll
        for (int v = 0; v < AV; ++v)
          xa[q][v] = *((const uint4*)(arow + (size_t)min(kb + q, kb1 - 1) * KB) + v);
    };
    f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
    auto multiply = [&](const uint4 (&wa)[U], const uint4 (&xa)[U][AV], int kb) {
#pragma unroll
      for (int q = 0; q < U; ++q) {
        if (kb + q < kb1) {
          if (INT8) {
            bf16x8 al, ah;
            widen_i8x16(wa[q], al, ah);
            uint4 x0 = xa[q][0], x1 = xa[q][AV - 1];
            acc = mfma(*(bf16x8*)&x0, al, acc);
            acc = mfma(*(bf16x8*)&x1, ah, acc);
          } else {
            acc = mfma(xa[q][0], wa[q], acc);
          }
        }
      }
    };
    if (kb0 < kb1) load_x(xa0, kb0);
    for (int kb = kb0; kb < kb1; kb += 2 * U) {
      if (kb + U < kb1) {
        load_w(wA1, kb + U);
        load_x(xa1, kb + U);
      }
      multiply(wA0, xa0, kb);
      if (kb + 2 * U < kb1) {
        load_w(wA0, kb + 2 * U);
        load_x(xa0, kb + 2 * U);
      }
      if (kb + U < kb1) multiply(wA1, xa1, kb + U);
    }
    partial = acc[0];  // D layout: lanes 0..15 (kq == 0), element 0 = row 0, column mm
  }
  if (kq == 0) red[wave][mm] = partial;
  __syncthreads();
  if (threadIdx.x >= 16) return;
  const int n = nb * 16 + mm;
  if (n >= p.n_rows) return;
  float o = 0.f;
  const int n_active = p.g.idx1 ? k : *p.g.n_active;
  for (int jj = 0; jj < k && jj < n_active; ++jj) {
    float y = red[jj * KS][mm];
#pragma unroll
    for (int sl = 1; sl < KS; ++sl) y += red[jj * KS + sl][mm];
    const int e = p.g.idx1 ? p.g.idx1[jj] : p.g.active[jj];
    if (INT8) y = y * p.sa[(size_t)e * p.n_rows + n];
    const int pair = p.g.idx1 ? jj : p.g.perm[p.g.offsets[e]];
    ((float*)p.out)[(size_t)pair * p.out_stride + n] = y;
    // The product must be rounded before it is added: an opaque multiply keeps the compiler
    // (-ffp-contract=fast in this file) from fusing it into an FMA.
    float prod;
    asm volatile("v_mul_f32 %0, %1, %2" : "=v"(prod) : "v"(w[pair]), "v"(y));
    o = o + prod;
  }
  if (residual) o = residual[n] + o;
  out[n] = o;
}

// Down projection + combine for ONE token, any k with a shared expert or without: the general
// form of the kernel above.  A workgroup owns a 16-row strip of W_d of every expert of the
// token and of the shared expert; its waves are dealt out as sr K slices per routed expert and
// ss slices of the shared one (k sr + ss <= 16, chosen by the host so that the slices are about
// equally long: the shared expert is usually several times as wide).  Partial sums meet in LDS
// in slice order, lanes 0..15 finish out[n] = sum_j w_j y_j[n] + s y_shared[n] (+ residual) with
// the combine kernel's arithmetic and order (src/moe/sparse.rs:226-233; shared expert and
// residual as in combine.hip), and y / y_shared are stored as the separate launches store them.
// One launch instead of three (routed down, shared down, combine).  With fewer strips than
// compute units (d = 2048: 128) every strip is shared by two workgroups of eight rows each.
//
// A slice is short here (22 blocks on the Qwen1.5-MoE and DeepSeek-MoE shapes), so the launch
// is a chain of memory round trips rather than a stream: a wave therefore requests up to kChunk
// weight blocks at once (all of its slice, usually) and the h rows are staged in LDS by the whole
// workgroup meanwhile (stage_h; needs idx1), instead of two small batches in turn with the h
// pieces fetched per lane.
template <bool INT8>
__global__ __launch_bounds__(1024) void ffn_down_combine1_kernel(
    StreamParams p, StreamParams ps, int k, int sr, int ss, int halves, int stage_h,
    const float* __restrict__ w, const float* __restrict__ sgate, const float* residual,
    float* out) {
  extern __shared__ __attribute__((aligned(16))) uint16_t sH[];  // [k][K routed] [K shared]
  const int nb = blockIdx.x / halves;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int kq = lane >> 4, mm = lane & 15;
  // halves == 2: the workgroup computes rows 8 h .. 8 h + 7 of the strip only and its lanes load
  // just those rows of every weight block (four full 128-byte lines of the block's eight).
  const bool lane_on = halves == 1 || (mm >> 3) == (int)(blockIdx.x - nb * halves);
  constexpr int KB = INT8 ? kKbInt8 : kKbBf16;
  constexpr int AV = INT8 ? 2 : 1;
  constexpr int kChunk = INT8 ? 11 : 22;  // weight blocks a wave requests at once
  // Every expert's K range is cut into the same eight slices as in the separate down launch
  // (eight waves per strip there) and the eight partial sums are added in the same order, so y
  // has the bits of that launch; a wave here takes 8 / sr (8 / ss) consecutive slices.
  __shared__ float red[16 * 8][16];
  const int routed_waves = k * sr;
  const bool is_shared = wave >= routed_waves;
  const int j = is_shared ? 0 : wave / sr;
  const int slice = is_shared ? wave - routed_waves : wave - j * sr;
  const int n_slices = is_shared ? ss : sr;
  const bool live = is_shared || p.g.idx1 || j < *p.g.n_active;  // uniform per wave
  const StreamParams& q = is_shared ? ps : p;
  const int subs = 8 / n_slices;
  const int kb8 = (q.nkb + 7) / 8;
  const int sub0 = slice * subs;
  const int kb0 = min(q.nkb, sub0 * kb8);
  const int kb1 = live ? min(q.nkb, (sub0 + subs) * kb8) : kb0;
  int e = 0, base = 0;
  if (live && !is_shared) {
    e = p.g.idx1 ? p.g.idx1[j] : p.g.active[j];
    base = p.g.idx1 ? j : p.g.offsets[e];
  }
  const uint4* pa = q.wa + (size_t)e * q.w_stride_u4 + (size_t)nb * q.nkb * 64 + lane;
  uint4 wreg[kChunk];
  auto load_w = [&](int kb) {
#pragma unroll
    for (int u = 0; u < kChunk; ++u)
      wreg[u] = (lane_on && kb + u < kb1) ? load_stream(pa + (size_t)(kb + u) * 64)
                                          : uint4{0u, 0u, 0u, 0u};
  };
  load_w(kb0);
  // h rows into LDS: row j of the routed experts (K = p.nkb * KB each), then the shared one.
  const int kr = p.nkb * KB, ksh = ss > 0 ? ps.nkb * KB : 0;
  if (stage_h) {
    const int cr = kr / 8, total = k * cr + ksh / 8;  // 16-byte pieces
    for (int c = threadIdx.x; c < total; c += blockDim.x) {
      const uint4* src;
      if (c < k * cr) {
        const int row = c / cr;
        src = (const uint4*)(p.a + (size_t)row * p.a_stride) + (c - row * cr);
      } else {
        src = (const uint4*)ps.a + (c - k * cr);
      }
      ((uint4*)sH)[c] = *src;
    }
    __syncthreads();
  }
  const uint16_t* xrow = stage_h ? sH + (is_shared ? k * kr : j * kr) + (KB / 4) * kq
                                 : q.a + (size_t)base * q.a_stride + (KB / 4) * kq;
  f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
  const int unit = is_shared ? k : j;
  int sub = sub0;
  int bound = min(q.nkb, (sub0 + 1) * kb8);  // first block of the next slice
  auto flush = [&] {  // D layout: lanes 0..15 (kq == 0), element 0 = row 0, column mm
    if (kq == 0) red[unit * 8 + sub][mm] = acc[0];
    acc = f32x4{0.f, 0.f, 0.f, 0.f};
    ++sub;
    bound = min(q.nkb, bound + kb8);
  };
  for (int kb = kb0; kb < kb1; kb += kChunk) {
    if (kb > kb0) load_w(kb);
#pragma unroll
    for (int u = 0; u < kChunk; ++u) {
      if (kb + u < kb1) {
        if (kb + u == bound) flush();
        const uint4* xp = (const uint4*)(xrow + (size_t)(kb + u) * KB);
        if (INT8) {
          bf16x8 al, ah;
          widen_i8x16(wreg[u], al, ah);
          uint4 x0 = xp[0], x1 = xp[AV - 1];
          acc = mfma(*(bf16x8*)&x0, al, acc);
          acc = mfma(*(bf16x8*)&x1, ah, acc);
        } else {
          acc = mfma(xp[0], wreg[u], acc);
        }
      }
    }
  }
  if (live)
    while (sub < sub0 + subs) flush();  // the last slice, and empty ones (a short K) as zeros
  __syncthreads();
  if (threadIdx.x >= 16 || !lane_on) return;
  const int n = nb * 16 + mm;
  if (n >= p.n_rows) return;
  float o = 0.f;
  const int n_active = p.g.idx1 ? k : *p.g.n_active;
  for (int jj = 0; jj < k && jj < n_active; ++jj) {
    float y = red[jj * 8][mm];
#pragma unroll
    for (int sl = 1; sl < 8; ++sl) y += red[jj * 8 + sl][mm];
    const int ee = p.g.idx1 ? p.g.idx1[jj] : p.g.active[jj];
    if (INT8) y = y * p.sa[(size_t)ee * p.n_rows + n];
    const int pair = p.g.idx1 ? jj : p.g.perm[p.g.offsets[ee]];
    ((float*)p.out)[(size_t)pair * p.out_stride + n] = y;
    // The product must be rounded before it is added: an opaque multiply keeps the compiler
    // (-ffp-contract=fast in this file) from fusing it into an FMA.
    float prod;
    asm volatile("v_mul_f32 %0, %1, %2" : "=v"(prod) : "v"(w[pair]), "v"(y));
    o = o + prod;
  }
  if (ss > 0) {
    float y = red[k * 8][mm];
#pragma unroll
    for (int sl = 1; sl < 8; ++sl) y += red[k * 8 + sl][mm];
    if (INT8) y = y * ps.sa[n];
    ((float*)ps.out)[n] = y;
    const float sc = sgate ? sgate[0] : 1.0f;
    float prod;
    asm volatile("v_mul_f32 %0, %1, %2" : "=v"(prod) : "v"(sc), "v"(y));
    o = o + prod;
  }
  if (residual) o = residual[n] + o;
  out[n] = o;
}

// Mid-batch form: experts that see a few dozen rows each.  Still bound by HBM (every weight
// byte is read once per 128 rows of its expert, straight into B-operand registers), but with
// that many rows the token rows can no longer come from L2 per wave: the NWV waves of a
// workgroup share them through LDS.  A wave owns its B strips over the whole K -- W_g and W_u
// of one strip in the gate/up phase, NBD adjacent strips of W_d in the down phase -- so there
// is no reduction across waves.  The workgroup's up to 128 token rows (eight 16-row tiles, A
// operand) pass through a ring of three LDS stages of JB weight blocks of k each (64 k with
// bf16 pairs or single int8 blocks, 128 k with int8 pairs), written from registers that were
// loaded one step earlier, one barrier per stage.  Only the row tiles that hold rows are staged
// and multiplied: ML (2, 4, 6 or 8) is the number of row tiles of the main loop, and a
// workgroup picks the smallest form that covers its rows (staging all 128 rows whatever the
// group held doubled the traffic of the launch at 32 rows per expert).  Weight blocks are
// requested NWB - 1 stages ahead into a ring of NWB register buffers.  Every load of the loop
// is issued unconditionally with a clamped stage index: a branch around a load makes the
// compiler wait for all loads in flight before every use.  16-byte chunk c of LDS row r sits
// at c ^ swz(r), which spreads the rows a fragment read touches over all banks.
// PG: int8 with one scale per output row and k group (see ffn_stream_kernel): every 64-k block
// is accumulated on its own and added to the running sum times the scale of its group; the
// scales travel through the register ring with the blocks they belong to.
template <bool INT8, bool UP, int NWV, int JB, int NWB, int NBD = 2, bool PG = false>
__global__ __launch_bounds__(64 * NWV, 8 / NWV) void ffn_mid_kernel(StreamParams p_routed,
                                                                    StreamParams p_shared,
                                                                    int shared_blocks) {
  constexpr int MT = 8, NB = UP ? 2 : NBD, NST = 3;
  constexpr int KB = INT8 ? kKbInt8 : kKbBf16;
  constexpr int CH = KB * JB / 8;  // 16-byte chunks per row and stage
  constexpr int ROWS = 16 * MT;
  __shared__ u32x4 lds_a[NST * ROWS * CH];

  // A shared expert rides in the same launch (its own weights, widths and rows: one group of
  // all T tokens): its row blocks are blockIdx.y = 0 .. shared_blocks - 1 (at z = 0), the routed
  // experts follow along y with their row blocks along z.  All of the shared expert comes first
  // in the grid that way, because its K can be several times the routed experts' and its
  // workgroups should not be the ones that start last (with its row blocks along z as well, the
  // later ones started behind every routed workgroup and ended the launch).
  const bool sh = (int)blockIdx.y < shared_blocks;
  const StreamParams& p = sh ? p_shared : p_routed;
  if ((int)blockIdx.x * (UP ? NWV : NWV * NB) * 16 >= p.n_pad) return;  // grid spans the wider
  const int u = sh ? 0 : (int)blockIdx.y - shared_blocks;
  if (u >= *p.g.n_active) return;
  const int e = p.g.active[u];
  const int base = p.g.offsets[e];
  const int cnt = p.g.offsets[e + 1] - base;
  // (a shared row block at z > 0 does not exist: it gets a block number past every row count)
  const int m0 = (sh ? (blockIdx.z ? 1 << 20 : (int)blockIdx.y) : (int)blockIdx.z) * ROWS;
  if (m0 >= cnt) return;
  const int mt_live = __builtin_amdgcn_readfirstlane(min(MT, (cnt - m0 + 15) >> 4));
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int kq = lane >> 4, mm = lane & 15;
  const int n_strips = p.n_pad >> 4;
  const int ns = p.nkb / JB;  // stages; the launcher admits K of whole stages only

  // The wave's two B strips.  A strip past the end is clamped to the last one: loaded and
  // multiplied like any other (the barriers need every wave), never stored.
  int strip[NB];
  const uint4* pw[NB];
  if (UP) {
    strip[0] = strip[1] = blockIdx.x * NWV + wave;
    const size_t off = (size_t)e * p.w_stride_u4 + (size_t)min(strip[0], n_strips - 1) * p.nkb * 64 + lane;
    pw[0] = p.wa + off;
    pw[1] = p.wb + off;
  } else {
#pragma unroll
    for (int t = 0; t < NB; ++t) {
      strip[t] = (blockIdx.x * NWV + wave) * NB + t;
      pw[t] = p.wa + (size_t)e * p.w_stride_u4 + (size_t)min(strip[t], n_strips - 1) * p.nkb * 64 + lane;
    }
  }
  // per-group scales of this lane's output row (column mm of the D layout) in each strip
  const float* psc[NB];
  if (PG) {
#pragma unroll
    for (int t = 0; t < NB; ++t)
      psc[t] = (UP && t == 1 ? p.sb : p.sa) + (size_t)e * p.n_kgroups * p.n_pad +
               min(strip[t], n_strips - 1) * 16 + mm;
  }
  // Ring of NWB register buffers of weight blocks: stage st lives in buffer st % NWB and is
  // requested NWB - 1 steps before it is multiplied.
  u32x4 wr[NWB][NB][JB];
  float wsc[NWB][PG ? NB : 1][PG ? JB : 1];
  // Workgroups walk K from different first stages (and wrap around): launched together and
  // paced by the same memory system, they would otherwise all read the same offset of their
  // 2^n-byte-spaced strips at the same time, i.e. the same few memory channels.
  // The first stage depends on the strip block and the expert only, not on where the expert sits
  // in the list of active ones or on the row block: the f32 sum of a (token, expert) pair is then
  // added up in the same order whatever else the batch holds (and the row blocks of an expert
  // walk K together, which lets the later ones find the weights in L2).
  const int rot = p.mid_rot ? (int)((blockIdx.x * 13u + (sh ? 5u : (unsigned)e * 29u)) % (unsigned)ns) : 0;
  auto stage_of = [&](int st) {
    const int sc = min(st, ns - 1) + rot;
    return sc >= ns ? sc - ns : sc;
  };
  auto load_w = [&](u32x4 (&w)[NB][JB], float (&sc_)[PG ? NB : 1][PG ? JB : 1], int st) {
    const int sc = stage_of(st);
#pragma unroll
    for (int t = 0; t < NB; ++t)
#pragma unroll
      for (int j = 0; j < JB; ++j) {
        w[t][j] = __builtin_nontemporal_load((const u32x4*)(pw[t] + (size_t)(sc * JB + j) * 64));
        if (PG) sc_[PG ? t : 0][PG ? j : 0] = psc[t][(size_t)((sc * JB + j) / p.group_blocks) * p.n_pad];
      }
  };
#pragma unroll
  for (int b = 0; b < NWB - 1; ++b) load_w(wr[b], wsc[b], b);

  // Chunk c of row r is stored at c ^ swz(r): eight consecutive rows then cover all banks
  // (rows of 128 bytes or more: r & 7; rows of 64 bytes pair up: (r >> 1) & 3).
  auto swz = [](int r) { return CH >= 8 ? (r & 7) : ((r >> 1) & 3); };

  f32x4 acc[NB][MT];
#pragma unroll
  for (int t = 0; t < NB; ++t)
#pragma unroll
    for (int i = 0; i < MT; ++i) acc[t][i] = f32x4{0.f, 0.f, 0.f, 0.f};
  const u32x4* frag = lds_a + mm * CH;
  const int sw = swz(mm);  // = swz(16 i + mm)

  auto run = [&](auto ml_c) {
    constexpr int ML = decltype(ml_c)::value;
    // Token rows of the 16 ML rows this form multiplies: the workgroup's threads share the
    // chunks of a stage, CPT (a power of two) consecutive chunks of one row each; surplus
    // threads repeat the first ones.  Rows past the end of the group repeat
    // its first row (an MFMA output row depends on its own input row only, and those rows are
    // never stored).
    constexpr int NT = 64 * NWV, NCH = 16 * ML * CH;
    constexpr int CPT = NCH <= NT ? 1 : NCH <= 2 * NT ? 2 : NCH <= 4 * NT ? 4 : 8;
    static_assert(CH % CPT == 0 && CPT * NT >= NCH, "mid-kernel staging");
    const int q0 = ((int)threadIdx.x * CPT) % NCH;
    const int ar = q0 / CH, ac = q0 % CH;
    int apos = m0 + ar;
    if (apos >= cnt) apos = m0;
    const size_t arow = UP ? (size_t)(p.g.perm[base + apos] / p.g.pair_div) : (size_t)(base + apos);
    const u32x4* ag = (const u32x4*)(p.a + arow * p.a_stride) + ac;
    auto load_a = [&](u32x4 (&ga)[CPT], int st) {
      const int sc = stage_of(st);
#pragma unroll
      for (int c = 0; c < CPT; ++c) ga[c] = ag[(size_t)sc * CH + c];
    };
    auto store_a = [&](const u32x4 (&ga)[CPT], int slot) {
#pragma unroll
      for (int c = 0; c < CPT; ++c)
        lds_a[(slot * ROWS + ar) * CH + ((ac + c) ^ swz(ar))] = ga[c];
    };
    auto compute = [&](const u32x4 (&w)[NB][JB], const float (&sc_)[PG ? NB : 1][PG ? JB : 1], int slot) {
      const u32x4* fs = frag + slot * ROWS * CH;
#pragma unroll
      for (int j = 0; j < JB; ++j) {
        if (INT8) {
          bf16x8 bl[NB], bh[NB];
#pragma unroll
          for (int t = 0; t < NB; ++t)
            widen_i8x16(make_uint4(w[t][j].x, w[t][j].y, w[t][j].z, w[t][j].w), bl[t], bh[t]);
#pragma unroll
          for (int i = 0; i < ML; ++i) {
            const u32x4 x0 = fs[16 * i * CH + ((j * 8 + 2 * kq) ^ sw)];
            const u32x4 x1 = fs[16 * i * CH + ((j * 8 + 2 * kq + 1) ^ sw)];
#pragma unroll
            for (int t = 0; t < NB; ++t) {
              if (PG) {
                f32x4 ta = mfma(*(const bf16x8*)&x0, bl[t], f32x4{0.f, 0.f, 0.f, 0.f});
                ta = mfma(*(const bf16x8*)&x1, bh[t], ta);
                acc[t][i] += ta * sc_[PG ? t : 0][PG ? j : 0];
              } else {
                acc[t][i] = mfma(*(const bf16x8*)&x0, bl[t], acc[t][i]);
                acc[t][i] = mfma(*(const bf16x8*)&x1, bh[t], acc[t][i]);
              }
            }
          }
        } else {
#pragma unroll
          for (int i = 0; i < ML; ++i) {
            const u32x4 x = fs[16 * i * CH + ((j * 4 + kq) ^ sw)];
#pragma unroll
            for (int t = 0; t < NB; ++t) acc[t][i] = mfma(*(const bf16x8*)&x, *(const bf16x8*)&w[t][j], acc[t][i]);
          }
        }
      }
    };
    // Step st: the registers hold the rows of stage st + 2, whose slot was read last in step
    // st - 1 (every wave is past that step's barrier); the rows of stage st + 3 and the weights
    // of stage st + NWB - 1 are requested, then stage st is multiplied.
    u32x4 ga[CPT];
    auto step = [&](int bc, int bl_, int st) {
      store_a(ga, (st + 2) % NST);
      load_a(ga, st + 3);
      load_w(wr[bl_], wsc[bl_], st + NWB - 1);
      if (st < ns) compute(wr[bc], wsc[bc], st % NST);
      __syncthreads();
    };
    load_a(ga, 0);
    store_a(ga, 0);
    load_a(ga, 1);
    store_a(ga, 1);
    load_a(ga, 2);
    __syncthreads();
    for (int st = 0; st < ns; st += NWB) {
#pragma unroll
      for (int b = 0; b < NWB; ++b) step(b, (b + NWB - 1) % NWB, st + b);
    }
  };
  if (mt_live <= 2)
    run(std::integral_constant<int, 2>{});
  else if (mt_live <= 4)
    run(std::integral_constant<int, 4>{});
  else if (mt_live <= 6)
    run(std::integral_constant<int, 6>{});
  else
    run(std::integral_constant<int, 8>{});

  // D layout: lane holds rows 4*kq + r (r = 0..3) of column mm.
#pragma unroll
  for (int t = 0; t < (UP ? 1 : NB); ++t) {
    const int n = strip[t] * 16 + mm;
    const bool n_ok = strip[t] < n_strips && n < p.n_rows;
    float sa = 1.f, sb = 1.f;
    if (INT8 && !PG) {
      sa = n_ok ? p.sa[(size_t)e * p.n_rows + n] : 0.f;
      if (UP) sb = n_ok ? p.sb[(size_t)e * p.n_rows + n] : 0.f;
    }
#pragma unroll
    for (int i = 0; i < MT; ++i) {
      if (i < mt_live) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int pos = m0 + 16 * i + 4 * kq + r;
          if (pos < cnt && strip[t] < n_strips) {
            if (UP) {
              const float g = acc[0][i][r] * sa;
              const float uu = acc[1][i][r] * sb;
              const float h = (g / (1.f + __expf(-g))) * uu;
              ((uint16_t*)p.out)[(size_t)(base + pos) * p.out_stride + n] = bf16_rne(h);
            } else if (n_ok) {
              const int pair = p.g.perm[base + pos];
              ((float*)p.out)[(size_t)pair * p.out_stride + n] = acc[t][i][r] * sa;
            }
          }
        }
      }
    }
  }
}

// Mid-batch launch.  Measured on the Mixtral shape (T = 64 ... 384): gate/up runs best as two
// workgroups of four waves per compute unit (the prologue of one overlaps the stream of the
// other) with 64-k stages and a weight ring of four (bf16) or six (int8) buffers; the down
// projection has few strips (d / 16) and a long K, so it takes one strip per wave and eight
// waves per workgroup: d / 128 workgroups per expert instead of d / 256.
template <bool INT8, bool UP>
hipError_t launch_mid(const StreamParams& p_in, int n_groups, int rows_max, hipStream_t s,
                      const StreamParams* shared) {
  StreamParams p = p_in, ps = shared ? *shared : p_in;
  p.mid_rot = ps.mid_rot = 1;
  const int n_pad = shared && shared->n_pad > p.n_pad ? shared->n_pad : p.n_pad;
  const int n_strips = n_pad / 16;
  const int per_wg = UP ? 4 : 8;
  const int row_blocks = (rows_max + 127) / 128;
  const int sb = shared ? row_blocks : 0;  // the shared expert has rows_max = T rows
  dim3 grid((n_strips + per_wg - 1) / per_wg, n_groups + sb, row_blocks);
  if constexpr (INT8) {
    if (p.group_blocks > 0) {  // per-group scales: a shorter ring leaves room for them
      if (UP)
        ffn_mid_kernel<true, true, 4, 1, 4, 2, true><<<grid, 256, 0, s>>>(p, ps, sb);
      else
        ffn_mid_kernel<true, false, 8, 2, 3, 1, true><<<grid, 512, 0, s>>>(p, ps, sb);
      return hipGetLastError();
    }
  }
  if (UP)
    ffn_mid_kernel<INT8, true, 4, INT8 ? 1 : 2, INT8 ? 6 : 4><<<grid, 256, 0, s>>>(p, ps, sb);
  else
    ffn_mid_kernel<INT8, false, 8, 2, 3, 1><<<grid, 512, 0, s>>>(p, ps, sb);
  return hipGetLastError();
}

template <bool INT8, bool UP>
hipError_t launch_stream(const StreamParams& p, int n_groups, int rows_max, hipStream_t s,
                         const StreamParams* shared) {
  // Up to 32 rows per expert per workgroup; larger groups take more workgroups along z.
  int mt = rows_max <= 16 ? 1 : 2;
  const StreamParams ps = shared ? *shared : p;
  // A shared expert rides as the last group of the grid, or as the first one when its K is much
  // longer than the routed experts' (its strips would otherwise start last and end the launch).
  const int shared_y = !shared ? -1 : (!UP && shared->nkb > p.nkb) ? 0 : n_groups;
  const int n_pad = shared && shared->n_pad > p.n_pad ? shared->n_pad : p.n_pad;
  // Two strips per workgroup once experts can have more than 16 rows:
  // int8 (per-row and per-group scales) in both phases, bf16 in the down phase.  Measured at T = 48 on the Mixtral shape:
  // int8 gate/up 177 -> 159 us, down 118 -> 97 us; bf16 down 170 -> 151 us, while the bf16
  // gate/up form (218 registers) is slower, 299 -> 331 us, and keeps one strip.
  // With a single row tile only the int8 down phase gains (T = 16: 86 -> 77 us), from 4 rows on.
  const bool two = (mt == 2 ? (INT8 || !UP) : (INT8 && !UP && rows_max >= 4)) &&
                   p.n_pad % 32 == 0 && (!shared || shared->n_pad % 32 == 0);
  dim3 grid(n_pad / (two ? 32 : 16), n_groups + (shared ? 1 : 0),
            (rows_max + 16 * mt - 1) / (16 * mt));
  // The down projection has few strips (d / 16) and a long K (f): eight K slices per strip
  // keep enough loads in flight; gate/up has 2f / 16 strips and uses four.
  constexpr int W = UP ? 4 : 8;
  if (INT8 && p.group_blocks > 0) {
    if (mt == 1 && two)
      ffn_stream_kernel<1, INT8, UP, W, INT8, 2><<<grid, 64 * W, 0, s>>>(p, ps, shared_y);
    else if (mt == 1 && UP && p.sel.logits)
      ffn_stream_kernel<1, INT8, UP, W, INT8, 1, UP><<<grid, 64 * W, 0, s>>>(p, ps, shared_y);
    else if (mt == 1)
      ffn_stream_kernel<1, INT8, UP, W, INT8><<<grid, 64 * W, 0, s>>>(p, ps, shared_y);
    else if (two)
      ffn_stream_kernel<2, INT8, UP, W, INT8, 2><<<grid, 64 * W, 0, s>>>(p, ps, shared_y);
    else
      ffn_stream_kernel<2, INT8, UP, W, INT8><<<grid, 64 * W, 0, s>>>(p, ps, shared_y);
    return hipGetLastError();
  }
  if constexpr (!UP) {
    // Short K (a strip of fewer than 64 blocks): four K slices instead of eight, so that a wave
    // still has a few batches of blocks to pipeline.  Measured (44 blocks per strip, 60-64
    // experts): down stage T = 16 36.3 -> 28.4 us and 52.1 -> 40.6 us, T = 8 26.9 -> 21.7, T = 19
    // (two row tiles, two strips per workgroup) 36.1 -> 29.6 and 59.0 -> 46.2; two
    // slices are slower again (T = 2 17.5 against 15.9 us).  A single token keeps eight: its
    // fused down + combine launch adds the slices up in that order, and the two must agree bit
    // for bit.
    constexpr int w4_below = 64;
    if (p.nkb < w4_below && rows_max > 1) {
      if (mt == 1 && two)
        ffn_stream_kernel<1, INT8, false, 4, false, 2><<<grid, 256, 0, s>>>(p, ps, shared_y);
      else if (mt == 1)
        ffn_stream_kernel<1, INT8, false, 4, false><<<grid, 256, 0, s>>>(p, ps, shared_y);
      else if (two)
        ffn_stream_kernel<2, INT8, false, 4, false, 2><<<grid, 256, 0, s>>>(p, ps, shared_y);
      else
        ffn_stream_kernel<2, INT8, false, 4, false><<<grid, 256, 0, s>>>(p, ps, shared_y);
      return hipGetLastError();
    }
  }
  if (mt == 1 && two)
    ffn_stream_kernel<1, INT8, UP, W, false, 2><<<grid, 64 * W, 0, s>>>(p, ps, shared_y);
  else if (mt == 1 && UP && p.sel.logits)
    ffn_stream_kernel<1, INT8, UP, W, false, 1, UP><<<grid, 64 * W, 0, s>>>(p, ps, shared_y);
  else if (mt == 1)
    ffn_stream_kernel<1, INT8, UP, W, false><<<grid, 64 * W, 0, s>>>(p, ps, shared_y);
  else if (two)
    ffn_stream_kernel<2, INT8, UP, W, false, 2><<<grid, 64 * W, 0, s>>>(p, ps, shared_y);
  else
    ffn_stream_kernel<2, INT8, UP, W, false><<<grid, 64 * W, 0, s>>>(p, ps, shared_y);
  return hipGetLastError();
}

}  // namespace

hipError_t launch_ffn_up_f32(const FfnArgs& a, hipStream_t s);
hipError_t launch_ffn_down_f32(const FfnArgs& a, hipStream_t s);

namespace {
StreamParams stream_params_up(const FfnArgs& a) {
  const bool int8 = a.wdtype == ATENIA_MOE_WEIGHT_INT8_W8A16;
  StreamParams p;
  p.wa = (const uint4*)a.gate.w;
  p.wb = (const uint4*)a.up.w;
  p.sa = a.gate.scale;
  p.sb = a.up.scale;
  p.group_blocks = a.gate.group_blocks;
  p.n_kgroups = a.gate.n_kgroups;
  p.w_stride_u4 = a.gate.expert_stride / 16;
  p.n_rows = a.gate.n_rows;
  p.n_pad = a.gate.n_pad;
  p.nkb = a.gate.k_pad / (int8 ? kKbInt8 : kKbBf16);
  p.a = (const uint16_t*)a.x;
  p.a_stride = a.x_stride;
  p.out = a.h;
  p.out_stride = a.h_stride;
  p.g = a.g;
  p.sel = a.sel;
  p.mid_rot = 0;
  return p;
}
StreamParams stream_params_down(const FfnArgs& a) {
  const bool int8 = a.wdtype == ATENIA_MOE_WEIGHT_INT8_W8A16;
  StreamParams p;
  p.wa = (const uint4*)a.down.w;
  p.wb = nullptr;
  p.sa = a.down.scale;
  p.sb = nullptr;
  p.group_blocks = a.down.group_blocks;
  p.n_kgroups = a.down.n_kgroups;
  p.w_stride_u4 = a.down.expert_stride / 16;
  p.n_rows = a.down.n_rows;
  p.n_pad = a.down.n_pad;
  p.nkb = a.down.k_pad / (int8 ? kKbInt8 : kKbBf16);
  p.a = (const uint16_t*)a.h;
  p.a_stride = a.h_stride;
  p.out = a.y;
  p.out_stride = a.y_stride;
  p.g = a.g;
  p.sel = InlineSelect{};
  p.mid_rot = 0;
  return p;
}
// The shared expert can ride in the routed experts' launch when both stream with the same
// kernel (no tiles, no f32 weights), are stored alike and see the same rows bound.
// In the down phase a strip's K is the expert's width: last in the grid, the strips of a shared
// expert much wider than the routed ones end the launch (measured: Qwen1.5-MoE, shared 4x as
// wide, T = 1: 20 us fused against 18 us as two launches).  With up to 32 rows it rides as the
// first group instead (launch_stream) and is hidden behind the routed experts: down stage
// T = 2 18.5 against 22.9 us as two launches, T = 16 52.2 / 60.1, T = 48 72.8 / 77.5; from
// 64 rows on, where its T rows take several passes over its weights, a shared expert more than
// twice as wide is faster in a launch of its own (T = 64 81.3 / 79.0, T = 128 100.9 / 85.5).
// The bound used is 48 rows.
bool can_fuse_shared(const FfnArgs& a, const FfnArgs* sh, bool down_phase) {
  if (!(sh && a.wdtype != ATENIA_MOE_WEIGHT_F32 && sh->wdtype == a.wdtype && !a.use_tiled &&
        !sh->use_tiled && sh->rows_max == a.rows_max &&
        (sh->gate.group_blocks > 0) == (a.gate.group_blocks > 0)))
    return false;
  if (a.use_mid != sh->use_mid) return false;
  // (the mid-batch launch starts all of the shared expert's workgroups first, which hides a
  // wider one: measured on the Qwen1.5-MoE shape, whole forward fused / a launch of its own
  // beyond 384 rows: T = 512 312 / 336 us, T = 768 339 / 365, T = 1024 363 / 386, T = 1280
  // 420 / 430: at every batch size.)
  if (a.use_mid) return true;
  constexpr int wide_rows = 48;
  if (!a.use_mid && down_phase && a.rows_max > 1 && a.rows_max <= wide_rows) return true;  // first in the grid
  return !down_phase || sh->down.k_pad <= 2 * a.down.k_pad;
}
}  // namespace

// K of whole stages (64 k for bf16 blocks, 128 k for int8 blocks).
bool ffn_mid_supported(const WeightSet& w, int wdtype) {
  if (wdtype == ATENIA_MOE_WEIGHT_F32) return false;
  if (w.group_blocks != 0 && wdtype != ATENIA_MOE_WEIGHT_INT8_W8A16) return false;
  const int kb = wdtype == ATENIA_MOE_WEIGHT_INT8_W8A16 ? kKbInt8 : kKbBf16;
  return w.k_pad % (2 * kb) == 0 && w.k_pad >= 2 * kb && w.n_pad >= 16;
}

bool ffn_stream_fuses_shared(const FfnArgs& a, const FfnArgs& shared, bool down_phase) {
  return can_fuse_shared(a, &shared, down_phase);
}

hipError_t launch_ffn_up(const FfnArgs& a, hipStream_t s, const FfnArgs* shared) {
  if (a.wdtype == ATENIA_MOE_WEIGHT_F32) return launch_ffn_up_f32(a, s);
  if (a.use_tiled) return launch_ffn_up_tiled(a, s);
  const bool int8 = a.wdtype == ATENIA_MOE_WEIGHT_INT8_W8A16;
  const StreamParams p = stream_params_up(a);
  if (a.use_mid) {
    if (!ffn_mid_supported(a.gate, a.wdtype) || !ffn_mid_supported(a.up, a.wdtype) || p.g.idx1 ||
        p.sel.logits)
      return hipErrorInvalidValue;
    StreamParams pm;
    const bool fuse_mid = can_fuse_shared(a, shared, false);
    if (fuse_mid) pm = stream_params_up(*shared);
    return int8 ? launch_mid<true, true>(p, a.n_groups_max, a.rows_max, s, fuse_mid ? &pm : nullptr)
                : launch_mid<false, true>(p, a.n_groups_max, a.rows_max, s, fuse_mid ? &pm : nullptr);
  }
  StreamParams ps;
  const bool fuse = can_fuse_shared(a, shared, false);
  if (fuse) ps = stream_params_up(*shared);
  return int8 ? launch_stream<true, true>(p, a.n_groups_max, a.rows_max, s, fuse ? &ps : nullptr)
              : launch_stream<false, true>(p, a.n_groups_max, a.rows_max, s, fuse ? &ps : nullptr);
}

hipError_t launch_ffn_down(const FfnArgs& a, hipStream_t s, const FfnArgs* shared) {
  if (a.wdtype == ATENIA_MOE_WEIGHT_F32) return launch_ffn_down_f32(a, s);
  if (a.use_tiled) return launch_ffn_down_tiled(a, s);
  const bool int8 = a.wdtype == ATENIA_MOE_WEIGHT_INT8_W8A16;
  const StreamParams p = stream_params_down(a);
  if (a.use_mid) {
    if (!ffn_mid_supported(a.down, a.wdtype) || p.g.idx1) return hipErrorInvalidValue;
    StreamParams pm;
    const bool fuse_mid = can_fuse_shared(a, shared, true);
    if (fuse_mid) pm = stream_params_down(*shared);
    return int8 ? launch_mid<true, false>(p, a.n_groups_max, a.rows_max, s, fuse_mid ? &pm : nullptr)
                : launch_mid<false, false>(p, a.n_groups_max, a.rows_max, s, fuse_mid ? &pm : nullptr);
  }
  StreamParams ps;
  const bool fuse = can_fuse_shared(a, shared, true);
  if (fuse) ps = stream_params_down(*shared);
  return int8 ? launch_stream<true, false>(p, a.n_groups_max, a.rows_max, s, fuse ? &ps : nullptr)
              : launch_stream<false, false>(p, a.n_groups_max, a.rows_max, s, fuse ? &ps : nullptr);
}

// Waves per routed expert (sr) and of the shared expert (ss) for the single-token down +
// combine launch: powers of two up to 8 (a wave takes 8 / sr of the eight K slices),
// k sr + ss <= 16 waves, the longest share as short as possible, then as many waves as
// possible.  False when the token's experts do not fit 16 waves.
static bool decode1_slices(int k, int nkb_r, int nkb_s, int* sr_out, int* ss_out) {
  long best = -1;
  for (int sr = 1; sr <= 8; sr *= 2) {
    for (int ss = nkb_s > 0 ? 1 : 0; ss <= (nkb_s > 0 ? 8 : 0); ss = ss ? ss * 2 : 9) {
      if (k * sr + ss > 16) continue;
      const int lr = (nkb_r + sr - 1) / sr, ls = ss ? (nkb_s + ss - 1) / ss : 0;
      const long cost = (long)(lr > ls ? lr : ls) * 64 - (k * sr + ss);
      if (best < 0 || cost < best) {
        best = cost;
        *sr_out = sr;
        *ss_out = ss;
      }
    }
  }
  return best >= 0;
}

bool ffn_down_decode1_supported(int T, const FfnArgs& a, int k, bool tiled, const FfnArgs* shared) {
  if (!(T == 1 && k >= 1 && a.wdtype != ATENIA_MOE_WEIGHT_F32 && !tiled &&
        a.down.group_blocks == 0))
    return false;
  if (!shared) return k <= 15;
  if (shared->wdtype != a.wdtype || shared->use_tiled || shared->down.group_blocks != 0 ||
      shared->down.n_rows != a.down.n_rows || shared->down.n_pad != a.down.n_pad)
    return false;
  int sr, ss;
  const int kb = a.wdtype == ATENIA_MOE_WEIGHT_INT8_W8A16 ? kKbInt8 : kKbBf16;
  return decode1_slices(k, a.down.k_pad / kb, shared->down.k_pad / kb, &sr, &ss);
}

hipError_t launch_ffn_down_decode1(const FfnArgs& a, hipStream_t s, const FfnArgs* shared) {
  const bool int8 = a.wdtype == ATENIA_MOE_WEIGHT_INT8_W8A16;
  const StreamParams p = stream_params_down(a);
  const dim3 grid(a.down.n_pad / 16);
  if (!shared && a.fuse_k <= 2) {
    const int threads = 64 * 8 * a.fuse_k;
    if (int8)
      ffn_down_decode1_kernel<true><<<grid, threads, 0, s>>>(p, a.fuse_k, a.fuse_w,
                                                             a.fuse_residual, a.fuse_out);
    else
      ffn_down_decode1_kernel<false><<<grid, threads, 0, s>>>(p, a.fuse_k, a.fuse_w,
                                                              a.fuse_residual, a.fuse_out);
    return hipGetLastError();
  }
  const StreamParams ps = shared ? stream_params_down(*shared) : p;
  int sr = 1, ss = 0;
  if (!decode1_slices(a.fuse_k, p.nkb, shared ? ps.nkb : 0, &sr, &ss)) return hipErrorInvalidValue;
  const int threads = 64 * (a.fuse_k * sr + ss);
  const int halves = (int)grid.x * 2 <= (a.n_cus > 0 ? a.n_cus : 256) ? 2 : 1;
  const dim3 g2(grid.x * halves);
  // h rows in LDS when the router left the token's experts in idx1 (row j = expert j's h) and
  // they fit next to the reduction buffer
  const size_t kb_elems = int8 ? kKbInt8 : kKbBf16;
  const size_t h_bytes = ((size_t)a.fuse_k * p.nkb + (shared ? ps.nkb : 0)) * kb_elems * 2;
  const int stage_h = a.g.idx1 != nullptr && h_bytes <= 48 * 1024;
  const size_t smem = stage_h ? h_bytes : 0;
  if (int8)
    ffn_down_combine1_kernel<true><<<g2, threads, smem, s>>>(p, ps, a.fuse_k, sr, ss, halves, stage_h,
                                                             a.fuse_w, a.fuse_sgate,
                                                             a.fuse_residual, a.fuse_out);
  else
    ffn_down_combine1_kernel<false><<<g2, threads, smem, s>>>(p, ps, a.fuse_k, sr, ss, halves, stage_h,
                                                              a.fuse_w, a.fuse_sgate,
                                                              a.fuse_residual, a.fuse_out);
  return hipGetLastError();
}

// ---- load-time repack of a row-major matrix into B blocks -------------------------------
namespace {
// One thread writes one 16-byte lane slot of one block.
__global__ void repack_blocks_kernel(const uint8_t* __restrict__ src, uint4* __restrict__ dst,
                                     int n_rows, int k_cols, int n_pad, int k_pad,
                                     int elem_bytes) {
  const int epl = 16 / elem_bytes;       // elements per lane slot
  const int KB = 4 * epl;                // k per block
  const int nkb = k_pad / KB;
  size_t slot = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  size_t total = (size_t)(n_pad / 16) * nkb * 64;
  if (slot >= total) return;
  int lane = slot & 63;
  size_t blk = slot >> 6;
  int kb = blk % nkb;
  int nb = blk / nkb;
  int row = nb * 16 + (lane & 15);
  int k0 = kb * KB + epl * (lane >> 4);
  alignas(16) uint8_t buf[16];
  for (int j = 0; j < 16; ++j) buf[j] = 0;
  if (row < n_rows) {
    for (int j = 0; j < epl; ++j) {
      int kk = k0 + j;
      if (kk < k_cols)
        for (int b = 0; b < elem_bytes; ++b)
          buf[j * elem_bytes + b] = src[((size_t)row * k_cols + kk) * elem_bytes + b];
    }
  }
  dst[slot] = *(const uint4*)buf;
}
}  // namespace

namespace {
// One thread converts one 16-byte lane slot of an int8 block (row r = lane % 16, 16 consecutive
// k) into the two lane slots of the bf16 block layout that hold the same elements.
__global__ void dequant_group_blocks_kernel(const uint4* __restrict__ q,
                                            const float* __restrict__ scales,
                                            uint4* __restrict__ out, int n_pad, int nkb8,
                                            int group_blocks, int n_kgroups, size_t total) {
  const size_t slot = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (slot >= total) return;
  const int lane = (int)(slot & 63);
  const size_t blk = slot >> 6;
  const int kb = (int)(blk % nkb8);
  const size_t strip = blk / nkb8;                 // g * (n_pad / 16) + nb
  const int nb = (int)(strip % (n_pad / 16));
  const size_t g = strip / (n_pad / 16);
  const int row = nb * 16 + (lane & 15), q4 = lane >> 4;
  // no scales: the int8 values themselves (every one is a bf16 value)
  const float sc = scales ? scales[(g * n_kgroups + kb / group_blocks) * n_pad + row] : 1.f;
  const uint4 v = q[slot];
  const uint32_t w[4] = {v.x, v.y, v.z, v.w};
  uint32_t o[8];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float f0 = (float)(int8_t)(w[i] & 0xff) * sc, f1 = (float)(int8_t)((w[i] >> 8) & 0xff) * sc;
    const float f2 = (float)(int8_t)((w[i] >> 16) & 0xff) * sc, f3 = (float)(int8_t)(w[i] >> 24) * sc;
    o[2 * i] = (uint32_t)bf16_rne(f0) | ((uint32_t)bf16_rne(f1) << 16);
    o[2 * i + 1] = (uint32_t)bf16_rne(f2) | ((uint32_t)bf16_rne(f3) << 16);
  }
  // int8 block kb, k offset 16 * q4 -> bf16 block 2 kb + q4 / 2, k offsets 8 * (2 (q4 % 2) + h)
  const size_t oblk = (strip * (size_t)(2 * nkb8) + (size_t)(2 * kb + (q4 >> 1))) * 64;
  const int olane = (lane & 15) + 16 * (2 * (q4 & 1));
  out[oblk + olane] = make_uint4(o[0], o[1], o[2], o[3]);
  out[oblk + olane + 16] = make_uint4(o[4], o[5], o[6], o[7]);
}
}  // namespace

hipError_t launch_dequant_group_blocks(const void* q_blocks, const float* scales, void* bf16_blocks,
                                       int G, int n_pad, int k_pad, int group_blocks, int n_kgroups,
                                       hipStream_t s) {
  const int nkb8 = k_pad / kKbInt8;
  const size_t total = (size_t)G * (n_pad / 16) * nkb8 * 64;
  if (total == 0) return hipSuccess;
  dequant_group_blocks_kernel<<<(unsigned)((total + 255) / 256), 256, 0, s>>>(
      (const uint4*)q_blocks, scales, (uint4*)bf16_blocks, n_pad, nkb8, group_blocks, n_kgroups, total);
  return hipGetLastError();
}

hipError_t launch_repack_blocks(const void* src, void* dst, int n_rows, int k_cols, int n_pad,
                                int k_pad, int elem_bytes, hipStream_t s) {
  const int KB = 4 * (16 / elem_bytes);
  size_t total = (size_t)(n_pad / 16) * (k_pad / KB) * 64;
  int blocks = (int)((total + 255) / 256);
  repack_blocks_kernel<<<blocks, 256, 0, s>>>((const uint8_t*)src, (uint4*)dst, n_rows, k_cols,
                                              n_pad, k_pad, elem_bytes);
  return hipGetLastError();
}

}  // namespace atenia_moe
