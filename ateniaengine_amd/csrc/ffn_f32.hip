// Kernel 3, f32-weight form: the reference's certified expert arithmetic on the GPU.
//
// f32 storage, f64 accumulation, and the reference's cast sequence
// (src/moe/dense.rs:74-77, 97-115, 253-270):
//   gate = (f32) sum_f64(W_g x);  up = (f32) sum_f64(W_u x)
//   h    = (f32)(silu_f64(gate)) * up        -- an f32 product
//   y    = (f32) sum_f64(W_d h)
// Only the order of the f64 additions differs from the CPU path (k is tiled), which moves a
// result by ~1e-16 relative before the final f32 rounding.  Two forms: the f64 matrix cores
// (ffn_f32_mfma_kernel, K a multiple of 8) and a scalar tile kernel for every other shape and
// for the f32-accumulating policies.
//
// F32ACC: the reference's other expert arithmetic (`matvec_f32`, src/moe/dense.rs:120-140, used
// under NumericPolicy::Strict and as the result `Fast` falls back to): the three projections
// accumulate in f32, acc = acc + w * x with the product and the sum rounded separately, c
// ascending.  A thread walks the k tiles in order, so its f32 sequence IS the reference's; the
// file is compiled without contraction so that no product is fused into the sum.  silu stays
// f64 -> f32 and the router stays f64 on every policy (src/moe/numeric_policy.rs:24-29).
#include <cstdlib>

#include "moe_internal.h"

namespace atenia_moe {

namespace {

constexpr int kTile = 32;
constexpr int kLdT = kTile + 1;

template <bool UP, bool F32ACC>
__global__ __launch_bounds__(256) void ffn_f32_kernel(
    const float* __restrict__ wa, const float* __restrict__ wb, int64_t w_stride, int n_rows,
    int k_cols, int n_pad, int k_pad, const float* __restrict__ a, int a_stride,
    float* __restrict__ out, int out_stride, GroupDesc g) {
  const int u = blockIdx.y;
  if (u >= *g.n_active) return;
  const int e = g.active[u];
  const int base = g.offsets[e];
  const int cnt = g.offsets[e + 1] - base;
  const int m0 = blockIdx.z * kTile;
  if (m0 >= cnt) return;
  const int n0 = blockIdx.x * kTile;
  const int tid = threadIdx.x, tx = tid & 31, ty = tid >> 5;

  __shared__ float sA[kTile * kLdT];
  __shared__ float sBa[kTile * kLdT];
  __shared__ float sBb[UP ? kTile * kLdT : 1];
  __shared__ int sRow[kTile];  // source row of A for each tile row, -1 = none

  if (tid < kTile) {
    int pos = m0 + tid;
    int row = -1;
    if (pos < cnt) row = UP ? g.perm[base + pos] / g.pair_div : base + pos;
    sRow[tid] = row;
  }
  const float* wae = wa + (size_t)e * w_stride;
  const float* wbe = UP ? wb + (size_t)e * w_stride : nullptr;
  // The 32 x 32 weight tile is four 1 KiB blocks (two strips of 16 rows x two blocks of 16 k): a
  // thread fetches one lane slot, 4 consecutive k of one row, as one 16-byte load.
  const int w_strip = n0 / 16 + (tid >> 7), w_kb2 = (tid >> 6) & 1, w_slot = tid & 63;
  const int w_r = 16 * (tid >> 7) + (w_slot & 15), w_c = 16 * w_kb2 + 4 * (w_slot >> 4);
  const int nkb = k_pad / kKbF32;
  const bool w_row_ok = w_strip < n_pad / 16;

  double acc_a[4] = {0, 0, 0, 0}, acc_b[4] = {0, 0, 0, 0};
  float facc_a[4] = {0.f, 0.f, 0.f, 0.f}, facc_b[4] = {0.f, 0.f, 0.f, 0.f};
  // A thread stages elements (r, c) = (tid / 32 + 8 q, tid % 32), q = 0..3, of each 32 x 32 tile.
  // The next tile's elements are fetched into registers before the current tile is multiplied,
  // so a k tile does not start with a memory round trip (the sums and their order are untouched).
  __syncthreads();  // sRow
  float ra[4];
  float4 rba, rbb;
  auto fetch = [&](int k0) {
    const int c = tid & 31, kk = k0 + c;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int r = (tid >> 5) + 8 * q;
      const int src = sRow[r];
      ra[q] = (src >= 0 && kk < k_cols) ? a[(size_t)src * a_stride + kk] : 0.f;
    }
    const int kb = k0 / kKbF32 + w_kb2;  // rows past n_rows and columns past k_cols hold zeros
    const bool ok = w_row_ok && kb < nkb;
    const size_t at = ((size_t)w_strip * nkb + kb) * 256 + w_slot * 4;
    rba = ok ? *(const float4*)(wae + at) : float4{0.f, 0.f, 0.f, 0.f};
    rbb = (UP && ok) ? *(const float4*)(wbe + at) : float4{0.f, 0.f, 0.f, 0.f};
  };
  fetch(0);
  for (int k0 = 0; k0 < k_cols; k0 += kTile) {
    __syncthreads();
    {
      const int c = tid & 31;
#pragma unroll
      for (int q = 0; q < 4; ++q) sA[((tid >> 5) + 8 * q) * kLdT + c] = ra[q];
      const float va[4] = {rba.x, rba.y, rba.z, rba.w}, vb[4] = {rbb.x, rbb.y, rbb.z, rbb.w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        sBa[w_r * kLdT + w_c + j] = va[j];
        if (UP) sBb[w_r * kLdT + w_c + j] = vb[j];
      }
    }
    __syncthreads();
    if (k0 + kTile < k_cols) fetch(k0 + kTile);
    if (F32ACC) {
      // tile columns past k_cols hold +0.0: acc + 0 * 0 leaves every sum as it was (a sum that
      // starts at +0.0 never becomes -0.0)
#pragma unroll 8
      for (int c = 0; c < kTile; ++c) {
        const float ba = sBa[tx * kLdT + c];
        const float bb = UP ? sBb[tx * kLdT + c] : 0.f;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float av = sA[(ty * 4 + i) * kLdT + c];
          facc_a[i] = facc_a[i] + ba * av;  // two roundings (no contraction in this file)
          if (UP) facc_b[i] = facc_b[i] + bb * av;
        }
      }
      continue;
    }
#pragma unroll 8
    for (int c = 0; c < kTile; ++c) {
      double ba = (double)sBa[tx * kLdT + c];
      double bb = UP ? (double)sBb[tx * kLdT + c] : 0.0;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        double av = (double)sA[(ty * 4 + i) * kLdT + c];
        acc_a[i] = fma(ba, av, acc_a[i]);
        if (UP) acc_b[i] = fma(bb, av, acc_b[i]);
      }
    }
  }
  const int n = n0 + tx;
  if (n >= n_rows) return;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    int pos = m0 + ty * 4 + i;
    if (pos >= cnt) continue;
    if (UP) {
      float gate = F32ACC ? facc_a[i] : (float)acc_a[i];
      float up = F32ACC ? facc_b[i] : (float)acc_b[i];
      double gd = (double)gate;
      float s = (float)(gd / (1.0 + exp(-gd)));
      out[(size_t)(base + pos) * out_stride + n] = __fmul_rn(s, up);
    } else {
      int pair = g.perm[base + pos];
      out[(size_t)pair * out_stride + n] = F32ACC ? facc_a[i] : (float)acc_a[i];
    }
  }
}

// ---- certified arithmetic on the f64 matrix cores ---------------------------------------------
// v_mfma_f64_16x16x4_f64: D[16 x 16] += A[16 x 4] * B[4 x 16] in f64.  Lane l supplies
// A[l % 16][l / 16] and B[l / 16][l % 16] (one double each) and holds D[4 * r + l / 16][l % 16],
// r = 0..3 (rows interleaved, unlike the f32 forms).  Here A = 16 weight rows, B = 16 token rows
// (transposed), so a lane's four results are weight rows l / 16, +4, +8, +12 of one token.
//
// f32 operands widen to f64 exactly and every product of two f32 values is exact in f64, so the
// only difference from the reference's c-ascending sum is the order of the f64 additions
// (~1e-16 relative before the f32 rounding) -- the same statement as for the scalar kernel above,
// at the matrix cores' rate.
//
// A workgroup owns a strip of 16 weight rows (gate and up strips in the gate/up phase) of one
// expert and up to MT * 16 of its token rows; its four waves split K and add their partial sums
// in wave order through LDS.  A lane holds 8 k of "its" row per step (row l % 16; two quads of 4
// consecutive k, the lane's slots of two weight blocks) for both operands; MFMA t of the step
// contracts element t of every lane's eight, i.e. k = k0 + 4 * (l / 16) + t for t < 4 and
// k0 + 16 + 4 * (l / 16) + t - 4 beyond -- any partition of k into groups of four is as good as
// another as long as A and B agree.  The weights come in 1 KiB blocks (moe_internal.h): read
// row-major, 16 lanes of a load touched 16 different rows, and the launch moved its bytes at
// 3 TB/s.
typedef __attribute__((__vector_size__(4 * sizeof(double)))) double f64x4;

// KS: waves that share one strip's K (4: one strip per workgroup, partial sums meet in LDS;
// 1: four strips per workgroup, one per wave, no reduction -- better when K is short).
template <bool UP, int MT, int KS>
__global__ __launch_bounds__(256) void ffn_f32_mfma_kernel(
    const float* __restrict__ wa, const float* __restrict__ wb, int64_t w_stride, int n_rows,
    int k_cols, int k_pad, const float* __restrict__ a, int a_stride, float* __restrict__ out,
    int out_stride, GroupDesc g) {
  const int u = blockIdx.y;
  if (u >= *g.n_active) return;
  const int e = g.active[u];
  const int base = g.offsets[e];
  const int cnt = g.offsets[e + 1] - base;
  const int m0 = blockIdx.z * 16 * MT;
  if (m0 >= cnt) return;
  const int mt_live = __builtin_amdgcn_readfirstlane(min(MT, (cnt - m0 + 15) >> 4));
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int n0 = (blockIdx.x * (4 / KS) + wave / KS) * 16;
  if (KS == 1 && n0 >= n_rows) return;  // whole wave past the last strip (no barrier follows)
  const int kslice = wave % KS;
  const int r16 = lane & 15, q = lane >> 4;
  constexpr int NACC = UP ? 2 : 1;

  // The strip's weights are 1 KiB blocks of 16 rows x 16 k, in k order: lane l's slot of a block
  // is row l % 16, k = 16 kb + 4 (l / 16) .. + 3, so a wave reads a block as one contiguous KiB
  // (rows past n_rows and columns past k_cols hold zeros).  A step takes two blocks: the lane's
  // eight k are 32 st + 4 q + {0..3} and 32 st + 16 + 4 q + {0..3}, for the token rows too.
  const int nkb = k_pad / kKbF32;
  const float* pa = wa + (size_t)e * w_stride + (size_t)(n0 / 16) * nkb * 256 + lane * 4;
  const float* pb = UP ? wb + (size_t)e * w_stride + (size_t)(n0 / 16) * nkb * 256 + lane * 4 : nullptr;
  const float* px[MT];
#pragma unroll
  for (int i = 0; i < MT; ++i) {
    int pos = m0 + 16 * i + r16;
    if (pos >= cnt) pos = m0;  // an output column depends on its own token only; never stored
    const int row = UP ? g.perm[base + pos] / g.pair_div : base + pos;
    px[i] = a + (size_t)row * a_stride + 4 * q;
  }

  // K in steps of 32 (8 per lane chunk), the steps dealt to the KS waves in contiguous runs
  const int nsteps = (k_cols + 31) / 32;
  const int per = (nsteps + KS - 1) / KS;
  const int s0 = kslice * per, s1 = min(nsteps, s0 + per);
  f64x4 acc[NACC][MT];
#pragma unroll
  for (int n = 0; n < NACC; ++n)
#pragma unroll
    for (int i = 0; i < MT; ++i) acc[n][i] = f64x4{0.0, 0.0, 0.0, 0.0};

  struct Chunk {
    float4 lo, hi;
  };
  // No branch around a load: with one the compiler cannot count the loads in flight any more
  // and waits for all of them before every use (one memory round trip per step).  A chunk past
  // the end of a row (k_cols is a multiple of 8: a chunk is whole or absent) is fetched from the
  // row's first columns and zeroed with selects; a step past the wave's range repeats its last.
  auto keep = [](float4& v, bool in) {
    v.x = in ? v.x : 0.f; v.y = in ? v.y : 0.f; v.z = in ? v.z : 0.f; v.w = in ? v.w : 0.f;
  };
  // token rows (row-major): the two quads of the step, each whole or absent (k_cols % 4 == 0)
  auto load8 = [&](const float* p, int st) {
    Chunk c;
    const bool in_lo = st * 32 + 4 * q < k_cols, in_hi = st * 32 + 16 + 4 * q < k_cols;
    c.lo = *(const float4*)(p + (in_lo ? (size_t)st * 32 : 0));
    c.hi = *(const float4*)(p + (in_hi ? (size_t)st * 32 + 16 : 0));
    keep(c.lo, in_lo);
    keep(c.hi, in_hi);
    return c;
  };
  // weights: blocks 2 st and 2 st + 1 of the strip (the second may lie past the last block)
  auto load_w = [&](const float* p, int st) {
    Chunk c;
    const bool in_hi = 2 * st + 1 < nkb;
    c.lo = *(const float4*)(p + (size_t)(2 * st) * 256);
    c.hi = *(const float4*)(p + (size_t)(in_hi ? 2 * st + 1 : 0) * 256);
    keep(c.hi, in_hi);
    return c;
  };
  auto elem = [](const Chunk& c, int t) {
    const float v[8] = {c.lo.x, c.lo.y, c.lo.z, c.lo.w, c.hi.x, c.hi.y, c.hi.z, c.hi.w};
    return (double)v[t];
  };
  Chunk wA[2], wB[2], xs[2][MT] = {};
  auto load_step = [&](int buf, int st) {
    st = min(st, s1 - 1);
    wA[buf] = load_w(pa, st);
    if (UP) wB[buf] = load_w(pb, st);
#pragma unroll
    for (int i = 0; i < MT; ++i) xs[buf][i] = load8(px[i], st);  // rows past the end: clamped
  };
  auto multiply = [&](int buf) {
#pragma unroll
    for (int t = 0; t < 8; ++t) {
      const double va = elem(wA[buf], t);
      const double vb = UP ? elem(wB[buf], t) : 0.0;
#pragma unroll
      for (int i = 0; i < MT; ++i) {
        if (i >= mt_live) continue;  // scalar branch: a 16-row tile without rows costs no MFMAs
        const double vx = elem(xs[buf][i], t);
        acc[0][i] = __builtin_amdgcn_mfma_f64_16x16x4f64(va, vx, acc[0][i], 0, 0, 0);
        if (UP) acc[NACC - 1][i] = __builtin_amdgcn_mfma_f64_16x16x4f64(vb, vx, acc[NACC - 1][i], 0, 0, 0);
      }
    }
  };
  if (s0 < s1) {
    load_step(0, s0);
    for (int st = s0; st < s1; st += 2) {
      load_step(1, st + 1);
      multiply(0);
      load_step(0, st + 2);
      if (st + 1 < s1) multiply(1);  // a scalar branch around matrix instructions only
    }
  }

  if (KS > 1) {  // partial sums of waves 1..3 to LDS, wave 0 adds them in wave order
    __shared__ f64x4 red[KS > 1 ? KS - 1 : 1][NACC][MT][64];
    if (wave > 0) {
#pragma unroll
      for (int n = 0; n < NACC; ++n)
#pragma unroll
        for (int i = 0; i < MT; ++i) red[wave - 1][n][i][lane] = acc[n][i];
    }
    __syncthreads();
    if (wave != 0) return;
#pragma unroll
    for (int w = 0; w < KS - 1; ++w)
#pragma unroll
      for (int n = 0; n < NACC; ++n)
#pragma unroll
        for (int i = 0; i < MT; ++i) acc[n][i] += red[w][n][i][lane];
  }

#pragma unroll
  for (int i = 0; i < MT; ++i) {
    const int pos = m0 + 16 * i + r16;  // the lane's token
    if (pos >= cnt) continue;
    const int pair = UP ? 0 : g.perm[base + pos];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int n = n0 + 4 * r + q;
      if (n >= n_rows) continue;
      if (UP) {
        const float gate = (float)acc[0][i][r];
        const float up = (float)acc[NACC - 1][i][r];
        const double gd = (double)gate;
        const float sv = (float)(gd / (1.0 + exp(-gd)));
        out[(size_t)(base + pos) * out_stride + n] = __fmul_rn(sv, up);
      } else {
        out[(size_t)pair * out_stride + n] = (float)acc[0][i][r];
      }
    }
  }
}

// The matrix-core form needs whole 8-element chunks and 16-byte aligned rows.
bool mfma_f64_ok(const FfnArgs& a, bool up) {
  const int k = up ? a.gate.k_cols : a.down.k_cols;
  const int stride = up ? a.x_stride : a.h_stride;
  const void* act = up ? a.x : a.h;
  return !a.f32_accumulate && k % 8 == 0 && stride % 4 == 0 && ((uintptr_t)act & 15) == 0;
}

// Four waves on one strip's K, or one strip per wave: split unless K is a few steps only.
bool mfma_f64_splits_k(int n_rows, int k_cols) {
  (void)n_rows;
  return k_cols >= 128;  // measured at d = 1024, f = 2048, T = 64: gate/up 53 against 59 us, down 32 against 69
}

}  // namespace

hipError_t launch_ffn_up_f32(const FfnArgs& a, hipStream_t s) {
  if (mfma_f64_ok(a, true)) {
    const int mt = a.rows_max <= 16 ? 1 : 2;
    const bool split = mfma_f64_splits_k(a.gate.n_rows, a.gate.k_cols);
    const int strips = (a.gate.n_rows + 15) / 16;
    dim3 grid(split ? strips : (strips + 3) / 4, a.n_groups_max, (a.rows_max + 16 * mt - 1) / (16 * mt));
    auto k = split ? (mt == 1 ? ffn_f32_mfma_kernel<true, 1, 4> : ffn_f32_mfma_kernel<true, 2, 4>)
                   : (mt == 1 ? ffn_f32_mfma_kernel<true, 1, 1> : ffn_f32_mfma_kernel<true, 2, 1>);
    k<<<grid, 256, 0, s>>>((const float*)a.gate.w, (const float*)a.up.w, a.gate.expert_stride,
                           a.gate.n_rows, a.gate.k_cols, a.gate.k_pad, (const float*)a.x, a.x_stride,
                           (float*)a.h, a.h_stride, a.g);
    return hipGetLastError();
  }
  dim3 grid((a.gate.n_rows + kTile - 1) / kTile, a.n_groups_max,
            (a.rows_max + kTile - 1) / kTile);
  auto k = a.f32_accumulate ? ffn_f32_kernel<true, true> : ffn_f32_kernel<true, false>;
  k<<<grid, 256, 0, s>>>((const float*)a.gate.w, (const float*)a.up.w, a.gate.expert_stride,
                         a.gate.n_rows, a.gate.k_cols, a.gate.n_pad, a.gate.k_pad, (const float*)a.x,
                         a.x_stride, (float*)a.h, a.h_stride, a.g);
  return hipGetLastError();
}

hipError_t launch_ffn_down_f32(const FfnArgs& a, hipStream_t s) {
  if (mfma_f64_ok(a, false)) {
    const int mt = a.rows_max <= 16 ? 1 : 2;
    const bool split = mfma_f64_splits_k(a.down.n_rows, a.down.k_cols);
    const int strips = (a.down.n_rows + 15) / 16;
    dim3 grid(split ? strips : (strips + 3) / 4, a.n_groups_max, (a.rows_max + 16 * mt - 1) / (16 * mt));
    auto k = split ? (mt == 1 ? ffn_f32_mfma_kernel<false, 1, 4> : ffn_f32_mfma_kernel<false, 2, 4>)
                   : (mt == 1 ? ffn_f32_mfma_kernel<false, 1, 1> : ffn_f32_mfma_kernel<false, 2, 1>);
    k<<<grid, 256, 0, s>>>((const float*)a.down.w, nullptr, a.down.expert_stride, a.down.n_rows,
                           a.down.k_cols, a.down.k_pad, (const float*)a.h, a.h_stride, a.y, a.y_stride,
                           a.g);
    return hipGetLastError();
  }
  dim3 grid((a.down.n_rows + kTile - 1) / kTile, a.n_groups_max,
            (a.rows_max + kTile - 1) / kTile);
  auto k = a.f32_accumulate ? ffn_f32_kernel<false, true> : ffn_f32_kernel<false, false>;
  k<<<grid, 256, 0, s>>>((const float*)a.down.w, nullptr, a.down.expert_stride, a.down.n_rows,
                         a.down.k_cols, a.down.n_pad, a.down.k_pad, (const float*)a.h, a.h_stride, a.y,
                         a.y_stride, a.g);
  return hipGetLastError();
}

}  // namespace atenia_moe
