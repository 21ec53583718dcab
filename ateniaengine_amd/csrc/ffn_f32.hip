// Kernel 3, f32-weight form: the reference's certified expert arithmetic on the GPU.
//
// f32 storage, f64 accumulation, and the reference's cast sequence
// (src/moe/dense.rs:74-77, 97-115, 253-270):
//   gate = (f32) sum_f64(W_g x);  up = (f32) sum_f64(W_u x)
//   h    = (f32)(silu_f64(gate)) * up        -- an f32 product
//   y    = (f32) sum_f64(W_d h)
// Only the order of the f64 additions differs from the CPU path (k is tiled), which moves a
// result by ~1e-16 relative before the final f32 rounding.  This path exists for parity
// with f32 checkpoints (1e-5 bar); it is FMA-bound and not the throughput path.
//
// F32ACC: the reference's other expert arithmetic (`matvec_f32`, src/moe/dense.rs:120-140, used
// under NumericPolicy::Strict and as the result `Fast` falls back to): the three projections
// accumulate in f32, acc = acc + w * x with the product and the sum rounded separately, c
// ascending.  A thread walks the k tiles in order, so its f32 sequence IS the reference's; the
// file is compiled without contraction so that no product is fused into the sum.  silu stays
// f64 -> f32 and the router stays f64 on every policy (src/moe/numeric_policy.rs:24-29).
#include "moe_internal.h"

namespace atenia_moe {

namespace {

constexpr int kTile = 32;
constexpr int kLdT = kTile + 1;

template <bool UP, bool F32ACC>
__global__ __launch_bounds__(256) void ffn_f32_kernel(
    const float* __restrict__ wa, const float* __restrict__ wb, int64_t w_stride, int n_rows,
    int k_cols, const float* __restrict__ a, int a_stride, float* __restrict__ out,
    int out_stride, GroupDesc g) {
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

  double acc_a[4] = {0, 0, 0, 0}, acc_b[4] = {0, 0, 0, 0};
  float facc_a[4] = {0.f, 0.f, 0.f, 0.f}, facc_b[4] = {0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < k_cols; k0 += kTile) {
    __syncthreads();
    for (int j = tid; j < kTile * kTile; j += 256) {
      int r = j >> 5, c = j & 31;
      int kk = k0 + c;
      int src = sRow[r];
      sA[r * kLdT + c] = (src >= 0 && kk < k_cols) ? a[(size_t)src * a_stride + kk] : 0.f;
      int n = n0 + r;
      bool ok = n < n_rows && kk < k_cols;
      sBa[r * kLdT + c] = ok ? wae[(size_t)n * k_cols + kk] : 0.f;
      if (UP) sBb[r * kLdT + c] = ok ? wbe[(size_t)n * k_cols + kk] : 0.f;
    }
    __syncthreads();
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

}  // namespace

hipError_t launch_ffn_up_f32(const FfnArgs& a, hipStream_t s) {
  dim3 grid((a.gate.n_rows + kTile - 1) / kTile, a.n_groups_max,
            (a.rows_max + kTile - 1) / kTile);
  auto k = a.f32_accumulate ? ffn_f32_kernel<true, true> : ffn_f32_kernel<true, false>;
  k<<<grid, 256, 0, s>>>((const float*)a.gate.w, (const float*)a.up.w, a.gate.expert_stride,
                         a.gate.n_rows, a.gate.k_cols, (const float*)a.x, a.x_stride, (float*)a.h,
                         a.h_stride, a.g);
  return hipGetLastError();
}

hipError_t launch_ffn_down_f32(const FfnArgs& a, hipStream_t s) {
  dim3 grid((a.down.n_rows + kTile - 1) / kTile, a.n_groups_max,
            (a.rows_max + kTile - 1) / kTile);
  auto k = a.f32_accumulate ? ffn_f32_kernel<false, true> : ffn_f32_kernel<false, false>;
  k<<<grid, 256, 0, s>>>((const float*)a.down.w, nullptr, a.down.expert_stride, a.down.n_rows,
                         a.down.k_cols, (const float*)a.h, a.h_stride, a.y, a.y_stride, a.g);
  return hipGetLastError();
}

}  // namespace atenia_moe
