// RMSNorm(x) * gamma for the decoder layer's FFN block: the step that precedes the MoE layer in
// src/moe/full_forward.rs:239-243 (graph: RmsNorm node + BroadcastMul node) and in
// src/moe/mla.rs:442, src/moe/decoder_layer.rs:97-107 (imperative, f64 accumulation).
//
// The normalised rows feed the router, so the arithmetic of the reference is kept, not just its
// value:
//   policy 0 (graph, src/nn/normalization.rs:8-37): sum of squares folded left to right in f32
//     (multiply and add rounded separately), mean = sum / max(cols, 1), inv = 1 / sqrt(mean + eps),
//     y = (x * inv) * gamma with both products rounded to f32.  The fold is a dependent chain of
//     `cols` additions per row and cannot be reassociated; the whole workgroup fetches a column
//     chunk and stores the (rounded) squares in LDS, then one lane per row adds them in order
//     while the next chunk is in flight; 4 rows per workgroup.
//   policy 1 (f64): sum of squares in f64 (the squares of f32 values are exact in f64), mean and
//     inverse root in f64, y = (float)(x * inv) * gamma.  The reference adds left to right; here 64
//     lanes per row add interleaved columns and the partial sums are added in lane order.  The two
//     orders differ by at most a few units of the f64 sum's last place, which the rounding of
//     x * inv to f32 hides except for values within ~1e-9 (relative) of a rounding boundary.
// HBM-bound at large T (reads x twice -- the second time from L2 -- and writes y once: 8 bytes of
// algorithmic traffic per element); at T <= 16 it is the latency of the fold.
#include "../../include/atenia_moe_hip.h"
#include "moe_internal.h"

// This file is compiled with -ffp-contract=off (see the Makefile): the reference rounds every
// product and every sum on its own, and hipcc would otherwise fuse `a * b + c` into one FMA
// (its default is -ffp-contract=fast, under which __fmul_rn / __fadd_rn are plain `*` and `+`
// and the fp-contract pragma is ignored).  sqrtf and `/` are hipcc's correctly rounded f32 forms;
// __fsqrt_rn is not.

namespace atenia_moe {

namespace {

constexpr int kRows = 4;           // rows (tokens) per workgroup: small, so several workgroups share a CU
constexpr int kChunk = 512;        // columns staged per step
constexpr int kPitch = kChunk + 4; // floats; 516 % 64 == 4: the walking lanes read disjoint banks
constexpr int kThreads = 256;
constexpr int kLanes = kThreads / kRows;  // f64 policy: lanes that share one row's sum
constexpr int kLoads = kRows * kChunk / 4 / kThreads;  // float4 per thread per chunk (2)

// Four consecutive floats of row `row` from column `col`; zero outside [0, T) x [0, d).
// VEC (d % 4 == 0, col % 4 == 0): one aligned 16-byte load from a clamped address, no branch.
template <bool VEC>
__device__ inline float4 load_x4(const float* __restrict__ x, int T, int d, int row, int col) {
  const bool ok = row < T && col < d;
  if (VEC) {
    const float4 v = *(const float4*)(x + (ok ? (size_t)row * d + col : 0));
    return ok ? v : make_float4(0.f, 0.f, 0.f, 0.f);
  }
  float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
  if (!ok) return v;
  const float* p = x + (size_t)row * d + col;
  v.x = p[0];
  if (col + 1 < d) v.y = p[1];
  if (col + 2 < d) v.z = p[2];
  if (col + 3 < d) v.w = p[3];
  return v;
}

template <int POLICY, bool VEC>
__global__ __launch_bounds__(kThreads) void rmsnorm_gamma_kernel(const float* __restrict__ x,
                                                                  const float* __restrict__ gamma,
                                                                  float eps, int T, int d,
                                                                  float* __restrict__ y) {
  __shared__ __attribute__((aligned(16))) float S[kRows * kPitch];
  __shared__ double part[kRows][kThreads / kRows];
  __shared__ double inv64[kRows];
  __shared__ float inv32[kRows];
  const int tid = threadIdx.x;
  const int t0 = blockIdx.x * kRows;
  const int n_chunks = (d + kChunk - 1) / kChunk;

  float4 pre[kLoads];
  auto fetch = [&](int chunk) {
#pragma unroll
    for (int i = 0; i < kLoads; ++i) {
      const int flat = i * kThreads + tid;
      pre[i] = load_x4<VEC>(x, T, d, t0 + flat / (kChunk / 4), chunk * kChunk + (flat % (kChunk / 4)) * 4);
    }
  };
  auto stash = [&]() {
#pragma unroll
    for (int i = 0; i < kLoads; ++i) {
      const int flat = i * kThreads + tid;
      float4 v = pre[i];
      if (POLICY == 0) {  // the walking lane only adds: every thread squares what it fetched
        v.x = v.x * v.x; v.y = v.y * v.y; v.z = v.z * v.z; v.w = v.w * v.w;
      }
      *(float4*)&S[(flat / (kChunk / 4)) * kPitch + (flat % (kChunk / 4)) * 4] = v;
    }
  };

  float s32 = 0.f;   // policy 0: the row's running sum (lanes 0..15 of wave 0)
  double s64 = 0.0;  // policy 1: this lane's share of row tid / kLanes
  fetch(0);
  for (int chunk = 0; chunk < n_chunks; ++chunk) {
    __syncthreads();  // the previous chunk has been consumed
    stash();
    __syncthreads();
    if (chunk + 1 < n_chunks) fetch(chunk + 1);  // in flight while the sums advance
    // Columns past d are zero in LDS and add +0 to a non-negative sum: no effect on any bit.
    const int width = min(kChunk, d - chunk * kChunk);
    if (POLICY == 0) {
      if (tid < kRows) {
        // Sixteen squares are added while the next sixteen are on their way from LDS (two
        // register sets, so nothing is copied).  Columns past `width` hold zeros.
        const float* row = S + tid * kPitch;
        float4 a0 = *(const float4*)(row), a1 = *(const float4*)(row + 4),
               a2 = *(const float4*)(row + 8), a3 = *(const float4*)(row + 12);
        for (int c = 0; c < width; c += 32) {
          const float4 b0 = *(const float4*)(row + c + 16), b1 = *(const float4*)(row + c + 20),
                       b2 = *(const float4*)(row + c + 24), b3 = *(const float4*)(row + c + 28);
          __builtin_amdgcn_sched_barrier(0);
          s32 += a0.x; s32 += a0.y; s32 += a0.z; s32 += a0.w;
          s32 += a1.x; s32 += a1.y; s32 += a1.z; s32 += a1.w;
          s32 += a2.x; s32 += a2.y; s32 += a2.z; s32 += a2.w;
          s32 += a3.x; s32 += a3.y; s32 += a3.z; s32 += a3.w;
          __builtin_amdgcn_sched_barrier(0);
          const int nc = (c + 32) & (kChunk - 1);  // past the chunk: a harmless re-read of column 0
          a0 = *(const float4*)(row + nc); a1 = *(const float4*)(row + nc + 4);
          a2 = *(const float4*)(row + nc + 8); a3 = *(const float4*)(row + nc + 12);
          __builtin_amdgcn_sched_barrier(0);
          s32 += b0.x; s32 += b0.y; s32 += b0.z; s32 += b0.w;
          s32 += b1.x; s32 += b1.y; s32 += b1.z; s32 += b1.w;
          s32 += b2.x; s32 += b2.y; s32 += b2.z; s32 += b2.w;
          s32 += b3.x; s32 += b3.y; s32 += b3.z; s32 += b3.w;
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    } else {
      const float* row = S + (tid / kLanes) * kPitch;
      for (int c = tid % kLanes; c < width; c += kLanes) {
        const double v = (double)row[c];
        s64 = fma(v, v, s64);  // v * v is exact in f64, so this is the separately rounded sum
      }
    }
  }

  if (POLICY == 0) {
    if (tid < kRows) {
      const float cols = (float)d;
      const float mean = s32 / (cols > 1.0f ? cols : 1.0f);
      inv32[tid] = 1.0f / sqrtf(mean + eps);
    }
  } else {
    part[tid / kLanes][tid % kLanes] = s64;
    __syncthreads();
    if (tid < kRows) {
      double ms = 0.0;
      for (int p = 0; p < kLanes; ++p) ms += part[tid][p];
      ms /= (double)d;
      inv64[tid] = 1.0 / sqrt(ms + (double)eps);
    }
  }
  __syncthreads();

  // y = (x * inv) * gamma, every product rounded on its own.  The rows of the group are
  // independent loads of one column block, so several are in flight per thread.
  const int d4 = (d + 3) / 4;
  for (int q = tid; q < d4; q += kThreads) {
    const int c = q * 4;
    const float4 g = load_x4<VEC>(gamma, 1, d, 0, c);
    float4 v[kRows];
#pragma unroll
    for (int r = 0; r < kRows; ++r) v[r] = load_x4<VEC>(x, T, d, t0 + r, c);
#pragma unroll
    for (int r = 0; r < kRows; ++r) {
      if (t0 + r >= T) break;
      float4 o;
      if (POLICY == 0) {
        const float i32 = inv32[r];
        o.x = (v[r].x * i32) * g.x; o.y = (v[r].y * i32) * g.y;
        o.z = (v[r].z * i32) * g.z; o.w = (v[r].w * i32) * g.w;
      } else {
        const double i64 = inv64[r];
        o.x = (float)((double)v[r].x * i64) * g.x; o.y = (float)((double)v[r].y * i64) * g.y;
        o.z = (float)((double)v[r].z * i64) * g.z; o.w = (float)((double)v[r].w * i64) * g.w;
      }
      float* out = y + (size_t)(t0 + r) * d + c;
      if (VEC) {
        *(float4*)out = o;
      } else {
        out[0] = o.x;
        if (c + 1 < d) out[1] = o.y;
        if (c + 2 < d) out[2] = o.z;
        if (c + 3 < d) out[3] = o.w;
      }
    }
  }
}

}  // namespace

hipError_t launch_rmsnorm_gamma(const NormArgs& a, hipStream_t s) {
  if (a.T <= 0 || a.d <= 0) return hipSuccess;
  const unsigned grid = (unsigned)((a.T + kRows - 1) / kRows);
  const bool vec = (a.d & 3) == 0;
#define ATENIA_NORM_LAUNCH(P, V) \
  rmsnorm_gamma_kernel<P, V><<<grid, kThreads, 0, s>>>(a.x, a.gamma, a.eps, a.T, a.d, a.y)
  if (a.policy == ATENIA_MOE_NORM_F64) {
    if (vec) ATENIA_NORM_LAUNCH(1, true); else ATENIA_NORM_LAUNCH(1, false);
  } else {
    if (vec) ATENIA_NORM_LAUNCH(0, true); else ATENIA_NORM_LAUNCH(0, false);
  }
#undef ATENIA_NORM_LAUNCH
  return hipGetLastError();
}

}  // namespace atenia_moe
