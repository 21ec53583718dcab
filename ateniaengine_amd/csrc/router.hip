// Kernel 1: router GEMV/GEMM + softmax + top-k, bit-exact with the reference's CPU router.
//
// Follows, operation for operation and cast for cast:
//   logits  = matvec(W_r, x)            src/moe/dense.rs:97-115, 325-337
//             one sequential, c-ascending f64 sum per (token, expert), rounded to f32 once
//   weights = softmax(logits)           src/moe/dense.rs:172-187
//             f32 max, f32 subtraction, f64 exp, sequential f64 sum, (f32)(e * (1/sum))
//   top-k                               src/moe/sparse.rs:142-191
//             order (f32 weight desc, index asc); selected indices emitted ascending;
//             f64 renormalisation over the selected weights in ascending order
//   shared-expert gate                  src/moe/layer.rs:436-443  sigmoid(f64 dot)
//
// Products of two f32 values are exact in f64, so fma(w, x, acc) rounds exactly like the
// reference's separate multiply and add.  Each (token, row) pair is owned by one thread
// that walks c = 0..d-1 in order, so the f64 sum is the reference's sum, not merely close.
#include "moe_internal.h"

namespace atenia_moe {

namespace {

constexpr int kRouterThreads = 256;
constexpr int kKc = 32;            // columns staged per step
constexpr int kLd = kKc + 1;       // padded LDS row stride (words)

__device__ inline float load_x(const float* x, size_t i) { return x[i]; }
__device__ inline float load_x(const uint16_t* x, size_t i) {
  return __uint_as_float(((uint32_t)x[i]) << 16);
}

// f32 -> bf16 bits, round to nearest even (NaN kept quiet).
__device__ inline uint16_t f32_to_bf16_rne(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

template <typename XT>
__global__ __launch_bounds__(kRouterThreads) void router_kernel(
    const XT* __restrict__ x, int T, int d, int E, int k, int renorm,
    const float* __restrict__ w_router, const float* __restrict__ bias,
    const float* __restrict__ gate_vec, int32_t* __restrict__ idx_out,
    float* __restrict__ w_out, float* __restrict__ sgate_out, uint16_t* __restrict__ xb,
    int d_pad, int32_t* __restrict__ status, int tokens_per_block) {
  const int R = E + (gate_vec ? 1 : 0);  // rows of the stacked [W_r ; gate] matrix
  const int TT = tokens_per_block;
  const int t0 = blockIdx.x * TT;
  const int tid = threadIdx.x;

  extern __shared__ float smem[];
  float* sW = smem;                       // [R][kLd]
  float* sX = sW + (size_t)R * kLd;       // [TT][kLd]
  // after the dot products the same memory is reused:
  //   sLogit [TT][R] f32, sExp [TT][E] f64, sWt [TT][E] f32, sSel [TT][E] i32

  const int tl = tid / R;  // local token
  const int r = tid - tl * R;
  const bool owner = tl < TT && (t0 + tl) < T;
  double acc = 0.0;

  const int c_end = xb ? (d_pad > d ? d_pad : d) : d;
  for (int c0 = 0; c0 < c_end; c0 += kKc) {
    __syncthreads();
    for (int j = tid; j < R * kKc; j += kRouterThreads) {
      int row = j / kKc, col = j - row * kKc;
      int c = c0 + col;
      float v = 0.f;
      if (c < d) v = row < E ? w_router[(size_t)row * d + c] : gate_vec[c];
      sW[row * kLd + col] = v;
    }
    for (int j = tid; j < TT * kKc; j += kRouterThreads) {
      int row = j / kKc, col = j - row * kKc;
      int c = c0 + col, t = t0 + row;
      float v = 0.f;
      if (t < T && c < d) v = load_x(x, (size_t)t * d + c);
      sX[row * kLd + col] = v;
      if (xb && t < T && c < d_pad) xb[(size_t)t * d_pad + c] = f32_to_bf16_rne(v);
    }
    __syncthreads();
    if (owner && c0 < d) {
      const float* wr = sW + r * kLd;
      const float* xr = sX + tl * kLd;
      // Columns past d hold zeros in both tiles: adding +0.0 leaves the sum unchanged.
#pragma unroll
      for (int c = 0; c < kKc; ++c) acc = fma((double)wr[c], (double)xr[c], acc);
    }
  }
  __syncthreads();

  float* sLogit = smem;                                   // [TT][R]
  double* sExp = (double*)(smem + ((TT * R + 1) & ~1));   // [TT][E]
  float* sWt = (float*)(sExp + (size_t)TT * E);           // [TT][E]
  int32_t* sSel = (int32_t*)(sWt + (size_t)TT * E);       // [TT][E]

  if (owner) {
    float logit = (float)acc;
    if (r < E) {
      if (bias) logit = logit + bias[r];
      sLogit[tl * R + r] = logit;
    } else {
      sgate_out[t0 + tl] = (float)(1.0 / (1.0 + exp(-acc)));
    }
  }
  __syncthreads();

  const bool expert_owner = owner && r < E;
  float my_logit = 0.f;
  if (expert_owner) {
    const float* lg = sLogit + tl * R;
    float mx = -INFINITY;
    for (int e = 0; e < E; ++e) mx = fmaxf(mx, lg[e]);  // skips NaN like f32::max
    my_logit = lg[r];
    sExp[tl * E + r] = exp((double)(my_logit - mx));    // f32 subtraction, then f64 exp
  }
  __syncthreads();
  float my_w = 0.f;
  if (expert_owner) {
    const double* ex = sExp + tl * E;
    double sum = 0.0;
    for (int e = 0; e < E; ++e) sum += ex[e];           // sequential fold, e ascending
    double inv = sum > 0.0 ? 1.0 / sum : 0.0;
    my_w = (float)(ex[r] * inv);
    sWt[tl * E + r] = my_w;
    if (!isfinite(my_w) || my_w < 0.f) {
      atomicMin(&status[0], -3);
      atomicMin(&status[1], ((t0 + tl) << 10) | r);
    }
  }
  __syncthreads();
  bool selected = false;
  if (expert_owner) {
    const float* wt = sWt + tl * E;
    int rank = 0;  // experts that sort before me under (weight desc, index asc)
    for (int e = 0; e < E; ++e) {
      float we = wt[e];
      rank += (we > my_w) || (we == my_w && e < r);
    }
    selected = rank < k;
    sSel[tl * E + r] = selected ? 1 : 0;
  }
  __syncthreads();
  if (expert_owner && selected) {
    const int32_t* sel = sSel + tl * E;
    const float* wt = sWt + tl * E;
    int slot = 0;
    double sum = 0.0;
    for (int e = 0; e < E; ++e) {
      if (sel[e]) {
        slot += e < r;
        sum += (double)wt[e];  // ascending e, as the reference sums the sorted selection
      }
    }
    double scale = renorm ? 1.0 / sum : 1.0;
    if (slot < k) {
      size_t o = (size_t)(t0 + tl) * k + slot;
      idx_out[o] = r;
      w_out[o] = (float)((double)my_w * scale);
    }
  }
}

}  // namespace

hipError_t launch_router(const RouterArgs& a, hipStream_t s) {
  const int R = a.E + (a.shared_gate ? 1 : 0);
  if (R > kMaxRouterRows || a.T <= 0) return hipErrorInvalidValue;
  int TT = kRouterThreads / R;
  if (TT < 1) TT = 1;
  // Keep enough blocks in flight for small batches.
  while (TT > 1 && (a.T + TT - 1) / TT < 256 && TT * R > 64) TT = (TT + 1) / 2;
  const int blocks = (a.T + TT - 1) / TT;
  size_t dot_bytes = ((size_t)R + TT) * kLd * sizeof(float);
  size_t post_bytes = (((size_t)TT * R + 1) & ~(size_t)1) * 4 + (size_t)TT * a.E * (8 + 4 + 4);
  size_t smem = dot_bytes > post_bytes ? dot_bytes : post_bytes;
  if (a.x_is_bf16) {
    router_kernel<uint16_t><<<blocks, kRouterThreads, smem, s>>>(
        (const uint16_t*)a.x, a.T, a.d, a.E, a.k, a.renorm, a.w_router, a.router_bias,
        a.shared_gate, a.idx, a.w, a.sgate, a.xb, a.d_pad, a.status, TT);
  } else {
    router_kernel<float><<<blocks, kRouterThreads, smem, s>>>(
        (const float*)a.x, a.T, a.d, a.E, a.k, a.renorm, a.w_router, a.router_bias,
        a.shared_gate, a.idx, a.w, a.sgate, a.xb, a.d_pad, a.status, TT);
  }
  return hipGetLastError();
}

}  // namespace atenia_moe
