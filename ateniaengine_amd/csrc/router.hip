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
// reference's separate multiply and add.  Two kernels compute the dot products:
//
//  * router_tile_kernel (any batch): each (token, row) pair is owned by one thread that walks
//    c = 0..d-1 in order, so the f64 sum IS the reference's sum.
//  * router_token_kernel (small batches, where that serial chain would dominate the layer):
//    one workgroup per token, every row split over a wavefront and reduced with shuffles.
//    A different summation order is only allowed when it provably cannot change the result:
//    every product is an integer multiple of 2^q (q = the smallest exponent of a product's
//    lowest set bit) and every partial sum of any subset is bounded by A = sum |product|;
//    if A < 2^(q+53) every such partial sum is exactly representable in f64, so EVERY
//    summation order -- the reference's included -- is free of rounding and yields the same
//    exact value.  The kernel checks this per row (true for bf16-valued operands in
//    practice); when it fails for any row of the token, the token's rows are recomputed in
//    the reference's order.
#include "moe_internal.h"

namespace atenia_moe {

namespace {

constexpr int kRouterThreads = 256;
constexpr int kKc = 32;            // columns staged per step
constexpr int kLd = kKc + 1;       // padded LDS row stride (words)
constexpr int kTokenThreads = 1024;
constexpr int kNoLsb = 32767;      // lsb exponent marker of a zero

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

// Exponent of the lowest set bit of a finite f32 (v = odd * 2^result); kNoLsb for zero,
// and a hugely negative value for inf/NaN so that no exactness claim survives them.
__device__ inline int lsb_exponent(float v) {
  uint32_t b = __float_as_uint(v);
  int e = (b >> 23) & 0xff;
  uint32_t m = b & 0x7fffffu;
  if (e == 0xff) return -100000;
  if (e == 0) {
    if (m == 0) return kNoLsb;
    return -149 + (__ffs((int)m) - 1);
  }
  m |= 0x800000u;
  return e - 150 + (__ffs((int)m) - 1);
}

// Softmax + top-k + renormalisation of ONE token by the threads r = 0..E-1 that call with
// `on`; every thread of the workgroup must call (barriers inside).  lg: [E] f32 logits,
// ex: [E] f64, wt: [E] f32, sel: [E] i32 scratch of this token.
__device__ inline void softmax_topk(bool on, int r, int E, int k, int renorm, int token,
                                    const float* lg, double* ex, float* wt, int32_t* sel,
                                    int32_t* __restrict__ idx_out, float* __restrict__ w_out,
                                    int32_t* __restrict__ status) {
  float my_logit = 0.f;
  if (on) {
    float mx = -INFINITY;
    for (int e = 0; e < E; ++e) mx = fmaxf(mx, lg[e]);  // skips NaN like f32::max
    my_logit = lg[r];
    ex[r] = exp((double)(my_logit - mx));                // f32 subtraction, then f64 exp
  }
  __syncthreads();
  float my_w = 0.f;
  if (on) {
    double sum = 0.0;
    for (int e = 0; e < E; ++e) sum += ex[e];            // sequential fold, e ascending
    double inv = sum > 0.0 ? 1.0 / sum : 0.0;
    my_w = (float)(ex[r] * inv);
    wt[r] = my_w;
    if (!isfinite(my_w) || my_w < 0.f) {
      atomicMin(&status[0], -3);
      atomicMin(&status[1], (token << 10) | r);
    }
  }
  __syncthreads();
  bool selected = false;
  if (on) {
    int rank = 0;  // experts that sort before me under (weight desc, index asc)
    for (int e = 0; e < E; ++e) {
      float we = wt[e];
      rank += (we > my_w) || (we == my_w && e < r);
    }
    selected = rank < k;
    sel[r] = selected ? 1 : 0;
  }
  __syncthreads();
  if (on && selected) {
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
      size_t o = (size_t)token * k + slot;
      idx_out[o] = r;
      w_out[o] = (float)((double)my_w * scale);
    }
  }
}

template <typename XT>
__global__ __launch_bounds__(kRouterThreads) void router_tile_kernel(
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
  const int tls = owner ? tl : 0;
  softmax_topk(owner && r < E, r, E, k, renorm, t0 + tls, sLogit + tls * R, sExp + tls * E,
               sWt + tls * E, sSel + tls * E, idx_out, w_out, status);
}

// Outputs of the expert grouping for the single-token case (see permute.hip for the contract).
struct FusedGrouping {
  int32_t *counts, *offsets, *perm, *inv, *active, *n_active, *shared_offsets;
  int32_t *tile_group, *tile_m0, *n_tiles, *shared_n_tiles;
};

template <typename XT>
__global__ __launch_bounds__(kTokenThreads) void router_token_kernel(
    const XT* __restrict__ x, int T, int d, int E, int k, int renorm,
    const float* __restrict__ w_router, const float* __restrict__ bias,
    const float* __restrict__ gate_vec, int32_t* __restrict__ idx_out,
    float* __restrict__ w_out, float* __restrict__ sgate_out, uint16_t* __restrict__ xb,
    int d_pad, int32_t* __restrict__ status, FusedGrouping fg) {
  const int R = E + (gate_vec ? 1 : 0);
  const int t = blockIdx.x;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  constexpr int NW = kTokenThreads / 64;

  extern __shared__ double smem_d[];
  double* sAcc = smem_d;                       // [R]
  double* sExp = sAcc + R;                     // [E]
  double* sPart = sExp + E;                    // [max(R, NW)]
  double* sPartA = sPart + (R > NW ? R : NW);  // [max(R, NW)]
  float* sX = (float*)(sPartA + (R > NW ? R : NW));  // [d]
  float* sLogit = sX + d;                      // [E]
  float* sWt = sLogit + E;                     // [E]
  int32_t* sSel = (int32_t*)(sWt + E);         // [E]
  int32_t* sBad = sSel + E;                    // [1]
  int32_t* sPartQ = sBad + 1;                  // [max(R, NW)]
  int16_t* sLx = (int16_t*)(sPartQ + (R > NW ? R : NW));  // [d]

  if (tid == 0) *sBad = 0;
  const int c_end = xb ? (d_pad > d ? d_pad : d) : d;
  for (int c = tid; c < c_end; c += kTokenThreads) {
    float v = c < d ? load_x(x, (size_t)t * d + c) : 0.f;
    if (c < d) {
      sX[c] = v;
      sLx[c] = (int16_t)max(lsb_exponent(v), -32000);
    }
    if (xb && c < d_pad) xb[(size_t)t * d_pad + c] = f32_to_bf16_rne(v);
  }
  __syncthreads();

  // Work items: (row, k slice).  With few rows each row is split over several waves so that
  // all 16 waves stream the router matrix.  Partial results meet in LDS; under the exactness
  // certificate their order of addition cannot change the sum.
  const int KS = R >= NW ? 1 : NW / R;              // k slices per row
  const int slice = ((d + KS - 1) / KS + 3) & ~3;   // multiple of 4 for float4 loads
  const bool vec_ok = (d & 3) == 0;
  for (int item = wave; item < R * KS; item += NW) {
    const int r = item / KS, ksl = item - r * KS;
    const float* wr = r < E ? w_router + (size_t)r * d : gate_vec;
    const int c_lo = ksl * slice, c_hi = min(d, c_lo + slice);
    double acc = 0.0, asum = 0.0;
    int qmin = kNoLsb;
    auto one = [&](float wv, int c) {
      float xv = sX[c];
      double wd = (double)wv, xd = (double)xv;
      acc = fma(wd, xd, acc);
      asum = fma(fabs(wd), fabs(xd), asum);
      int lx = sLx[c];
      int lw = lsb_exponent(wv);
      if (lx != kNoLsb && lw != kNoLsb) qmin = min(qmin, lx + lw);
    };
    if (vec_ok) {
#pragma unroll 4
      for (int c = c_lo + lane * 4; c < c_hi; c += 256) {
        float4 w4 = *(const float4*)(wr + c);
        one(w4.x, c);
        one(w4.y, c + 1);
        one(w4.z, c + 2);
        one(w4.w, c + 3);
      }
    } else {
      for (int c = c_lo + lane; c < c_hi; c += 64) one(wr[c], c);
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
      acc += __shfl_xor(acc, off);
      asum += __shfl_xor(asum, off);
      qmin = min(qmin, __shfl_xor(qmin, off));
    }
    if (lane == 0) {
      sPart[item] = acc;
      sPartA[item] = asum;
      sPartQ[item] = qmin;
    }
  }
  __syncthreads();
  if (tid < R) {
    double acc = 0.0, asum = 0.0;
    int qmin = kNoLsb;
    for (int ksl = 0; ksl < KS; ++ksl) {
      acc += sPart[tid * KS + ksl];
      asum += sPartA[tid * KS + ksl];
      qmin = min(qmin, sPartQ[tid * KS + ksl]);
    }
    // Exact in every order iff sum|p| < 2^(q+53); asum itself carries a relative error of
    // at most d * 2^-53, covered by the margin.
    bool exact = qmin == kNoLsb || (qmin > -2000 && asum * 1.000001 < ldexp(1.0, qmin + 53));
    sAcc[tid] = acc;
    if (!exact) *sBad = 1;
  }
  __syncthreads();
  if (*sBad) {
    // The reference's own order: one sequential c-ascending f64 sum per row.
    for (int r = tid; r < R; r += kTokenThreads) {
      const float* wr = r < E ? w_router + (size_t)r * d : gate_vec;
      double acc = 0.0;
      for (int c = 0; c < d; ++c) acc = fma((double)wr[c], (double)sX[c], acc);
      sAcc[r] = acc;
    }
    __syncthreads();
  }
  if (tid < R) {
    double acc = sAcc[tid];
    if (tid < E) {
      float logit = (float)acc;
      if (bias) logit = logit + bias[tid];
      sLogit[tid] = logit;
    } else {
      sgate_out[t] = (float)(1.0 / (1.0 + exp(-acc)));
    }
  }
  __syncthreads();
  softmax_topk(tid < E, tid, E, k, renorm, t, sLogit, sExp, sWt, sSel, idx_out, w_out, status);
  if (fg.counts) {  // T == 1: the grouping of a single token follows from its top-k
    __syncthreads();
    if (tid == 0) {
      int run = 0;
      for (int e = 0; e < E; ++e) {
        const int c = sSel[e] ? 1 : 0;
        fg.counts[e] = c;
        fg.offsets[e] = run;
        if (c && run < k) {
          fg.active[run] = e;
          fg.perm[run] = run;
          fg.inv[run] = run;
          fg.tile_group[run] = e;
          fg.tile_m0[run] = 0;
          ++run;
        }
      }
      fg.offsets[E] = run;
      *fg.n_active = run;
      *fg.n_tiles = run;
      *fg.shared_n_tiles = 1;
      fg.shared_offsets[0] = 0;
      fg.shared_offsets[1] = 1;
    }
  }
}

}  // namespace

hipError_t launch_router(const RouterArgs& a, hipStream_t s, int* fused_permute) {
  const int R = a.E + (a.shared_gate ? 1 : 0);
  if (fused_permute) *fused_permute = 0;
  if (R > kMaxRouterRows || a.T <= 0) return hipErrorInvalidValue;
  if (a.T <= a.token_kernel_max_tokens) {
    const size_t np = R > kTokenThreads / 64 ? R : kTokenThreads / 64;
    size_t smem = ((size_t)R + a.E + 2 * np) * 8 + (size_t)a.d * 4 + (size_t)a.E * 12 + 4 +
                  np * 4 + (size_t)a.d * 2 + 16;
    if (smem <= 64 * 1024) {
      FusedGrouping fg{};
      if (a.T == 1 && a.fuse_permute) {
        const PermuteArgs& pa = *a.fuse_permute;
        fg = FusedGrouping{pa.counts, pa.offsets, pa.perm, pa.inv, pa.active, pa.n_active,
                           pa.shared_offsets, pa.tile_group, pa.tile_m0, pa.n_tiles,
                           pa.shared_n_tiles};
        if (fused_permute) *fused_permute = 1;
      }
      if (a.x_is_bf16)
        router_token_kernel<uint16_t><<<a.T, kTokenThreads, smem, s>>>(
            (const uint16_t*)a.x, a.T, a.d, a.E, a.k, a.renorm, a.w_router, a.router_bias,
            a.shared_gate, a.idx, a.w, a.sgate, a.xb, a.d_pad, a.status, fg);
      else
        router_token_kernel<float><<<a.T, kTokenThreads, smem, s>>>(
            (const float*)a.x, a.T, a.d, a.E, a.k, a.renorm, a.w_router, a.router_bias,
            a.shared_gate, a.idx, a.w, a.sgate, a.xb, a.d_pad, a.status, fg);
      return hipGetLastError();
    }
  }
  int TT = kRouterThreads / R;
  if (TT < 1) TT = 1;
  // Keep enough blocks in flight for small batches.
  while (TT > 1 && (a.T + TT - 1) / TT < 256 && TT * R > 64) TT = (TT + 1) / 2;
  const int blocks = (a.T + TT - 1) / TT;
  size_t dot_bytes = ((size_t)R + TT) * kLd * sizeof(float);
  size_t post_bytes = (((size_t)TT * R + 1) & ~(size_t)1) * 4 + (size_t)TT * a.E * (8 + 4 + 4);
  size_t smem = dot_bytes > post_bytes ? dot_bytes : post_bytes;
  if (a.x_is_bf16) {
    router_tile_kernel<uint16_t><<<blocks, kRouterThreads, smem, s>>>(
        (const uint16_t*)a.x, a.T, a.d, a.E, a.k, a.renorm, a.w_router, a.router_bias,
        a.shared_gate, a.idx, a.w, a.sgate, a.xb, a.d_pad, a.status, TT);
  } else {
    router_tile_kernel<float><<<blocks, kRouterThreads, smem, s>>>(
        (const float*)a.x, a.T, a.d, a.E, a.k, a.renorm, a.w_router, a.router_bias,
        a.shared_gate, a.idx, a.w, a.sgate, a.xb, a.d_pad, a.status, TT);
  }
  return hipGetLastError();
}

}  // namespace atenia_moe
