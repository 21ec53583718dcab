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
#include <cstdlib>

#include "moe_internal.h"

#include <mutex>

namespace atenia_moe {

namespace {

constexpr int kRouterThreads = 256;
constexpr int kKc = 32;            // columns staged per step
constexpr int kLd = kKc + 1;       // padded LDS row stride (words)
constexpr int kTokenThreads = 1024;

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
constexpr int kNoLsb = 32767;
__device__ inline int lsb_exponent(float v) {  // selects only: it sits in unrolled loops
  const uint32_t b = __float_as_uint(v);
  const int e = (b >> 23) & 0xff;
  const uint32_t m = b & 0x7fffffu;
  const uint32_t mm = e ? (m | 0x800000u) : m;  // normal numbers carry the implicit one
  int r = (e ? e - 150 : -149) + (__ffs((int)mm) - 1);
  r = mm == 0 ? kNoLsb : r;
  return e == 0xff ? -100000 : r;
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
#pragma unroll 8
    for (int e = 0; e < E; ++e) mx = fmaxf(mx, lg[e]);  // skips NaN like f32::max
    my_logit = lg[r];
    ex[r] = exp((double)(my_logit - mx));                // f32 subtraction, then f64 exp
  }
  __syncthreads();
  float my_w = 0.f;
  if (on) {
    double sum = 0.0;
#pragma unroll 8
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
#pragma unroll 8
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
    int d_pad, int32_t* __restrict__ status, float* __restrict__ logits_out, int tokens_per_block) {
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
      if (logits_out) logits_out[(size_t)(t0 + tl) * E + r] = logit;
    } else {
      sgate_out[t0 + tl] = (float)(1.0 / (1.0 + exp(-acc)));
    }
  }
  __syncthreads();
  if (logits_out) return;  // routing is decided by another kernel from the raw logits
  const int tls = owner ? tl : 0;
  softmax_topk(owner && r < E, r, E, k, renorm, t0 + tls, sLogit + tls * R, sExp + tls * E,
               sWt + tls * E, sSel + tls * E, idx_out, w_out, status);
}

// Softmax + top-k + renormalisation of a block of TT tokens at once, same arithmetic and order
// as softmax_topk.  The steps that the reference does as sequential folds over the experts
// (f64 sum of the exponentials, f64 sum of the selected weights) are dependent chains, so one
// thread per token runs them for all tokens of the block side by side; the element-wise steps
// (exp, weight, rank) are spread over all threads.  lg: [TT][R] f32 logits in LDS; scratch:
// ex [TT][E] f64, wt [TT][E] f32, sel [TT][E] u8, tok [TT] f64 (max, then 1/sum).
__device__ inline void softmax_topk_block(int TT, int R, int E, int k, int renorm, int t0, int T,
                                          const float* lg, double* ex, float* wt, uint8_t* sel,
                                          double* tok, int32_t* __restrict__ idx_out,
                                          float* __restrict__ w_out,
                                          int32_t* __restrict__ status) {
  const int tid = threadIdx.x, nthr = blockDim.x;
  const int pairs = TT * E;
  if (tid < TT) {
    const float* l = lg + tid * R;
    float mx = -INFINITY;
#pragma unroll 8
    for (int e = 0; e < E; ++e) mx = fmaxf(mx, l[e]);  // skips NaN like f32::max
    tok[tid] = (double)mx;
  }
  __syncthreads();
  for (int pr = tid; pr < pairs; pr += nthr) {
    const int t = pr / E, e = pr - t * E;
    ex[pr] = exp((double)(lg[t * R + e] - (float)tok[t]));  // f32 subtraction, then f64 exp
  }
  __syncthreads();
  if (tid < TT) {
    const double* x = ex + tid * E;
    double sum = 0.0;
#pragma unroll 8
    for (int e = 0; e < E; ++e) sum += x[e];  // sequential fold, e ascending
    tok[tid] = sum > 0.0 ? 1.0 / sum : 0.0;
  }
  __syncthreads();
  for (int pr = tid; pr < pairs; pr += nthr) {
    const int t = pr / E, e = pr - t * E;
    const float w = (float)(ex[pr] * tok[t]);
    wt[pr] = w;
    if ((!isfinite(w) || w < 0.f) && t0 + t < T) {
      atomicMin(&status[0], -3);
      atomicMin(&status[1], ((t0 + t) << 10) | e);
    }
  }
  __syncthreads();
  for (int pr = tid; pr < pairs; pr += nthr) {
    const int t = pr / E, e = pr - t * E;
    const float* w = wt + t * E;
    const float my_w = w[e];
    int rank = 0;  // experts that sort before me under (weight desc, index asc)
#pragma unroll 8
    for (int o = 0; o < E; ++o) {
      const float wo = w[o];
      rank += (wo > my_w) || (wo == my_w && o < e);
    }
    sel[pr] = rank < k ? 1 : 0;
  }
  __syncthreads();
  if (tid < TT && t0 + tid < T) {
    const float* w = wt + tid * E;
    const uint8_t* sl = sel + tid * E;
    double sum = 0.0;
#pragma unroll 8
    for (int e = 0; e < E; ++e)
      if (sl[e]) sum += (double)w[e];  // ascending e, as the reference sums the sorted selection
    const double scale = renorm ? 1.0 / sum : 1.0;
    size_t o = (size_t)(t0 + tid) * k;
    int slot = 0;
    for (int e = 0; e < E && slot < k; ++e) {
      if (sl[e]) {
        idx_out[o + slot] = e;
        w_out[o + slot] = (float)((double)w[e] * scale);
        ++slot;
      }
    }
  }
}

// Batched form of the sequential kernel for up to 64 rows.  Same arithmetic and order as
// router_tile_kernel (one c-ascending f64 fma chain per (token, row)); what changes is how the
// chains are fed:
//   * a thread owns TPT tokens and RPT rows (rows rg, rg + RG, ...), so a value read from
//     LDS serves several chains and the chains of one thread hide each other's fma latency;
//   * tiles of KC columns are converted to f64 once while they are stored to LDS, so the
//     inner loop is ds_read_b128 (two consecutive columns) + fma only;
//   * the global loads of tile s+2 are issued into registers before tile s is multiplied.
template <typename XT> struct XVec;
template <> struct XVec<float> {
  typedef float4 type;
  static __device__ inline float4 load(const float* p) { return *(const float4*)p; }
  static __device__ inline void unpack(float4 v, float (&f)[4]) { f[0] = v.x; f[1] = v.y; f[2] = v.z; f[3] = v.w; }
  static __device__ inline float4 zero() { return make_float4(0.f, 0.f, 0.f, 0.f); }
};
template <> struct XVec<uint16_t> {
  typedef uint2 type;
  static __device__ inline uint2 load(const uint16_t* p) { return *(const uint2*)p; }
  static __device__ inline void unpack(uint2 v, float (&f)[4]) {
    f[0] = __uint_as_float(v.x << 16); f[1] = __uint_as_float(v.x & 0xffff0000u);
    f[2] = __uint_as_float(v.y << 16); f[3] = __uint_as_float(v.y & 0xffff0000u);
  }
  static __device__ inline uint2 zero() { return make_uint2(0u, 0u); }
};

template <typename XT, int RPT, int TPT, int KC>
__global__ __launch_bounds__(kRouterThreads) void router_batch_kernel(
    const XT* __restrict__ x, int T, int d, int E, int k, int renorm,
    const float* __restrict__ w_router, const float* __restrict__ bias,
    const float* __restrict__ gate_vec, int32_t* __restrict__ idx_out,
    float* __restrict__ w_out, float* __restrict__ sgate_out, uint16_t* __restrict__ xb,
    int d_pad, int32_t* __restrict__ status, float* __restrict__ logits_out) {
  constexpr int RG = 16;                   // row groups = threads per token
  constexpr int TG = kRouterThreads / RG;  // 16 token groups = threads per row group
  constexpr int TT = TG * TPT;             // tokens per block: a thread owns tokens tg, tg + TG, ...
  constexpr int RW = RG * RPT;             // rows of the staged weight tile (>= R)
  constexpr int LD = KC + 2;               // f64 row stride: rows 4 banks apart, 16-byte aligned
  constexpr int KV = KC / 4;               // 4-column vectors per tile row
  constexpr int NX = (TT * KV + kRouterThreads - 1) / kRouterThreads;
  constexpr int NW = (RW * KV + kRouterThreads - 1) / kRouterThreads;
  typedef XVec<XT> XV;
  const int R = E + (gate_vec ? 1 : 0);
  const int t0 = blockIdx.x * TT;
  // More than RW rows: blockIdx.y picks the block of RW rows (only when the logits go to
  // `logits_out`, since the softmax below needs all rows of a token in one workgroup).
  const int r_lo = blockIdx.y * RW;
  const int tid = threadIdx.x;
  const int tg = tid / RG, rg = tid - tg * RG;

  extern __shared__ double smem_b[];
  double* sX = smem_b;            // [TT][LD]
  double* sW = sX + TT * LD;      // [RW][LD]

  typedef typename XV::type xvec_t;
  auto load_tile = [&](xvec_t (&xr)[NX], float4 (&wr)[NW], int c0) {
#pragma unroll
    for (int i = 0; i < NX; ++i) {
      const int j = tid + i * kRouterThreads;
      const int row = j / KV, c = c0 + (j - row * KV) * 4;
      xr[i] = XV::zero();
      if (j < TT * KV && t0 + row < T && c < d) xr[i] = XV::load(x + (size_t)(t0 + row) * d + c);
    }
#pragma unroll
    for (int i = 0; i < NW; ++i) {
      const int j = tid + i * kRouterThreads;
      const int row = j / KV, c = c0 + (j - row * KV) * 4;
      wr[i] = make_float4(0.f, 0.f, 0.f, 0.f);
      if (j < RW * KV && r_lo + row < R && c < d)
        wr[i] = *(const float4*)((r_lo + row < E ? w_router + (size_t)(r_lo + row) * d : gate_vec) + c);
    }
  };
  auto store_tile = [&](const xvec_t (&xr)[NX], const float4 (&wr)[NW], int c0) {
#pragma unroll
    for (int i = 0; i < NX; ++i) {
      const int j = tid + i * kRouterThreads;
      if (j < TT * KV) {
        const int row = j / KV, cl = (j - row * KV) * 4;
        float f[4];
        XV::unpack(xr[i], f);
        double* dst = sX + row * LD + cl;
        *(double2*)dst = make_double2((double)f[0], (double)f[1]);
        *(double2*)(dst + 2) = make_double2((double)f[2], (double)f[3]);
        const int c = c0 + cl;
        if (xb && blockIdx.y == 0 && t0 + row < T && c < d_pad) {
          uint2 b;
          b.x = f32_to_bf16_rne(f[0]) | ((uint32_t)f32_to_bf16_rne(f[1]) << 16);
          b.y = f32_to_bf16_rne(f[2]) | ((uint32_t)f32_to_bf16_rne(f[3]) << 16);
          *(uint2*)(xb + (size_t)(t0 + row) * d_pad + c) = b;
        }
      }
    }
#pragma unroll
    for (int i = 0; i < NW; ++i) {
      const int j = tid + i * kRouterThreads;
      if (j < RW * KV) {
        const int row = j / KV, cl = (j - row * KV) * 4;
        double* dst = sW + row * LD + cl;
        *(double2*)dst = make_double2((double)wr[i].x, (double)wr[i].y);
        *(double2*)(dst + 2) = make_double2((double)wr[i].z, (double)wr[i].w);
      }
    }
  };

  double acc[TPT][RPT];
#pragma unroll
  for (int j = 0; j < TPT; ++j)
#pragma unroll
    for (int i = 0; i < RPT; ++i) acc[j][i] = 0.0;
  // Columns from d up to c_end exist only to zero-fill the padding of xb; both staged tiles
  // hold +0.0 there, which leaves every sum unchanged.
  const int c_end = xb ? (d_pad > d ? d_pad : d) : d;
  // Two register sets: the loads of tile s+2 are issued while tile s is multiplied, so a
  // load has two multiply phases to land before its tile is stored to LDS.
  xvec_t xr0[NX], xr1[NX];
  float4 wr0[NW], wr1[NW];
  // Workgroup barrier that orders LDS traffic only.  __syncthreads() would also wait for
  // every outstanding global load, which is exactly the latency the prefetch is there to hide.
  auto lds_barrier = [] {
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
  };
  auto step = [&](xvec_t (&xr)[NX], float4 (&wr)[NW], int c0) {
    lds_barrier();  // everyone is done reading the previous tile
    store_tile(xr, wr, c0);
    lds_barrier();
    if (c0 + 2 * KC < c_end) load_tile(xr, wr, c0 + 2 * KC);
    // Columns are taken in groups of CG: the LDS reads of group g+1 are issued before the
    // fma chain steps of group g (two register sets), so no read latency sits between them.
    const double* xs = sX + tg * LD;
    const double* ws = sW + rg * LD;
    constexpr int CG = TPT * RPT <= 4 ? 8 : 4, NV = CG / 2;
    double2 xa[TPT][NV], wa[RPT][NV], xb2[TPT][NV], wb2[RPT][NV];
    auto rd = [&](double2 (&xv)[TPT][NV], double2 (&wv)[RPT][NV], int c) {
#pragma unroll
      for (int u = 0; u < NV; ++u) {
#pragma unroll
        for (int j = 0; j < TPT; ++j) xv[j][u] = *(const double2*)(xs + j * TG * LD + c + 2 * u);
#pragma unroll
        for (int i = 0; i < RPT; ++i) wv[i][u] = *(const double2*)(ws + i * RG * LD + c + 2 * u);
      }
    };
    auto mul = [&](const double2 (&xv)[TPT][NV], const double2 (&wv)[RPT][NV]) {
#pragma unroll
      for (int u = 0; u < NV; ++u)
#pragma unroll
        for (int i = 0; i < RPT; ++i)
#pragma unroll
          for (int j = 0; j < TPT; ++j) {
            acc[j][i] = fma(wv[i][u].x, xv[j][u].x, acc[j][i]);
            acc[j][i] = fma(wv[i][u].y, xv[j][u].y, acc[j][i]);
          }
    };
    static_assert(KC % (2 * CG) == 0, "tile width must hold whole pairs of column groups");
    rd(xa, wa, 0);
    for (int c = 0; c < KC; c += 2 * CG) {
      rd(xb2, wb2, c + CG);
      __builtin_amdgcn_sched_barrier(0);
      mul(xa, wa);
      __builtin_amdgcn_sched_barrier(0);
      if (c + 2 * CG < KC) rd(xa, wa, c + 2 * CG);
      __builtin_amdgcn_sched_barrier(0);
      mul(xb2, wb2);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  load_tile(xr0, wr0, 0);
  if (KC < c_end) load_tile(xr1, wr1, KC);
  for (int c0 = 0; c0 < c_end; c0 += 2 * KC) {
    step(xr0, wr0, c0);
    if (c0 + KC < c_end) step(xr1, wr1, c0 + KC);
  }
  __syncthreads();

  // reuse of the tile memory: logits of the block, then the softmax scratch
  float* sLogit = (float*)smem_b;                          // [TT][R]
  double* sExp = smem_b + ((TT * R + 1) / 2);              // [TT][E]
  double* sTok = sExp + TT * E;                            // [TT]
  float* sWt = (float*)(sTok + TT);                        // [TT][E]
  uint8_t* sSel = (uint8_t*)(sWt + TT * E);                // [TT][E]
#pragma unroll
  for (int j = 0; j < TPT; ++j) {
    const int tl = tg + j * TG;
    if (t0 + tl >= T) continue;
#pragma unroll
    for (int i = 0; i < RPT; ++i) {
      const int r = r_lo + rg + i * RG;
      if (r < E) {
        float logit = (float)acc[j][i];
        if (bias) logit = logit + bias[r];
        sLogit[tl * R + r] = logit;
        if (logits_out) logits_out[(size_t)(t0 + tl) * E + r] = logit;
      } else if (r < R) {
        sgate_out[t0 + tl] = (float)(1.0 / (1.0 + exp(-acc[j][i])));
      }
    }
  }
  __syncthreads();
  if (logits_out) return;  // routing is decided by another kernel from the raw logits
  softmax_topk_block(TT, R, E, k, renorm, t0, T, sLogit, sExp, sWt, sSel, sTok, idx_out, w_out,
                     status);
}

template <typename XT, int RPT, int TPT, int KC>
hipError_t launch_router_batch(const RouterArgs& a, hipStream_t s) {
  constexpr int TT = kRouterThreads / 16 * TPT, RW = 16 * RPT, LD = KC + 2;
  const int R = a.E + (a.shared_gate ? 1 : 0);
  size_t dot_bytes = (size_t)(TT + RW) * LD * 8;
  size_t post_bytes = (((size_t)TT * R + 1) / 2) * 8 + (size_t)TT * a.E * (8 + 4 + 1) + TT * 8 + 16;
  size_t smem = dot_bytes > post_bytes ? dot_bytes : post_bytes;
  if (smem > 64 * 1024) {
    // per instantiation: largest size the attribute was set for (layers may launch from
    // several host threads)
    static std::mutex attr_mu;
    static size_t attr_bytes = 0;
    std::lock_guard<std::mutex> lock(attr_mu);
    if (smem > attr_bytes) {
      hipError_t e = hipFuncSetAttribute((const void*)router_batch_kernel<XT, RPT, TPT, KC>,
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
      if (e != hipSuccess) return e;
      attr_bytes = smem;
    }
  }
  const int blocks = (a.T + TT - 1) / TT;
  const int row_blocks = (R + RW - 1) / RW;
  if (row_blocks > 1 && !a.logits_out) return hipErrorInvalidValue;
  router_batch_kernel<XT, RPT, TPT, KC><<<dim3(blocks, row_blocks), kRouterThreads, smem, s>>>(
      (const XT*)a.x, a.T, a.d, a.E, a.k, a.renorm, a.w_router, a.router_bias, a.shared_gate,
      a.idx, a.w, a.sgate, a.xb, a.d_pad, a.status, a.logits_out);
  return hipGetLastError();
}

// ---- batches on the f64 matrix cores, any summation order made safe by a certificate ---------
// v_mfma_f64_16x16x4_f64 (operand layout: see ffn_f32.hip): A = 16 rows of [W_r ; gate], B = 16
// tokens, so lane l holds D[4 r + l / 16][l % 16] = rows 4 r + l / 16 of token l % 16.  A
// workgroup owns 16 tokens and all rows (RB blocks of 16); its four waves split k and add their
// partial sums in wave order.  f32 operands widen exactly and their products are exact in f64,
// so the result differs from the reference's c-ascending sum only by the order of the f64
// additions.  That is accepted only under the same two certificates as in router_token_kernel:
//   interval : any order lands within g = d 2^-53 sum|p| of the true sum, and sum|p| is bounded
//              here by |w_r| |x_t| (Cauchy-Schwarz; |x_t|^2 is accumulated next to the matrix
//              instructions, |w_r|^2 comes with the layer); if [acc - 2g, acc + 2g] rounds to
//              one f32 (one f32 sigmoid for the gate row) that value is the reference's;
//   exactness: for the few sums that fail it, one wave checks that every product is a multiple
//              of 2^q and sum|p| < 2^(q+53), which makes every order exact (bf16-valued
//              operands pass);
// and a sum that fails both is recomputed in the reference's order by one lane.
// Against one sequential chain per (token, row) this is 3-4x faster at 4096 tokens.
typedef __attribute__((__vector_size__(4 * sizeof(double)))) double f64x4_t;

template <typename XT> struct XChunk;
template <> struct XChunk<float> {
  float4 lo, hi;
  __device__ inline void load(const float* p) { lo = *(const float4*)p; hi = *(const float4*)(p + 4); }
  __device__ inline void keep(bool k) {  // selects, no branch
    lo.x = k ? lo.x : 0.f; lo.y = k ? lo.y : 0.f; lo.z = k ? lo.z : 0.f; lo.w = k ? lo.w : 0.f;
    hi.x = k ? hi.x : 0.f; hi.y = k ? hi.y : 0.f; hi.z = k ? hi.z : 0.f; hi.w = k ? hi.w : 0.f;
  }
  __device__ inline void get(float (&f)[8]) const {
    f[0] = lo.x; f[1] = lo.y; f[2] = lo.z; f[3] = lo.w; f[4] = hi.x; f[5] = hi.y; f[6] = hi.z; f[7] = hi.w;
  }
};
template <> struct XChunk<uint16_t> {
  uint4 v;
  __device__ inline void load(const uint16_t* p) { v = *(const uint4*)p; }
  __device__ inline void keep(bool k) {
    v.x = k ? v.x : 0u; v.y = k ? v.y : 0u; v.z = k ? v.z : 0u; v.w = k ? v.w : 0u;
  }
  __device__ inline void get(float (&f)[8]) const {
    const uint32_t u[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f[2 * i] = __uint_as_float(u[i] << 16);
      f[2 * i + 1] = __uint_as_float(u[i] & 0xffff0000u);
    }
  }
  // min(key, |bits| - 1 of each of the eight values) as unsigned numbers: magnitudes order like
  // their bit patterns, and a zero wraps to the largest key, so the result names the smallest
  // non-zero magnitude seen (bf16_key_lsb below turns it into a last-bit exponent).
  __device__ inline uint32_t min_key(uint32_t key) const {
    const uint32_t u[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i)
      key = min(key, min((u[i] & 0x7fffu) - 1u, ((u[i] >> 16) & 0x7fffu) - 1u));
    return key;
  }
};
// A bf16 value with exponent field e is a multiple of 2^(e - 134) (2^-133 for a denormal), so
// the exponent field of the smallest non-zero magnitude among some values bounds the last-bit
// exponent of every one of them from below: cheaper to follow than the exact last set bit, and
// the exactness test it feeds has bits to spare.  kNoLsb: every value was zero.  (An inf or a
// NaN is not seen here; it makes the norm that the same test compares infinite or NaN.)
constexpr uint32_t kNoKey = 0xffffffffu;
__device__ inline int bf16_key_lsb(uint32_t key) {
  return key == kNoKey ? kNoLsb : (int)((key + 1u) >> 7) - 134;
}

// Softmax + top-k from logits that another launch left in HBM, one wavefront per token (up to 64
// experts; wave_select_token in select_wave.h).
constexpr int kWaveSelectThreads = 256;
__global__ __launch_bounds__(kWaveSelectThreads) void wave_select_kernel(
    const float* __restrict__ logits, int T, int E, int k, int renorm,
    int32_t* __restrict__ idx_out, float* __restrict__ w_out, int32_t* __restrict__ status) {
  const int lane = threadIdx.x & 63;
  const int t = blockIdx.x * (kWaveSelectThreads / 64) + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  if (t >= T) return;
  wave_select_token(logits + (size_t)t * E, E, k, renorm, t, lane, idx_out, w_out, status);
}

template <typename XT, int RB, int NBUF, int NWV>
__global__ __launch_bounds__(64 * NWV) void router_mfma_kernel(
    const XT* __restrict__ x, int T, int d, int E, int k, int renorm,
    const float* __restrict__ w_router, const float* __restrict__ bias,
    const float* __restrict__ gate_vec, int32_t* __restrict__ idx_out,
    float* __restrict__ w_out, float* __restrict__ sgate_out, int32_t* __restrict__ status,
    float* __restrict__ logits_out, const int32_t* __restrict__ w_lsb,
    const uint16_t* __restrict__ w_t8, int Rp, const double* __restrict__ w_norm2) {
  // gridDim.y > 1 (only with logits_out): this workgroup owns the rows row0 .. row0 + R - 1 of
  // the stacked matrix [W_r ; gate] and leaves the logits to another launch; otherwise all rows.
  constexpr int TT = 16;
  const int R_all = E + (gate_vec ? 1 : 0);
  const int row0 = blockIdx.y * 16 * RB;
  const int R = min(16 * RB, R_all - row0);
  const int t0 = blockIdx.x * TT;
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int r16 = lane & 15, q = lane >> 4;

  extern __shared__ double smem_m[];
  constexpr int NT = 64 * NWV;                    // NWV waves split k
  double* sPart = smem_m;                         // [NWV][RB][4][64] partial sums
  double* sXsq = sPart + NWV * RB * 4 * 64;       // [NWV][16]  partial |x_t|^2
  double* sAcc = sXsq + NWV * 16;                 // [16][R]
  double* sXn2 = sAcc + 16 * R;                   // [16]
  double* sWn2 = sXn2 + 16;                       // [R]
  float* sLogit = (float*)(sWn2 + R);             // [16][R]
  uint32_t* sXq = (uint32_t*)(sLogit + 16 * R);   // [NWV][16] key of the smallest |x_t| (partial)
  uint8_t* sFlag = (uint8_t*)(sXq + NWV * 16);    // [16][R] 1 = the interval certificate failed
  // A lower bound of the last-bit exponent of the token's activations is followed beside the
  // matrix instructions when there are several row blocks.  f64 matrix instructions and vector
  // instructions do not overlap on this chip (a step costs the sum of both), and with one block
  // of 8 matrix instructions per step the extra ones cost more than the second looks they
  // save: 25.8 -> 27.6 us on 8 rows, d = 4096.
  constexpr bool kTrackLsb = RB >= 2;
  static_assert(sizeof(XT) == 2, "the last-bit bound below reads bf16 bit patterns");
  uint32_t xq = kNoKey;

  const int tok = min(t0 + r16, T - 1);  // rows past T repeat the last token; never written out
  const XT* px = x + (size_t)tok * d + 8 * q;
  // The stacked matrix comes from its bf16 copy in chunk-major order [d / 8][Rp][8] (made when
  // the layer is created; rows past the last one and chunks past d are zeros): the 16 rows of a
  // block lie side by side, so a load instruction reads 4 x 256 contiguous bytes instead of 64
  // bytes from each of 16 rows -- the row-major f32 matrix cost the load path a fifth of the
  // loop -- and neither a clamp nor a select is needed.
  const uint16_t* pw[RB];
#pragma unroll
  for (int b = 0; b < RB; ++b) pw[b] = w_t8 + ((size_t)q * Rp + row0 + 16 * b + r16) * 8;
  const size_t w_step = (size_t)32 * Rp;  // four chunks
  if (tid < R) sWn2[tid] = w_norm2[row0 + tid];  // |w_r|^2, read after the barriers below
  // k in steps of 32 (8 per lane), the steps dealt to the four waves in contiguous runs
  const int nsteps = (d + 31) / 32;
  const int per = (nsteps + NWV - 1) / NWV;
  const int s0 = wave * per, s1 = min(nsteps, s0 + per);

  // One row block: two accumulators in turn, so that consecutive matrix instructions do not
  // wait for each other's result (summed once at the end; any order is as good).  With more
  // blocks their instructions interleave anyway and the registers are better spent on a second
  // workgroup per compute unit.
  constexpr int NACC = RB == 1 ? 2 : 1;
  f64x4_t acc[RB][NACC];
#pragma unroll
  for (int b = 0; b < RB; ++b)
#pragma unroll
    for (int n = 0; n < NACC; ++n) acc[b][n] = f64x4_t{0.0, 0.0, 0.0, 0.0};
  double xsq = 0.0;

  XChunk<XT> xc[NBUF];
  XChunk<uint16_t> wc[NBUF][RB];
  // Every step issues the same loads whatever the lane or the step: a chunk past d is fetched
  // from the row's first columns and zeroed with selects, a step past the wave's range repeats
  // its last one.  With a branch around a load the compiler can no longer count the loads in
  // flight and waits for all of them (s_waitcnt vmcnt(0)) before every use -- the first cut of
  // this kernel did, and ran one memory round trip per step.
  auto load_step = [&](int buf, int st) {
    st = min(st, s1 - 1);
    const bool in = st * 32 + 8 * q < d;  // d is a multiple of 8: a chunk is whole or absent
    const size_t off = in ? (size_t)st * 32 : 0;
    xc[buf].load(px + off);
    xc[buf].keep(in);
#pragma unroll
    for (int b = 0; b < RB; ++b) wc[buf][b].load(pw[b] + (size_t)st * w_step);
  };
  auto multiply = [&](int buf) {
    float xf[8];
    xc[buf].get(xf);
    if (kTrackLsb) xq = xc[buf].min_key(xq);
    double xd[8];
#pragma unroll
    for (int t = 0; t < 8; ++t) {
      xd[t] = (double)xf[t];
      xsq = fma(xd[t], xd[t], xsq);
    }
#pragma unroll
    for (int b = 0; b < RB; ++b) {
      float wf[8];
      wc[buf][b].get(wf);
#pragma unroll
      for (int t = 0; t < 8; ++t) {
        const double wd = (double)wf[t];
        acc[b][t % NACC] = __builtin_amdgcn_mfma_f64_16x16x4f64(wd, xd[t], acc[b][t % NACC], 0, 0, 0);
      }
    }
  };
  if (s0 < s1) {
#pragma unroll
    for (int i = 0; i < NBUF - 1; ++i) load_step(i, s0 + i);
    for (int st = s0; st < s1; st += NBUF) {
#pragma unroll
      for (int i = 0; i < NBUF; ++i) {
        load_step((i + NBUF - 1) % NBUF, st + i + NBUF - 1);
        if (st + i < s1) multiply(i);  // scalar branch around matrix instructions only
      }
    }
  }

  // partial sums and norms of this wave -> LDS
#pragma unroll
  for (int b = 0; b < RB; ++b) {
#pragma unroll
    for (int r = 0; r < 4; ++r)
      sPart[((wave * RB + b) * 4 + r) * 64 + lane] = NACC == 2 ? acc[b][0][r] + acc[b][NACC - 1][r] : acc[b][0][r];
  }
  {
    double v = xsq;
    v += __shfl_xor(v, 16);
    v += __shfl_xor(v, 32);
    if (q == 0) sXsq[wave * 16 + r16] = v;
    if (kTrackLsb) {
      xq = min(xq, __shfl_xor(xq, 16));
      xq = min(xq, __shfl_xor(xq, 32));
      if (q == 0) sXq[wave * 16 + r16] = xq;
    }
  }
  __syncthreads();

  // thread (token t, row class rr) finishes rows rr, rr + 16, ...
  const int t = tid & 15, rr = tid >> 4;
  double xn2 = 0.0;
#pragma unroll
  for (int w = 0; w < NWV; ++w) xn2 += sXsq[w * 16 + t];
  if (rr == 0) sXn2[t] = xn2;
  int xq_t = kNoLsb;
  if (kTrackLsb) {
    uint32_t key = kNoKey;
#pragma unroll
    for (int w = 0; w < NWV; ++w) key = min(key, sXq[w * 16 + t]);
    xq_t = bf16_key_lsb(key);
  }
  const double gfac = (double)(2 * d + 4) * 1.1102230246251565e-16 * 1.001;
  for (int r = rr; r < R; r += NT / 16) {
    const int b = r >> 4, rho = r & 15, reg = rho >> 2, qq = rho & 3;
    double a = 0.0;
#pragma unroll
    for (int w = 0; w < NWV; ++w) a += sPart[((w * RB + b) * 4 + reg) * 64 + qq * 16 + t];
    const double wn2 = sWn2[r];
    // sum|p| <= |w_r| |x_t|; the factor 1.001 covers the roundings of the norms and the root
    const double e = sqrt(xn2 * wn2) * gfac;
    const double lo = a - e, hi = a + e;
    bool ok;
    if (row0 + r < E) {
      const float flo = (float)lo, fhi = (float)hi;
      ok = flo == fhi && isfinite(flo);
    } else {
      const float glo = (float)(1.0 / (1.0 + exp(-lo))), ghi = (float)(1.0 / (1.0 + exp(-hi)));
      ok = glo == ghi;
    }
    if (kTrackLsb && !ok && w_lsb) {
      // Exactness from the two minima alone: every product of the pair is a multiple of
      // 2^(q_x + q_w), so with sum|p| < 2^(q_x + q_w + 53) every partial sum of every order is
      // exact -- the test of the second look with a lower bound for q, which most flagged sums
      // pass without either row being read again (all zeros on one side: the sum is exactly 0).
      const int wq = w_lsb[min(row0 + r, E)];
      if (xq_t == kNoLsb || wq == kNoLsb) {
        ok = true;
      } else {
        const int ql = xq_t + wq;
        ok = ql > -2000 && sqrt(xn2 * wn2) * 1.001 < ldexp(1.0, ql + 53);
      }
    }
    sAcc[t * R + r] = a;
    sFlag[t * R + r] = ok ? 0 : 1;
  }
  __syncthreads();

  // Second look at the flagged sums (about one in a thousand, so about one per workgroup and
  // five in the unluckiest): the partial-sum area is free now and holds their list.  The
  // exactness test reads both rows of a flagged sum once; those reads are dealt to the waves in
  // pieces of 512 columns, whichever sum they belong to, so a workgroup with one flagged sum
  // and one with five both keep all their waves busy.  The sums that fail this test too (a
  // product with a very low last bit: one tiny activation is enough) go on a second list.
  int* sList = (int*)sPart;          // [<= 16 R] flagged entries
  int* sList2 = sList + 16 * R;      // [<= 16 R] entries that want the reference's own order
  int* sQ = sList2 + 16 * R;         // [<= 16 R] lowest last-bit exponent of a flagged entry's products
  int* sCount = sQ + 16 * R;         // [0] flagged, [1] for the chain
  constexpr int kSeqChunk = 512;     // 8 KiB: with the lists it fits the smallest partial-sum area
  double2* sSeq = (double2*)(((uintptr_t)(sCount + 2) + 15) & ~(uintptr_t)15);
  static_assert(3 * 16 * 16 * RB * 4 + 8 + 16 + kSeqChunk * 16 <= NWV * RB * 4 * 64 * 8,
                "lists and staging area must fit the partial-sum area");
  if (tid < 2) sCount[tid] = 0;
  __syncthreads();
  for (int ent = tid; ent < 16 * R; ent += NT)
    if (sFlag[ent]) {
      const int at = atomicAdd(sCount, 1);
      sList[at] = ent;
      sQ[at] = kNoLsb;
    }
  __syncthreads();
  const int n_flagged = *sCount;
  const int pieces = (d + 511) / 512;
  const int n_items = n_flagged * pieces;
  constexpr int NB = 4;  // pieces a wave has in flight: their loads leave together
  for (int it0 = wave; it0 < n_items; it0 += NWV * NB) {  // wave-uniform
    XChunk<XT> xn[NB];
    XChunk<float> wn[NB];
    int ent[NB];
    bool in[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      const int it = it0 + b * NWV;
      const bool valid = it < n_items;  // a piece past the end re-reads the first one
      const int itc = valid ? it : it0;
      const int i = itc / pieces, piece = itc - i * pieces;
      const int ei = sList[i];
      const int ft = ei / R, fr = ei - ft * R;
      const XT* xr = x + (size_t)min(t0 + ft, T - 1) * d;
      const float* wr = row0 + fr < E ? w_router + (size_t)(row0 + fr) * d : gate_vec;
      const int c = piece * 512 + lane * 8;  // eight columns per lane
      in[b] = valid && c < d;                // d is a multiple of 8: a chunk is whole or absent
      ent[b] = i;
      xn[b].load(xr + (c < d ? c : 0));
      wn[b].load(wr + (c < d ? c : 0));
    }
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      float xf[8], wf[8];
      xn[b].get(xf);
      wn[b].get(wf);
      int qmin = kNoLsb;
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int lx = lsb_exponent(xf[u]), lw = lsb_exponent(wf[u]);
        qmin = min(qmin, (in[b] && lx != kNoLsb && lw != kNoLsb) ? lx + lw : kNoLsb);
      }
#pragma unroll
      for (int off = 32; off >= 1; off >>= 1) qmin = min(qmin, __shfl_xor(qmin, off));
      if (lane == 0 && qmin != kNoLsb) atomicMin(sQ + ent[b], qmin);
    }
  }
  __syncthreads();
  for (int i = tid; i < n_flagged; i += NT) {
    const int ei = sList[i], qmin = sQ[i];
    const int ft = ei / R, fr = ei - ft * R;
    const double bound = sqrt(sXn2[ft] * sWn2[fr]) * 1.001;
    const bool exact = qmin == kNoLsb || (qmin > -2000 && bound < ldexp(1.0, qmin + 53));
    if (!exact) sList2[atomicAdd(sCount + 1, 1)] = ei;
  }
  __syncthreads();
  // The reference's own order for those: one sequential c-ascending f64 sum.  The workgroup
  // widens kSeqChunk columns at a time into LDS and one thread walks them, so each step of the
  // chain waits for an LDS read instead of two trips to L2 (d = 2048: ~10 us instead of ~115).
  const int n_chain = sCount[1];
  for (int i = 0; i < n_chain; ++i) {
    const int ei = sList2[i];
    const int ft = ei / R, fr = ei - ft * R;
    const XT* xr = x + (size_t)min(t0 + ft, T - 1) * d;
    const float* wr = row0 + fr < E ? w_router + (size_t)(row0 + fr) * d : gate_vec;
    double a = 0.0;
    for (int c0 = 0; c0 < d; c0 += kSeqChunk) {
      const int n = min(kSeqChunk, d - c0);
      for (int c = tid; c < n; c += NT)
        sSeq[c] = double2{(double)wr[c0 + c], (double)load_x(xr, c0 + c)};
      __syncthreads();
      if (tid == 0) {
#pragma unroll 8
        for (int c = 0; c < n; ++c) a = fma(sSeq[c].x, sSeq[c].y, a);
      }
      __syncthreads();
    }
    if (tid == 0) sAcc[ei] = a;
  }
  if (n_chain) __syncthreads();

  for (int ent = tid; ent < 16 * R; ent += NT) {
    const int ft = ent / R, fr = ent - ft * R;
    const double a = sAcc[ent];
    if (row0 + fr < E) {
      float logit = (float)a;
      if (bias) logit = logit + bias[row0 + fr];
      sLogit[ent] = logit;
      if (logits_out && t0 + ft < T) logits_out[(size_t)(t0 + ft) * E + row0 + fr] = logit;
    } else if (t0 + ft < T) {
      sgate_out[t0 + ft] = (float)(1.0 / (1.0 + exp(-a)));
    }
  }
  if (logits_out) return;  // routing is decided by another launch from the logits
  __syncthreads();
  if (E <= 64) {
    // Softmax and top-k with lane r = expert r, a wave taking the tokens wave, wave + NWV, ...
    // Same arithmetic, casts and order as softmax_topk (and wave_softmax_topk in select_wave.h);
    // what is laid out for speed is the two loops of 64 steps: the reference's sequential fold
    // of the exponentials is run for all 16 tokens at once by 16 lanes reading LDS, and the
    // selection takes k maxima over the wave instead of ranking every expert against every
    // other.
    constexpr int TPW = TT / NWV;
    double* sExp = smem_m;            // [16][64]: the partial-sum area again
    double* sInv = sExp + TT * 64;    // [16]
    static_assert((TT * 64 + TT) * 8 <= NWV * RB * 4 * 64 * 8, "softmax scratch must fit");
    const bool on = lane < E;
    double ex[TPW];
#pragma unroll
    for (int j = 0; j < TPW; ++j) {
      const int tk = wave + j * NWV;
      const float my = on ? sLogit[tk * R + lane] : -INFINITY;
      // a NaN logit is skipped, as f32::max skips it
      const float mx = wave_max_f32(fmaxf(-INFINITY, my));
      ex[j] = on ? exp((double)(my - mx)) : 0.0;  // f32 subtraction, then f64 exp
      sExp[tk * 64 + lane] = ex[j];
    }
    __syncthreads();
    if (tid < TT) {
      const double* xe = sExp + tid * 64;
      double sum = 0.0;
      for (int e0 = 0; e0 < E; e0 += 8) {  // sequential fold, e ascending; the padding adds +0
#pragma unroll
        for (int u = 0; u < 8; ++u) sum += xe[e0 + u];
      }
      sInv[tid] = sum > 0.0 ? 1.0 / sum : 0.0;
    }
    __syncthreads();
    float wt[TPW];
    int token[TPW];
    bool valid[TPW];
#pragma unroll
    for (int j = 0; j < TPW; ++j) {
      const int tk = wave + j * NWV;
      token[j] = t0 + tk;
      valid[j] = token[j] < T;  // wave-uniform
      wt[j] = (float)(ex[j] * sInv[tk]);
      if (valid[j] && on && (!isfinite(wt[j]) || wt[j] < 0.f)) {
        atomicMin(&status[0], -3);
        atomicMin(&status[1], (token[j] << 10) | lane);
      }
    }
    wave_topk_write_n<TPW>(wt, on, lane, k, renorm, token, valid, idx_out, w_out);
    return;
  }
  // the partial-sum area is free now: softmax scratch
  double* sExp = smem_m;                          // [16][E]
  double* sTok = sExp + 16 * E;                   // [16]
  float* sWt = (float*)(sTok + 16);               // [16][E]
  uint8_t* sSel = (uint8_t*)(sWt + 16 * E);       // [16][E]
  softmax_topk_block(TT, R, E, k, renorm, t0, T, sLogit, sExp, sWt, sSel, sTok, idx_out, w_out,
                     status);
}

template <typename XT, int RB, int NBUF, int NWV>
hipError_t launch_router_mfma_rb(const RouterArgs& a, int R, hipStream_t s) {
  const size_t smem = ((size_t)NWV * RB * 4 * 64 + NWV * 16 + (size_t)16 * R + 16 + R) * 8 +
                      (size_t)16 * R * 4 + (size_t)NWV * 16 * 4 + (size_t)16 * R + 16;
  if (smem > 64 * 1024 || 16 * RB > a.w_rows_pad) return hipErrorInvalidValue;
  // (The selection stays inside this kernel, four tokens per wave: with the logits in HBM and a
  // second launch that gives every token a wave of its own the route stage measured 3-8 us
  // longer at 8192-16384 tokens.)
  router_mfma_kernel<XT, RB, NBUF, NWV><<<(a.T + 15) / 16, 64 * NWV, smem, s>>>(
      (const XT*)a.x, a.T, a.d, a.E, a.k, a.renorm, a.w_router, a.router_bias, a.shared_gate,
      a.idx, a.w, a.sgate, a.status, nullptr, a.w_lsb_min, a.w_t8, a.w_rows_pad, a.w_norm2);
  return hipGetLastError();
}

// (defined further down: selection from logits in HBM with one thread per expert, up to 256 experts)
constexpr int kSelectThreads = 256;
__global__ __launch_bounds__(kSelectThreads) void softmax_select_kernel(
    const float* __restrict__ logits, int T, int E, int k, int renorm,
    int32_t* __restrict__ idx_out, float* __restrict__ w_out, int32_t* __restrict__ status,
    FusedGrouping fg);

// The same kernel with the rows dealt to workgroups in blocks of 16 (eight waves split k), the
// logits left in HBM and the routing decided by a second launch, one wave per token: with many
// rows and a batch that gives fewer workgroups of 16 tokens than the chip has compute units,
// four times as many workgroups of a quarter of the length.
template <typename XT>
hipError_t launch_router_mfma_split(const RouterArgs& a, int R, hipStream_t s) {
  constexpr int NWV = 8, RB = 1, RL = 16;
  const size_t smem = ((size_t)NWV * RB * 4 * 64 + NWV * 16 + (size_t)16 * RL + 16 + RL) * 8 +
                      (size_t)16 * RL * 4 + (size_t)NWV * 16 * 4 + (size_t)16 * RL + 16;
  if ((R + 15) / 16 * 16 > a.w_rows_pad) return hipErrorInvalidValue;
  router_mfma_kernel<XT, RB, 4, NWV><<<dim3((a.T + 15) / 16, (R + 15) / 16), 64 * NWV, smem, s>>>(
      (const XT*)a.x, a.T, a.d, a.E, a.k, a.renorm, a.w_router, a.router_bias, a.shared_gate,
      a.idx, a.w, a.sgate, a.status, a.logits_out ? a.logits_out : a.logits_tmp, a.w_lsb_min,
      a.w_t8, a.w_rows_pad, a.w_norm2);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess || a.logits_out) return e;  // the caller's own launch routes from the logits
  if (a.E <= 64) {
    constexpr int per = kWaveSelectThreads / 64;
    wave_select_kernel<<<(a.T + per - 1) / per, kWaveSelectThreads, 0, s>>>(
        a.logits_tmp, a.T, a.E, a.k, a.renorm, a.idx, a.w, a.status);
  } else {
    const int TT = kSelectThreads / a.E;
    softmax_select_kernel<<<(a.T + TT - 1) / TT, kSelectThreads, 0, s>>>(
        a.logits_tmp, a.T, a.E, a.k, a.renorm, a.idx, a.w, a.status, FusedGrouping{});
  }
  return hipGetLastError();
}

// Up to 80 rows, d a multiple of 8, routing decided in the same launch, no bf16 copy of x to
// write (bf16 activations of unpadded width: the store would sit in the loop).
bool router_mfma_ok(const RouterArgs& a, int R) {
  static const bool off = [] {
    const char* e = getenv("ATENIA_MOE_ROUTER_MFMA");  // tuning knob: 0 = sequential chains
    return e && atoi(e) == 0;
  }();
  // Against the sequential kernel (route stage, us): 8 rows, d = 4096: T = 4096 32 / 57-75,
  // 8192 48 / 89, 16384 89 / 160; 61-64 rows, d = 2048: T = 4096 59 / 92-97, 8192 86 / 87,
  // 12288 127 / 178, 16384 155 / 180: at every batch size.
  // Only with operands that make the exactness test pass -- bf16 activations and router rows whose
  // f32 values fit bf16: otherwise every sum the interval test flags (one in a thousand) costs a
  // sequential chain in its workgroup, and the launch lasts as long as the slowest of them.
  const bool operands = !off && a.d % 8 == 0 && !a.xb && a.x_is_bf16 &&
                        a.w_fits_bf16 && a.w_t8 && a.w_norm2 && a.E >= a.k;
  if (R < 0) return operands;  // the form that deals the rows to workgroups takes any row count
  return operands && R <= 80 && !a.logits_out;
}

// When the rows are dealt to workgroups.  Measured on MI355X, d = 2048, route stage in us,
// split / one workgroup per 16 tokens: 64 rows T = 600 26 / 54, 1024 25 / 54, 2048 36 / 57,
// 3072 57 / 58, 4096 64 / 59, 8192 116 / 87; 32 rows T = 1024 24 / 29, 2048 25 / (29-32),
// 4096 37 / 32; 48 rows, d = 4096, T = 2048 54 / 81.  Against the per-token kernel below 512
// tokens (64 rows): T = 16 23 / 15, 32 24 / 19, 48 24 / 23, 56 24 / 27, 64 24 / 29, 128 24 / 28,
// 256 24 / 32, 384 25 / 47, 512 25 / 50; 32 rows: T = 128 23 / 20, 512 23 / 35.
bool router_mfma_split_wanted(const RouterArgs& a, int R) {
  constexpr int max_t = 2048;
  const int lo = R > 32 ? 52 : 192;
  if (R <= 16 || a.T < lo || !router_mfma_ok(a, -1)) return false;
  // The raw logits are wanted (another launch routes), or more rows than one workgroup holds:
  // no other form on the matrix cores, so at every batch size.  DeepSeek-V3 router shape (256
  // rows, d = 7168, logits for the group-limited selection), route stage in us, this form /
  // the per-token kernel up to 512 tokens and the sequential-order kernel beyond: T = 64
  // 74 / 249, 256 130 / 249, 512 164 / 251, 1024 220 / 260, 2048 354 / 316, 4096 626 / 645,
  // 8192 1172 / 1302 (30 GFLOP of f64 there: 25 TFLOP/s against 78.6 at the f64 matrix peak;
  // several blocks of 16 tokens per workgroup, to read the 7 MB matrix less often, and two or
  // four row blocks per workgroup, to read the tokens less often, both measured no faster).
  if (a.logits_out) return true;
  if (!a.logits_tmp || a.E > kSelectThreads) return false;
  return R > 80 || a.T <= max_t;
}

template <typename XT>
hipError_t launch_router_mfma(const RouterArgs& a, int R, hipStream_t s) {
  // few rows: eight waves split k, so that a batch of 4096 tokens (256 workgroups, one per
  // compute unit) still puts two waves on every SIMD
  if (R <= 16) return launch_router_mfma_rb<XT, 1, 4, 8>(a, R, s);
  if (R <= 32) return launch_router_mfma_rb<XT, 2, 3, 8>(a, R, s);
  if (R <= 48) return launch_router_mfma_rb<XT, 3, 3, 4>(a, R, s);
  if (R <= 64) return launch_router_mfma_rb<XT, 4, 3, 4>(a, R, s);
  return launch_router_mfma_rb<XT, 5, 3, 4>(a, R, s);
}

template <typename XT>
hipError_t dispatch_router_batch(const RouterArgs& a, int R, hipStream_t s) {
  if (R <= 16) return launch_router_batch<XT, 1, 1, 128>(a, s);
  if (R <= 32) return launch_router_batch<XT, 2, 1, 64>(a, s);
  // Many rows and many tokens: a thread takes two tokens as well (each w value read from LDS
  // serves two chains, eight independent f64 chains per thread) while the grid still covers
  // the chip.
  // measured on MI355X at 64 rows, d = 2048: two tokens per thread pay from 8192 tokens on
  const long long work = (long long)a.T * ((R + 63) / 64);  // row blocks count like more tokens
  const int tpt = work >= 8192 ? 2 : 1;
  if (tpt >= 2) return launch_router_batch<XT, 4, 2, 64>(a, s);
  return launch_router_batch<XT, 4, 1, 64>(a, s);
}

// The expert grouping of ONE token from its selection flags (what kernel 2 would produce).
// Called by the threads e = 0..E-1 of the workgroup (sel in LDS, already synchronised): thread e
// counts the selected experts before it and writes its own entries.
__device__ inline void write_single_token_grouping(const FusedGrouping& fg, const int32_t* sel,
                                                   int e, int E, int k) {
  if (e >= E) return;
  int run = 0, total = 0;
#pragma unroll 8
  for (int o = 0; o < E; ++o) {
    const int c = sel[o] ? 1 : 0;
    run += o < e ? c : 0;
    total += c;
  }
  const int c = sel[e] ? 1 : 0;
  fg.counts[e] = c;
  fg.offsets[e] = run;
  if (c && run < k) {
    fg.active[run] = e;
    fg.perm[run] = run;
    fg.inv[run] = run;
    fg.tile_group[run] = e;
    fg.tile_m0[run] = 0;
  }
  if (e == 0) {
    fg.offsets[E] = total;
    *fg.n_active = total;
    *fg.n_tiles = total;
    *fg.shared_n_tiles = 1;
    fg.shared_offsets[0] = 0;
    fg.shared_offsets[1] = 1;
  }
}

// Softmax + top-k from logits that another launch left in HBM: used when the rows of the
// router matrix were spread over several workgroups per token (many experts, few tokens), so
// no single workgroup holds all logits of a token.  256 / E tokens per workgroup.
__global__ __launch_bounds__(kSelectThreads) void softmax_select_kernel(
    const float* __restrict__ logits, int T, int E, int k, int renorm,
    int32_t* __restrict__ idx_out, float* __restrict__ w_out, int32_t* __restrict__ status,
    FusedGrouping fg) {
  __shared__ double sExp[kSelectThreads];
  __shared__ float sWt[kSelectThreads], sLg[kSelectThreads];
  __shared__ int32_t sSel[kSelectThreads];
  const int TT = kSelectThreads / E;
  const int tid = threadIdx.x;
  const int tl = tid / E, r = tid - tl * E;
  const int t = blockIdx.x * TT + tl;
  const bool on = tl < TT && t < T;
  const int ts = on ? t : 0, ls = on ? tl : 0;
  sLg[tid] = on ? logits[(size_t)t * E + r] : 0.f;  // one coalesced read; the folds walk LDS
  __syncthreads();
  softmax_topk(on, r, E, k, renorm, ts, sLg + ls * E, sExp + ls * E, sWt + ls * E, sSel + ls * E,
               idx_out, w_out, status);
  if (fg.counts) {  // T == 1: the workgroup holds token 0 only
    __syncthreads();
    write_single_token_grouping(fg, sSel, tid, E, k);
  }
}

template <typename XT>
__global__ __launch_bounds__(kTokenThreads) void router_token_kernel(
    const XT* __restrict__ x, int T, int d, int E, int k, int renorm,
    const float* __restrict__ w_router, const float* __restrict__ bias,
    const float* __restrict__ gate_vec, int32_t* __restrict__ idx_out,
    float* __restrict__ w_out, float* __restrict__ sgate_out, uint16_t* __restrict__ xb,
    int d_pad, int32_t* __restrict__ status, float* __restrict__ logits_out, FusedGrouping fg) {
  // gridDim.y > 1 (only when the logits go to `logits_out`): this workgroup computes rows
  // row_lo .. row_lo + R - 1 of the stacked matrix; otherwise all of them.
  const int R_all = E + (gate_vec ? 1 : 0);
  const int rows_per_block = (R_all + gridDim.y - 1) / gridDim.y;
  const int row_lo = blockIdx.y * rows_per_block;
  const int R = min(rows_per_block, R_all - row_lo);
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
  int32_t* sBad = sSel + E;                    // [2]: second look wanted, sequential order wanted
  int32_t* sNeed = sBad + 2;                   // [R]
  int32_t* sPartQ = sNeed + R;                 // [max(R, NW)]

  if (tid < 2) sBad[tid] = 0;
  // Work items: (row, k slice).  With few rows each row is split over several waves so that
  // all 16 waves stream the router matrix.  Partial results meet in LDS; under the interval
  // certificate below their order of addition cannot change what the sum rounds to.
  const int KS = R >= NW ? 1 : NW / R;              // k slices per row
  const int slice = ((d + KS - 1) / KS + 3) & ~3;   // multiple of 4 for float4 loads
  const bool vec_ok = (d & 3) == 0;
  const int c_end = xb ? (d_pad > d ? d_pad : d) : d;
  for (int c = tid; c < c_end; c += kTokenThreads) {
    float v = c < d ? load_x(x, (size_t)t * d + c) : 0.f;
    if (c < d) sX[c] = v;
    if (xb && blockIdx.y == 0 && c < d_pad) xb[(size_t)t * d_pad + c] = f32_to_bf16_rne(v);
  }
  __syncthreads();

  for (int item = wave; item < R * KS; item += NW) {
    const int r = item / KS, ksl = item - r * KS;
    const float* wr = row_lo + r < E ? w_router + (size_t)(row_lo + r) * d : gate_vec;
    const int c_lo = ksl * slice, c_hi = min(d, c_lo + slice);
    double acc = 0.0, asum = 0.0;
    auto one = [&](float wv, int c) {
      float xv = sX[c];
      double wd = (double)wv, xd = (double)xv;
      acc = fma(wd, xd, acc);
      asum = fma(fabs(wd), fabs(xd), asum);
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
    }
    if (lane == 0) {
      sPart[item] = acc;
      sPartA[item] = asum;
    }
  }
  __syncthreads();
  if (tid < R) {
    double acc = 0.0, asum = 0.0;
    for (int ksl = 0; ksl < KS; ++ksl) {
      acc += sPart[tid * KS + ksl];
      asum += sPartA[tid * KS + ksl];
    }
    bool exact;
    {
      // The certificate: any order of d exact products summed in f64 lands within
      // g = d * 2^-53 * sum|p| of the true sum (standard bound, 1 / (1 - d u) absorbed by the
      // margin; asum's own relative error of d * 2^-53 likewise), so this sum and the
      // reference's sequential one differ by at most 2 g.  If both ends of [acc - 2g, acc + 2g]
      // round to the same f32 (the same f32 sigmoid for the gate row), the reference's result is
      // that value, whatever its order.  Rounding is monotone; the two extra units of 2^-53
      // cover the roundings of acc -/+ e themselves.  About one sum in a thousand sits close
      // enough to an f32 rounding boundary to fail this; those rows get the second look below.
      const double e = asum * ((double)(2 * d + 4) * 1.1102230246251565e-16) * 1.0001;
      const double lo = acc - e, hi = acc + e;
      if (row_lo + tid < E) {
        const float flo = (float)lo, fhi = (float)hi;
        exact = flo == fhi && isfinite(flo);
      } else {
        const float glo = (float)(1.0 / (1.0 + exp(-lo))), ghi = (float)(1.0 / (1.0 + exp(-hi)));
        exact = glo == ghi;
      }
    }
    sAcc[tid] = acc;
    sNeed[tid] = exact ? 0 : 1;
    if (!exact) {
      sPartA[tid * KS] = asum;  // this thread's own entries: nobody else reads them
      sBad[0] = 1;
    }
  }
  __syncthreads();
  if (sBad[0]) {
    // Second look, for the flagged rows only: when every product of a row is a multiple of 2^q
    // and sum|p| < 2^(q+53), every partial sum of every order is exact in f64, so the sum
    // above IS the reference's sequential one (bf16-valued operands satisfy this).  asum carries
    // a relative error of at most d * 2^-53, covered by the margin.
    for (int item = wave; item < R * KS; item += NW) {
      const int r = item / KS, ksl = item - r * KS;
      int qmin = kNoLsb;
      if (sNeed[r]) {
        const float* wr = row_lo + r < E ? w_router + (size_t)(row_lo + r) * d : gate_vec;
        const int c_lo = ksl * slice, c_hi = min(d, c_lo + slice);
        for (int c = c_lo + lane; c < c_hi; c += 64) {
          const int lx = lsb_exponent(sX[c]), lw = lsb_exponent(wr[c]);
          if (lx != kNoLsb && lw != kNoLsb) qmin = min(qmin, lx + lw);
        }
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) qmin = min(qmin, __shfl_xor(qmin, off));
      }
      if (lane == 0) sPartQ[item] = qmin;
    }
    __syncthreads();
    if (tid < R && sNeed[tid]) {
      int qmin = kNoLsb;
      for (int ksl = 0; ksl < KS; ++ksl) qmin = min(qmin, sPartQ[tid * KS + ksl]);
      const double asum = sPartA[tid * KS];
      const bool exact = qmin == kNoLsb || (qmin > -2000 && asum * 1.000001 < ldexp(1.0, qmin + 53));
      if (!exact) sBad[1] = 1;
    }
    __syncthreads();
  }
  if (sBad[1]) {
    // The reference's own order: one sequential c-ascending f64 sum per row.
    for (int r = tid; r < R; r += kTokenThreads) {
      const float* wr = row_lo + r < E ? w_router + (size_t)(row_lo + r) * d : gate_vec;
      double acc = 0.0;
      for (int c = 0; c < d; ++c) acc = fma((double)wr[c], (double)sX[c], acc);
      sAcc[r] = acc;
    }
    __syncthreads();
  }
  if (tid < R) {
    double acc = sAcc[tid];
    const int gr = row_lo + tid;
    if (gr < E) {
      float logit = (float)acc;
      if (bias) logit = logit + bias[gr];
      sLogit[tid] = logit;  // indexed by expert when the workgroup holds all rows (row_lo == 0)
      if (logits_out) logits_out[(size_t)t * E + gr] = logit;
    } else {
      sgate_out[t] = (float)(1.0 / (1.0 + exp(-acc)));
    }
  }
  __syncthreads();
  if (logits_out) return;  // routing is decided by another kernel from the raw logits
  softmax_topk(tid < E, tid, E, k, renorm, t, sLogit, sExp, sWt, sSel, idx_out, w_out, status);
  if (fg.counts) {  // T == 1: the grouping of a single token follows from its top-k
    __syncthreads();
    write_single_token_grouping(fg, sSel, tid, E, k);
  }
}

}  // namespace

hipError_t launch_router(const RouterArgs& a, hipStream_t s, int* fused_permute) {
  const int R = a.E + (a.shared_gate ? 1 : 0);
  if (fused_permute) *fused_permute = 0;
  if (R > kMaxRouterRows || a.T <= 0) return hipErrorInvalidValue;
  // The per-token kernel re-reads the whole stacked matrix for every token; with many rows
  // (row blocks, logits mode) that only pays for a handful of tokens.
  const bool mfma = router_mfma_ok(a, R);
  if (router_mfma_split_wanted(a, R))
    return launch_router_mfma_split<uint16_t>(a, R, s);  // bf16 activations only (router_mfma_ok)
  const bool token_ok = a.T <= a.token_kernel_max_tokens &&
                        (R <= 64 || (long long)a.T * R * a.d <= (16ll << 20));
  if (token_ok) {
    const size_t np = R > kTokenThreads / 64 ? R : kTokenThreads / 64;
    size_t smem = ((size_t)R + a.E + 2 * np) * 8 + (size_t)a.d * 4 + (size_t)a.E * 12 + 8 +
                  ((size_t)R + np) * 4 + 16;
    if (smem <= 64 * 1024) {
      // Many rows, few tokens: one workgroup per token would stream the whole stacked matrix
      // through a single CU.  The rows are spread over workgroups instead (four rows each, a
      // row split over four waves), the logits go to HBM, and the selection runs as a second,
      // tiny launch -- the caller's own one (logits_out) or softmax_select_kernel here.
      // Measured (61-65 rows, d = 2048): spread 29 / 30 / 35 / 46 us at T = 33 / 48 / 64 / 96
      // against 40-43 us for one workgroup per token, so the rows are spread up to 64 tokens.
      const bool spread = R > 32 && (a.logits_out || (a.logits_tmp && a.T <= 64 &&
                                                      a.E <= kSelectThreads));
      float* lg = a.logits_out ? a.logits_out : (spread ? a.logits_tmp : nullptr);
      FusedGrouping fg{};
      if (a.T == 1 && a.fuse_permute && !a.logits_out) {
        const PermuteArgs& pa = *a.fuse_permute;
        fg = FusedGrouping{pa.counts, pa.offsets, pa.perm, pa.inv, pa.active, pa.n_active,
                           pa.shared_offsets, pa.tile_group, pa.tile_m0, pa.n_tiles,
                           pa.shared_n_tiles};
        if (fused_permute) *fused_permute = 1;
      }
      const FusedGrouping fg_token = spread ? FusedGrouping{} : fg;
      const int row_blocks = spread ? (R + 3) / 4 : 1;
      const dim3 grid(a.T, row_blocks);
      if (a.x_is_bf16)
        router_token_kernel<uint16_t><<<grid, kTokenThreads, smem, s>>>(
            (const uint16_t*)a.x, a.T, a.d, a.E, a.k, a.renorm, a.w_router, a.router_bias,
            a.shared_gate, a.idx, a.w, a.sgate, a.xb, a.d_pad, a.status, lg, fg_token);
      else
        router_token_kernel<float><<<grid, kTokenThreads, smem, s>>>(
            (const float*)a.x, a.T, a.d, a.E, a.k, a.renorm, a.w_router, a.router_bias,
            a.shared_gate, a.idx, a.w, a.sgate, a.xb, a.d_pad, a.status, lg, fg_token);
      if (spread && !a.logits_out && a.defer_select && a.T == 1 && a.E <= 64 && fg.counts) {
        // the caller's next launch routes the token itself from the logits (select_wave.h)
        if (fused_permute) *fused_permute = 2;
        return hipGetLastError();
      }
      if (spread && !a.logits_out) {
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
        if (a.E <= 64 && !fg.counts) {  // one wave per token
          constexpr int per = kWaveSelectThreads / 64;
          wave_select_kernel<<<(a.T + per - 1) / per, kWaveSelectThreads, 0, s>>>(
              lg, a.T, a.E, a.k, a.renorm, a.idx, a.w, a.status);
          return hipGetLastError();
        }
        const int TT = kSelectThreads / a.E;
        softmax_select_kernel<<<(a.T + TT - 1) / TT, kSelectThreads, 0, s>>>(
            lg, a.T, a.E, a.k, a.renorm, a.idx, a.w, a.status, fg);
      }
      return hipGetLastError();
    }
  }
  if (mfma)
    return launch_router_mfma<uint16_t>(a, R, s);
  // Up to 64 rows per workgroup; more rows only when the logits leave the kernel (row blocks).
  if ((R <= 64 || a.logits_out) && a.d % 4 == 0 && (!a.xb || a.d_pad % 4 == 0)) {
    return a.x_is_bf16 ? dispatch_router_batch<uint16_t>(a, R, s)
                       : dispatch_router_batch<float>(a, R, s);
  }
  // More than 64 rows with softmax routing: the same row-block launch into the scratch logits,
  // then the selection as a second launch.
  if (a.logits_tmp && a.E <= kSelectThreads && a.d % 4 == 0 && (!a.xb || a.d_pad % 4 == 0)) {
    RouterArgs b = a;
    b.logits_out = a.logits_tmp;
    hipError_t e = a.x_is_bf16 ? dispatch_router_batch<uint16_t>(b, R, s)
                               : dispatch_router_batch<float>(b, R, s);
    if (e != hipSuccess) return e;
    const int TT = kSelectThreads / a.E;
    softmax_select_kernel<<<(a.T + TT - 1) / TT, kSelectThreads, 0, s>>>(
        a.logits_tmp, a.T, a.E, a.k, a.renorm, a.idx, a.w, a.status, FusedGrouping{});
    return hipGetLastError();
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
        a.shared_gate, a.idx, a.w, a.sgate, a.xb, a.d_pad, a.status, a.logits_out, TT);
  } else {
    router_tile_kernel<float><<<blocks, kRouterThreads, smem, s>>>(
        (const float*)a.x, a.T, a.d, a.E, a.k, a.renorm, a.w_router, a.router_bias,
        a.shared_gate, a.idx, a.w, a.sgate, a.xb, a.d_pad, a.status, a.logits_out, TT);
  }
  return hipGetLastError();
}

}  // namespace atenia_moe
