// DeepSeek-V3 routing: sigmoid scores, bias-corrected selection, group-limited top-k, scaled
// combine weights (src/moe/v3_router.rs:206-309), from the raw f32 logits the router kernels
// leave in HBM.  All arithmetic in f64 as in the reference:
//   score_e  = 1 / (1 + exp(-logit_e));  choice_e = score_e + bias_e
//   group score = sum of the group's two largest choices; the topk_group best groups stay
//   (ties: lower group), experts of other groups are masked to -inf; the top_k best remaining
//   experts are selected (ties: lower index) and emitted ascending;
//   weight = score (not choice), / (sum of selected scores, ascending, + 1e-20) when
//   norm_topk_prob, * routed_scaling_factor, rounded to f32.
// "The k best under (value desc, index asc)" is computed as a rank count per element, which is
// what the reference's stable sort yields.  One thread per (token, expert); a workgroup holds
// 256 / E tokens.  A non-finite logit is reported through the status words like a non-finite
// routing weight of the softmax router (the reference fails with NonFinite{router_logits, index}).
#include "moe_internal.h"

namespace atenia_moe {

namespace {

constexpr int kV3Threads = 256;

__global__ __launch_bounds__(kV3Threads) void v3_route_kernel(
    const float* __restrict__ logits, const float* __restrict__ bias, int T, int E, int k,
    int n_group, int topk_group, int norm_topk_prob, double scale, int32_t* __restrict__ idx_out,
    float* __restrict__ w_out, int32_t* __restrict__ status) {
  __shared__ double sScore[kV3Threads];   // [TT][E]
  __shared__ double sChoice[kV3Threads];  // [TT][E]
  __shared__ double sGroup[kV3Threads / 2];    // [TT][n_group]
  __shared__ uint8_t sGroupSel[kV3Threads / 2];
  __shared__ uint8_t sSel[kV3Threads];      // slot of a selected thread
  __shared__ double sList[kV3Threads];      // [TT][k] scores of the selected experts, ascending
  __shared__ unsigned long long sWaveVote[kV3Threads / 64];
  const int TT = kV3Threads / E;  // >= 1: the launcher refuses E > 256
  const int tid = threadIdx.x;
  const int tl = tid / E, r = tid - tl * E;
  const int t = blockIdx.x * TT + tl;
  const bool on = tl < TT && t < T;
  const int epg = E / n_group;
  const int base = tl * E, gbase = tl * n_group;

  if (on) {
    const float lg = logits[(size_t)t * E + r];
    if (!isfinite(lg)) {
      atomicMin(&status[0], -3);
      atomicMin(&status[1], (t << 10) | r);
    }
    const double sc = 1.0 / (1.0 + exp(-(double)lg));
    sScore[base + r] = sc;
    sChoice[base + r] = sc + (double)bias[r];
  }
  __syncthreads();
  if (on && r < n_group) {  // the two largest choices of group r
    const double* c = sChoice + base + r * epg;
    double m1 = -INFINITY, m2 = -INFINITY;
#pragma unroll 8
    for (int j = 0; j < epg; ++j) {
      const double v = c[j];  // finite: fmax / fmin are plain comparisons here
      m2 = fmax(m2, fmin(m1, v));
      m1 = fmax(m1, v);
    }
    sGroup[gbase + r] = m1 + m2;
  }
  __syncthreads();
  if (on && r < n_group) {
    const double mine = sGroup[gbase + r];
    int rank = 0;  // groups that sort before this one under (score desc, index asc)
    for (int g = 0; g < n_group; ++g) {
      const double o = sGroup[gbase + g];
      rank += (o > mine) || (o == mine && g < r);
    }
    sGroupSel[gbase + r] = rank < topk_group;
  }
  __syncthreads();
  // Only experts of the kept groups compete; an expert's rank counts those that sort before it
  // under (choice desc, index asc).  Masked experts never enter: top_k <= experts in the kept
  // groups (checked when the router is configured).
  bool selected = false;
  double my_score = 0.0;
  if (on && sGroupSel[gbase + r / epg]) {
    const double mine = sChoice[base + r];
    int rank = 0;
    for (int g = 0; g < n_group; ++g) {
      if (!sGroupSel[gbase + g]) continue;  // uniform across the workgroup when it holds one token
      const double* c = sChoice + base + g * epg;
      const int e0 = g * epg;
#pragma unroll 8
      for (int j = 0; j < epg; ++j) {
        const double o = c[j];
        rank += (o > mine) || (o == mine && e0 + j < r);
      }
    }
    selected = rank < k;
    my_score = sScore[base + r];
  }
  // Ascending slots: selected lanes before this one in its wave (ballot) plus the selected
  // lanes of the earlier waves that belong to the same token.
  const unsigned long long vote = __ballot(selected);
  const int lane = tid & 63, wave = tid >> 6;
  if (lane == 0) sWaveVote[wave] = vote;
  __syncthreads();
  if (selected) {
    int slot = 0;
    const int first = base, last = base + r;  // thread ids of this token before this expert
    for (int w = first >> 6; w <= wave; ++w) {
      unsigned long long m = sWaveVote[w];
      const int lo = w * 64;
      if (first > lo) m &= ~0ull << (first - lo);
      if (last < lo + 64) m &= (last - lo) >= 64 ? ~0ull : ((1ull << (last - lo)) - 1ull);
      slot += __popcll(m);
    }
    if (slot < k) {
      sList[tl * k + slot] = my_score;
      idx_out[(size_t)t * k + slot] = r;
    }
    sSel[tid] = (uint8_t)slot;
  }
  __syncthreads();
  if (selected) {
    const int slot = sSel[tid];
    double denom = 0.0;
    for (int j = 0; j < k; ++j) denom += sList[tl * k + j];  // ascending index, as the sorted selection is summed
    denom += 1e-20;
    double w = my_score;
    if (norm_topk_prob) w /= denom;
    w *= scale;
    if (slot < k) w_out[(size_t)t * k + slot] = (float)w;
  }
}

}  // namespace

hipError_t launch_v3_route(const V3RouteArgs& a, hipStream_t s) {
  if (a.T <= 0) return hipSuccess;
  if (a.E <= 0 || a.E > kV3Threads || a.n_group <= 0 || a.E % a.n_group != 0 ||
      a.n_group > kV3Threads / 2)
    return hipErrorInvalidValue;
  const int TT = kV3Threads / a.E;
  const unsigned grid = (unsigned)((a.T + TT - 1) / TT);
  v3_route_kernel<<<grid, kV3Threads, 0, s>>>(a.logits, a.bias, a.T, a.E, a.k, a.n_group,
                                              a.topk_group, a.norm_topk_prob,
                                              a.routed_scaling_factor, a.idx, a.w, a.status);
  return hipGetLastError();
}

}  // namespace atenia_moe
