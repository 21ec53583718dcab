// Softmax + top-k of ONE token inside a single wavefront, and the expert grouping that follows
// from it.  Same arithmetic, casts and order as softmax_topk in router.hip (dense.rs:172-187,
// sparse.rs:142-191): lane r holds expert r (E <= 64), the two sequential folds of the reference
// (f64 sum of the exponentials, f64 sum of the selected weights, both e ascending) run over
// v_readlane values, so every wave that calls this on the same logits gets the same bits.
// Used where a launch that needs the routing of a single token computes it itself instead of
// waiting for a launch of its own.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <math.h>

namespace atenia_moe {

// Outputs of the expert grouping for the single-token case (see permute.hip for the contract).
struct FusedGrouping {
  int32_t *counts, *offsets, *perm, *inv, *active, *n_active, *shared_offsets;
  int32_t *tile_group, *tile_m0, *n_tiles, *shared_n_tiles;
};

// What a launch needs to route the single token itself: the raw logits [E] (bias added) that
// the router launch left in HBM, and where the routing and the grouping go.
struct InlineSelect {
  const float* logits;  // null = routing was done by the router launch
  int E, k, renorm;
  int32_t* idx;     // [k] experts ascending
  float* w;         // [k]
  int32_t* status;  // [2]
  FusedGrouping fg;
};

struct WaveRouting {
  unsigned long long mask;  // selected experts
  int slot;                 // this lane's position among them (valid when selected)
  float w;                  // this lane's routing weight after renormalisation
  bool selected;
  bool bad;                 // softmax weight not finite or negative
};

__device__ inline float readlane_f32(float v, int l) {
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), l));
}
__device__ inline double readlane_f64(double v, int l) {
  const long long b = __double_as_longlong(v);
  const unsigned lo = (unsigned)__builtin_amdgcn_readlane((int)(b & 0xffffffffll), l);
  const unsigned hi = (unsigned)__builtin_amdgcn_readlane((int)(b >> 32), l);
  return __longlong_as_double((long long)(((unsigned long long)hi << 32) | lo));
}

// Every lane of the wave must call (lanes >= E idle along).
__device__ inline WaveRouting wave_softmax_topk(const float* lg, int E, int k, int renorm, int lane) {
  const bool on = lane < E;
  const float my = on ? lg[lane] : -INFINITY;
  float mx = fmaxf(-INFINITY, my);  // a NaN logit is skipped, as f32::max skips it
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off));
  const double ex = on ? exp((double)(my - mx)) : 0.0;  // f32 subtraction, then f64 exp
  double sum = 0.0;
  for (int e = 0; e < E; ++e) sum += readlane_f64(ex, e);  // sequential fold, e ascending
  const double inv = sum > 0.0 ? 1.0 / sum : 0.0;
  const float wt = (float)(ex * inv);
  WaveRouting r;
  r.bad = on && (!isfinite(wt) || wt < 0.f);
  int rank = 0;  // experts that sort before this one under (weight desc, index asc)
  for (int e = 0; e < E; ++e) {
    const float we = readlane_f32(wt, e);
    rank += (we > wt) || (we == wt && e < lane);
  }
  r.selected = on && rank < k;
  r.mask = __ballot(r.selected);
  r.slot = __popcll(r.mask & ((1ull << lane) - 1ull));
  double ssum = 0.0;  // ascending e, as the reference sums the sorted selection
  for (unsigned long long m = r.mask; m; m &= m - 1) ssum += (double)readlane_f32(wt, __ffsll((long long)m) - 1);
  const double scale = renorm ? 1.0 / ssum : 1.0;
  r.w = (float)((double)wt * scale);
  return r;
}

// Expert of group u (the u-th selected expert, ascending), or -1.
__device__ inline int wave_selected_expert(unsigned long long mask, int u) {
  for (int i = 0; i < u && mask; ++i) mask &= mask - 1;
  return mask ? __ffsll((long long)mask) - 1 : -1;
}

// One wave writes the token's routing and, when fg.counts is set, its expert grouping.
__device__ inline void wave_write_routing(const InlineSelect& s, const WaveRouting& r, int lane) {
  if (r.bad) {
    atomicMin(&s.status[0], -3);
    atomicMin(&s.status[1], lane);  // token 0
  }
  if (r.selected && r.slot < s.k) {
    s.idx[r.slot] = lane;
    s.w[r.slot] = r.w;
  }
  const FusedGrouping& fg = s.fg;
  if (!fg.counts) return;
  const int total = __popcll(r.mask);
  if (lane < s.E) {
    fg.counts[lane] = r.selected ? 1 : 0;
    fg.offsets[lane] = r.slot;
    if (r.selected && r.slot < s.k) {
      fg.active[r.slot] = lane;
      fg.perm[r.slot] = r.slot;
      fg.inv[r.slot] = r.slot;
      fg.tile_group[r.slot] = lane;
      fg.tile_m0[r.slot] = 0;
    }
  }
  if (lane == 0) {
    fg.offsets[s.E] = total;
    *fg.n_active = total;
    *fg.n_tiles = total;
    *fg.shared_n_tiles = 1;
    fg.shared_offsets[0] = 0;
    fg.shared_offsets[1] = 1;
  }
}

}  // namespace atenia_moe
