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

// Largest value over the 64 lanes of a wave, in every lane: four DPP steps make each row of 16
// lanes uniform (swap neighbours, swap pairs, mirror the half row, mirror the row), the four row
// values meet on the scalar side.
__device__ inline int wave_max_i32(int v) {
  v = max(v, __builtin_amdgcn_update_dpp(v, v, 0xB1, 0xf, 0xf, false));   // quad_perm [1,0,3,2]
  v = max(v, __builtin_amdgcn_update_dpp(v, v, 0x4E, 0xf, 0xf, false));   // quad_perm [2,3,0,1]
  v = max(v, __builtin_amdgcn_update_dpp(v, v, 0x141, 0xf, 0xf, false));  // row_half_mirror
  v = max(v, __builtin_amdgcn_update_dpp(v, v, 0x140, 0xf, 0xf, false));  // row_mirror
  return max(max(__builtin_amdgcn_readlane(v, 0), __builtin_amdgcn_readlane(v, 16)),
             max(__builtin_amdgcn_readlane(v, 32), __builtin_amdgcn_readlane(v, 48)));
}

// Top-k of one token from its softmax weights (lane r = expert r) and the routing written out:
// the k experts that sort first under (weight desc, index asc) are found as k times the largest
// weight still available, the lowest lane among equals.  Weights are >= +0, so their bit
// patterns order like integers (-1 = not available; a NaN weight is reported by the caller).
// The weights of the selection are summed e ascending, as the reference sums its sorted
// selection (dense.rs:172-187, sparse.rs:142-191).
__device__ inline void wave_topk_write(float wt, bool on, int lane, int k, int renorm, int token,
                                       int32_t* __restrict__ idx_out, float* __restrict__ w_out) {
  const int wbits = on ? __float_as_int(wt) : -1;
  unsigned long long avail = ~0ull, mask = 0ull;
  for (int r = 0; r < k; ++r) {
    const int v = (avail >> lane) & 1ull ? wbits : -1;
    const int m = wave_max_i32(v);
    const unsigned long long cand = __ballot(v == m && m >= 0);
    if (!cand) break;  // wave-uniform; k <= E makes it unreachable
    const unsigned long long win = cand & (~cand + 1ull);
    mask |= win;
    avail &= ~win;
  }
  const bool selected = (mask >> lane) & 1ull;
  const int slot = __popcll(mask & ((1ull << lane) - 1ull));
  double ssum = 0.0;
  for (unsigned long long m = mask; m; m &= m - 1)
    ssum += (double)readlane_f32(wt, __ffsll((long long)m) - 1);
  const double scale = renorm ? 1.0 / ssum : 1.0;
  if (selected && slot < k) {
    const size_t o = (size_t)token * k + slot;
    idx_out[o] = lane;
    w_out[o] = (float)((double)wt * scale);
  }
}

// The same for N tokens of one wave at once (lane r = expert r of each): the N selections are
// independent chains of cross-lane steps, and run interleaved they hide each other's latency.
// Token j is written only when valid[j].  Same results as N calls of wave_topk_write.
template <int N>
__device__ inline void wave_topk_write_n(const float (&wt)[N], bool on, int lane, int k, int renorm,
                                         const int (&token)[N], const bool (&valid)[N],
                                         int32_t* __restrict__ idx_out, float* __restrict__ w_out) {
  int wbits[N];
  unsigned long long avail[N], mask[N];
#pragma unroll
  for (int j = 0; j < N; ++j) {
    wbits[j] = on ? __float_as_int(wt[j]) : -1;
    avail[j] = ~0ull;
    mask[j] = 0ull;
  }
  for (int r = 0; r < k; ++r) {
#pragma unroll
    for (int j = 0; j < N; ++j) {
      const int v = (avail[j] >> lane) & 1ull ? wbits[j] : -1;
      const int m = wave_max_i32(v);
      const unsigned long long cand = __ballot(v == m && m >= 0);
      const unsigned long long win = cand & (~cand + 1ull);  // nothing left: no bit, no change
      mask[j] |= win;
      avail[j] &= ~win;
    }
  }
#pragma unroll
  for (int j = 0; j < N; ++j) {
    if (!valid[j]) continue;  // wave-uniform
    const bool selected = (mask[j] >> lane) & 1ull;
    const int slot = __popcll(mask[j] & ((1ull << lane) - 1ull));
    double ssum = 0.0;
    for (unsigned long long m = mask[j]; m; m &= m - 1)
      ssum += (double)readlane_f32(wt[j], __ffsll((long long)m) - 1);
    const double scale = renorm ? 1.0 / ssum : 1.0;
    if (selected && slot < k) {
      const size_t o = (size_t)token[j] * k + slot;
      idx_out[o] = lane;
      w_out[o] = (float)((double)wt[j] * scale);
    }
  }
}

// Largest of 64 non-NaN floats, in every lane (the steps of wave_max_i32).
__device__ inline float wave_max_f32(float f) {
  int v = __float_as_int(f);
  auto mx = [](int a, int b) { return __float_as_int(fmaxf(__int_as_float(a), __int_as_float(b))); };
  v = mx(v, __builtin_amdgcn_update_dpp(v, v, 0xB1, 0xf, 0xf, false));
  v = mx(v, __builtin_amdgcn_update_dpp(v, v, 0x4E, 0xf, 0xf, false));
  v = mx(v, __builtin_amdgcn_update_dpp(v, v, 0x141, 0xf, 0xf, false));
  v = mx(v, __builtin_amdgcn_update_dpp(v, v, 0x140, 0xf, 0xf, false));
  return fmaxf(fmaxf(readlane_f32(__int_as_float(v), 0), readlane_f32(__int_as_float(v), 16)),
               fmaxf(readlane_f32(__int_as_float(v), 32), readlane_f32(__int_as_float(v), 48)));
}

// Softmax + top-k of token t from its logits row in memory, by one wavefront (up to 64 experts).
// Same arithmetic, casts and order as softmax_topk in router.hip; the sequential fold of the
// exponentials runs over v_readlane values.  Every lane of the wave must call.
__device__ inline void wave_select_token(const float* __restrict__ lg, int E, int k, int renorm,
                                         int t, int lane, int32_t* __restrict__ idx_out,
                                         float* __restrict__ w_out, int32_t* __restrict__ status) {
  const bool on = lane < E;
  const float my = on ? lg[lane] : -INFINITY;
  float mx = fmaxf(-INFINITY, my);  // a NaN logit is skipped, as f32::max skips it
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off));
  const double ex = on ? exp((double)(my - mx)) : 0.0;  // f32 subtraction, then f64 exp
  double sum = 0.0;
  for (int e0 = 0; e0 < E; e0 += 8) {  // sequential fold, e ascending; lanes past E add +0
#pragma unroll
    for (int u = 0; u < 8; ++u) sum += readlane_f64(ex, e0 + u);
  }
  const double inv = sum > 0.0 ? 1.0 / sum : 0.0;
  const float wt = (float)(ex * inv);
  if (on && (!isfinite(wt) || wt < 0.f)) {
    atomicMin(&status[0], -3);
    atomicMin(&status[1], (t << 10) | lane);
  }
  wave_topk_write(wt, on, lane, k, renorm, t, idx_out, w_out);
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
