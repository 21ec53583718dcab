// Kernel 2: histogram, prefix scan and stable permutation that groups (token, slot) pairs
// by expert.
//
// The reference has no such step: it visits tokens one after another
// (src/moe/graph_op.rs:345-348) and, inside a token, the selected experts in ascending
// index order (src/moe/sparse.rs:175).  The grouping contract is derived from that visiting
// order: pairs are numbered p = t*k + slot, counts[e] is the number of pairs routed to e,
// offsets is the exclusive scan of counts, and perm lists the pair ids expert by expert,
// ascending in p inside each expert (a stable counting sort).  All integer work; results are
// unique, so they must match the CPU oracle bit for bit.
//
// Small batches (P <= 1024 pairs) take one launch of one block; up to 16 blocks of 1024 pairs
// still one launch, every block counting the whole list for itself.  Larger ones take three:
// per-block histograms, one block that scans them, and a scatter pass that recomputes each
// block's stable ranks.
#include <algorithm>
#include <cstdlib>

#include "moe_internal.h"

namespace atenia_moe {

namespace {

constexpr int kWaves = kPermuteBlock / 64;

// Stable rank of this thread's pair among the pairs of the same expert inside the block.
// sWaveCnt: [kWaves][E] scratch.  On return sWaveCnt[w][e] holds the exclusive prefix over
// waves and sBlkCnt[e] the block total.  All threads of the block must call.
__device__ int block_stable_rank(int e, bool valid, int E, int32_t* sWaveCnt,
                                 int32_t* sBlkCnt) {
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  for (int j = tid; j < kWaves * E; j += kPermuteBlock) sWaveCnt[j] = 0;
  __syncthreads();
  // The lanes of this wave with the same expert: one ballot per bit of the expert index, each
  // lane keeping the side its own bit is on (eight ballots for up to 256 experts, where a loop
  // over the distinct experts of the wave took one round of ballot + shuffle per expert).
  const unsigned long long lt = lane == 0 ? 0ull : (~0ull >> (64 - lane));
  unsigned long long m = __ballot(valid);
  for (int b = 0; (1 << b) < E; ++b) {  // wave-uniform trip count
    const bool bit = (e >> b) & 1;
    const unsigned long long B = __ballot(bit);
    m &= bit ? B : ~B;
  }
  const int my_rank = __popcll(m & lt);
  if (valid && (m & lt) == 0ull) sWaveCnt[wave * E + e] = __popcll(m);  // the first lane of its group
  __syncthreads();
  for (int ee = tid; ee < E; ee += kPermuteBlock) {
    int run = 0;
    for (int w = 0; w < kWaves; ++w) {
      int c = sWaveCnt[w * E + ee];
      sWaveCnt[w * E + ee] = run;
      run += c;
    }
    sBlkCnt[ee] = run;
  }
  __syncthreads();
  return valid ? sWaveCnt[wave * E + e] + my_rank : 0;
}

// counts -> offsets / active list, done by one thread (E <= a few hundred).
struct TileOut {
  int32_t* tile_group;
  int32_t* tile_m0;
  int32_t* n_tiles;
  int32_t* shared_n_tiles;
  int32_t* tile_rows;  // rows of each tile (may be null)
  int32_t* tile_li;    // index of the tile inside its expert | (tiles of the expert << 16) (may be null)
  int max_groups;      // 32-row groups a tile may hold: 8 (256-row tiles) or 9
};

// Row tiles of an expert with c rows.  max_groups == 8: whole 256-row tiles and one tile with
// the rest.  max_groups == 9: the expert's 32-row groups are dealt evenly over as few tiles as
// hold them, so that a rest of up to 32 rows per tile rides in a tile of nine groups instead of
// becoming a tile of its own (which would stream a whole weight panel for a handful of rows).
__device__ inline int expert_tiles(int c, int max_groups) {
  if (max_groups <= 8) return (c + kTileM - 1) / kTileM;
  const int G = (c + 31) >> 5;
  return (G + max_groups - 1) / max_groups;
}
__device__ inline void expert_tile(int c, int max_groups, int nt, int i, int& m0, int& rows) {
  if (max_groups <= 8) {
    m0 = i * kTileM;
    rows = min(kTileM, c - m0);
    return;
  }
  const int G = (c + 31) >> 5;
  const int q = G / nt, r = G - q * nt;          // the first r tiles hold q + 1 groups
  const int g0 = i * q + min(i, r);
  m0 = g0 * 32;
  rows = min((q + (i < r ? 1 : 0)) * 32, c - m0);
}

// counts -> offsets / active list / row-tile list.  Block-cooperative: every thread of the
// block calls it (barriers inside), thread e owns expert e.  Three prefix sums over the experts
// (rows, active flags, row tiles) replace a serial walk whose stores and loads through generic
// pointers waited for each other (12 us for 60 experts).  E <= kMaxRouterRows.
// s_offsets (LDS, [E + 1], may be null) receives the offsets as well; valid after the caller's
// next barrier.  write_out = false: only s_offsets is wanted (another block writes the lists).
__device__ void finish_offsets(int E, const int32_t* counts, int32_t* offsets, int32_t* active,
                               int32_t* n_active, int32_t* shared_offsets, int T, TileOut to,
                               int32_t* s_offsets = nullptr, bool write_out = true) {
  // exclusive prefixes over the experts, totals at [kMaxRouterRows]
  __shared__ int32_t sRows[kMaxRouterRows + 1], sAct[kMaxRouterRows + 1], sTiles[kMaxRouterRows + 1];
  const int tid = threadIdx.x;
  const bool mine = tid < E;
  const int c = mine ? counts[tid] : 0;
  const int a = c > 0 ? 1 : 0;
  const int nt = to.tile_group ? expert_tiles(c, to.max_groups) : 0;
  if (tid < 64) {
    // One wave scans all three: a lane owns EPL consecutive experts, the lane totals are
    // scanned with six shuffles each (barrier-free; sixteen barriers of 1024 threads for a
    // step-by-step scan in LDS took longer than everything else in the launch).
    constexpr int EPL = kMaxRouterRows / 64;
    int cr[EPL], ca[EPL], ct[EPL];
    int r = 0, q = 0, t = 0;
#pragma unroll
    for (int j = 0; j < EPL; ++j) {
      const int ee = EPL * tid + j;
      const int cc = ee < E ? counts[ee] : 0;
      cr[j] = r;
      ca[j] = q;
      ct[j] = t;
      r += cc;
      q += cc > 0 ? 1 : 0;
      t += to.tile_group ? expert_tiles(cc, to.max_groups) : 0;
    }
    int ir = r, iq = q, it = t;  // inclusive over the lanes
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const int ur = __shfl_up(ir, off), uq = __shfl_up(iq, off), ut = __shfl_up(it, off);
      if (tid >= off) {
        ir += ur;
        iq += uq;
        it += ut;
      }
    }
#pragma unroll
    for (int j = 0; j < EPL; ++j) {
      sRows[EPL * tid + j] = ir - r + cr[j];
      sAct[EPL * tid + j] = iq - q + ca[j];
      sTiles[EPL * tid + j] = it - t + ct[j];
    }
    if (tid == 63) {
      sRows[kMaxRouterRows] = ir;
      sAct[kMaxRouterRows] = iq;
      sTiles[kMaxRouterRows] = it;
    }
  }
  __syncthreads();
  if (mine && s_offsets) s_offsets[tid] = sRows[tid];
  if (tid == 0 && s_offsets) s_offsets[E] = sRows[kMaxRouterRows];
  if (!write_out) return;
  if (mine) {
    offsets[tid] = sRows[tid];
    if (a) active[sAct[tid]] = tid;
    const int t0 = sTiles[tid];
    for (int i = 0; i < nt; ++i) {
      int m0, rows;
      expert_tile(c, to.max_groups, nt, i, m0, rows);
      to.tile_group[t0 + i] = tid;
      to.tile_m0[t0 + i] = m0;
      if (to.tile_rows) to.tile_rows[t0 + i] = rows;
      if (to.tile_li) to.tile_li[t0 + i] = i | (nt << 16);
    }
  }
  if (tid == 0) {
    offsets[E] = sRows[kMaxRouterRows];
    *n_active = sAct[kMaxRouterRows];
    if (to.n_tiles) *to.n_tiles = sTiles[kMaxRouterRows];
    if (to.shared_n_tiles) *to.shared_n_tiles = (T + kTileM - 1) / kTileM;
    if (shared_offsets) {
      shared_offsets[0] = 0;
      shared_offsets[1] = T;
    }
  }
}

__global__ __launch_bounds__(kPermuteBlock) void permute_single_kernel(
    const int32_t* __restrict__ idx, int P, int E, int T, int32_t* counts, int32_t* offsets,
    int32_t* perm, int32_t* inv, int32_t* active, int32_t* n_active, int32_t* shared_offsets,
    TileOut to) {
  extern __shared__ int32_t sm[];
  int32_t* sWaveCnt = sm;               // [kWaves][E]
  int32_t* sBlkCnt = sm + kWaves * E;   // [E]
  int32_t* sOff = sBlkCnt + E;          // [E+1]
  const int p = threadIdx.x;
  const bool valid = p < P;
  const int e = valid ? idx[p] : 0;
  int rank = block_stable_rank(e, valid, E, sWaveCnt, sBlkCnt);
  for (int ee = threadIdx.x; ee < E; ee += kPermuteBlock) counts[ee] = sBlkCnt[ee];
  // the exclusive scan of the counts comes out of finish_offsets' parallel prefix (one thread
  // walking the experts in LDS took 3-4 us with 60 of them)
  finish_offsets(E, sBlkCnt, offsets, active, n_active, shared_offsets, T, to, sOff);
  __syncthreads();
  if (valid) {
    int pos = sOff[e] + rank;
    perm[pos] = p;
    inv[p] = pos;
  }
}

// A few thousand pairs in ONE launch: block b places the pairs b * 1024 .. of the list, and
// counts for itself what the three-launch form below passes through HBM -- every block reads
// the whole index list (at most kMultiBlocks * 1024 entries, from L2) and keeps, per expert,
// the total and the number of pairs in the blocks before its own.  Block 0 writes the lists.
constexpr int kMultiBlocks = 16;
__global__ __launch_bounds__(kPermuteBlock) void permute_multi_kernel(
    const int32_t* __restrict__ idx, int P, int E, int T, int32_t* counts, int32_t* offsets,
    int32_t* perm, int32_t* inv, int32_t* active, int32_t* n_active, int32_t* shared_offsets,
    TileOut to) {
  extern __shared__ int32_t sm[];
  int32_t* sWaveCnt = sm;               // [kWaves][E]
  int32_t* sBlkCnt = sm + kWaves * E;   // [E]
  int32_t* sOff = sBlkCnt + E;          // [E+1]
  int32_t* sTot = sOff + E + 1;         // [E]
  int32_t* sBefore = sTot + E;          // [E]
  const int tid = threadIdx.x, blk = blockIdx.x, nblk = gridDim.x;
  for (int j = tid; j < E; j += kPermuteBlock) {
    sTot[j] = 0;
    sBefore[j] = 0;
  }
  __syncthreads();
  int e = 0;
  for (int c = 0; c < nblk; ++c) {
    const int q = c * kPermuteBlock + tid;
    if (q < P) {
      const int ee = idx[q];
      atomicAdd(&sTot[ee], 1);
      if (c < blk) atomicAdd(&sBefore[ee], 1);
      if (c == blk) e = ee;
    }
  }
  const int p = blk * kPermuteBlock + tid;
  const bool valid = p < P;
  int rank = block_stable_rank(e, valid, E, sWaveCnt, sBlkCnt);  // barriers inside: the counts are complete
  if (blk == 0)
    for (int ee = tid; ee < E; ee += kPermuteBlock) counts[ee] = sTot[ee];
  finish_offsets(E, sTot, offsets, active, n_active, shared_offsets, T, to, sOff, blk == 0);
  __syncthreads();
  if (valid) {
    int pos = sOff[e] + sBefore[e] + rank;
    perm[pos] = p;
    inv[p] = pos;
  }
}

__global__ __launch_bounds__(kPermuteBlock) void permute_hist_kernel(
    const int32_t* __restrict__ idx, int P, int E, int32_t* __restrict__ blk_counts) {
  extern __shared__ int32_t sm[];
  for (int j = threadIdx.x; j < E; j += kPermuteBlock) sm[j] = 0;
  __syncthreads();
  int p = blockIdx.x * kPermuteBlock + threadIdx.x;
  if (p < P) atomicAdd(&sm[idx[p]], 1);
  __syncthreads();
  for (int j = threadIdx.x; j < E; j += kPermuteBlock)
    blk_counts[(size_t)blockIdx.x * E + j] = sm[j];
}

// One block: for every expert, turn the per-block counts into per-block bases.  The blocks are
// cut into nseg contiguous segments and thread (segment, expert) walks its own segment, so the
// two passes over the nblk x E table take nblk / nseg dependent steps instead of nblk (96 blocks
// of 1024 pairs at 16384 tokens x 6: 39 us when one thread per expert walked them all).
__global__ __launch_bounds__(kPermuteBlock) void permute_scan_kernel(
    int E, int nblk, int T, int32_t* __restrict__ blk_counts, int32_t* counts,
    int32_t* offsets, int32_t* active, int32_t* n_active, int32_t* shared_offsets, TileOut to) {
  extern __shared__ int32_t sm[];  // [E] totals, [E+1] offsets, [nseg][E] segment sums
  int32_t* sTot = sm;
  int32_t* sOff = sm + E;
  int32_t* sSeg = sOff + E + 1;
  int nseg = kPermuteBlock / E;
  if (nseg > nblk) nseg = nblk;
  if (nseg < 1) nseg = 1;
  const int bps = (nblk + nseg - 1) / nseg;  // blocks per segment
  const int tid = threadIdx.x;
  const int seg = tid / E, e = tid - seg * E;
  const bool on = seg < nseg;
  const int b_lo = seg * bps, b_hi = min(nblk, b_lo + bps);
  if (on) {
    int run = 0;
    for (int b = b_lo; b < b_hi; ++b) run += blk_counts[(size_t)b * E + e];
    sSeg[seg * E + e] = run;
  }
  __syncthreads();
  if (tid < E) {  // totals; the segment sums become exclusive prefixes over the segments
    int run = 0;
    for (int sg = 0; sg < nseg; ++sg) {
      const int c = sSeg[sg * E + tid];
      sSeg[sg * E + tid] = run;
      run += c;
    }
    sTot[tid] = run;
    counts[tid] = run;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int run = 0;
    for (int ee = 0; ee < E; ++ee) {
      sOff[ee] = run;
      run += sTot[ee];
    }
    sOff[E] = run;
  }
  __syncthreads();
  finish_offsets(E, sTot, offsets, active, n_active, shared_offsets, T, to);
  if (on) {
    int run = sOff[e] + sSeg[seg * E + e];
    for (int b = b_lo; b < b_hi; ++b) {
      const int c = blk_counts[(size_t)b * E + e];
      blk_counts[(size_t)b * E + e] = run;  // becomes the block's base for expert e
      run += c;
    }
  }
}

__global__ __launch_bounds__(kPermuteBlock) void permute_scatter_kernel(
    const int32_t* __restrict__ idx, int P, int E, const int32_t* __restrict__ blk_base,
    int32_t* __restrict__ perm, int32_t* __restrict__ inv) {
  extern __shared__ int32_t sm[];
  int32_t* sWaveCnt = sm;
  int32_t* sBlkCnt = sm + kWaves * E;
  const int p = blockIdx.x * kPermuteBlock + threadIdx.x;
  const bool valid = p < P;
  const int e = valid ? idx[p] : 0;
  int rank = block_stable_rank(e, valid, E, sWaveCnt, sBlkCnt);
  if (valid) {
    int pos = blk_base[(size_t)blockIdx.x * E + e] + rank;
    perm[pos] = p;
    inv[p] = pos;
  }
}

__global__ void fill_i32_kernel(int32_t* p, int n, int32_t v, int32_t step) {
  int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = v + step * i;
}

}  // namespace

hipError_t launch_permute(const PermuteArgs& a, hipStream_t s, int* n_launches) {
  const int P = a.T * a.k, E = a.E;
  if (P <= 0) return hipErrorInvalidValue;
  TileOut to{a.tile_group, a.tile_m0, a.n_tiles, a.shared_n_tiles, a.tile_rows, a.tile_li,
             a.max_tile_groups > 0 ? a.max_tile_groups : 8};
  if (P <= kPermuteBlock) {
    size_t sm = ((size_t)kWaves * E + E + E + 1) * sizeof(int32_t);
    permute_single_kernel<<<1, kPermuteBlock, sm, s>>>(a.idx, P, E, a.T, a.counts, a.offsets,
                                                       a.perm, a.inv, a.active, a.n_active,
                                                       a.shared_offsets, to);
    if (n_launches) *n_launches = 1;
    return hipGetLastError();
  }
  const int nblk = (P + kPermuteBlock - 1) / kPermuteBlock;
  if (nblk <= kMultiBlocks) {
    size_t sm = ((size_t)kWaves * E + 4 * (size_t)E + 1) * sizeof(int32_t);
    permute_multi_kernel<<<nblk, kPermuteBlock, sm, s>>>(a.idx, P, E, a.T, a.counts, a.offsets,
                                                         a.perm, a.inv, a.active, a.n_active,
                                                         a.shared_offsets, to);
    if (n_launches) *n_launches = 1;
    return hipGetLastError();
  }
  permute_hist_kernel<<<nblk, kPermuteBlock, (size_t)E * sizeof(int32_t), s>>>(a.idx, P, E,
                                                                                 a.blk_counts);
  const int nseg = std::max(1, std::min(nblk, kPermuteBlock / E));
  permute_scan_kernel<<<1, kPermuteBlock, ((size_t)2 * E + 1 + (size_t)nseg * E) * sizeof(int32_t), s>>>(
      E, nblk, a.T, a.blk_counts, a.counts, a.offsets, a.active, a.n_active, a.shared_offsets,
      to);
  permute_scatter_kernel<<<nblk, kPermuteBlock, ((size_t)kWaves * E + E) * sizeof(int32_t), s>>>(
      a.idx, P, E, a.blk_counts, a.perm, a.inv);
  if (n_launches) *n_launches = 3;
  return hipGetLastError();
}

hipError_t launch_fill_i32(int32_t* p, int n, int32_t v, int32_t step, hipStream_t s) {
  if (n <= 0) return hipSuccess;
  fill_i32_kernel<<<(n + 255) / 256, 256, 0, s>>>(p, n, v, step);
  return hipGetLastError();
}

}  // namespace atenia_moe
