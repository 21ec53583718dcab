// Kernel 4: weighted combine back to token order.
//
// out[t] = sum over the token's slots (ascending expert id) of w[t,slot] * y[t,slot], then
// += scale[t] * y_shared[t]      (src/moe/sparse.rs:226-233, src/moe/layer.rs:415-429), and,
// for the decoder layer's FFN block, out[t] = residual[t] + that (src/moe/full_forward.rs:251).
// The reference multiplies and adds in f32 with two roundings and a fixed order; the same
// sequence is kept here (no fused multiply-add, no atomics), so given equal expert outputs
// the combine is bit-identical.  Expert outputs are stored by pair id t*k+slot, so a token's
// k rows are adjacent and every read and write is a coalesced float4.  When the down phase
// split the k range of some tiles, an expert output there is the f32 sum of its partial
// buffers, added in buffer order.  The bf16 tiled down kernels may leave the expert outputs as
// bf16 (half the bytes both ways); they are widened here, exactly, before the same arithmetic.
#include "moe_internal.h"

// This file is compiled with -ffp-contract=off (see the Makefile): the reference rounds every
// product and every sum on its own, and hipcc would otherwise fuse `a * b + c` into one FMA
// (its default is -ffp-contract=fast, under which __fmul_rn / __fadd_rn are plain `*` and `+`
// and the fp-contract pragma is ignored).

namespace atenia_moe {

namespace {

// Expert outputs are read exactly once: a streaming (non-temporal) load leaves the caches to the
// kernels around this one.
typedef float f32x4_t __attribute__((ext_vector_type(4)));
__device__ inline float4 load_once(const float* p) {
  const f32x4_t v = __builtin_nontemporal_load((const f32x4_t*)p);
  return make_float4(v.x, v.y, v.z, v.w);
}

// CPT consecutive expert-output values: f32 (CPT = 4, streaming load) or bf16 widened to f32
// (CPT = 4 or 8: 8 or 16 bytes per lane)
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
template <bool BF16, int CPT>
__device__ inline void load_vec(const void* base, size_t elem, bool once, float (&v)[CPT]) {
  if (BF16) {
    uint32_t q[CPT / 2];
    const uint16_t* p = (const uint16_t*)base + elem;
    if (CPT == 8) {
      const u32x4_t t = once ? __builtin_nontemporal_load((const u32x4_t*)p) : *(const u32x4_t*)p;
      q[0] = t.x; q[1] = t.y; q[CPT / 2 - 2] = t.z; q[CPT / 2 - 1] = t.w;
    } else {
      const u32x2_t t = once ? __builtin_nontemporal_load((const u32x2_t*)p) : *(const u32x2_t*)p;
      q[0] = t.x; q[1] = t.y;
    }
#pragma unroll
    for (int j = 0; j < CPT / 2; ++j) {
      v[2 * j] = __uint_as_float(q[j] << 16);
      v[2 * j + 1] = __uint_as_float(q[j] & 0xffff0000u);
    }
  } else {
    const float* p = (const float*)base + elem;
    const float4 q = once ? load_once(p) : *(const float4*)p;
    v[0] = q.x; v[1] = q.y; v[2] = q.z; v[3] = q.w;
  }
}
template <bool BF16>
__device__ inline float load1(const void* base, size_t elem) {
  if (BF16) return __uint_as_float((uint32_t)((const uint16_t*)base)[elem] << 16);
  return ((const float*)base)[elem];
}

// CPT: columns per thread (8 only when both y and y_shared -- if any -- are bf16 and d % 8 == 0).
template <bool YB, bool SB, int CPT>
__global__ __launch_bounds__(256) void combine_kernel(int T, int k, int d,
                                                      const float* __restrict__ w,
                                                      const void* __restrict__ y, int y_stride,
                                                      const uint8_t* __restrict__ part_flags,
                                                      int flag_cols, size_t y_part_stride,
                                                      const void* __restrict__ y_shared,
                                                      const float* __restrict__ sgate,
                                                      const float* residual, float* out) {
  constexpr int PER_BLOCK = 256 * CPT;
  const int chunks = (d + PER_BLOCK - 1) / PER_BLOCK;
  const int t = blockIdx.x / chunks;
  const int c = ((blockIdx.x - t * chunks) * 256 + threadIdx.x) * CPT;
  if (c >= d) return;
  const bool vec = (c + CPT - 1 < d) && ((y_stride & (CPT - 1)) == 0) && ((d & (CPT - 1)) == 0);
  float o[CPT];
#pragma unroll
  for (int j = 0; j < CPT; ++j) o[j] = 0.f;
  for (int slot = 0; slot < k; ++slot) {
    const float ws = w[(size_t)t * k + slot];
    const size_t yr = ((size_t)t * k + slot) * y_stride + c;
    const int y_parts = part_flags ? part_flags[((size_t)t * k + slot) * flag_cols + c / 256] : 1;
    float v[CPT];
#pragma unroll
    for (int j = 0; j < CPT; ++j) v[j] = 0.f;
    if (vec) {
      load_vec<YB, CPT>(y, yr, true, v);
      for (int part = 1; part < y_parts; ++part) {
        float q[CPT];
        load_vec<YB, CPT>(y, yr + part * y_part_stride, false, q);
#pragma unroll
        for (int j = 0; j < CPT; ++j) v[j] = __fadd_rn(v[j], q[j]);
      }
    } else {
      for (int j = 0; j < CPT && c + j < d; ++j) {
        v[j] = load1<YB>(y, yr + j);
        for (int part = 1; part < y_parts; ++part)
          v[j] = __fadd_rn(v[j], load1<YB>(y, yr + part * y_part_stride + j));
      }
    }
#pragma unroll
    for (int j = 0; j < CPT; ++j) o[j] = __fadd_rn(o[j], __fmul_rn(ws, v[j]));
  }
  if (y_shared) {
    const float sc = sgate ? sgate[t] : 1.0f;
    const size_t yr = (size_t)t * y_stride + c;
    float v[CPT];
#pragma unroll
    for (int j = 0; j < CPT; ++j) v[j] = 0.f;
    if (vec) {
      load_vec<SB, CPT>(y_shared, yr, true, v);
    } else {
      for (int j = 0; j < CPT && c + j < d; ++j) v[j] = load1<SB>(y_shared, yr + j);
    }
#pragma unroll
    for (int j = 0; j < CPT; ++j) o[j] = __fadd_rn(o[j], __fmul_rn(sc, v[j]));
  }
  if (residual) {  // may alias `out`: each element is read and written by this thread only
    const float* rr = residual + (size_t)t * d + c;
    if (vec) {
#pragma unroll
      for (int j4 = 0; j4 < CPT; j4 += 4) {
        const float4 q = *(const float4*)(rr + j4);
        o[j4] = __fadd_rn(q.x, o[j4]); o[j4 + 1] = __fadd_rn(q.y, o[j4 + 1]);
        o[j4 + 2] = __fadd_rn(q.z, o[j4 + 2]); o[j4 + 3] = __fadd_rn(q.w, o[j4 + 3]);
      }
    } else {
      for (int j = 0; j < CPT && c + j < d; ++j) o[j] = __fadd_rn(rr[j], o[j]);
    }
  }
  float* orow = out + (size_t)t * d + c;
  if (vec) {
#pragma unroll
    for (int j4 = 0; j4 < CPT; j4 += 4)
      *(float4*)(orow + j4) = make_float4(o[j4], o[j4 + 1], o[j4 + 2], o[j4 + 3]);
  } else {
    for (int j = 0; j < CPT && c + j < d; ++j) orow[j] = o[j];
  }
}

}  // namespace

hipError_t launch_combine(const CombineArgs& a, hipStream_t s) {
  // bf16 expert outputs: 8 columns (16 bytes of each row) per thread
  const bool wide = a.y_bf16 && (!a.y_shared || a.ys_bf16) && a.d % 8 == 0 && a.y_stride % 8 == 0;
  const int per_block = 256 * (wide ? 8 : 4);
  const unsigned grid = (unsigned)((a.d + per_block - 1) / per_block) * (unsigned)a.T;
#define ATENIA_COMBINE(YB, SB, CPT)                                                                 \
  combine_kernel<YB, SB, CPT><<<grid, 256, 0, s>>>(a.T, a.k, a.d, a.w, a.y, a.y_stride,             \
                                                   a.part_flags, a.flag_cols, a.y_part_stride,      \
                                                   a.y_shared, a.sgate, a.residual, a.out)
  if (wide) ATENIA_COMBINE(true, true, 8);
  else if (a.y_bf16 && a.ys_bf16) ATENIA_COMBINE(true, true, 4);
  else if (a.y_bf16) ATENIA_COMBINE(true, false, 4);
  else if (a.ys_bf16) ATENIA_COMBINE(false, true, 4);
  else ATENIA_COMBINE(false, false, 4);
#undef ATENIA_COMBINE
  return hipGetLastError();
}

}  // namespace atenia_moe
