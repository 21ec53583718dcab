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

// four consecutive expert-output values: f32 (streaming load) or bf16 widened to f32
template <bool BF16>
__device__ inline void load4(const void* base, size_t elem, bool once, float (&v)[4]) {
  if (BF16) {
    const uint2 q = *(const uint2*)((const uint16_t*)base + elem);
    v[0] = __uint_as_float(q.x << 16); v[1] = __uint_as_float(q.x & 0xffff0000u);
    v[2] = __uint_as_float(q.y << 16); v[3] = __uint_as_float(q.y & 0xffff0000u);
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

template <bool YB, bool SB>
__global__ __launch_bounds__(256) void combine_kernel(int T, int k, int d,
                                                      const float* __restrict__ w,
                                                      const void* __restrict__ y, int y_stride,
                                                      const uint8_t* __restrict__ part_flags,
                                                      int flag_cols, size_t y_part_stride,
                                                      const void* __restrict__ y_shared,
                                                      const float* __restrict__ sgate,
                                                      const float* residual, float* out) {
  const int chunks = (d + 1023) / 1024;
  const int t = blockIdx.x / chunks;
  const int c = ((blockIdx.x - t * chunks) * 256 + threadIdx.x) * 4;
  if (c >= d) return;
  const bool vec = (c + 3 < d) && ((y_stride & 3) == 0) && ((d & 3) == 0);
  float o[4] = {0.f, 0.f, 0.f, 0.f};
  for (int slot = 0; slot < k; ++slot) {
    const float ws = w[(size_t)t * k + slot];
    const size_t yr = ((size_t)t * k + slot) * y_stride + c;
    const int y_parts = part_flags ? part_flags[((size_t)t * k + slot) * flag_cols + c / 256] : 1;
    float v[4] = {0.f, 0.f, 0.f, 0.f};
    if (vec) {
      load4<YB>(y, yr, true, v);
      for (int part = 1; part < y_parts; ++part) {
        float q[4];
        load4<YB>(y, yr + part * y_part_stride, false, q);
        v[0] = __fadd_rn(v[0], q[0]); v[1] = __fadd_rn(v[1], q[1]);
        v[2] = __fadd_rn(v[2], q[2]); v[3] = __fadd_rn(v[3], q[3]);
      }
    } else {
      for (int j = 0; j < 4 && c + j < d; ++j) {
        v[j] = load1<YB>(y, yr + j);
        for (int part = 1; part < y_parts; ++part)
          v[j] = __fadd_rn(v[j], load1<YB>(y, yr + part * y_part_stride + j));
      }
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) o[j] = __fadd_rn(o[j], __fmul_rn(ws, v[j]));
  }
  if (y_shared) {
    const float sc = sgate ? sgate[t] : 1.0f;
    const size_t yr = (size_t)t * y_stride + c;
    float v[4] = {0.f, 0.f, 0.f, 0.f};
    if (vec) {
      load4<SB>(y_shared, yr, true, v);
    } else {
      for (int j = 0; j < 4 && c + j < d; ++j) v[j] = load1<SB>(y_shared, yr + j);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) o[j] = __fadd_rn(o[j], __fmul_rn(sc, v[j]));
  }
  if (residual) {  // may alias `out`: each element is read and written by this thread only
    const float* rr = residual + (size_t)t * d + c;
    if (vec) {
      const float4 q = *(const float4*)rr;
      o[0] = __fadd_rn(q.x, o[0]); o[1] = __fadd_rn(q.y, o[1]);
      o[2] = __fadd_rn(q.z, o[2]); o[3] = __fadd_rn(q.w, o[3]);
    } else {
      for (int j = 0; j < 4 && c + j < d; ++j) o[j] = __fadd_rn(rr[j], o[j]);
    }
  }
  float* orow = out + (size_t)t * d + c;
  if (vec) {
    *(float4*)orow = make_float4(o[0], o[1], o[2], o[3]);
  } else {
    for (int j = 0; j < 4 && c + j < d; ++j) orow[j] = o[j];
  }
}

}  // namespace

hipError_t launch_combine(const CombineArgs& a, hipStream_t s) {
  const unsigned grid = (unsigned)((a.d + 1023) / 1024) * (unsigned)a.T;
#define ATENIA_COMBINE(YB, SB)                                                                      \
  combine_kernel<YB, SB><<<grid, 256, 0, s>>>(a.T, a.k, a.d, a.w, a.y, a.y_stride, a.part_flags,    \
                                              a.flag_cols, a.y_part_stride, a.y_shared, a.sgate,    \
                                              a.residual, a.out)
  if (a.y_bf16 && a.ys_bf16) ATENIA_COMBINE(true, true);
  else if (a.y_bf16) ATENIA_COMBINE(true, false);
  else if (a.ys_bf16) ATENIA_COMBINE(false, true);
  else ATENIA_COMBINE(false, false);
#undef ATENIA_COMBINE
  return hipGetLastError();
}

}  // namespace atenia_moe
