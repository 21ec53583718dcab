// INT8 -> BF16 dequantisation of a row-major [K, N] weight on the device: the two launchers of
// the reference's W8A16 path (src/cuda/int8_to_bf16.cu:24-71 per channel, :91-141 per group),
// under the symbol names and with the argument lists its FFI block binds
// (src/cuda/int8_to_bf16.rs:63-81), plus stream-taking forms.
//
//   per channel : out[k, n] = trunc_bf16((float)q[k, n] * scales[n])
//   per group   : out[k, n] = trunc_bf16((float)q[k, n] * scales[(k / group_size) * N + n])
//
// One f32 multiply and a 16-bit truncation per element, so results are bit-identical to the
// reference kernel.  The bound is HBM: 1 byte read and 2 bytes written per element.  A thread
// converts 8 consecutive elements of a row (one 8-byte load, one 16-byte store), so a wavefront
// reads 512 and writes 1024 contiguous bytes per step, in four rows at a time to keep several
// loads in flight.  Shapes whose rows are not multiples of 8 elements, or unaligned pointers,
// take a one-element-per-thread kernel with the same arithmetic.
#include <hip/hip_runtime.h>

#include <cstdint>
#include <type_traits>

#include "../../include/atenia_moe_hip.h"

namespace {

constexpr int kThreads = 256;
constexpr int kSteps = 4;  // rows per thread

typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

__device__ inline uint32_t bf16_trunc_pair(float a, float b) {
  return (__float_as_uint(a) >> 16) | (__float_as_uint(b) & 0xffff0000u);
}

// Chunks of 8 elements (N % 8 == 0, so a chunk never crosses a row).  The workgroup is a
// TX x (256 / TX) patch of (column chunk, row) positions and walks kSteps such patches down the
// rows: a thread keeps its column, so the scales of a per-channel weight are loaded once per
// thread and those of a per-group weight once per group it crosses -- no index division per
// element.  group_size == 0: per channel.
template <int TX>
__global__ __launch_bounds__(kThreads) void int8_to_bf16_vec_kernel(
    const uint2* __restrict__ q, const float* __restrict__ scales, uint4* __restrict__ out, int K,
    int N, int group_size) {
  constexpr int TY = kThreads / TX;
  const int chunks_per_row = N >> 3;
  const int cx = blockIdx.x * TX + (threadIdx.x % TX);
  const int r0 = blockIdx.y * (TY * kSteps) + threadIdx.x / TX;
  if (cx >= chunks_per_row) return;
  uint2 v[kSteps];
#pragma unroll
  for (int s = 0; s < kSteps; ++s) {
    const int r = r0 + s * TY;
    v[s] = make_uint2(0u, 0u);
    if (r < K) {  // read once: streaming load
      const u32x2 t = __builtin_nontemporal_load((const u32x2*)(q + (size_t)r * chunks_per_row + cx));
      v[s] = make_uint2(t.x, t.y);
    }
  }
  const float* sp = scales + cx * 8;
  int g_loaded = -1;
  float4 s0 = make_float4(0.f, 0.f, 0.f, 0.f), s1 = s0;
#pragma unroll
  for (int s = 0; s < kSteps; ++s) {
    const int r = r0 + s * TY;
    if (r >= K) continue;
    const int g = group_size > 0 ? r / group_size : 0;
    if (g != g_loaded) {
      s0 = *(const float4*)(sp + (size_t)g * N);
      s1 = *(const float4*)(sp + (size_t)g * N + 4);
      g_loaded = g;
    }
    const uint32_t lo = v[s].x, hi = v[s].y;
    uint4 o;
    o.x = bf16_trunc_pair((float)(int8_t)(lo & 0xff) * s0.x, (float)(int8_t)((lo >> 8) & 0xff) * s0.y);
    o.y = bf16_trunc_pair((float)(int8_t)((lo >> 16) & 0xff) * s0.z, (float)(int8_t)(lo >> 24) * s0.w);
    o.z = bf16_trunc_pair((float)(int8_t)(hi & 0xff) * s1.x, (float)(int8_t)((hi >> 8) & 0xff) * s1.y);
    o.w = bf16_trunc_pair((float)(int8_t)((hi >> 16) & 0xff) * s1.z, (float)(int8_t)(hi >> 24) * s1.w);
    // written once and not read again by this kernel: streaming store
    __builtin_nontemporal_store(u32x4{o.x, o.y, o.z, o.w},
                                (u32x4*)(out + (size_t)r * chunks_per_row + cx));
  }
}

__global__ __launch_bounds__(kThreads) void int8_to_bf16_elem_kernel(
    const int8_t* __restrict__ q, const float* __restrict__ scales, uint16_t* __restrict__ out,
    long long total, int N, int group_size) {
  const long long stride = (long long)gridDim.x * kThreads;
  for (long long i = (long long)blockIdx.x * kThreads + threadIdx.x; i < total; i += stride) {
    const long long row = i / N;
    const int col = (int)(i - row * N);
    const float s = scales[(group_size > 0 ? (row / group_size) * N : 0) + col];
    out[i] = (uint16_t)(__float_as_uint((float)q[i] * s) >> 16);
  }
}

int launch(const void* d_int8, const float* d_scales, void* d_bf16, int k, int n, int group_size,
           hipStream_t stream) {
  const long long total = (long long)k * (long long)n;
  const bool aligned = (((uintptr_t)d_int8 | (uintptr_t)d_bf16 | (uintptr_t)d_scales) & 15) == 0;
  // the vector kernel puts row blocks on grid.y (at most 65535 of them)
  if (n % 8 == 0 && aligned && (long long)k <= 65535LL * kSteps) {
    const int cpr = n / 8;
    auto go = [&](auto tx_c) {
      constexpr int TX = decltype(tx_c)::value;
      const long long rows_per_block = (long long)(kThreads / TX) * kSteps;
      const long long by = (k + rows_per_block - 1) / rows_per_block;
      dim3 grid((cpr + TX - 1) / TX, (unsigned)by);
      int8_to_bf16_vec_kernel<TX><<<grid, kThreads, 0, stream>>>(
          (const uint2*)d_int8, d_scales, (uint4*)d_bf16, k, n, group_size);
    };
    if (cpr >= 256) go(std::integral_constant<int, 256>{});
    else if (cpr >= 64) go(std::integral_constant<int, 64>{});
    else if (cpr >= 16) go(std::integral_constant<int, 16>{});
    else go(std::integral_constant<int, 4>{});
  } else {
    long long blocks = (total + kThreads - 1) / kThreads;
    if (blocks > (1 << 20)) blocks = 1 << 20;  // grid-stride loop covers the rest
    int8_to_bf16_elem_kernel<<<(unsigned)blocks, kThreads, 0, stream>>>(
        (const int8_t*)d_int8, d_scales, (uint16_t*)d_bf16, total, n, group_size);
  }
  return (int)hipGetLastError();
}

}  // namespace

extern "C" {

int atenia_moe_int8_to_bf16_per_channel_launch_device(const void* d_int8, const float* d_scales,
                                                      void* d_bf16, int k, int n, void* stream) {
  if ((long long)k * (long long)n <= 0) return 0;
  if (!d_int8 || !d_scales || !d_bf16) return -1;
  return launch(d_int8, d_scales, d_bf16, k, n, 0, (hipStream_t)stream);
}

int atenia_moe_int8_to_bf16_per_group_launch_device(const void* d_int8, const float* d_scales,
                                                    void* d_bf16, int k, int n, int group_size,
                                                    void* stream) {
  if ((long long)k * (long long)n <= 0) return 0;
  if (group_size <= 0) return -2;
  if (!d_int8 || !d_scales || !d_bf16) return -1;
  return launch(d_int8, d_scales, d_bf16, k, n, group_size, (hipStream_t)stream);
}

// The reference's own symbol names and argument lists (default stream, asynchronous, return the
// runtime's launch status): a host that binds src/cuda/int8_to_bf16.rs:63-81 links unchanged.
int int8_to_bf16_per_channel_launch_device(const void* d_int8, const float* d_scales,
                                           void* d_bf16, int k, int n) {
  return atenia_moe_int8_to_bf16_per_channel_launch_device(d_int8, d_scales, d_bf16, k, n, nullptr);
}

int int8_to_bf16_per_group_launch_device(const void* d_int8, const float* d_scales, void* d_bf16,
                                         int k, int n, int group_size) {
  return atenia_moe_int8_to_bf16_per_group_launch_device(d_int8, d_scales, d_bf16, k, n, group_size,
                                                         nullptr);
}

}  // extern "C"
