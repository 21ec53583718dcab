// extern "C" surface of libatenia_moe_hip.so: layer handles, weight upload, workspace and the
// forward pipeline  router -> permute -> expert gate/up -> expert down -> combine.
//
// The handle plays the part of the reference's registry entry (src/moe/graph_op.rs:207-232):
// it owns the layer, here resident in HBM.  The reference's residency tiers
// (src/moe/residency.rs) collapse to this single tier.
#include "../../include/atenia_moe_hip.h"

#include <climits>
#include <cstdarg>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <atomic>
#include <thread>
#include <mutex>
#include <memory>
#include <new>
#include <string>
#include <vector>

#include "moe_internal.h"

using namespace atenia_moe;

// Workspace of atenia_moe_hip_layer_forward_device_noalloc: device memory the library owns from
// load time on, for callers that must not allocate.  Every GPU the library runs on holds its own
// copy of the array at its own address for the life of the process.  In host code the NAME of the
// array is only a stand-in for hipGetSymbolAddress -- it is not a device address and is never
// passed to a kernel or a runtime call; resolve_static_scratch() below keeps the real address
// per device.
constexpr size_t kStaticScratchBytes = (size_t)16 << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace {

thread_local std::string g_last_error;

int fail(int rc, const char* fmt, ...) {
  char buf[512];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof buf, fmt, ap);
  va_end(ap);
  g_last_error = buf;
  return rc;
}

int hip_rc(hipError_t e, const char* what) {
  if (e == hipSuccess) return ATENIA_MOE_OK;
  int rc = e == hipErrorOutOfMemory ? ATENIA_MOE_ERR_OOM : ATENIA_MOE_ERR_LAUNCH;
  return fail(rc, "%s: %s", what, hipGetErrorString(e));
}

#define HIP_TRY(expr)                               \
  do {                                              \
    int rc__ = hip_rc((expr), #expr);               \
    if (rc__ != ATENIA_MOE_OK) return rc__;         \
  } while (0)

// Device address of `scratch` on GPU `device`, looked up once per device with that device
// current (each GPU has its own copy of the array).  *out may be nullptr to only warm the table.
constexpr int kMaxDevices = 64;
int resolve_static_scratch(int device, unsigned char** out) {
  static std::mutex mu;
  static unsigned char* table[kMaxDevices] = {};
  if (device < 0 || device >= kMaxDevices)
    return fail(ATENIA_MOE_ERR_UNSUPPORTED, "device ordinal %d out of range", device);
  std::lock_guard<std::mutex> lock(mu);
  if (!table[device]) {
    int cur = -1;
    HIP_TRY(hipGetDevice(&cur));
    if (cur != device) HIP_TRY(hipSetDevice(device));
    void* ptr = nullptr;
    const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (cur != device) (void)hipSetDevice(cur);
    if (e != hipSuccess || !ptr)
      return fail(ATENIA_MOE_ERR_LAUNCH, "hipGetSymbolAddress(scratch) on device %d: %s", device,
                  hipGetErrorString(e));
    table[device] = (unsigned char*)ptr;
  }
  if (out) *out = table[device];
  return ATENIA_MOE_OK;
}

struct DevBuf {
  void* p = nullptr;
  size_t bytes = 0;
  ~DevBuf() { release(); }
  void release() {
    if (p) (void)hipFree(p);
    p = nullptr;
    bytes = 0;
  }
  // Grow-only; contents are zeroed on (re)allocation.
  int ensure(size_t want) {
    if (want <= bytes) return ATENIA_MOE_OK;
    release();
    HIP_TRY(hipMalloc(&p, want));
    HIP_TRY(hipMemset(p, 0, want));
    bytes = want;
    return ATENIA_MOE_OK;
  }
  template <typename T>
  T* as() const { return (T*)p; }
};

size_t elem_bytes_of(int wdtype) {
  return wdtype == ATENIA_MOE_WEIGHT_F32 ? 4 : wdtype == ATENIA_MOE_WEIGHT_BF16 ? 2 : 1;
}
int kb_of(int wdtype) { return wdtype == ATENIA_MOE_WEIGHT_INT8_W8A16 ? kKbInt8 : kKbBf16; }

}  // namespace

// Pointers into one workspace (device memory beyond the inputs and outputs of a forward).
struct WsView {
  int cap_tokens = 0;  // tokens the view was laid out for
  int y_parts = 1;     // partial output buffers of the tiled down phase it has room for
  uint16_t* xb = nullptr;
  int32_t *idx = nullptr, *counts = nullptr, *offsets = nullptr, *active = nullptr,
          *n_active = nullptr, *perm = nullptr, *inv = nullptr, *blk_counts = nullptr,
          *shared_desc = nullptr, *ident = nullptr, *tile_group = nullptr, *tile_m0 = nullptr,
          *tile_rows = nullptr, *tile_li = nullptr,
          *s_tile_group = nullptr, *s_tile_m0 = nullptr;
  float *w = nullptr, *sgate = nullptr, *y = nullptr, *ys = nullptr, *logits = nullptr;
  void *h = nullptr, *hs = nullptr;
  uint8_t* part_flags = nullptr;
};

struct AteniaMoeLayer {
  uint32_t magic = 0x4d6f4541u;
  int E = 0, k = 0, d = 0, f = 0, fs = 0, conv = 0, wdtype = 0;
  int d_kpad = 0;   // K padding of x rows (gate/up projections)
  int f_kpad = 0;   // K padding of h rows (down projection)
  int fs_kpad = 0;
  int device = 0;
  int group_size = 0;  // per-group int8: input elements per scale (0 = per-row scales)

  DevBuf w_router, router_bias, shared_gate;
  bool router_fits_bf16 = false;  // every router / gate value is exactly a bf16 value
  DevBuf router_lsb;              // [E + 1] i32: lowest last-bit exponent of each router row / the gate
  DevBuf router_t8;               // bf16 [ceil(d / 32) * 4][router_rows_pad][8]: RouterArgs::w_t8
  DevBuf router_norm2;            // f64 [router_rows_pad]: squared norms of the stacked rows
  int router_rows_pad = 0;
  DevBuf wg, wu, wd, sg, su, sd;        // routed experts
  DevBuf swg, swu, swd, ssg, ssu, ssd;  // shared expert
  WeightSet gate{}, up{}, down{}, s_gate{}, s_up{}, s_down{};
  int64_t bytes_per_expert = 0;

  // workspace (grow-only in tokens): one slab carved by ws_layout; `cur` is the view the most
  // recent forward ran on (the handle's own, or the static scratch of the no-alloc entry point)
  DevBuf slab, x_in, out, status;
  WsView ws{}, cur{};
  DevBuf xn, gamma_in;  // block forward: normalised rows [T, d] f32; gamma of the host variant
  // DeepSeek-V3 routing (off while v3_n_group == 0): the router kernels leave raw logits in
  // `logits` and v3_route_kernel decides from them
  int v3_n_group = 0, v3_topk_group = 0, v3_norm = 0;
  double v3_scale = 1.0;
  DevBuf v3_bias;
  // per-group int8: bf16 copies for the MFMA-tiled (prefill) kernels, made on first use
  DevBuf pg_wg, pg_wu, pg_wd, pg_swg, pg_swu, pg_swd;
  WeightSet gate_b{}, up_b{}, down_b{}, s_gate_b{}, s_up_b{}, s_down_b{};
  bool pg_ready = false;
  bool q_copy_off = false;  // W8A16: the copy could not be allocated once; int8 tiled kernels from then on
  int normed_T = 0;     // rows of xn the last block forward wrote
  int last_T = 0;
  int stage_T[4] = {-1, -1, -1, -1};  // token count each pipeline stage last completed for
  int nf_token = -1, nf_expert = -1;  // location of the last non-finite routing weight reported
  bool last_split = false;  // the last forward's down phase may have split tail tiles
  bool last_y_bf16 = false, last_ys_bf16 = false;  // ... and may have left y / ys as bf16

  hipStream_t stream = nullptr;
  // Host-buffer entry point, large batches: page-locked staging (two slots each way); the
  // events tell the host when the copy engine has emptied / filled a slot.
  void *pin_in = nullptr, *pin_out = nullptr;
  size_t pin_bytes = 0;  // per slot
  hipEvent_t ev_h2d[2] = {}, ev_d2h[2] = {};
  bool staging_ready = false;
  std::mutex mu;
  // Ordering of asynchronous forwards on one handle: a forward on another stream than the
  // previous one (`done_stream`) first waits for that stream's work, so two streams never use
  // the workspace at the same time (skipped while a stream is being captured into a graph).
  hipEvent_t done = nullptr;
  // a shared expert that takes launches of its own runs beside the routed experts (run_forward)
  hipStream_t side = nullptr;
  hipEvent_t ev_fork = nullptr, ev_join = nullptr;
  hipStream_t done_stream = nullptr;
  bool done_valid = false;
  bool done_recorded = false;  // `done` marks the end of the last forward on done_stream

  bool profiling = false;
  int policy = ATENIA_MOE_POLICY_CERTIFIED;  // expert arithmetic of f32 layers
  hipEvent_t ev[ATENIA_MOE_N_STAGES] = {};
  bool ev_valid = false;
  int32_t launches[ATENIA_MOE_N_STAGES] = {};
};

namespace {

// Compute units of the current device (read once per process).
constexpr int kMaxYParts = 4;  // partial output buffers of the tiled down phase

int device_cu_count() {
  static const int v = [] {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
      return 256;
    return n;
  }();
  return v;
}

// Largest batch served by the weight-streaming expert kernels when set from outside (tuning
// knob: ATENIA_MOE_STREAM_MAX_TOKENS, read once per process); 0 = the built-in rule below.
int stream_max_tokens_override() {
  static const int v = [] {
    const char* e = getenv("ATENIA_MOE_STREAM_MAX_TOKENS");
    int n = e ? atoi(e) : 0;
    return n > 0 ? n : 0;
  }();
  return v;
}
constexpr int kStreamMaxTokens = 56;
// Whether a batch of T tokens whose experts see rows_num / rows_den rows each on average
// (T * k / E) is served by the weight-streaming kernels.  Those pass over an expert's weights
// once per 32 of its rows, while the tiled kernels cost about the same from about 50 tokens to a
// few hundred, so beyond 56 tokens the choice goes by the average rows per expert.  Measured
// cross-overs on MI355X: 15-21 rows for bf16 weights (Mixtral shape T = 85, Qwen1.5-MoE shape
// T = 256, DeepSeek-V2-Lite shape T = 175), 35 for int8 with per-row or per-group scales
// (Mixtral shape T = 140; the tiled int8 kernel widens every weight in the VALU however few rows
// it multiplies, and per-group layers run the tiled kernels on a bf16 copy).
bool batch_streams(int T, long long rows_num, long long rows_den, int max_avg_rows) {
  if (const int n = stream_max_tokens_override()) return T <= n;
  if (T <= kStreamMaxTokens) return true;
  return rows_num <= rows_den * max_avg_rows;
}
// Largest batch routed by the one-workgroup-per-token router kernel (tuning knob:
// ATENIA_MOE_ROUTER_TOKEN_MAX, read once per process).
int router_token_max() {
  static const int v = [] {
    const char* e = getenv("ATENIA_MOE_ROUTER_TOKEN_MAX");
    int n = e ? atoi(e) : -1;
    return n >= 0 ? n : 512;
  }();
  return v;
}

bool valid_handle(const AteniaMoeLayer* L) { return L && L->magic == 0x4d6f4541u; }

// Uploads one projection family [G, n_rows, k_cols] (row-major per expert at
// host + g*host_stride) into `dst` and fills `ws`.
int upload_family(const void* host, size_t host_stride_elems, int G, int n_rows, int k_cols,
                  int wdtype, DevBuf& dst, WeightSet& ws, DevBuf& staging) {
  const size_t eb = elem_bytes_of(wdtype);
  ws.n_rows = n_rows;
  ws.k_cols = k_cols;
  // f32: the same 1 KiB blocks with 16 k each (a lane slot = 4 consecutive k of one row), so a
  // wave reads a strip of 16 rows in whole blocks; expert_stride stays in elements.
  const bool f32w = wdtype == ATENIA_MOE_WEIGHT_F32;
  const int KB = f32w ? kKbF32 : kb_of(wdtype);
  ws.n_pad = round_up(n_rows, 16);
  ws.k_pad = round_up(k_cols, KB);
  const int64_t expert_bytes = (int64_t)ws.n_pad * ws.k_pad * (int64_t)eb;
  ws.expert_stride = f32w ? expert_bytes / 4 : expert_bytes;  // elements (f32) or bytes
  int rc = dst.ensure((size_t)G * expert_bytes);
  if (rc) return rc;
  rc = staging.ensure((size_t)n_rows * k_cols * eb);
  if (rc) return rc;
  for (int g = 0; g < G; ++g) {
    HIP_TRY(hipMemcpy(staging.p, (const uint8_t*)host + (size_t)g * host_stride_elems * eb,
                      (size_t)n_rows * k_cols * eb, hipMemcpyHostToDevice));
    HIP_TRY(launch_repack_blocks(staging.p, (uint8_t*)dst.p + (size_t)g * expert_bytes,
                                 n_rows, k_cols, ws.n_pad, ws.k_pad, (int)eb, nullptr));
    HIP_TRY(hipDeviceSynchronize());
  }
  ws.w = dst.p;
  return ATENIA_MOE_OK;
}

int upload_f32(const float* host, size_t n, DevBuf& dst) {
  int rc = dst.ensure(n * 4);
  if (rc) return rc;
  HIP_TRY(hipMemcpy(dst.p, host, n * 4, hipMemcpyHostToDevice));
  return ATENIA_MOE_OK;
}

// Per-group scales [G, n_rows, n_kgroups] (host) -> [G][n_kgroups][n_pad] (device): for a fixed
// k group the rows are adjacent, so the 16 rows of a strip are one 64-byte read for the
// streaming kernel and a row tile is contiguous for the dequantising kernel.  Rows past n_rows
// get scale 0.
int upload_group_scales(const float* host, int G, int n_rows, int k_cols, int group_size,
                        DevBuf& dst, WeightSet& ws) {
  const int ng = (k_cols + group_size - 1) / group_size;
  const int n_pad = round_up(n_rows, 16);
  std::vector<float> re((size_t)G * n_pad * ng, 0.0f);
  for (int g = 0; g < G; ++g)
    for (int n = 0; n < n_rows; ++n)
      for (int kg = 0; kg < ng; ++kg)
        re[((size_t)g * ng + kg) * n_pad + n] = host[((size_t)g * n_rows + n) * ng + kg];
  int rc = upload_f32(re.data(), re.size(), dst);
  if (rc) return rc;
  ws.scale = dst.as<float>();
  ws.group_blocks = group_size / kKbInt8;
  ws.n_kgroups = ng;
  return ATENIA_MOE_OK;
}

// bf16 copy of an int8 family (made on the first batch that takes the MFMA-tiled kernels on it):
// same rows and K padding, bf16 blocks.  Per-group scales: value = bf16(q * scale of its group),
// no scales left.  One scale per row: value = q itself (exact in bf16), and the copy keeps the
// row scales for the kernel's epilogue.
int make_bf16_copy(const WeightSet& q, int G, DevBuf& dst, WeightSet& out) {
  const bool per_group = q.group_blocks > 0;
  out = q;
  out.scale = per_group ? nullptr : q.scale;
  out.group_blocks = 0;
  out.n_kgroups = 0;
  out.expert_stride = (int64_t)q.n_pad * q.k_pad * 2;  // bytes
  int rc = dst.ensure((size_t)G * out.expert_stride);
  if (rc) return rc;
  out.w = dst.p;
  HIP_TRY(launch_dequant_group_blocks(q.w, per_group ? q.scale : nullptr, dst.p, G, q.n_pad, q.k_pad,
                                      per_group ? q.group_blocks : 1, per_group ? q.n_kgroups : 1,
                                      nullptr));
  return ATENIA_MOE_OK;
}

// Lays a workspace for T tokens out from `base` (256-byte aligned pieces) and returns its size;
// with v == nullptr only the size is computed.  y_parts: partial output buffers of the down phase.
size_t ws_layout(const AteniaMoeLayer* L, int T, int y_parts, uint8_t* base, WsView* v) {
  const size_t P = (size_t)T * L->k;
  const bool f32w = L->wdtype == ATENIA_MOE_WEIGHT_F32;
  const size_t act = f32w ? 4 : 2;
  size_t off = 0;
  auto take = [&](size_t bytes) {
    uint8_t* p = base ? base + off : nullptr;
    off += (bytes + 255) / 256 * 256;
    return p;
  };
  WsView t{};
  t.cap_tokens = T;
  t.y_parts = y_parts;
  if (!f32w) t.xb = (uint16_t*)take((size_t)T * L->d_kpad * 2);
  t.idx = (int32_t*)take(P * 4);
  t.w = (float*)take(P * 4);
  t.sgate = (float*)take((size_t)T * 4);
  t.counts = (int32_t*)take((size_t)L->E * 4);
  t.offsets = (int32_t*)take((size_t)(L->E + 1) * 4);
  t.active = (int32_t*)take((size_t)L->E * 4);
  t.n_active = (int32_t*)take(4);
  t.perm = (int32_t*)take(P * 4);
  t.inv = (int32_t*)take(P * 4);
  t.blk_counts = (int32_t*)take(((P + kPermuteBlock - 1) / kPermuteBlock) * L->E * 4);
  // [0..1] offsets {0,T}, [2] active {0}, [3] n_active {1}, [4] routed row tiles, [5] shared row tiles
  t.shared_desc = (int32_t*)take(32);
  const size_t max_tiles = (P + kTileM - 1) / kTileM + L->E;
  t.tile_group = (int32_t*)take(max_tiles * 4);
  t.tile_m0 = (int32_t*)take(max_tiles * 4);
  t.tile_rows = (int32_t*)take(max_tiles * 4);
  t.tile_li = (int32_t*)take(max_tiles * 4);
  t.s_tile_group = (int32_t*)take(((size_t)T / kTileM + 1) * 4);
  t.s_tile_m0 = (int32_t*)take(((size_t)T / kTileM + 1) * 4);
  t.ident = (int32_t*)take((size_t)T * 4);
  t.logits = (float*)take((size_t)T * L->E * 4);
  t.h = take(P * (size_t)L->f_kpad * act);
  t.y = (float*)take((size_t)y_parts * P * L->d * 4);  // one buffer per k range of tail tiles
  t.part_flags = (uint8_t*)take(P * (size_t)((L->d + 255) / 256));
  if (L->fs > 0) {
    t.hs = take((size_t)T * L->fs_kpad * act);
    t.ys = (float*)take((size_t)T * L->d * 4);
  }
  if (v) *v = t;
  return off;
}

// What a workspace must hold before its first forward: the identity row list and the row tiles
// of the shared expert, its group descriptor, and zeros in the K padding of the h rows (the
// expert kernels multiply the padding with zero weights, which only helps if it is finite).
// A kernel, not memsets, so that the no-alloc entry point stays capturable into a graph.
__global__ void workspace_init_kernel(int32_t* ident, int T, int32_t* s_tile_group,
                                      int32_t* s_tile_m0, int n_s_tiles, int32_t* shared_desc,
                                      uint16_t* h, int h_rows, int f, int f_kpad, uint16_t* hs,
                                      int fs, int fs_kpad) {
  const int stride = gridDim.x * blockDim.x;
  const int i0 = blockIdx.x * blockDim.x + threadIdx.x;
  for (int i = i0; i < T; i += stride) ident[i] = i;
  for (int i = i0; i < n_s_tiles; i += stride) {
    s_tile_group[i] = 0;
    s_tile_m0[i] = i * kTileM;
  }
  if (i0 < 8) shared_desc[i0] = i0 == 3 ? 1 : 0;
  const int pad = f_kpad - f;
  if (h && pad > 0)
    for (long long i = i0; i < (long long)h_rows * pad; i += stride)
      h[(i / pad) * f_kpad + f + (i % pad)] = 0;
  const int spad = fs_kpad - fs;
  if (hs && spad > 0)
    for (long long i = i0; i < (long long)T * spad; i += stride)
      hs[(i / spad) * fs_kpad + fs + (i % spad)] = 0;
}

hipError_t launch_workspace_init(const AteniaMoeLayer* L, const WsView& V, int T, hipStream_t s) {
  const bool f32w = L->wdtype == ATENIA_MOE_WEIGHT_F32;  // f32 rows carry no K padding
  const long long work = (long long)T * L->k * (f32w ? 0 : L->f_kpad - L->f) + T;
  const int blocks = (int)std::min<long long>(256, (work + 255) / 256);
  workspace_init_kernel<<<blocks, 256, 0, s>>>(
      V.ident, T, V.s_tile_group, V.s_tile_m0, T / kTileM + 1, V.shared_desc,
      f32w ? nullptr : (uint16_t*)V.h, T * L->k, L->f, L->f_kpad,
      f32w ? nullptr : (uint16_t*)V.hs, L->fs, L->fs_kpad);
  return hipGetLastError();
}

int ensure_workspace(AteniaMoeLayer* L, int T) {
  if (T <= L->ws.cap_tokens) return ATENIA_MOE_OK;
  // the slab may be in use by a forward still running on some stream
  HIP_TRY(hipDeviceSynchronize());
  const size_t bytes = ws_layout(L, T, kMaxYParts, nullptr, nullptr);
  L->ws = WsView{};
  L->cur = WsView{};
  for (int st = 0; st < 4; ++st) L->stage_T[st] = -1;
  L->last_T = 0;
  int rc = L->slab.ensure(bytes);
  if (rc) return rc;
  WsView v{};
  ws_layout(L, T, kMaxYParts, (uint8_t*)L->slab.p, &v);
  if ((rc = L->x_in.ensure((size_t)T * L->d * 4))) return rc;
  if ((rc = L->out.ensure((size_t)T * L->d * 4))) return rc;
  HIP_TRY(launch_workspace_init(L, v, T, nullptr));
  HIP_TRY(hipDeviceSynchronize());
  L->ws = v;
  return ATENIA_MOE_OK;
}

struct StageTimer {
  AteniaMoeLayer* L;
  hipStream_t s;
  int next = 0;
  void mark() {
    if (L->profiling && next < ATENIA_MOE_N_STAGES) (void)hipEventRecord(L->ev[next], s);
    ++next;
  }
};

// Pipeline stages for run_forward's [first, last] range.
enum { kStageRouter = 0, kStagePermute = 1, kStageFfn = 2, kStageCombine = 3 };

// Runs stages first..last of the pipeline on `s`.  A stage reads what the stages before it
// left in the handle's workspace, so a range that does not start at the router is only valid
// after the earlier stages ran for the same n_tokens (checked) on the same activations.
// Per-group int8: the bf16 copy of the experts that batches for the MFMA-tiled kernels run on.
// Made at `create` when max_tokens_hint announces such batches, else by the first such batch.
int ensure_pg_copy(AteniaMoeLayer* L) {
  if (L->pg_ready) return ATENIA_MOE_OK;
  if (L->group_size == 0) {
    // W8A16: the copy is optional; a cap on its size keeps a layer on the int8 kernels (tuning
    // knob ATENIA_MOE_INT8_COPY_MAX_MB, read once; unset = no cap).
    static const long long cap_mb = [] {
      const char* e = getenv("ATENIA_MOE_INT8_COPY_MAX_MB");
      return e ? atoll(e) : -1ll;
    }();
    auto bytes_of = [](const WeightSet& w, int G) { return (long long)G * w.n_pad * w.k_pad * 2; };
    long long need = bytes_of(L->gate, L->E) + bytes_of(L->up, L->E) + bytes_of(L->down, L->E);
    if (L->fs > 0) need += bytes_of(L->s_gate, 1) + bytes_of(L->s_up, 1) + bytes_of(L->s_down, 1);
    if (cap_mb >= 0 && need > (cap_mb << 20))
      return fail(ATENIA_MOE_ERR_UNSUPPORTED, "bf16 copy of %lld bytes is over the cap of %lld MiB",
                  need, cap_mb);
  }
  int rc = make_bf16_copy(L->gate, L->E, L->pg_wg, L->gate_b);
  if (!rc) rc = make_bf16_copy(L->up, L->E, L->pg_wu, L->up_b);
  if (!rc) rc = make_bf16_copy(L->down, L->E, L->pg_wd, L->down_b);
  if (!rc && L->fs > 0) {
    rc = make_bf16_copy(L->s_gate, 1, L->pg_swg, L->s_gate_b);
    if (!rc) rc = make_bf16_copy(L->s_up, 1, L->pg_swu, L->s_up_b);
    if (!rc) rc = make_bf16_copy(L->s_down, 1, L->pg_swd, L->s_down_b);
  }
  if (rc) return rc;
  HIP_TRY(hipDeviceSynchronize());
  L->pg_ready = true;
  return ATENIA_MOE_OK;
}
void release_pg_copy(AteniaMoeLayer* L) {
  for (DevBuf* b : {&L->pg_wg, &L->pg_wu, &L->pg_wd, &L->pg_swg, &L->pg_swu, &L->pg_swd}) b->release();
  L->gate_b = L->up_b = L->down_b = L->s_gate_b = L->s_up_b = L->s_down_b = WeightSet{};
  L->pg_ready = false;
}

// Which expert kernels a batch of T tokens takes (a pure function of the layer and T).
enum { kFamStream = 0, kFamMid = 1, kFamTiled = 2 };
struct BatchPlan {
  int up, down;         // kernel family of the gate/up phase and of the down phase (kFam*)
  bool routed_streams;  // gate/up phase: weight-streaming kernels (either form), not the tiled ones
  bool routed_mid;      // gate/up phase in the mid-batch form (token rows shared through LDS)
  bool pg_prefill;      // per-group int8 layer running the tiled kernels on its bf16 copy
  bool q_copy;          // W8A16 layer running the bf16 tiled kernels on a bf16 copy of its int8
                        // values (exact), row scales applied to the f32 results
  bool tall_tiles;      // row tiles of up to nine 32-row groups (bf16 pipelined kernels only)
  bool duo_up, duo_down;  // tiled phase on the two-workgroups-per-compute-unit form (short K)
};
// Longest K (padded) for which a tiled bf16 phase takes the form with two workgroups per compute
// unit (tuning knob ATENIA_MOE_DUO_MAX_K, read once; 0 switches the form off).
int duo_max_k() {
  static const int v = [] {
    const char* e = getenv("ATENIA_MOE_DUO_MAX_K");
    return e ? atoi(e) : 0;
  }();
  return v;
}
// Rows per expert on average from which a W8A16 layer's tiled phases run on the bf16 copy of its
// int8 values (tuning knob ATENIA_MOE_INT8_COPY_MIN_ROWS, read once; 0 = never, no copy is made).
int int8_copy_min_rows() {
  static const int v = [] {
    const char* e = getenv("ATENIA_MOE_INT8_COPY_MIN_ROWS");
    return e ? atoi(e) : 256;
  }();
  return v;
}
// Tiles of uneven height can be switched off (tuning knob ATENIA_MOE_TALL_TILES=0, read once).
bool tall_tiles_enabled() {
  static const bool v = [] {
    const char* e = getenv("ATENIA_MOE_TALL_TILES");
    return !(e && atoi(e) == 0);
  }();
  return v;
}
// Batch sizes served by the mid-batch streaming kernel (routed experts, and the shared one in
// the same launches): from `min_tokens` tokens and `lo` rows per expert on average (T k / E) up
// to `hi` rows.  Measured cross-overs on MI355X, whole forward, mid-batch kernel / the other one:
//  * against the register-resident streaming kernel, without a shared expert: bf16 at 14-16 rows
//    (Mixtral shape T = 48 0.476 / 0.465 ms, T = 64 0.481 / 0.487, T = 96 0.491 / 0.529), int8 at
//    8-10 rows (T = 32 0.281 / 0.274, T = 40 0.258 / 0.267, T = 56 0.262 / 0.287);
//  * with a shared expert that the kernel takes along, whose T rows cost the streaming kernel
//    a pass per 32 tokens: from 40 tokens whatever the routed experts see (DeepSeek-V2-Lite
//    shape T = 24 0.133 / 0.132, T = 40 0.147 / 0.157, T = 64 0.168 / 0.198, T = 128
//    0.206 / 0.281; Qwen1.5-MoE shape T = 24 0.200 / 0.203, T = 40 0.230 / 0.247, T = 56
//    0.240 / 0.259, T = 128 0.268 / 0.302; below 40 tokens the gate/up phase of the
//    register-resident kernel is the faster one, Qwen T = 32 108 against 117 us);
//  * against the tiled kernels at 52-72 rows for bf16 (Mixtral T = 192 0.522 / 0.540, T = 224
//    equal; Qwen T = 1024 0.468 / 0.479, T = 1536 0.555 / 0.541; DeepSeek T = 640 0.415 / 0.437,
//    T = 768 equal) and at about 110 rows for int8, whose tiled kernel widens every weight in the
//    VALU (Mixtral int8 T = 192 0.346 / 0.526, T = 320 0.467 / 0.535, T = 448 0.562 / 0.572).
// Tuning knobs ATENIA_MOE_MID_MIN_TOKENS / ATENIA_MOE_MID_MIN_AVG / ATENIA_MOE_MID_MAX_AVG (read
// once) replace the three bounds; a maximum of 0 switches the kernel off.
struct MidBounds {
  int min_tokens, max_tokens;  // gate/up phase: batch sizes
  double lo, hi;               // gate/up phase: rows per expert on average
  int down_min_tokens;         // down phase: from this batch size ...
  double down_hi;              // ... up to this many rows per expert on average
};
MidBounds mid_bounds(const AteniaMoeLayer* L) {
  static const double env_lo = [] {
    const char* e = getenv("ATENIA_MOE_MID_MIN_AVG");
    return e ? atof(e) : -1.0;
  }();
  static const double env_hi = [] {
    const char* e = getenv("ATENIA_MOE_MID_MAX_AVG");
    return e ? atof(e) : -1.0;
  }();
  static const int env_min_tokens = [] {
    const char* e = getenv("ATENIA_MOE_MID_MIN_TOKENS");
    return e ? atoi(e) : 0;
  }();
  const bool int8w = L->wdtype == ATENIA_MOE_WEIGHT_INT8_W8A16;
  // a shared expert that the mid-batch kernel can take along
  const bool rides = L->fs > 0 && ffn_mid_supported(L->s_gate, L->wdtype) &&
                     ffn_mid_supported(L->s_up, L->wdtype) && ffn_mid_supported(L->s_down, L->wdtype);
  MidBounds b;
  b.min_tokens = rides || int8w ? 40 : kStreamMaxTokens + 1;
  b.max_tokens = INT_MAX;
  b.lo = rides ? 0.0 : int8w ? 10.0 : 14.0;
  b.hi = int8w ? 104.0 : rides ? 68.0 : 52.0;
  // The down phase alone gains from the mid-batch form from 20 tokens on when its K is long: it
  // has d / 16 strips only, which that form spreads over d / 128 workgroups of eight waves that
  // each own a strip over the whole K (no reduction through LDS).  Down launch, mid-batch /
  // register-resident: Mixtral int8 T = 24 79 / 83 us, T = 48 80 / 97; Mixtral bf16 T = 24
  // 142 / 144, T = 56 145 / 157.
  b.down_min_tokens = 20;
  b.down_hi = b.hi;
  // Narrow experts (a down strip of fewer than 64 blocks, which the register-resident launch
  // cuts into four K slices): that launch is the better one for longer, and the mid-batch form
  // then stays ahead of the tiled kernels for longer, phase by phase (us, DeepSeek-V2-Lite /
  // Qwen1.5-MoE shapes, stream | mid | tiled):
  //   gate/up  T = 32 64 | 67, 110 | 117;  T = 48 77 | 74, 125 | 123;  T = 128 137 | 106 | 136,
  //            158 | 132 | 175;  T = 512 181 | 186 (mid | tiled), 178 | 184;  T = 640 202 | 187,
  //            186 | 183;  T = 768 223 | 195, 196 | 186
  //   down     T = 32 35 | 43, 56 | 72;  T = 48 48 | 47, 77 | 80;  T = 64 57 | 52, 78 | 84;
  //            T = 128 84 | 65, 85 | 101;  T = 256 132 | 90, 122 | 122;  T = 384 179 | 109 | 154,
  //            159 | 132 | 188;  T = 1024 168 | 181 (mid | tiled), 156 | 199;  T = 1536 224 | 198,
  //            186 | 206;  T = 2048 278 | 220, 272 | 215
  // (the Qwen shape's shared expert is 4x as wide as a routed one and keeps a down launch of its
  // own beside the register-resident kernel, which is why that kernel holds out to 256 tokens.)
  const int kb = int8w ? kKbInt8 : kKbBf16;
  if (L->down.k_pad / kb < 64 && L->group_size == 0) {
    const bool wide_shared = L->fs > 0 && L->s_down.k_pad > 2 * L->down.k_pad;
    if (rides) {
      b.min_tokens = 48;
      b.max_tokens = 640;
      b.hi = 52.0;
    }
    b.down_min_tokens = wide_shared ? 256 : 56;
    // (with the shared expert's row blocks first in the mid-batch grid, whole forward in us,
    // default | mid-batch everywhere | tiled everywhere: Qwen shape T = 1024 360 | 387 | 426,
    // T = 1536 499 | 496 | 499 with down alone 206 tiled against 170 mid-batch, T = 2048 down 216
    // against 230; DeepSeek shape T = 1024 432 | 482 | 446, T = 1536 501 | 635 | 499.  A shared
    // expert much wider than the routed ones has few tiles of a long K in a tiled launch of its
    // own, which the mid-batch launch hides: that shape keeps the mid-batch down launch longer.)
    b.down_hi = wide_shared ? 125.0 : 100.0;
  }
  if (env_lo >= 0.0) b.lo = env_lo;
  if (env_hi >= 0.0) b.hi = b.down_hi = env_hi;
  if (env_min_tokens > 0) b.min_tokens = b.down_min_tokens = env_min_tokens;
  return b;
}
// The measured cross-overs as they stand: family of each phase at batch size T.
void rule_families(const AteniaMoeLayer* L, int T, int& up, int& down) {
  const bool int8w = L->wdtype == ATENIA_MOE_WEIGHT_INT8_W8A16;
  const bool base_streams = batch_streams(T, (long long)T * L->k, L->E, int8w ? 32 : 16);
  const double avg = (double)T * L->k / L->E;
  up = down = base_streams ? kFamStream : kFamTiled;
  if (stream_max_tokens_override() == 0 &&
      ffn_mid_supported(L->gate, L->wdtype) && ffn_mid_supported(L->up, L->wdtype) &&
      ffn_mid_supported(L->down, L->wdtype)) {
    const MidBounds b = mid_bounds(L);
    if (T >= b.min_tokens && T <= b.max_tokens && avg >= b.lo && avg <= b.hi) up = kFamMid;
    if (b.hi > 0.0 && T >= b.down_min_tokens && avg <= b.down_hi)
      down = kFamMid;
    else if (up == kFamMid && T < b.down_min_tokens)
      down = kFamStream;  // narrow experts: the register-resident down launch holds out longer
    // a per-group layer runs the tiled kernels on a bf16 copy: both phases or neither
    if (L->group_size > 0 && (up == kFamTiled) != (down == kFamTiled)) up = down = kFamTiled;
  }
}
// The bounds above are fitted to the shapes that were measured; on other shapes they can cross
// (few experts: the rows per expert pass the mid-batch form's upper bound while the batch is
// still small enough to stream; a wide shared expert: the down phase would enter the mid-batch
// form after the tiled kernels have already taken it).  A phase never goes back to a
// smaller-batch family as T grows: it takes the largest family the rule names at any batch size
// up to T.  The rule only changes at its bounds, so those are the batch sizes to look at.
BatchPlan plan_batch(const AteniaMoeLayer* L, int T) {
  BatchPlan p;
  rule_families(L, T, p.up, p.down);
  {
    const MidBounds b = mid_bounds(L);
    const double per = (double)L->E / L->k;  // tokens per row-per-expert
    const double marks[] = {(double)kStreamMaxTokens, 16.0 * per, 32.0 * per, (double)b.min_tokens,
                            (double)b.max_tokens, b.lo * per, b.hi * per, (double)b.down_min_tokens,
                            b.down_hi * per, (double)stream_max_tokens_override()};
    for (double mk : marks)
      for (int dt = -1; dt <= 1; ++dt) {
        const double c = std::floor(mk) + dt;
        if (c < 1.0 || c >= (double)T) continue;
        int u, dn;
        rule_families(L, (int)c, u, dn);
        p.up = std::max(p.up, u);      // kFamStream < kFamMid < kFamTiled
        p.down = std::max(p.down, dn);
      }
    if (L->group_size > 0 && (p.up == kFamTiled) != (p.down == kFamTiled)) p.up = p.down = kFamTiled;
  }
  p.routed_streams = p.up != kFamTiled;
  p.routed_mid = p.up == kFamMid;
  p.pg_prefill = L->group_size > 0 && p.up == kFamTiled && L->d_kpad % 64 == 0 &&
                 L->f_kpad % 64 == 0 && (L->fs == 0 || L->fs_kpad % 64 == 0);
  // the routed experts on the bf16 pipelined kernel (K a multiple of 64, >= 128)
  // W8A16: the int8 tiled kernel widens every weight in the VALU next to the matrix
  // instructions and has no tiles of nine row groups; once a batch is bound by the matrix cores
  // rather than by the weight stream (from int8_copy_min_rows() rows per expert on average) the
  // bf16 kernel on a bf16 copy of the int8 values is the faster one, for three times the
  // layer's footprint.  Both phases or neither (the row-tile lists differ), and only where the
  // shared expert's widths fit the same kernel.
  const bool dims64 = L->d_kpad % 64 == 0 && L->d_kpad >= 128 && L->f_kpad % 64 == 0 && L->f_kpad >= 128 &&
                      (L->fs == 0 || (L->fs_kpad % 64 == 0 && L->fs_kpad >= 128));
  p.q_copy = L->wdtype == ATENIA_MOE_WEIGHT_INT8_W8A16 && L->group_size == 0 && p.up == kFamTiled &&
             p.down == kFamTiled &&
             dims64 && int8_copy_min_rows() > 0 && !L->q_copy_off &&
             (double)T * L->k / L->E >= (double)int8_copy_min_rows();
  const bool bf16_tiles = L->wdtype == ATENIA_MOE_WEIGHT_BF16 || p.pg_prefill || p.q_copy;
  const bool pipe_ok = bf16_tiles && L->d_kpad % 64 == 0 && L->d_kpad >= 128 && L->f_kpad % 64 == 0 &&
                       L->f_kpad >= 128;
  static const int duo_phases = [] {
    const char* e = getenv("ATENIA_MOE_DUO_PHASES");
    return e ? atoi(e) : 3;
  }();
  p.duo_up = pipe_ok && p.up == kFamTiled && L->d_kpad <= duo_max_k() && (duo_phases & 1);
  p.duo_down = pipe_ok && p.down == kFamTiled && L->f_kpad <= duo_max_k() && (duo_phases & 2);
  // (the two-workgroup form cuts 256-row tiles in two, so a batch that uses it keeps those)
  p.tall_tiles = tall_tiles_enabled() && (p.up == kFamTiled || p.down == kFamTiled) && pipe_ok &&
                 !p.duo_up && !p.duo_down;
  return p;
}

// Partial output buffers the no-alloc workspace of a T-token batch needs (the tiled down phase
// may split tail tiles over k; the streaming kernels write one buffer).
int noalloc_y_parts(const AteniaMoeLayer* L, int T) {
  return plan_batch(L, T).down != kFamTiled || L->wdtype == ATENIA_MOE_WEIGHT_F32 ? 1 : kMaxYParts;
}

// Expert outputs of bf16 layers as bf16 between the tiled down launch and the combine (tuning
// knob ATENIA_MOE_Y_BF16=0 keeps them f32; read once).
bool y_bf16_enabled() {
  static const bool on = [] {
    const char* e = getenv("ATENIA_MOE_Y_BF16");
    return !(e && atoi(e) == 0);
  }();
  return on;
}

// Routed and shared experts' tiled launches of a phase as one launch where both are on the
// caller's stream (tuning knob ATENIA_MOE_PAIR_LAUNCHES=0: always two; read once).
bool pair_launches_enabled() {
  static const bool on = [] {
    const char* e = getenv("ATENIA_MOE_PAIR_LAUNCHES");
    return !(e && atoi(e) == 0);
  }();
  return on;
}

bool side_stream_enabled() {
  static const bool on = [] {
    const char* e = getenv("ATENIA_MOE_SHARED_SIDE_STREAM");  // 0 = everything on the caller's stream
    return !(e && atoi(e) == 0);
  }();
  return on;
}

bool stream_is_capturing(hipStream_t s) {
  hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(s, &st) != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  return st != hipStreamCaptureStatusNone;
}

// Family of the shared expert in a phase where the routed experts take `fam`: the same one where
// its widths allow it; beside the mid-batch kernel, if they do not, the tiled ones.
void shared_family(FfnArgs& fsd, int fam, int ffn_dtype) {
  const bool mid_ok = ffn_mid_supported(fsd.gate, ffn_dtype) && ffn_mid_supported(fsd.up, ffn_dtype) &&
                      ffn_mid_supported(fsd.down, ffn_dtype);
  const bool tiles_ok = tiled_supported(fsd.gate, ffn_dtype) && tiled_supported(fsd.down, ffn_dtype);
  fsd.use_mid = fam == kFamMid && mid_ok;
  fsd.use_tiled = (fam == kFamTiled || (fam == kFamMid && !mid_ok)) && tiles_ok;
}

// Everything run_forward decides about the expert kernels of a T-token batch, from the layer's
// dimensions alone (no device state): the same function answers atenia_moe_hip_plan_batch.
int family_name(int f) {
  return f == kFamMid ? ATENIA_MOE_KERNELS_MID : f == kFamTiled ? ATENIA_MOE_KERNELS_TILED : ATENIA_MOE_KERNELS_STREAM;
}
struct ResolvedPlan {
  BatchPlan plan;
  int ffn_dtype;         // element type the expert kernels see (bf16 for a per-group layer's copy)
  int fam_up, fam_down;  // routed experts, per phase (kFam*)
  bool duo_up, duo_down; // tiled phase on the two-workgroup form
  bool split_tail;       // tiled down launch may split the k range of tail tiles
  bool y_bf16, ys_bf16;  // expert outputs left as bf16 for the combine (routed / shared)
  int s_fam_up, s_fam_down;  // shared expert (-1: none)
};
// A per-group layer's bf16 copy has the dimensions of the int8 blocks and no group scales.
WeightSet dims_of(const AteniaMoeLayer* L, const WeightSet& w, bool pg_prefill) {
  WeightSet o = w;
  if (pg_prefill) {
    o.scale = nullptr;
    o.group_blocks = 0;
    o.n_kgroups = 0;
  }
  return o;
}
ResolvedPlan resolve_plan(const AteniaMoeLayer* L, int T) {
  ResolvedPlan r{};
  r.plan = plan_batch(L, T);
  const bool pg = r.plan.pg_prefill;
  // (a W8A16 layer's copy keeps its row scales and has the int8 blocks' dimensions)
  r.ffn_dtype = pg || r.plan.q_copy ? ATENIA_MOE_WEIGHT_BF16 : L->wdtype;
  const WeightSet gate = dims_of(L, L->gate, pg), down = dims_of(L, L->down, pg);
  const bool tiles_ok = tiled_supported(gate, r.ffn_dtype) && tiled_supported(down, r.ffn_dtype);
  r.fam_up = r.plan.up == kFamTiled && !tiles_ok ? kFamStream : r.plan.up;
  r.fam_down = r.plan.down == kFamTiled && !tiles_ok ? kFamStream : r.plan.down;
  r.duo_up = r.fam_up == kFamTiled && r.plan.duo_up;
  r.duo_down = r.fam_down == kFamTiled && r.plan.duo_down;
  r.split_tail = r.fam_down == kFamTiled && !r.duo_down && tiled_down_splits_tail(down, r.ffn_dtype);
  // bf16 layers on the bf16 tiled kernels leave the expert outputs as bf16 for the combine (half
  // the bytes written and read back; the bf16 rounding of h already sets this path's error).
  auto pipe = [&](const WeightSet& w) {
    return r.ffn_dtype == ATENIA_MOE_WEIGHT_BF16 && w.k_pad % 64 == 0 && w.k_pad >= 128 &&
           w.n_rows % 8 == 0;  // (a lane of the bf16 epilogue stores 8 columns at once)
  };
  r.y_bf16 = y_bf16_enabled() && L->wdtype == ATENIA_MOE_WEIGHT_BF16 && r.fam_down == kFamTiled &&
             pipe(down);
  r.s_fam_up = r.s_fam_down = -1;
  if (L->fs > 0 && L->wdtype != ATENIA_MOE_WEIGHT_F32) {
    FfnArgs fsd{};
    fsd.gate = dims_of(L, L->s_gate, pg);
    fsd.up = dims_of(L, L->s_up, pg);
    fsd.down = dims_of(L, L->s_down, pg);
    shared_family(fsd, r.fam_up, r.ffn_dtype);
    r.s_fam_up = fsd.use_mid ? kFamMid : fsd.use_tiled ? kFamTiled : kFamStream;
    shared_family(fsd, r.fam_down, r.ffn_dtype);
    r.s_fam_down = fsd.use_mid ? kFamMid : fsd.use_tiled ? kFamTiled : kFamStream;
    r.ys_bf16 = r.y_bf16 && fsd.use_tiled && pipe(fsd.down);
  }
  return r;
}

// `view`: the workspace to run on (nullptr = the handle's own).  no_alloc: fail instead of
// allocating anything.
int run_forward_impl(AteniaMoeLayer* L, const void* d_x, int x_dtype, int T, float* d_out,
                     hipStream_t s, int first, int last, const float* d_residual,
                     const WsView* view, bool no_alloc);

// A stream that this library did not make and that is not one of the runtime's own (null, legacy,
// per-thread): its owner may destroy it between two calls on the handle.
bool caller_owned_stream(const AteniaMoeLayer* L, hipStream_t s) {
  return (uintptr_t)s > 15 && s != L->stream && s != L->side;
}

int run_forward(AteniaMoeLayer* L, const void* d_x, int x_dtype, int T, float* d_out,
                hipStream_t s, int first, int last, const float* d_residual = nullptr,
                const WsView* view = nullptr, bool no_alloc = false) {
  const int rc = run_forward_impl(L, d_x, x_dtype, T, d_out, s, first, last, d_residual, view, no_alloc);
  // (see the ordering note in run_forward_impl; nothing is recorded into a graph being captured)
  if (L->done_valid && L->done_stream == s && caller_owned_stream(L, s) && !stream_is_capturing(s)) {
    if (hipEventRecord(L->done, s) == hipSuccess) L->done_recorded = true;
    else (void)hipGetLastError();
  }
  return rc;
}

int run_forward_impl(AteniaMoeLayer* L, const void* d_x, int x_dtype, int T, float* d_out,
                     hipStream_t s, int first, int last, const float* d_residual,
                     const WsView* view, bool no_alloc) {
  for (int st = 0; st < first; ++st)
    if (L->stage_T[st] != T)
      return fail(ATENIA_MOE_ERR_DIM, "stage %d has not run for %d tokens on this handle", st, T);
  for (int st = first; st < 4; ++st) L->stage_T[st] = -1;
  const bool f32w = L->wdtype == ATENIA_MOE_WEIGHT_F32;
  if (f32w && x_dtype != ATENIA_MOE_ACT_F32)
    return fail(ATENIA_MOE_ERR_UNSUPPORTED, "f32 weights need f32 activations");
  if (first > kStageRouter && view == nullptr && L->cur.idx != L->ws.idx)
    return fail(ATENIA_MOE_ERR_DIM, "the earlier stages ran on another workspace");
  // A W8A16 layer's bf16 copy only makes large batches faster: when it cannot be made (no room
  // left for twice the int8 bytes) the layer keeps the int8 tiled kernels from then on.  Decided
  // here, before the grouping stage lays out row tiles for either kernel.
  if (!f32w && !no_alloc && !L->pg_ready && !L->q_copy_off && plan_batch(L, T).q_copy &&
      ensure_pg_copy(L) != ATENIA_MOE_OK) {
    release_pg_copy(L);
    (void)hipGetLastError();
    L->q_copy_off = true;
  }
  const WsView V = view ? *view : L->ws;
  L->cur = V;
  // A forward still running on another stream uses the same workspace: wait for it.  Nothing
  // is recorded while calls stay on the null stream or the handle's own stream (an event per
  // forward would cost a decode step several microseconds): those cannot go away, so when the
  // stream changes the previous one is marked then -- the mark covers everything submitted to it
  // so far -- and the new one waits for the mark.  A stream the caller made may be gone by the
  // next call (and its handle value reused), so it is never touched again: run_forward marks it
  // at the end of each forward it submits there (`done_recorded`), and the next stream waits for
  // that mark.
  const bool capturing = stream_is_capturing(s);
  if (!capturing) {
    if (L->done_valid && L->done_stream != s) {
      if (L->done_recorded) {
        HIP_TRY(hipStreamWaitEvent(s, L->done, 0));
      } else if (hipEventRecord(L->done, L->done_stream) == hipSuccess) {
        HIP_TRY(hipStreamWaitEvent(s, L->done, 0));
      } else {
        (void)hipGetLastError();
        HIP_TRY(hipDeviceSynchronize());
      }
    }
    L->done_valid = true;
    L->done_stream = s;
    L->done_recorded = false;
  }
  StageTimer tm{L, s};
  for (int i = 0; i < ATENIA_MOE_N_STAGES; ++i) L->launches[i] = 0;
  tm.mark();  // ev[0]: start

  const bool x_bf16 = x_dtype == ATENIA_MOE_ACT_BF16;
  const bool need_xb = !f32w && !(x_bf16 && L->d_kpad == L->d);
  RouterArgs ra{};
  ra.x = d_x;
  ra.x_is_bf16 = x_bf16;
  ra.T = T;
  ra.d = L->d;
  ra.E = L->E;
  ra.k = L->k;
  ra.renorm = L->conv == ATENIA_MOE_CONVENTION_ATENIA;
  ra.w_router = L->w_router.as<float>();
  ra.w_fits_bf16 = L->router_fits_bf16;
  ra.w_lsb_min = L->router_lsb.as<int32_t>();
  ra.w_t8 = L->router_t8.as<uint16_t>();
  ra.w_rows_pad = L->router_rows_pad;
  ra.w_norm2 = L->router_norm2.as<double>();
  ra.router_bias = L->router_bias.as<float>();
  const bool gated = L->fs > 0 && L->conv == ATENIA_MOE_CONVENTION_HUGGINGFACE_QWEN &&
                     L->shared_gate.p != nullptr && L->v3_n_group == 0;
  ra.shared_gate = gated ? L->shared_gate.as<float>() : nullptr;
  ra.idx = V.idx;
  ra.w = V.w;
  ra.sgate = V.sgate;
  ra.xb = need_xb ? V.xb : nullptr;
  ra.d_pad = L->d_kpad;
  ra.status = L->status.as<int32_t>();
  // f32 layers: the sums of f32-valued products are not exact in every order, but the per-token
  // kernel's interval certificate settles all but about one sum in a thousand (those rows are
  // recomputed in the reference's order inside the kernel), so small batches take it as well
  // (router stage, d = 1024, 8 rows, per-token kernel / one sequential chain per (token, row):
  // T = 1 9.6 / 18.5 us, 16 13.5 / 19.0, 64 15.5 / 19.4, 128 14.9 / 19.4, 256 19.9 / 19.4,
  // 512 29.9 / 19.3).  Tuning knob ATENIA_MOE_ROUTER_TOKEN_MAX_F32 (read once).
  static const int f32_token_max = [] {
    const char* e = getenv("ATENIA_MOE_ROUTER_TOKEN_MAX_F32");
    return e ? atoi(e) : 192;
  }();
  ra.token_kernel_max_tokens = f32w ? f32_token_max : router_token_max();
  PermuteArgs pa{};
  pa.idx = V.idx;
  pa.T = T;
  pa.k = L->k;
  pa.E = L->E;
  pa.counts = V.counts;
  pa.offsets = V.offsets;
  pa.perm = V.perm;
  pa.inv = V.inv;
  pa.active = V.active;
  pa.n_active = V.n_active;
  pa.blk_counts = V.blk_counts;
  pa.shared_offsets = V.shared_desc;
  pa.tile_group = V.tile_group;
  pa.tile_m0 = V.tile_m0;
  pa.n_tiles = V.shared_desc + 4;
  pa.shared_n_tiles = V.shared_desc + 5;
  pa.tile_rows = V.tile_rows;
  pa.tile_li = V.tile_li;
  pa.max_tile_groups = plan_batch(L, T).tall_tiles ? 9 : 8;
  ra.fuse_permute = last >= kStagePermute ? &pa : nullptr;
  const bool v3 = L->v3_n_group > 0;
  if (v3 || L->E > 31) ra.logits_tmp = V.logits;
  if (v3) {
    ra.logits_out = V.logits;
    ra.shared_gate = nullptr;  // the V3 block adds its shared experts ungated
  }
  // One token through the streaming gate/up launch: that launch can route the token itself from
  // the logits, so a router launch that spreads its rows need not be followed by a launch that
  // only selects.
  ra.defer_select = T == 1 && last >= kStageFfn && !v3 && !f32w && L->E <= 64 &&
                    plan_batch(L, T).routed_streams;
  int fused = 0;
  if (first <= kStageRouter) {
    HIP_TRY(launch_router(ra, s, &fused));
    L->launches[0] = 1;
    if (v3) {
      V3RouteArgs va{};
      va.logits = V.logits;
      va.bias = L->v3_bias.as<float>();
      va.T = T;
      va.E = L->E;
      va.k = L->k;
      va.n_group = L->v3_n_group;
      va.topk_group = L->v3_topk_group;
      va.norm_topk_prob = L->v3_norm;
      va.routed_scaling_factor = L->v3_scale;
      va.idx = V.idx;
      va.w = V.w;
      va.status = L->status.as<int32_t>();
      HIP_TRY(launch_v3_route(va, s));
      L->launches[0] = 2;
    }
    L->stage_T[kStageRouter] = T;
  }
  tm.mark();  // ev[1]: router done
  L->last_T = T;
  if (last < kStagePermute) return ATENIA_MOE_OK;

  if (first <= kStagePermute) {
    int nl = 0;
    if (!fused) HIP_TRY(launch_permute(pa, s, &nl));
    L->launches[1] = nl;
    L->stage_T[kStagePermute] = T;
  }
  tm.mark();  // ev[2]: permute done
  if (last < kStageFfn) return ATENIA_MOE_OK;

  const void* a_x = f32w ? d_x : (need_xb ? (const void*)V.xb : d_x);
  const int a_stride = f32w ? L->d : L->d_kpad;

  // Per-group int8 and a batch for the MFMA-tiled kernels: those take one scale per row, so the
  // layer keeps a bf16 copy of its experts for such batches: q * group scale rounded to the
  // nearest bf16 (the reference's GPU dequantiser truncates instead,
  // src/cuda/int8_to_bf16.cu:91-110; rounding halves the error against the q * scale the
  // reference's CPU path multiplies with).  Decode batches stream the int8 weights themselves.
  // A W8A16 layer does the same from int8_copy_min_rows() rows per expert on, with the int8
  // values themselves in the copy (exact) and the row scales applied to the f32 results.
  const BatchPlan plan = plan_batch(L, T);
  const bool pg_prefill = plan.pg_prefill || plan.q_copy;
  if (pg_prefill && !L->pg_ready && no_alloc)
    return fail(ATENIA_MOE_ERR_UNSUPPORTED,
                "int8 layer: a batch of %d tokens needs the layer's bf16 copy, which is made by "
                "the first such batch through an allocating entry point", T);
  if (pg_prefill && !L->pg_ready) {
    int rc = ensure_pg_copy(L);
    if (rc) return rc;
  }
  const int ffn_dtype = pg_prefill ? ATENIA_MOE_WEIGHT_BF16 : L->wdtype;

  FfnArgs fa{};
  fa.wdtype = ffn_dtype;
  fa.f32_accumulate = L->policy != ATENIA_MOE_POLICY_CERTIFIED;
  fa.g.offsets = V.offsets;
  fa.g.active = V.active;
  fa.g.n_active = V.n_active;
  fa.g.perm = V.perm;
  fa.g.pair_div = L->k;
  fa.g.idx1 = T == 1 && fused ? V.idx : nullptr;
  if (fused == 2) {  // the router left the logits: the gate/up launch selects and groups
    fa.sel.logits = V.logits;
    fa.sel.E = L->E;
    fa.sel.k = L->k;
    fa.sel.renorm = ra.renorm;
    fa.sel.idx = V.idx;
    fa.sel.w = V.w;
    fa.sel.status = L->status.as<int32_t>();
    fa.sel.fg = FusedGrouping{pa.counts, pa.offsets, pa.perm, pa.inv, pa.active, pa.n_active,
                              pa.shared_offsets, pa.tile_group, pa.tile_m0, pa.n_tiles,
                              pa.shared_n_tiles};
  }
  fa.n_groups_max = (int)std::min<long long>(L->E, (long long)T * L->k);
  fa.rows_max = T;
  fa.gate = pg_prefill ? L->gate_b : L->gate;
  fa.up = pg_prefill ? L->up_b : L->up;
  fa.down = pg_prefill ? L->down_b : L->down;
  fa.x = a_x;
  fa.x_stride = a_stride;
  fa.h = V.h;
  fa.h_stride = L->f_kpad;
  fa.y = V.y;
  fa.y_stride = L->d;
  // Tiled (MFMA-bound) kernels once an expert can see more rows than the streaming kernel
  // keeps in registers; below that the weights are streamed once (HBM-bound).
  // (each phase has its own family; a tiled phase whose widths the tiled kernels do not take
  // falls back to the register-resident streaming kernel)
  const ResolvedPlan rp = resolve_plan(L, T);
  const int fam_up = rp.fam_up, fam_down = rp.fam_down;
  const bool tiled = fam_up == kFamTiled;  // gate/up phase
  fa.use_tiled = fam_up == kFamTiled;
  fa.use_mid = fam_up == kFamMid;
  fa.use_duo = rp.duo_up;
  fa.tall_tiles = plan.tall_tiles;
  fa.tile_group = V.tile_group;
  fa.tile_m0 = V.tile_m0;
  fa.n_tiles = V.shared_desc + 4;
  fa.tile_rows = V.tile_rows;
  fa.tile_li = V.tile_li;
  fa.max_row_tiles = (int)(((size_t)T * L->k + kTileM - 1) / kTileM +
                           std::min<long long>(L->E, (long long)T * L->k));
  const bool duo_down = rp.duo_down;
  const bool split_tail = rp.split_tail;
  fa.y_parts = split_tail ? std::min(kMaxYParts, V.y_parts) : 1;
  fa.y_part_stride = (size_t)T * L->k * L->d;
  fa.part_flags = split_tail ? V.part_flags : nullptr;
  fa.n_cus = device_cu_count();
  L->last_split = split_tail;
  fa.y_bf16 = rp.y_bf16;
  L->last_y_bf16 = fa.y_bf16;
  L->last_ys_bf16 = false;

  FfnArgs fsd{};
  if (L->fs > 0) {
    fsd = fa;
    fsd.y_bf16 = 0;
    fsd.use_duo = 0;
    fsd.tall_tiles = 0;  // the shared expert's rows are cut into whole 256-row tiles
    fsd.sel = InlineSelect{};
    const int32_t* sd = V.shared_desc;
    fsd.g.offsets = sd;
    fsd.g.active = sd + 2;
    fsd.g.n_active = sd + 3;
    fsd.g.perm = V.ident;
    fsd.g.pair_div = 1;
    fsd.g.idx1 = T == 1 ? sd : nullptr;  // sd[0] = 0: the one group, its one row
    fsd.n_groups_max = 1;
    fsd.rows_max = T;
    fsd.gate = pg_prefill ? L->s_gate_b : L->s_gate;
    fsd.up = pg_prefill ? L->s_up_b : L->s_up;
    fsd.down = pg_prefill ? L->s_down_b : L->s_down;
    fsd.h = V.hs;
    fsd.h_stride = L->fs_kpad;
    fsd.y = V.ys;
    fsd.y_parts = 1;
    fsd.part_flags = nullptr;
    // The shared expert follows the routed ones (it then rides in their launches): it is small
    // next to E routed experts, so its extra passes (one per 32 tokens) cost less than the
    // launches of its own that the tiled form would need.
    // (With the routed experts on the mid-batch kernel it takes that kernel too, one pass over
    // its weights per 128 tokens; if its widths do not fit that kernel, the tiled ones.)
    shared_family(fsd, fam_up, ffn_dtype);
    fsd.tile_group = V.s_tile_group;
    fsd.tile_m0 = V.s_tile_m0;
    fsd.n_tiles = V.shared_desc + 5;
    fsd.tile_rows = nullptr;  // the shared expert's rows are cut into whole 256-row tiles
    fsd.tile_li = nullptr;
    fsd.max_row_tiles = (T + kTileM - 1) / kTileM;
  }

  // Small batches stream both the routed experts and the shared one: one launch per phase.
  const bool fuse_shared_up = L->fs > 0 && ffn_stream_fuses_shared(fa, fsd, false);
  // A shared expert with tiled launches of its own: its gate/up and down depend on nothing the
  // routed experts compute, and each is a launch of few tiles (T / 256 row tiles; the down
  // launch of a wide shared expert fills a quarter of the chip for the length of its long K).
  // They go to a stream of the handle's own, between an event the caller's stream records after
  // the grouping and one it waits for before the first launch that reads the shared expert's
  // results, so that the hardware deals the tiles of both to the compute units as they free up.
  // Not under stream capture (no cross-stream dependencies are recorded into a caller's graph),
  // not from the entry point that allocates nothing (its callers get launches on their own
  // stream and nothing else) and not with stage profiling on (the stage events sit on the
  // caller's stream only).  While
  // the shared expert's down launch has fewer tiles than the chip has compute units; beyond,
  // its launches fill the chip by themselves and two kernels at once only share L2 worse.
  // Whole forward, one stream / two (us): Qwen1.5-MoE shape T = 1536 468 / 437, 2048 524 / 442,
  // 3072 646 / 561, 4096 783 / 711, 8192 1249 / 1239, 16384 2313 / 2336; DeepSeek-V2-Lite shape
  // T = 1024 436 / 409, 1536 497 / 442, 2048 561 / 514, 3072 717 / 658, 4096 834 / 813,
  // 8192 1360 / 1379, 16384 2546 / 2592.
  const long long shared_down_tiles =
      (long long)((T + kTileM - 1) / kTileM) * ((L->d + 255) / 256);
  // Where both are on the bf16 pipelined kernel the routed and the shared expert's tiles of a
  // phase are ONE launch instead (the shared expert's tiles behind the routed ones in the gate/up
  // phase, in front of them in the down phase where its K is the longer one): the compute units
  // that the last tiles of one part leave idle start on the other part at once, where each launch
  // by itself ends on a partly filled round of tiles, and the two parts never compete for an
  // XCD's L2.  One-stream stage times, two launches / one (us), gate/up and down: Qwen1.5-MoE
  // shape T = 2048 271 / 238 and 213 / 149, 4096 429 / 386 and 272 / 222, 12288 1045 / 1002 and
  // 613 / 560; DeepSeek-V2-Lite shape T = 4096 450 / 433 and 297 / 269, 12288 1092 / 1062 and
  // 680 / 650.  Whole forward, second stream / paired launches (ms): Qwen T = 768 0.344 / 0.332,
  // 1024 0.371 / 0.358, 2048 0.447 / 0.439, 3072 0.579 / 0.559, 4096 0.712 / 0.700, 6144
  // 1.018 / 1.002; DeepSeek T = 768 0.369 / 0.359, 1024 0.416 / 0.405, 1536 0.444 / 0.446, 2048
  // 0.509 / 0.495, 3072 0.670 / 0.657, 6144 1.104 / 1.091; two launches on one stream / paired:
  // Qwen T = 8192 1.261 / 1.249, 12288 1.848 / 1.769; DeepSeek T = 8192 1.367 / 1.335, 16384
  // 2.527 / 2.490.  The second stream stays for the layers that cannot pair (int8 tiles).
  const bool pair_up = pair_launches_enabled() && L->fs > 0 && !fuse_shared_up &&
                       tiled_up_pair_supported(fa, fsd);
  const bool side_run = side_stream_enabled() && L->fs > 0 && !fuse_shared_up && tiled && L->side &&
                        shared_down_tiles < fa.n_cus && first <= kStageFfn && !L->profiling &&
                        !no_alloc && !pair_up && !stream_is_capturing(s);
  bool side_open = false;
  if (first <= kStageFfn) {
    if (side_run) {
      HIP_TRY(hipEventRecord(L->ev_fork, s));
      HIP_TRY(hipStreamWaitEvent(L->side, L->ev_fork, 0));
      side_open = true;
    }
    if (pair_up) {
      HIP_TRY(launch_ffn_up_tiled_pair(fa, fsd, s));
      L->launches[2] = 1;
    } else {
      HIP_TRY(launch_ffn_up(fa, s, fuse_shared_up ? &fsd : nullptr));
      L->launches[2] = 1;
      if (L->fs > 0 && !fuse_shared_up) {
        HIP_TRY(launch_ffn_up(fsd, side_run ? L->side : s));
        L->launches[2] = 2;
      }
    }
  }
  auto side_join = [&]() -> hipError_t {  // the caller's stream waits for the side stream's work
    if (!side_open) return hipSuccess;
    side_open = false;
    hipError_t e = hipEventRecord(L->ev_join, L->side);
    return e != hipSuccess ? e : hipStreamWaitEvent(s, L->ev_join, 0);
  };
  tm.mark();  // ev[3]: gate/up done
  // the down phase may take another family than gate/up did
  fa.use_tiled = fam_down == kFamTiled;
  fa.use_mid = fam_down == kFamMid;
  fa.use_duo = duo_down;
  if (L->fs > 0) {
    shared_family(fsd, fam_down, ffn_dtype);
    fsd.y_bf16 = rp.ys_bf16;
    L->last_ys_bf16 = fsd.y_bf16;
  }
  const bool fuse_shared_down = L->fs > 0 && ffn_stream_fuses_shared(fa, fsd, true);
  // One token, whole pipeline requested: the down launch covers the routed experts and the
  // shared one and finishes the combine as well (one launch instead of two or three).
  const bool fuse1 = first <= kStageFfn && last >= kStageCombine && L->group_size == 0 &&
                     ffn_down_decode1_supported(T, fa, L->k, tiled, L->fs > 0 ? &fsd : nullptr);
  bool pair_down = false;
  if (first <= kStageFfn) {
    if (fuse1) {
      fa.fuse_w = V.w;
      fa.fuse_out = d_out;
      fa.fuse_residual = d_residual;
      fa.fuse_sgate = gated ? V.sgate : nullptr;
      fa.fuse_k = L->k;
      HIP_TRY(launch_ffn_down_decode1(fa, s, L->fs > 0 ? &fsd : nullptr));
    } else {
      if (fuse_shared_down) HIP_TRY(side_join());  // the fused launch reads the shared expert's h
      // one launch for both, the shared expert's tiles (the longer K) first
      pair_down = pair_launches_enabled() && L->fs > 0 && !fuse_shared_down && !side_open &&
                  tiled_down_pair_supported(fsd, fa);
      if (pair_down) HIP_TRY(launch_ffn_down_tiled_pair(fsd, fa, s));
      else HIP_TRY(launch_ffn_down(fa, s, fuse_shared_down ? &fsd : nullptr));
    }
    L->launches[3] = 1;
    if (L->fs > 0 && !fuse_shared_down && !fuse1 && !pair_down) {
      HIP_TRY(launch_ffn_down(fsd, side_open ? L->side : s));
      L->launches[3] = 2;
    }
    HIP_TRY(side_join());
    L->stage_T[kStageFfn] = T;
  }
  tm.mark();  // ev[4]: down done
  if (last < kStageCombine) return ATENIA_MOE_OK;
  if (fuse1) {
    L->launches[4] = 0;
    L->stage_T[kStageCombine] = T;
    tm.mark();  // ev[5]: nothing left to do
    L->launches[5] = L->launches[0] + L->launches[1] + L->launches[2] + L->launches[3];
    return ATENIA_MOE_OK;
  }

  CombineArgs ca{};
  ca.T = T;
  ca.k = L->k;
  ca.d = L->d;
  ca.w = V.w;
  ca.y = V.y;
  ca.y_stride = L->d;
  ca.part_flags = fa.part_flags;
  ca.flag_cols = (L->d + 255) / 256;
  ca.y_part_stride = fa.y_part_stride;
  ca.y_bf16 = fa.y_bf16;
  ca.y_shared = L->fs > 0 ? V.ys : nullptr;
  ca.ys_bf16 = L->fs > 0 && fsd.y_bf16;
  ca.sgate = gated ? V.sgate : nullptr;
  ca.residual = d_residual;
  ca.out = d_out;
  HIP_TRY(launch_combine(ca, s));
  L->launches[4] = 1;
  L->stage_T[kStageCombine] = T;
  tm.mark();  // ev[5]: combine done
  L->launches[5] = L->launches[0] + L->launches[1] + L->launches[2] + L->launches[3] + 1;
  return ATENIA_MOE_OK;
}

int read_status(AteniaMoeLayer* L, hipStream_t s, int32_t* token, int32_t* expert) {
  if (hipStreamSynchronize(s) != hipSuccess)
    return fail(ATENIA_MOE_ERR_SYNC, "stream synchronisation failed");
  int32_t st[2] = {0, INT_MAX};
  if (!L->status.p) return ATENIA_MOE_OK;
  HIP_TRY(hipMemcpy(st, L->status.p, 8, hipMemcpyDeviceToHost));
  if (st[0] == 0) return ATENIA_MOE_OK;
  int tk = st[1] >> 10, ex = st[1] & 1023;
  if (token) *token = tk;
  if (expert) *expert = ex;
  L->nf_token = tk;
  L->nf_expert = ex;
  int32_t reset[2] = {0, INT_MAX};
  HIP_TRY(hipMemcpy(L->status.p, reset, 8, hipMemcpyHostToDevice));
  return fail(ATENIA_MOE_ERR_NON_FINITE, "non-finite routing weight at token %d, expert %d", tk,
              ex);
}

// ---- host-buffer entry point, large batches -----------------------------------------------------
// A batch from pageable host memory travels through page-locked staging in chunks of
// kHostChunkTokens: the calling thread copies chunk c + 1 into a staging slot while the copy
// engine moves chunk c to the device; after the one forward over the whole batch the output comes
// back the same way (the copy engine fills one slot while the thread empties the other).  The
// caller's pages cannot be registered on the fly (hipHostRegister is not available on every
// host), hence the staging copy; it runs at memcpy speed, about twice what the runtime's own
// pageable copies reach.  Everything is ordered on the handle's stream; the events only tell the
// host when a slot is free or full.
constexpr int kHostChunkTokens = 1024;

// Page-locked caller memory (hipHostMalloc and the like) is copied by the DMA engines directly;
// staging it would only add a copy.
bool is_page_locked(const void* p) {
  hipPointerAttribute_t at{};
  if (hipPointerGetAttributes(&at, p) != hipSuccess) {
    (void)hipGetLastError();  // ordinary memory: the query fails and leaves its error behind
    return false;
  }
  return at.type == hipMemoryTypeHost;
}

int ensure_host_staging(AteniaMoeLayer* L) {
  const size_t need = (size_t)kHostChunkTokens * L->d * 4;
  if (!L->staging_ready) {
    for (int i = 0; i < 2; ++i) {
      HIP_TRY(hipEventCreateWithFlags(&L->ev_h2d[i], hipEventDisableTiming));
      HIP_TRY(hipEventCreateWithFlags(&L->ev_d2h[i], hipEventDisableTiming));
    }
    L->staging_ready = true;
  }
  if (L->pin_bytes < need) {
    if (L->pin_in) (void)hipHostFree(L->pin_in);
    if (L->pin_out) (void)hipHostFree(L->pin_out);
    L->pin_in = L->pin_out = nullptr;
    L->pin_bytes = 0;
    HIP_TRY(hipHostMalloc(&L->pin_in, 2 * need, hipHostMallocDefault));
    HIP_TRY(hipHostMalloc(&L->pin_out, 2 * need, hipHostMallocDefault));
    L->pin_bytes = need;
  }
  return ATENIA_MOE_OK;
}

// The staging copies (pageable caller memory <-> page-locked slots) are what the calling thread
// would otherwise spend most of the call on: one core moves about half of what the copy engine
// does.  For each of the two copy phases of a staged call (input in, output out -- not while the
// forward itself runs, during which helpers would only spin) a few helper threads take a slice
// of every chunk each (tuning knob ATENIA_MOE_HOST_COPY_THREADS, read once: threads in all,
// 1 = the caller alone).  A thread that cannot be started is done without.
class CopyCrew {
 public:
  explicit CopyCrew(int helpers) {
    th_.reserve(helpers > 0 ? helpers : 0);
    for (int i = 0; i < helpers; ++i) {
      try {
        th_.emplace_back([this, i] { run(i + 1); });
      } catch (...) {  // no exception may cross the C boundary: copy with the threads there are
        break;
      }
    }
  }
  ~CopyCrew() {
    quit_ = true;
    gen_.fetch_add(1, std::memory_order_release);
    for (auto& t : th_) t.join();
  }
  void copy(void* dst, const void* src, size_t bytes) {
    dst_ = (char*)dst;
    src_ = (const char*)src;
    bytes_ = bytes;
    done_.store(0, std::memory_order_relaxed);
    gen_.fetch_add(1, std::memory_order_release);
    slice(0);
    while (done_.load(std::memory_order_acquire) < (int)th_.size()) std::this_thread::yield();
  }

 private:
  void slice(int i) {
    const size_t n = th_.size() + 1;
    const size_t per = ((bytes_ + n - 1) / n + 4095) & ~(size_t)4095;
    const size_t lo = std::min(bytes_, (size_t)i * per), hi = std::min(bytes_, lo + per);
    if (hi > lo) memcpy(dst_ + lo, src_ + lo, hi - lo);
  }
  void run(int i) {
    int seen = 0;
    for (;;) {
      int g;
      while ((g = gen_.load(std::memory_order_acquire)) == seen) std::this_thread::yield();
      seen = g;
      if (quit_) return;
      slice(i);
      done_.fetch_add(1, std::memory_order_release);
    }
  }
  std::vector<std::thread> th_;
  std::atomic<int> gen_{0}, done_{0};
  std::atomic<bool> quit_{false};
  char* dst_ = nullptr;
  const char* src_ = nullptr;
  size_t bytes_ = 0;
};
int host_copy_threads() {
  static const int v = [] {
    const char* e = getenv("ATENIA_MOE_HOST_COPY_THREADS");
    const int n = e ? atoi(e) : 4;
    return std::max(1, std::min(n, 16));
  }();
  return v;
}

int forward_host_staged(AteniaMoeLayer* L, const float* x_host, int T, float* out_host) {
  int rc = ensure_host_staging(L);
  if (rc) return rc;
  const size_t row = (size_t)L->d * 4;
  const int n_chunks = (T + kHostChunkTokens - 1) / kHostChunkTokens;
  auto tokens_of = [&](int c) { return std::min(kHostChunkTokens, T - c * kHostChunkTokens); };
  {
    CopyCrew crew(host_copy_threads() - 1);
    for (int c = 0; c < n_chunks; ++c) {
      const int slot = c & 1;
      const size_t off = (size_t)c * kHostChunkTokens * row, bytes = (size_t)tokens_of(c) * row;
      // the slot is free once the copy of chunk c - 2 has left it
      if (c >= 2) HIP_TRY(hipEventSynchronize(L->ev_h2d[slot]));
      crew.copy((char*)L->pin_in + slot * L->pin_bytes, (const char*)x_host + off, bytes);
      HIP_TRY(hipMemcpyAsync((char*)L->x_in.p + off, (char*)L->pin_in + slot * L->pin_bytes, bytes,
                             hipMemcpyHostToDevice, L->stream));
      HIP_TRY(hipEventRecord(L->ev_h2d[slot], L->stream));
    }
  }
  rc = run_forward(L, L->x_in.p, ATENIA_MOE_ACT_F32, T, L->out.as<float>(), L->stream,
                   kStageRouter, kStageCombine);
  if (rc) return rc;
  std::unique_ptr<CopyCrew> crew;  // started when the first output chunk has arrived
  auto drain = [&](int c) -> int {  // chunk c's output: staging -> caller
    const int slot = c & 1;
    HIP_TRY(hipEventSynchronize(L->ev_d2h[slot]));
    if (!crew) crew.reset(new (std::nothrow) CopyCrew(host_copy_threads() - 1));
    void* dst = (char*)out_host + (size_t)c * kHostChunkTokens * row;
    const void* src = (char*)L->pin_out + slot * L->pin_bytes;
    if (crew) crew->copy(dst, src, (size_t)tokens_of(c) * row);
    else memcpy(dst, src, (size_t)tokens_of(c) * row);
    return ATENIA_MOE_OK;
  };
  for (int c = 0; c < n_chunks; ++c) {
    const int slot = c & 1;
    const size_t off = (size_t)c * kHostChunkTokens * row, bytes = (size_t)tokens_of(c) * row;
    // the slot is free once the caller has chunk c - 2's rows
    if (c >= 2 && (rc = drain(c - 2))) return rc;
    HIP_TRY(hipMemcpyAsync((char*)L->pin_out + slot * L->pin_bytes, (char*)L->out.p + off, bytes,
                           hipMemcpyDeviceToHost, L->stream));
    HIP_TRY(hipEventRecord(L->ev_d2h[slot], L->stream));
  }
  for (int c = std::max(0, n_chunks - 2); c < n_chunks; ++c)
    if ((rc = drain(c))) return rc;
  return read_status(L, L->stream, nullptr, nullptr);
}

}  // namespace

extern "C" {

int atenia_moe_hip_available(void) {
  static int cached = [] {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess || n <= 0) return 0;
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, 0) != hipSuccess) return 0;
    return strncmp(prop.gcnArchName, "gfx950", 6) == 0 ? 1 : 0;
  }();
  return cached;
}

const char* atenia_moe_hip_last_error_string(void) { return g_last_error.c_str(); }

int atenia_moe_hip_layer_create(const AteniaMoeLayerDesc* D, AteniaMoeLayer** out_layer) {
  if (!D || !out_layer) return fail(ATENIA_MOE_ERR_DIM, "null descriptor or output pointer");
  *out_layer = nullptr;
  if (D->num_experts < 1 || D->d_model < 1 || D->d_ff < 1 || D->d_ff_shared < 0)
    return fail(ATENIA_MOE_ERR_DIM, "bad dimensions E=%d d=%d f=%d f_s=%d", D->num_experts,
                D->d_model, D->d_ff, D->d_ff_shared);
  if (D->top_k < 1 || D->top_k > D->num_experts)
    return fail(ATENIA_MOE_ERR_K, "bad k=%d for %d experts", D->top_k, D->num_experts);
  if (D->convention != ATENIA_MOE_CONVENTION_ATENIA &&
      D->convention != ATENIA_MOE_CONVENTION_HUGGINGFACE_QWEN)
    return fail(ATENIA_MOE_ERR_DIM, "unknown convention %d", D->convention);
  if (D->weight_dtype < 0 || D->weight_dtype > ATENIA_MOE_WEIGHT_INT8_PER_GROUP)
    return fail(ATENIA_MOE_ERR_DIM, "unknown weight dtype %d", D->weight_dtype);
  const bool per_group = D->weight_dtype == ATENIA_MOE_WEIGHT_INT8_PER_GROUP;
  if (per_group && (D->group_size <= 0 || D->group_size % kKbInt8 != 0))
    return fail(ATENIA_MOE_ERR_DIM, "per-group int8 needs group_size > 0 and a multiple of %d (got %d)",
                kKbInt8, D->group_size);
  if (per_group && !D->w_up)
    return fail(ATENIA_MOE_ERR_UNSUPPORTED, "per-group int8 takes separate gate and up tensors");
  if (!D->w_router || !D->w_gate || !D->w_down)
    return fail(ATENIA_MOE_ERR_DIM, "router / gate / down weights are required");
  const bool int8 = D->weight_dtype == ATENIA_MOE_WEIGHT_INT8_W8A16 || per_group;
  if (int8 && (!D->scale_gate || !D->scale_up || !D->scale_down))
    return fail(ATENIA_MOE_ERR_DIM, "int8 weights need per-row scales");
  if (D->d_ff_shared > 0) {
    if (!D->s_gate || !D->s_up || !D->s_down)
      return fail(ATENIA_MOE_ERR_DIM, "shared expert weights missing");
    if (int8 && (!D->s_scale_gate || !D->s_scale_up || !D->s_scale_down))
      return fail(ATENIA_MOE_ERR_DIM, "int8 shared expert needs per-row scales");
  }
  if (D->num_experts + (D->shared_gate ? 1 : 0) > kMaxRouterRows)
    return fail(ATENIA_MOE_ERR_UNSUPPORTED, "at most %d router rows (experts + shared-expert gate)",
                kMaxRouterRows);
  if (!atenia_moe_hip_available())
    return fail(ATENIA_MOE_ERR_LAUNCH, "no gfx950 device available");

  AteniaMoeLayer* L = new (std::nothrow) AteniaMoeLayer();
  if (!L) return fail(ATENIA_MOE_ERR_OOM, "host allocation failed");
  L->E = D->num_experts;
  L->k = D->top_k;
  L->d = D->d_model;
  L->f = D->d_ff;
  L->fs = D->d_ff_shared;
  L->conv = D->convention;
  // Per-group int8 is stored and streamed like per-row int8; only the scales differ.
  L->wdtype = per_group ? ATENIA_MOE_WEIGHT_INT8_W8A16 : D->weight_dtype;
  L->group_size = per_group ? D->group_size : 0;
  const int KB = L->wdtype == ATENIA_MOE_WEIGHT_F32 ? 1 : kb_of(L->wdtype);
  L->d_kpad = round_up(L->d, KB);
  L->f_kpad = round_up(L->f, KB);
  L->fs_kpad = round_up(L->fs, KB);

  int rc = ATENIA_MOE_OK;
  auto bail = [&](int code) {
    delete L;
    return code;
  };
  if (hipStreamCreate(&L->stream) != hipSuccess)
    return bail(fail(ATENIA_MOE_ERR_LAUNCH, "hipStreamCreate failed"));
  const size_t E = L->E, d = L->d, f = L->f, fs = L->fs;
  if ((rc = upload_f32(D->w_router, E * d, L->w_router))) return bail(rc);
  if (D->router_bias && (rc = upload_f32(D->router_bias, E, L->router_bias))) return bail(rc);
  if (D->shared_gate && (rc = upload_f32(D->shared_gate, d, L->shared_gate))) return bail(rc);
  {
    // Router rows (and the gate vector) whose f32 values all fit bf16, as they do when the
    // checkpoint was bf16: with bf16 activations every product then has few enough significant
    // bits that a sum in any order is exact in f64, which is what lets the router use the
    // matrix cores without a slow path (router.hip).
    auto fits_bf16 = [](const float* p, size_t n) {
      uint32_t low = 0;
      for (size_t i = 0; i < n; ++i) {
        uint32_t u;
        memcpy(&u, p + i, 4);
        low |= u;
      }
      return (low & 0xffffu) == 0;
    };
    L->router_fits_bf16 = fits_bf16(D->w_router, E * d) &&
                          (!D->shared_gate || fits_bf16(D->shared_gate, d));
    // Lowest last-bit exponent over each row (v = odd * 2^q; 32767 = the row is all zeros, a
    // hugely negative value = it holds an inf or a NaN): with the same minimum over a token's
    // activations it bounds the last bit of every product of the pair from below, which settles
    // most of the sums the router's interval test flags without reading either row again.
    auto row_lsb = [](const float* p, size_t n) {
      int q = 32767;
      for (size_t i = 0; i < n; ++i) {
        uint32_t u;
        memcpy(&u, p + i, 4);
        const int e = (u >> 23) & 0xff;
        const uint32_t m = u & 0x7fffffu, mm = e ? (m | 0x800000u) : m;
        if (e == 0xff) return -100000;
        if (mm == 0) continue;
        q = std::min(q, (e ? e - 150 : -149) + __builtin_ctz(mm));
      }
      return q;
    };
    std::vector<int32_t> lsb(E + 1, 32767);
    for (size_t r = 0; r < E; ++r) lsb[r] = row_lsb(D->w_router + r * d, d);
    if (D->shared_gate) lsb[E] = row_lsb(D->shared_gate, d);
    if ((rc = L->router_lsb.ensure(lsb.size() * 4))) return bail(rc);
    if (hipMemcpy(L->router_lsb.p, lsb.data(), lsb.size() * 4, hipMemcpyHostToDevice) != hipSuccess)
      return bail(fail(ATENIA_MOE_ERR_LAUNCH, "upload of the router row table failed"));
    if (L->router_fits_bf16 && d % 8 == 0) {
      // The copy the matrix-core router streams: bf16 (exact: the values fit), eight columns
      // of all rows side by side, zero rows up to a multiple of 16 and zero chunks up to a
      // multiple of 32 columns; and |row|^2 for its bound on sum|p|.
      const size_t R = E + (D->shared_gate ? 1 : 0), Rp = (R + 15) / 16 * 16;
      const size_t chunks = (d + 31) / 32 * 4;
      std::vector<uint16_t> t8(chunks * Rp * 8, 0);
      std::vector<double> n2(Rp, 0.0);
      for (size_t r = 0; r < R; ++r) {
        const float* row = r < E ? D->w_router + r * d : D->shared_gate;
        double acc = 0.0;
        for (size_t c = 0; c < d; ++c) {
          uint32_t u;
          memcpy(&u, row + c, 4);
          t8[((c / 8) * Rp + r) * 8 + c % 8] = (uint16_t)(u >> 16);
          acc += (double)row[c] * (double)row[c];
        }
        n2[r] = acc;
      }
      if ((rc = L->router_t8.ensure(t8.size() * 2)) || (rc = L->router_norm2.ensure(n2.size() * 8)))
        return bail(rc);
      if (hipMemcpy(L->router_t8.p, t8.data(), t8.size() * 2, hipMemcpyHostToDevice) != hipSuccess ||
          hipMemcpy(L->router_norm2.p, n2.data(), n2.size() * 8, hipMemcpyHostToDevice) != hipSuccess)
        return bail(fail(ATENIA_MOE_ERR_LAUNCH, "upload of the router's bf16 copy failed"));
      L->router_rows_pad = (int)Rp;
    }
  }

  DevBuf staging;
  const size_t eb = elem_bytes_of(L->wdtype);
  const bool packed = D->w_up == nullptr;
  const void* gate_h = D->w_gate;
  const void* up_h = packed ? (const void*)((const uint8_t*)D->w_gate + f * d * eb) : D->w_up;
  const size_t gu_stride = packed ? 2 * f * d : f * d;
  if ((rc = upload_family(gate_h, gu_stride, L->E, L->f, L->d, L->wdtype, L->wg, L->gate,
                          staging)))
    return bail(rc);
  if ((rc = upload_family(up_h, gu_stride, L->E, L->f, L->d, L->wdtype, L->wu, L->up, staging)))
    return bail(rc);
  if ((rc = upload_family(D->w_down, d * f, L->E, L->d, L->f, L->wdtype, L->wd, L->down,
                          staging)))
    return bail(rc);
  if (per_group) {
    const int gs = L->group_size;
    if ((rc = upload_group_scales(D->scale_gate, L->E, L->f, L->d, gs, L->sg, L->gate))) return bail(rc);
    if ((rc = upload_group_scales(D->scale_up, L->E, L->f, L->d, gs, L->su, L->up))) return bail(rc);
    if ((rc = upload_group_scales(D->scale_down, L->E, L->d, L->f, gs, L->sd, L->down))) return bail(rc);
  } else if (int8) {
    if ((rc = upload_f32(D->scale_gate, E * f, L->sg))) return bail(rc);
    if ((rc = upload_f32(D->scale_up, E * f, L->su))) return bail(rc);
    if ((rc = upload_f32(D->scale_down, E * d, L->sd))) return bail(rc);
    L->gate.scale = L->sg.as<float>();
    L->up.scale = L->su.as<float>();
    L->down.scale = L->sd.as<float>();
  }
  if (fs > 0) {
    if ((rc = upload_family(D->s_gate, fs * d, 1, L->fs, L->d, L->wdtype, L->swg, L->s_gate,
                            staging)))
      return bail(rc);
    if ((rc = upload_family(D->s_up, fs * d, 1, L->fs, L->d, L->wdtype, L->swu, L->s_up,
                            staging)))
      return bail(rc);
    if ((rc = upload_family(D->s_down, d * fs, 1, L->d, L->fs, L->wdtype, L->swd, L->s_down,
                            staging)))
      return bail(rc);
    if (per_group) {
      const int gs = L->group_size;
      if ((rc = upload_group_scales(D->s_scale_gate, 1, L->fs, L->d, gs, L->ssg, L->s_gate))) return bail(rc);
      if ((rc = upload_group_scales(D->s_scale_up, 1, L->fs, L->d, gs, L->ssu, L->s_up))) return bail(rc);
      if ((rc = upload_group_scales(D->s_scale_down, 1, L->d, L->fs, gs, L->ssd, L->s_down))) return bail(rc);
    } else if (int8) {
      if ((rc = upload_f32(D->s_scale_gate, fs, L->ssg))) return bail(rc);
      if ((rc = upload_f32(D->s_scale_up, fs, L->ssu))) return bail(rc);
      if ((rc = upload_f32(D->s_scale_down, d, L->ssd))) return bail(rc);
      L->s_gate.scale = L->ssg.as<float>();
      L->s_up.scale = L->ssu.as<float>();
      L->s_down.scale = L->ssd.as<float>();
    }
  }
  // Algorithmic bytes of one routed expert as stored (weights + int8 scales).
  L->bytes_per_expert = (int64_t)(3 * d * f * eb) + (int8 ? (int64_t)(2 * f + d) * 4 : 0);
  if (per_group)  // one scale per row and group instead of one per row
    L->bytes_per_expert = (int64_t)(3 * d * f * eb) +
                          ((int64_t)2 * f * ((d + L->group_size - 1) / L->group_size) +
                           (int64_t)d * ((f + L->group_size - 1) / L->group_size)) * 4;
  if ((rc = L->status.ensure(8))) return bail(rc);
  {
    const int32_t st[2] = {0, INT_MAX};
    if (hipMemcpy(L->status.p, st, 8, hipMemcpyHostToDevice) != hipSuccess)
      return bail(fail(ATENIA_MOE_ERR_LAUNCH, "status upload failed"));
  }
  if (hipEventCreateWithFlags(&L->done, hipEventDisableTiming) != hipSuccess)
    return bail(fail(ATENIA_MOE_ERR_LAUNCH, "hipEventCreate failed"));
  if (L->fs > 0 && side_stream_enabled()) {
    if (hipStreamCreateWithFlags(&L->side, hipStreamNonBlocking) != hipSuccess ||
        hipEventCreateWithFlags(&L->ev_fork, hipEventDisableTiming) != hipSuccess ||
        hipEventCreateWithFlags(&L->ev_join, hipEventDisableTiming) != hipSuccess)
      return bail(fail(ATENIA_MOE_ERR_LAUNCH, "stream / event creation failed"));
  }
  if (hipGetDevice(&L->device) != hipSuccess)
    return bail(fail(ATENIA_MOE_ERR_LAUNCH, "hipGetDevice failed"));
  if ((rc = resolve_static_scratch(L->device, nullptr))) return bail(rc);
  if (D->max_tokens_hint > 0) {
    if ((rc = ensure_workspace(L, D->max_tokens_hint))) return bail(rc);
    const BatchPlan hp = plan_batch(L, D->max_tokens_hint);
    if ((hp.pg_prefill || hp.q_copy) && (rc = ensure_pg_copy(L))) return bail(rc);
  }
  if (hipDeviceSynchronize() != hipSuccess)
    return bail(fail(ATENIA_MOE_ERR_SYNC, "device synchronisation failed after upload"));
  *out_layer = L;
  return ATENIA_MOE_OK;
}

int atenia_moe_hip_layer_destroy(AteniaMoeLayer* L) {
  if (!valid_handle(L)) return fail(ATENIA_MOE_ERR_HANDLE, "invalid layer handle");
  {
    std::lock_guard<std::mutex> lock(L->mu);
    (void)hipDeviceSynchronize();
    if (L->ev_valid)
      for (auto& e : L->ev) (void)hipEventDestroy(e);
    if (L->done) (void)hipEventDestroy(L->done);
    if (L->ev_fork) (void)hipEventDestroy(L->ev_fork);
    if (L->ev_join) (void)hipEventDestroy(L->ev_join);
    if (L->side) (void)hipStreamDestroy(L->side);
    if (L->staging_ready) {
      for (int i = 0; i < 2; ++i) {
        (void)hipEventDestroy(L->ev_h2d[i]);
        (void)hipEventDestroy(L->ev_d2h[i]);
      }
    }
    if (L->pin_in) (void)hipHostFree(L->pin_in);
    if (L->pin_out) (void)hipHostFree(L->pin_out);
    if (L->stream) (void)hipStreamDestroy(L->stream);
    L->magic = 0;
  }
  delete L;
  return ATENIA_MOE_OK;
}

int atenia_moe_hip_layer_forward_device(AteniaMoeLayer* L, const void* d_x, int x_dtype,
                                        int n_tokens, float* d_out, void* stream) {
  if (!valid_handle(L)) return fail(ATENIA_MOE_ERR_HANDLE, "invalid layer handle");
  if (n_tokens < 0) return fail(ATENIA_MOE_ERR_DIM, "negative token count");
  if (n_tokens == 0) return ATENIA_MOE_OK;
  if (!d_x || !d_out) return fail(ATENIA_MOE_ERR_DIM, "null activation pointer");
  if (x_dtype != ATENIA_MOE_ACT_F32 && x_dtype != ATENIA_MOE_ACT_BF16)
    return fail(ATENIA_MOE_ERR_DIM, "unknown activation dtype %d", x_dtype);
  if ((long long)n_tokens * L->k > (long long)INT_MAX / 4)
    return fail(ATENIA_MOE_ERR_DIM, "too many tokens");
  std::lock_guard<std::mutex> lock(L->mu);
  int rc = ensure_workspace(L, n_tokens);
  if (rc) return rc;
  return run_forward(L, d_x, x_dtype, n_tokens, d_out, (hipStream_t)stream, kStageRouter,
                     kStageCombine);
}

int atenia_moe_hip_layer_forward_device_noalloc(AteniaMoeLayer* L, const void* d_x, int x_dtype,
                                                int n_tokens, float* d_out, void* stream) {
  if (!valid_handle(L)) return fail(ATENIA_MOE_ERR_HANDLE, "invalid layer handle");
  if (n_tokens < 0) return fail(ATENIA_MOE_ERR_DIM, "negative token count");
  if (n_tokens == 0) return ATENIA_MOE_OK;
  if (!d_x || !d_out) return fail(ATENIA_MOE_ERR_DIM, "null activation pointer");
  if (x_dtype != ATENIA_MOE_ACT_F32 && x_dtype != ATENIA_MOE_ACT_BF16)
    return fail(ATENIA_MOE_ERR_DIM, "unknown activation dtype %d", x_dtype);
  if ((long long)n_tokens * L->k > (long long)INT_MAX / 4)
    return fail(ATENIA_MOE_ERR_DIM, "too many tokens");
  std::lock_guard<std::mutex> lock(L->mu);
  const int y_parts = noalloc_y_parts(L, n_tokens);
  const size_t need = ws_layout(L, n_tokens, y_parts, nullptr, nullptr);
  if (need > kStaticScratchBytes)
    return fail(ATENIA_MOE_ERR_UNSUPPORTED,
                "a batch of %d tokens needs %zu bytes of workspace; the static buffer of the "
                "no-alloc entry point holds %zu", n_tokens, need, kStaticScratchBytes);
  int dev = -1;
  HIP_TRY(hipGetDevice(&dev));
  unsigned char* base = nullptr;  // the array's address on this GPU, never the array's name
  int rc = resolve_static_scratch(dev, &base);
  if (rc) return rc;
  WsView v{};
  ws_layout(L, n_tokens, y_parts, base, &v);
  hipStream_t s = (hipStream_t)stream;
  // The buffer keeps the last call's contents (possibly another layer's, laid out otherwise):
  // what must start from a known state is rewritten by a kernel on the call's own stream.
  HIP_TRY(launch_workspace_init(L, v, n_tokens, s));
  return run_forward(L, d_x, x_dtype, n_tokens, d_out, s, kStageRouter, kStageCombine, nullptr, &v,
                     true);
}

int atenia_moe_hip_layer_forward(AteniaMoeLayer* L, const float* x_host, int n_tokens,
                                 float* out_host) {
  if (!valid_handle(L)) return fail(ATENIA_MOE_ERR_HANDLE, "invalid layer handle");
  if (n_tokens < 0) return fail(ATENIA_MOE_ERR_DIM, "negative token count");
  if (n_tokens == 0) return ATENIA_MOE_OK;
  if (!x_host || !out_host) return fail(ATENIA_MOE_ERR_DIM, "null activation pointer");
  std::lock_guard<std::mutex> lock(L->mu);
  int rc = ensure_workspace(L, n_tokens);
  if (rc) return rc;
  if (n_tokens >= 2 * kHostChunkTokens && !(is_page_locked(x_host) && is_page_locked(out_host)))
    return forward_host_staged(L, x_host, n_tokens, out_host);
  const size_t bytes = (size_t)n_tokens * L->d * 4;
  HIP_TRY(hipMemcpyAsync(L->x_in.p, x_host, bytes, hipMemcpyHostToDevice, L->stream));
  rc = run_forward(L, L->x_in.p, ATENIA_MOE_ACT_F32, n_tokens, L->out.as<float>(), L->stream,
                   kStageRouter, kStageCombine);
  if (rc) return rc;
  HIP_TRY(hipMemcpyAsync(out_host, L->out.p, bytes, hipMemcpyDeviceToHost, L->stream));
  return read_status(L, L->stream, nullptr, nullptr);
}

namespace {
// RMSNorm * gamma into the handle's xn, then the whole pipeline on xn with x1 as the residual.
int run_block(AteniaMoeLayer* L, const float* d_x1, int T, const float* d_gamma, float eps,
              int norm_policy, float* d_out, hipStream_t s) {
  int rc = ensure_workspace(L, T);
  if (rc) return rc;
  if ((rc = L->xn.ensure((size_t)L->ws.cap_tokens * L->d * 4))) return rc;
  NormArgs na{};
  na.x = d_x1;
  na.gamma = d_gamma;
  na.eps = eps;
  na.policy = norm_policy;
  na.T = T;
  na.d = L->d;
  na.y = L->xn.as<float>();
  HIP_TRY(launch_rmsnorm_gamma(na, s));
  L->normed_T = T;
  return run_forward(L, L->xn.p, ATENIA_MOE_ACT_F32, T, d_out, s, kStageRouter, kStageCombine,
                     d_x1);
}

int block_prologue(AteniaMoeLayer* L, int n_tokens, const void* x1, const void* gamma,
                   const void* out, float eps, int norm_policy) {
  if (!valid_handle(L)) return fail(ATENIA_MOE_ERR_HANDLE, "invalid layer handle");
  if (n_tokens < 0) return fail(ATENIA_MOE_ERR_DIM, "negative token count");
  if (n_tokens > 0 && (!x1 || !gamma || !out))
    return fail(ATENIA_MOE_ERR_DIM, "null activation or gamma pointer");
  if (norm_policy != ATENIA_MOE_NORM_GRAPH_F32 && norm_policy != ATENIA_MOE_NORM_F64)
    return fail(ATENIA_MOE_ERR_DIM, "unknown norm policy %d", norm_policy);
  if (!(eps >= 0.0f)) return fail(ATENIA_MOE_ERR_DIM, "eps must be a non-negative number");
  if ((long long)n_tokens * L->k > (long long)INT_MAX / 4)
    return fail(ATENIA_MOE_ERR_DIM, "too many tokens");
  return ATENIA_MOE_OK;
}
}  // namespace

int atenia_moe_hip_layer_block_forward_device(AteniaMoeLayer* L, const float* d_x1, int n_tokens,
                                              const float* d_gamma, float eps, int norm_policy,
                                              float* d_out, void* stream) {
  int rc = block_prologue(L, n_tokens, d_x1, d_gamma, d_out, eps, norm_policy);
  if (rc || n_tokens == 0) return rc;
  std::lock_guard<std::mutex> lock(L->mu);
  return run_block(L, d_x1, n_tokens, d_gamma, eps, norm_policy, d_out, (hipStream_t)stream);
}

int atenia_moe_hip_layer_block_forward(AteniaMoeLayer* L, const float* x1_host, int n_tokens,
                                       const float* gamma_host, float eps, int norm_policy,
                                       float* out_host) {
  int rc = block_prologue(L, n_tokens, x1_host, gamma_host, out_host, eps, norm_policy);
  if (rc || n_tokens == 0) return rc;
  std::lock_guard<std::mutex> lock(L->mu);
  if ((rc = ensure_workspace(L, n_tokens))) return rc;
  if ((rc = L->gamma_in.ensure((size_t)L->d * 4))) return rc;
  const size_t bytes = (size_t)n_tokens * L->d * 4;
  HIP_TRY(hipMemcpyAsync(L->x_in.p, x1_host, bytes, hipMemcpyHostToDevice, L->stream));
  HIP_TRY(hipMemcpyAsync(L->gamma_in.p, gamma_host, (size_t)L->d * 4, hipMemcpyHostToDevice,
                         L->stream));
  rc = run_block(L, L->x_in.as<float>(), n_tokens, L->gamma_in.as<float>(), eps, norm_policy,
                 L->out.as<float>(), L->stream);
  if (rc) return rc;
  HIP_TRY(hipMemcpyAsync(out_host, L->out.p, bytes, hipMemcpyDeviceToHost, L->stream));
  return read_status(L, L->stream, nullptr, nullptr);
}

int atenia_moe_hip_layer_last_normed(AteniaMoeLayer* L, float* h2_host) {
  if (!valid_handle(L)) return fail(ATENIA_MOE_ERR_HANDLE, "invalid layer handle");
  if (!h2_host) return fail(ATENIA_MOE_ERR_DIM, "null output pointer");
  std::lock_guard<std::mutex> lock(L->mu);
  if (L->normed_T <= 0 || !L->xn.p) return fail(ATENIA_MOE_ERR_DIM, "no block forward has run on this handle");
  HIP_TRY(hipDeviceSynchronize());
  HIP_TRY(hipMemcpy(h2_host, L->xn.p, (size_t)L->normed_T * L->d * 4, hipMemcpyDeviceToHost));
  return ATENIA_MOE_OK;
}

namespace {
int stage_prologue(AteniaMoeLayer* L, int n_tokens) {
  if (!valid_handle(L)) return fail(ATENIA_MOE_ERR_HANDLE, "invalid layer handle");
  if (n_tokens <= 0) return fail(ATENIA_MOE_ERR_DIM, "token count must be positive");
  if ((long long)n_tokens * L->k > (long long)INT_MAX / 4)
    return fail(ATENIA_MOE_ERR_DIM, "too many tokens");
  return ATENIA_MOE_OK;
}
}  // namespace

int atenia_moe_router_launch_device(AteniaMoeLayer* L, const void* d_x, int x_dtype,
                                    int n_tokens, int32_t* d_idx, float* d_w, void* stream) {
  int rc = stage_prologue(L, n_tokens);
  if (rc) return rc;
  if (!d_x) return fail(ATENIA_MOE_ERR_DIM, "null activation pointer");
  if (x_dtype != ATENIA_MOE_ACT_F32 && x_dtype != ATENIA_MOE_ACT_BF16)
    return fail(ATENIA_MOE_ERR_DIM, "unknown activation dtype %d", x_dtype);
  std::lock_guard<std::mutex> lock(L->mu);
  rc = ensure_workspace(L, n_tokens);
  if (rc) return rc;
  hipStream_t s = (hipStream_t)stream;
  rc = run_forward(L, d_x, x_dtype, n_tokens, nullptr, s, kStageRouter, kStageRouter);
  if (rc) return rc;
  const size_t n = (size_t)n_tokens * L->k;
  const WsView& V = L->cur;
  if (d_idx) HIP_TRY(hipMemcpyAsync(d_idx, V.idx, n * 4, hipMemcpyDeviceToDevice, s));
  if (d_w) HIP_TRY(hipMemcpyAsync(d_w, V.w, n * 4, hipMemcpyDeviceToDevice, s));
  return ATENIA_MOE_OK;
}

int atenia_moe_permute_launch_device(AteniaMoeLayer* L, int n_tokens, int32_t* d_counts,
                                     int32_t* d_offsets, int32_t* d_perm, void* stream) {
  int rc = stage_prologue(L, n_tokens);
  if (rc) return rc;
  std::lock_guard<std::mutex> lock(L->mu);
  hipStream_t s = (hipStream_t)stream;
  rc = run_forward(L, nullptr, L->wdtype == ATENIA_MOE_WEIGHT_F32 ? ATENIA_MOE_ACT_F32 : ATENIA_MOE_ACT_BF16,
                   n_tokens, nullptr, s, kStagePermute, kStagePermute);
  if (rc) return rc;
  const WsView& V = L->cur;
  if (d_counts)
    HIP_TRY(hipMemcpyAsync(d_counts, V.counts, (size_t)L->E * 4, hipMemcpyDeviceToDevice, s));
  if (d_offsets)
    HIP_TRY(hipMemcpyAsync(d_offsets, V.offsets, ((size_t)L->E + 1) * 4,
                           hipMemcpyDeviceToDevice, s));
  if (d_perm)
    HIP_TRY(hipMemcpyAsync(d_perm, V.perm, (size_t)n_tokens * L->k * 4,
                           hipMemcpyDeviceToDevice, s));
  return ATENIA_MOE_OK;
}

int atenia_moe_expert_ffn_launch_device(AteniaMoeLayer* L, const void* d_x, int x_dtype,
                                        int n_tokens, void* stream) {
  int rc = stage_prologue(L, n_tokens);
  if (rc) return rc;
  if (!d_x) return fail(ATENIA_MOE_ERR_DIM, "null activation pointer");
  if (x_dtype != ATENIA_MOE_ACT_F32 && x_dtype != ATENIA_MOE_ACT_BF16)
    return fail(ATENIA_MOE_ERR_DIM, "unknown activation dtype %d", x_dtype);
  std::lock_guard<std::mutex> lock(L->mu);
  return run_forward(L, d_x, x_dtype, n_tokens, nullptr, (hipStream_t)stream, kStageFfn, kStageFfn);
}

int atenia_moe_combine_launch_device(AteniaMoeLayer* L, int n_tokens, float* d_out,
                                     void* stream) {
  int rc = stage_prologue(L, n_tokens);
  if (rc) return rc;
  if (!d_out) return fail(ATENIA_MOE_ERR_DIM, "null output pointer");
  std::lock_guard<std::mutex> lock(L->mu);
  return run_forward(L, nullptr, L->wdtype == ATENIA_MOE_WEIGHT_F32 ? ATENIA_MOE_ACT_F32 : ATENIA_MOE_ACT_BF16,
                     n_tokens, d_out, (hipStream_t)stream, kStageCombine, kStageCombine);
}

int atenia_moe_hip_layer_status(AteniaMoeLayer* L, void* stream, int32_t* token,
                                int32_t* expert) {
  if (!valid_handle(L)) return fail(ATENIA_MOE_ERR_HANDLE, "invalid layer handle");
  std::lock_guard<std::mutex> lock(L->mu);
  return read_status(L, (hipStream_t)stream, token, expert);
}

int atenia_moe_hip_layer_last_non_finite(AteniaMoeLayer* L, int32_t* token, int32_t* expert) {
  if (!valid_handle(L)) return fail(ATENIA_MOE_ERR_HANDLE, "invalid layer handle");
  std::lock_guard<std::mutex> lock(L->mu);
  if (token) *token = L->nf_token;
  if (expert) *expert = L->nf_expert;
  return ATENIA_MOE_OK;
}

int atenia_moe_hip_layer_set_v3_router(AteniaMoeLayer* L, int n_group, int topk_group,
                                       double routed_scaling_factor, int norm_topk_prob,
                                       const float* e_score_correction_bias_host) {
  if (!valid_handle(L)) return fail(ATENIA_MOE_ERR_HANDLE, "invalid layer handle");
  // V3RouterConfig::validate (src/moe/v3_router.rs:148-181), same order, same texts.
  if (n_group <= 0) return fail(ATENIA_MOE_ERR_K, "v3-router: n_group must be > 0");
  if (topk_group <= 0) return fail(ATENIA_MOE_ERR_K, "v3-router: topk_group must be > 0");
  if (L->E % n_group != 0)
    return fail(ATENIA_MOE_ERR_K, "v3-router: n_routed_experts (%d) not divisible by n_group (%d)",
                L->E, n_group);
  const int epg = L->E / n_group;
  if (epg < 2)
    return fail(ATENIA_MOE_ERR_K, "v3-router: experts_per_group (%d) < 2 (HF takes top-2 per group)",
                epg);
  if (topk_group > n_group)
    return fail(ATENIA_MOE_ERR_K, "v3-router: topk_group (%d) > n_group (%d)", topk_group, n_group);
  if (L->k > topk_group * epg)
    return fail(ATENIA_MOE_ERR_K, "v3-router: top_k (%d) exceeds experts in selected groups (%d)",
                L->k, topk_group * epg);
  if (!e_score_correction_bias_host)
    return fail(ATENIA_MOE_ERR_DIM, "v3-router: e_score_correction_bias length 0 != n_routed_experts %d",
                L->E);
  for (int i = 0; i < L->E; ++i)
    if (!std::isfinite(e_score_correction_bias_host[i]))
      return fail(ATENIA_MOE_ERR_NON_FINITE, "v3-router: e_score_correction_bias at %d is non-finite", i);
  if (!std::isfinite(routed_scaling_factor))
    return fail(ATENIA_MOE_ERR_NON_FINITE, "v3-router: routed_scaling_factor is non-finite");
  if (L->router_bias.p)
    return fail(ATENIA_MOE_ERR_UNSUPPORTED, "v3-router: the layer was created with an additive router bias");
  if (L->E > 256) return fail(ATENIA_MOE_ERR_UNSUPPORTED, "v3-router: at most 256 experts");
  std::lock_guard<std::mutex> lock(L->mu);
  int rc = upload_f32(e_score_correction_bias_host, (size_t)L->E, L->v3_bias);
  if (rc) return rc;
  L->v3_n_group = n_group;
  L->v3_topk_group = topk_group;
  L->v3_norm = norm_topk_prob ? 1 : 0;
  L->v3_scale = routed_scaling_factor;
  for (int st = 0; st < 4; ++st) L->stage_T[st] = -1;
  return ATENIA_MOE_OK;
}

int atenia_moe_hip_layer_route(AteniaMoeLayer* L, const float* x_host, int n_tokens,
                               int32_t* idx_host, float* w_host) {
  if (!valid_handle(L)) return fail(ATENIA_MOE_ERR_HANDLE, "invalid layer handle");
  if (n_tokens < 0) return fail(ATENIA_MOE_ERR_DIM, "negative token count");
  if (n_tokens == 0) return ATENIA_MOE_OK;
  if (!x_host || !idx_host || !w_host) return fail(ATENIA_MOE_ERR_DIM, "null pointer");
  std::lock_guard<std::mutex> lock(L->mu);
  int rc = ensure_workspace(L, n_tokens);
  if (rc) return rc;
  HIP_TRY(hipMemcpyAsync(L->x_in.p, x_host, (size_t)n_tokens * L->d * 4, hipMemcpyHostToDevice,
                         L->stream));
  rc = run_forward(L, L->x_in.p, ATENIA_MOE_ACT_F32, n_tokens, nullptr, L->stream, kStageRouter,
                   kStageRouter);
  if (rc) return rc;
  rc = read_status(L, L->stream, nullptr, nullptr);
  if (rc) return rc;
  const size_t P = (size_t)n_tokens * L->k;
  const WsView& V = L->cur;
  HIP_TRY(hipMemcpy(idx_host, V.idx, P * 4, hipMemcpyDeviceToHost));
  HIP_TRY(hipMemcpy(w_host, V.w, P * 4, hipMemcpyDeviceToHost));
  return ATENIA_MOE_OK;
}

int atenia_moe_hip_layer_permute(AteniaMoeLayer* L, const int32_t* idx_host, int n_tokens,
                                 int32_t* counts_host, int32_t* offsets_host,
                                 int32_t* perm_host) {
  if (!valid_handle(L)) return fail(ATENIA_MOE_ERR_HANDLE, "invalid layer handle");
  if (n_tokens < 0) return fail(ATENIA_MOE_ERR_DIM, "negative token count");
  if (!idx_host || !counts_host || !offsets_host || (n_tokens > 0 && !perm_host))
    return fail(ATENIA_MOE_ERR_DIM, "null pointer");
  if (n_tokens == 0) {
    for (int e = 0; e < L->E; ++e) counts_host[e] = 0;
    for (int e = 0; e <= L->E; ++e) offsets_host[e] = 0;
    return ATENIA_MOE_OK;
  }
  const size_t P = (size_t)n_tokens * L->k;
  for (size_t p = 0; p < P; ++p)
    if (idx_host[p] < 0 || idx_host[p] >= L->E)
      return fail(ATENIA_MOE_ERR_DIM, "expert index %d out of range at pair %zu", idx_host[p], p);
  std::lock_guard<std::mutex> lock(L->mu);
  int rc = ensure_workspace(L, n_tokens);
  if (rc) return rc;
  const WsView& V = L->ws;
  L->cur = V;
  // the routing, the grouping and the row tiles no longer describe one forward
  for (int st = 0; st < 4; ++st) L->stage_T[st] = -1;
  L->last_T = 0;
  HIP_TRY(hipDeviceSynchronize());  // a forward may still be using the workspace on some stream
  HIP_TRY(hipMemcpyAsync(V.idx, idx_host, P * 4, hipMemcpyHostToDevice, L->stream));
  PermuteArgs pa{};
  pa.idx = V.idx;
  pa.T = n_tokens;
  pa.k = L->k;
  pa.E = L->E;
  pa.counts = V.counts;
  pa.offsets = V.offsets;
  pa.perm = V.perm;
  pa.inv = V.inv;
  pa.active = V.active;
  pa.n_active = V.n_active;
  pa.blk_counts = V.blk_counts;
  pa.shared_offsets = nullptr;
  pa.tile_group = nullptr;
  pa.tile_m0 = nullptr;
  pa.n_tiles = nullptr;
  pa.shared_n_tiles = nullptr;
  pa.tile_rows = nullptr;
  pa.tile_li = nullptr;
  pa.max_tile_groups = 8;
  HIP_TRY(launch_permute(pa, L->stream, nullptr));
  if (hipStreamSynchronize(L->stream) != hipSuccess)
    return fail(ATENIA_MOE_ERR_SYNC, "stream synchronisation failed");
  HIP_TRY(hipMemcpy(counts_host, V.counts, (size_t)L->E * 4, hipMemcpyDeviceToHost));
  HIP_TRY(hipMemcpy(offsets_host, V.offsets, (size_t)(L->E + 1) * 4, hipMemcpyDeviceToHost));
  HIP_TRY(hipMemcpy(perm_host, V.perm, P * 4, hipMemcpyDeviceToHost));
  return ATENIA_MOE_OK;
}

int atenia_moe_hip_layer_last_routing(AteniaMoeLayer* L, int32_t* idx_host, float* w_host,
                                      int32_t* counts_host, int32_t* offsets_host,
                                      int32_t* perm_host) {
  if (!valid_handle(L)) return fail(ATENIA_MOE_ERR_HANDLE, "invalid layer handle");
  std::lock_guard<std::mutex> lock(L->mu);
  if (L->last_T <= 0) return fail(ATENIA_MOE_ERR_DIM, "no forward has run on this handle");
  if (hipDeviceSynchronize() != hipSuccess)
    return fail(ATENIA_MOE_ERR_SYNC, "device synchronisation failed");
  const size_t P = (size_t)L->last_T * L->k;
  const WsView& V = L->cur;
  if (idx_host) HIP_TRY(hipMemcpy(idx_host, V.idx, P * 4, hipMemcpyDeviceToHost));
  if (w_host) HIP_TRY(hipMemcpy(w_host, V.w, P * 4, hipMemcpyDeviceToHost));
  if (counts_host)
    HIP_TRY(hipMemcpy(counts_host, V.counts, (size_t)L->E * 4, hipMemcpyDeviceToHost));
  if (offsets_host)
    HIP_TRY(hipMemcpy(offsets_host, V.offsets, (size_t)(L->E + 1) * 4, hipMemcpyDeviceToHost));
  if (perm_host) HIP_TRY(hipMemcpy(perm_host, V.perm, P * 4, hipMemcpyDeviceToHost));
  return ATENIA_MOE_OK;
}

int atenia_moe_hip_layer_last_expert_outputs(AteniaMoeLayer* L, float* y_host,
                                             float* y_shared_host) {
  if (!valid_handle(L)) return fail(ATENIA_MOE_ERR_HANDLE, "invalid layer handle");
  std::lock_guard<std::mutex> lock(L->mu);
  if (L->last_T <= 0) return fail(ATENIA_MOE_ERR_DIM, "no forward has run on this handle");
  if (hipDeviceSynchronize() != hipSuccess)
    return fail(ATENIA_MOE_ERR_SYNC, "device synchronisation failed");
  const size_t P = (size_t)L->last_T * L->k;
  const WsView& V = L->cur;
  // one buffer of expert outputs as f32, whatever it is stored as
  auto fetch = [&](float* dst, const float* src, size_t n, bool bf16) -> int {
    if (!bf16) {
      HIP_TRY(hipMemcpy(dst, src, n * 4, hipMemcpyDeviceToHost));
      return ATENIA_MOE_OK;
    }
    std::vector<uint16_t> bits(n);
    HIP_TRY(hipMemcpy(bits.data(), src, n * 2, hipMemcpyDeviceToHost));
    for (size_t i = 0; i < n; ++i) {
      const uint32_t u = (uint32_t)bits[i] << 16;
      memcpy(dst + i, &u, 4);
    }
    return ATENIA_MOE_OK;
  };
  if (y_host) {
    const size_t n = P * L->d;
    const size_t part_bytes = n * (L->last_y_bf16 ? 2 : 4);  // between the partial buffers
    int rc = fetch(y_host, V.y, n, L->last_y_bf16);
    if (rc) return rc;
    if (L->last_split) {  // add the partial buffers the down phase wrote for split tail tiles
      const int fc = (L->d + 255) / 256;
      std::vector<uint8_t> flags(P * fc);
      HIP_TRY(hipMemcpy(flags.data(), V.part_flags, flags.size(), hipMemcpyDeviceToHost));
      std::vector<float> part(n);
      for (int i = 1; i < kMaxYParts; ++i) {
        bool any = false;
        for (uint8_t f : flags) any = any || f > i;
        if (!any) break;
        if ((rc = fetch(part.data(), (const float*)((const uint8_t*)V.y + (size_t)i * part_bytes), n,
                        L->last_y_bf16)))
          return rc;
        for (size_t pr = 0; pr < P; ++pr)
          for (int c = 0; c < L->d; ++c)
            if (flags[pr * fc + c / 256] > i) y_host[pr * L->d + c] += part[pr * L->d + c];
      }
    }
  }
  if (y_shared_host && L->fs > 0) {
    int rc = fetch(y_shared_host, V.ys, (size_t)L->last_T * L->d, L->last_ys_bf16);
    if (rc) return rc;
  }
  return ATENIA_MOE_OK;
}

int atenia_moe_hip_layer_last_down_split(AteniaMoeLayer* L, uint8_t* parts_host) {
  if (!valid_handle(L)) return fail(ATENIA_MOE_ERR_HANDLE, "invalid layer handle");
  if (!parts_host) return fail(ATENIA_MOE_ERR_DIM, "null pointer");
  std::lock_guard<std::mutex> lock(L->mu);
  if (L->last_T <= 0) return fail(ATENIA_MOE_ERR_DIM, "no forward has run on this handle");
  if (hipDeviceSynchronize() != hipSuccess)
    return fail(ATENIA_MOE_ERR_SYNC, "device synchronisation failed");
  const size_t n = (size_t)L->last_T * L->k * ((L->d + 255) / 256);
  if (L->last_split) HIP_TRY(hipMemcpy(parts_host, L->cur.part_flags, n, hipMemcpyDeviceToHost));
  else memset(parts_host, 1, n);
  return ATENIA_MOE_OK;
}

int atenia_moe_hip_layer_set_numeric_policy(AteniaMoeLayer* L, int policy) {
  if (!valid_handle(L)) return fail(ATENIA_MOE_ERR_HANDLE, "invalid layer handle");
  if (policy != ATENIA_MOE_POLICY_CERTIFIED && policy != ATENIA_MOE_POLICY_STRICT &&
      policy != ATENIA_MOE_POLICY_FAST)
    return fail(ATENIA_MOE_ERR_DIM, "unknown numeric policy %d", policy);
  std::lock_guard<std::mutex> lock(L->mu);
  L->policy = policy;
  return ATENIA_MOE_OK;
}

int atenia_moe_hip_layer_set_profiling(AteniaMoeLayer* L, int enabled) {
  if (!valid_handle(L)) return fail(ATENIA_MOE_ERR_HANDLE, "invalid layer handle");
  std::lock_guard<std::mutex> lock(L->mu);
  if (enabled && !L->ev_valid) {
    for (auto& e : L->ev) HIP_TRY(hipEventCreate(&e));
    L->ev_valid = true;
  }
  L->profiling = enabled != 0;
  return ATENIA_MOE_OK;
}

int atenia_moe_hip_layer_stage_ms(AteniaMoeLayer* L, float ms[ATENIA_MOE_N_STAGES]) {
  if (!valid_handle(L)) return fail(ATENIA_MOE_ERR_HANDLE, "invalid layer handle");
  if (!ms) return fail(ATENIA_MOE_ERR_DIM, "null pointer");
  std::lock_guard<std::mutex> lock(L->mu);
  if (!L->profiling || !L->ev_valid || L->last_T <= 0)
    return fail(ATENIA_MOE_ERR_DIM, "profiling is off or no forward has run");
  if (hipEventSynchronize(L->ev[ATENIA_MOE_N_STAGES - 1]) != hipSuccess)
    return fail(ATENIA_MOE_ERR_SYNC, "event synchronisation failed");
  for (int i = 0; i < ATENIA_MOE_N_STAGES - 1; ++i)
    HIP_TRY(hipEventElapsedTime(&ms[i], L->ev[i], L->ev[i + 1]));
  HIP_TRY(hipEventElapsedTime(&ms[ATENIA_MOE_N_STAGES - 1], L->ev[0],
                              L->ev[ATENIA_MOE_N_STAGES - 1]));
  return ATENIA_MOE_OK;
}

int atenia_moe_hip_layer_stage_launches(AteniaMoeLayer* L, int32_t n[ATENIA_MOE_N_STAGES]) {
  if (!valid_handle(L)) return fail(ATENIA_MOE_ERR_HANDLE, "invalid layer handle");
  if (!n) return fail(ATENIA_MOE_ERR_DIM, "null pointer");
  std::lock_guard<std::mutex> lock(L->mu);
  for (int i = 0; i < ATENIA_MOE_N_STAGES; ++i) n[i] = L->launches[i];
  return ATENIA_MOE_OK;
}

int atenia_moe_hip_layer_expert_kernels(const AteniaMoeLayer* L, int64_t n_tokens,
                                        int32_t family[2]) {
  if (!valid_handle(L)) return fail(ATENIA_MOE_ERR_HANDLE, "invalid layer handle");
  if (!family) return fail(ATENIA_MOE_ERR_DIM, "null pointer");
  if (n_tokens <= 0 || n_tokens > INT32_MAX) return fail(ATENIA_MOE_ERR_DIM, "n_tokens = %lld", (long long)n_tokens);
  const int T = (int)n_tokens;
  if (L->wdtype == ATENIA_MOE_WEIGHT_F32) {
    family[0] = ATENIA_MOE_KERNELS_F32;
    family[1] = L->fs > 0 ? ATENIA_MOE_KERNELS_F32 : -1;
    return ATENIA_MOE_OK;
  }
  const ResolvedPlan r = resolve_plan(L, T);  // the decisions run_forward takes
  family[0] = family_name(r.fam_up);
  family[1] = L->fs > 0 ? family_name(r.s_fam_up) : -1;
  return ATENIA_MOE_OK;
}

int atenia_moe_hip_plan_batch(int num_experts, int top_k, int d_model, int d_ff, int d_ff_shared,
                              int weight_dtype, int group_size, int64_t n_tokens,
                              int32_t plan[8]) {
  if (!plan) return fail(ATENIA_MOE_ERR_DIM, "null pointer");
  if (num_experts < 1 || d_model < 1 || d_ff < 1 || d_ff_shared < 0)
    return fail(ATENIA_MOE_ERR_DIM, "bad dimensions E=%d d=%d f=%d f_s=%d", num_experts, d_model,
                d_ff, d_ff_shared);
  if (top_k < 1 || top_k > num_experts)
    return fail(ATENIA_MOE_ERR_K, "bad k=%d for %d experts", top_k, num_experts);
  if (weight_dtype < 0 || weight_dtype > ATENIA_MOE_WEIGHT_INT8_PER_GROUP)
    return fail(ATENIA_MOE_ERR_DIM, "unknown weight dtype %d", weight_dtype);
  const bool per_group = weight_dtype == ATENIA_MOE_WEIGHT_INT8_PER_GROUP;
  if (per_group && (group_size <= 0 || group_size % kKbInt8 != 0))
    return fail(ATENIA_MOE_ERR_DIM, "per-group int8 needs group_size > 0 and a multiple of %d (got %d)",
                kKbInt8, group_size);
  if (n_tokens <= 0 || n_tokens > INT32_MAX) return fail(ATENIA_MOE_ERR_DIM, "n_tokens = %lld", (long long)n_tokens);
  // a layer of these dimensions, as `create` fills them in (no device memory behind it)
  AteniaMoeLayer L;
  L.E = num_experts;
  L.k = top_k;
  L.d = d_model;
  L.f = d_ff;
  L.fs = d_ff_shared;
  L.wdtype = per_group ? ATENIA_MOE_WEIGHT_INT8_W8A16 : weight_dtype;
  L.group_size = per_group ? group_size : 0;
  const bool f32w = L.wdtype == ATENIA_MOE_WEIGHT_F32;
  const int KB = f32w ? 1 : kb_of(L.wdtype);
  L.d_kpad = round_up(L.d, KB);
  L.f_kpad = round_up(L.f, KB);
  L.fs_kpad = round_up(L.fs, KB);
  auto dims = [&](WeightSet& w, int n_rows, int k_cols) {
    w.n_rows = n_rows;
    w.k_cols = k_cols;
    w.n_pad = f32w ? n_rows : round_up(n_rows, 16);
    w.k_pad = f32w ? k_cols : round_up(k_cols, KB);
    if (per_group) {
      w.group_blocks = group_size / kKbInt8;
      w.n_kgroups = (k_cols + group_size - 1) / group_size;
    }
  };
  dims(L.gate, L.f, L.d);
  dims(L.up, L.f, L.d);
  dims(L.down, L.d, L.f);
  if (L.fs > 0) {
    dims(L.s_gate, L.fs, L.d);
    dims(L.s_up, L.fs, L.d);
    dims(L.s_down, L.d, L.fs);
  }
  for (int i = 0; i < 8; ++i) plan[i] = 0;
  if (f32w) {
    plan[0] = plan[1] = ATENIA_MOE_KERNELS_F32;
    plan[2] = plan[3] = L.fs > 0 ? ATENIA_MOE_KERNELS_F32 : -1;
    return ATENIA_MOE_OK;
  }
  const ResolvedPlan r = resolve_plan(&L, (int)n_tokens);
  plan[0] = family_name(r.fam_up);
  plan[1] = family_name(r.fam_down);
  plan[2] = L.fs > 0 ? family_name(r.s_fam_up) : -1;
  plan[3] = L.fs > 0 ? family_name(r.s_fam_down) : -1;
  plan[4] = r.y_bf16;
  plan[5] = r.ys_bf16;
  plan[6] = r.plan.tall_tiles;
  plan[7] = (r.duo_up ? 1 : 0) | (r.duo_down ? 2 : 0) | (r.plan.q_copy ? 4 : 0);
  return ATENIA_MOE_OK;
}

int atenia_moe_hip_layer_info(const AteniaMoeLayer* L, int64_t info[8]) {
  if (!valid_handle(L)) return fail(ATENIA_MOE_ERR_HANDLE, "invalid layer handle");
  if (!info) return fail(ATENIA_MOE_ERR_DIM, "null pointer");
  info[0] = L->E;
  info[1] = L->k;
  info[2] = L->d;
  info[3] = L->f;
  info[4] = L->fs;
  info[5] = L->conv;
  info[6] = L->wdtype;
  info[7] = L->bytes_per_expert;
  return ATENIA_MOE_OK;
}

int atenia_moe_quantize_per_group_i8(const float* w, size_t rows, size_t cols, size_t group_size,
                                     int8_t* q_out, float* scales_out) {
  if (!w || !q_out || !scales_out) return fail(ATENIA_MOE_ERR_DIM, "null pointer");
  if (group_size == 0) return fail(ATENIA_MOE_ERR_DIM, "group_size must be > 0");
  const size_t ng = (cols + group_size - 1) / group_size;
  for (size_t r = 0; r < rows; ++r)
    for (size_t g = 0; g < ng; ++g) {
      const size_t c0 = g * group_size, c1 = std::min(cols, c0 + group_size);
      float max_abs = 0.0f;
      for (size_t c = c0; c < c1; ++c) {
        const float v = std::fabs(w[r * cols + c]);
        if (v > max_abs) max_abs = v;
      }
      const float sc = std::max(max_abs / 127.0f, 1e-12f);
      scales_out[r * ng + g] = sc;
      for (size_t c = c0; c < c1; ++c) {
        float qf = std::round(w[r * cols + c] / sc);  // half away from zero, like f32::round
        qf = std::min(127.0f, std::max(-127.0f, qf));
        q_out[r * cols + c] = (int8_t)(int32_t)qf;
      }
    }
  return ATENIA_MOE_OK;
}

int atenia_moe_quantize_per_row_i8(const float* w, size_t rows, size_t cols, int8_t* q,
                                   float* scales) {
  if (!w || !q || !scales) return fail(ATENIA_MOE_ERR_DIM, "null pointer");
  for (size_t r = 0; r < rows; ++r) {
    const float* row = w + r * cols;
    float amax = 0.0f;
    for (size_t c = 0; c < cols; ++c) amax = fmaxf(amax, fabsf(row[c]));
    const float scale = amax > 0.0f ? amax / 127.0f : 1.0f;
    scales[r] = scale;
    const float inv = 1.0f / scale;
    for (size_t c = 0; c < cols; ++c) {
      float v = roundf(row[c] * inv);
      v = v < -127.0f ? -127.0f : (v > 127.0f ? 127.0f : v);
      q[r * cols + c] = (int8_t)v;
    }
  }
  return ATENIA_MOE_OK;
}

int atenia_moe_absmax_per_group_symmetric(const float* w, size_t k, size_t n, size_t group_size,
                                          int8_t* q, float* scales) {
  if (!w || !q || !scales) return fail(ATENIA_MOE_ERR_DIM, "null pointer");
  if (group_size == 0) return fail(ATENIA_MOE_ERR_DIM, "group size must be positive");
  // one pass per group of rows: column maxima into the group's scale row, then the quotients
  for (size_t k0 = 0; k0 < k; k0 += group_size) {
    const size_t k1 = k0 + group_size < k ? k0 + group_size : k;
    float* sc = scales + (k0 / group_size) * n;
    for (size_t c = 0; c < n; ++c) sc[c] = 0.0f;
    for (size_t r = k0; r < k1; ++r)
      for (size_t c = 0; c < n; ++c) sc[c] = fmaxf(sc[c], fabsf(w[r * n + c]));
    for (size_t c = 0; c < n; ++c) sc[c] = fmaxf(sc[c] / 127.0f, 1e-12f);
    for (size_t r = k0; r < k1; ++r)
      for (size_t c = 0; c < n; ++c) {
        float v = roundf(w[r * n + c] / sc[c]);
        v = v < -127.0f ? -127.0f : (v > 127.0f ? 127.0f : v);
        q[r * n + c] = (int8_t)v;
      }
  }
  return ATENIA_MOE_OK;
}

int atenia_moe_absmax_per_channel_symmetric(const float* w, size_t k, size_t n, int8_t* q,
                                            float* scales) {
  // one group spanning all of K
  return atenia_moe_absmax_per_group_symmetric(w, k, n, k > 0 ? k : 1, q, scales);
}

int atenia_moe_f32_to_bf16_trunc(const float* src, size_t n, uint16_t* dst) {
  if (!src || !dst) return fail(ATENIA_MOE_ERR_DIM, "null pointer");
  for (size_t i = 0; i < n; ++i) {
    uint32_t u;
    memcpy(&u, src + i, 4);
    dst[i] = (uint16_t)(u >> 16);
  }
  return ATENIA_MOE_OK;
}

}  // extern "C"
