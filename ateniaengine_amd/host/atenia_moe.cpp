// Implementation of the host mirror over the C ABI (see atenia_moe.hpp for the reference
// interface each part follows).
#include "atenia_moe.hpp"

#include <algorithm>
#include <cstdlib>
#include <cctype>
#include <atomic>
#include <cmath>
#include <cstring>
#include <map>
#include <utility>

#include "../../include/atenia_moe_hip.h"

namespace atenia {
namespace moe {

// ---- error text: the reference's Display implementations -------------------------------------
std::string MoeConfigError::to_string() const {
  switch (kind) {  // src/moe/layer.rs:56-75
    case ZeroExperts: return "moe-config: num_experts is 0";
    case ZeroExpertsPerToken: return "moe-config: experts_per_token is 0";
    case ExpertsPerTokenExceedsCount:
      return "moe-config: experts_per_token (" + std::to_string(per_token) + ") > num_experts (" +
             std::to_string(total) + ")";
    case ZeroDModel: return "moe-config: d_model is 0";
    case ZeroDFf: return "moe-config: d_ff is 0";
  }
  return "moe-config";
}

std::string MoeDenseError::to_string() const {
  switch (kind) {  // src/moe/dense.rs:51-69
    case DimMismatch:
      return std::string("moe-dense: ") + what + " dim mismatch: expected " +
             std::to_string(expected) + ", got " + std::to_string(actual);
    case WeightShapeMismatch:
      return std::string("moe-dense: ") + what + " weight shape mismatch: expected " +
             std::to_string(expected) + " elems, got " + std::to_string(actual);
    case NoExperts: return "moe-dense: layer has no experts";
    case RouterExpertCountMismatch:
      return "moe-dense: router expert count (" + std::to_string(expected) + ") != experts (" +
             std::to_string(actual) + ")";
  }
  return "moe-dense";
}

std::string MoeSparseError::to_string() const {
  switch (kind) {  // src/moe/sparse.rs:52-72
    case ZeroK: return "moe-sparse: k must be > 0";
    case KExceedsExperts:
      return "moe-sparse: k (" + std::to_string(k) + ") exceeds num_experts (" +
             std::to_string(num_experts) + ")";
    case NonFiniteWeight:
      return "moe-sparse: routing weight at " + std::to_string(index) + " is non-finite";
    case NegativeWeight:
      return "moe-sparse: routing weight at " + std::to_string(index) + " is negative";
    case SelectedSumNonPositive: return "moe-sparse: selected top-k weights sum to <= 0";
    case Dense: return "moe-sparse: " + dense.to_string();
  }
  return "moe-sparse";
}

std::string MoeBindingError::to_string() const {
  const std::string L = std::to_string(layer_id);
  switch (kind) {  // src/moe/binding.rs:72-113
    case LayerNotFound: return "moe-binding: layer " + L + " has no MoE weights";
    case NoExperts: return "moe-binding: layer " + L + " has no experts";
    case IncompleteExpert:
      return "moe-binding: layer " + L + " expert " + std::to_string(expert_id) +
             " is missing a gate/up/down projection";
    case MissingRouter: return "moe-binding: layer " + L + " has no router tensor";
    case UnresolvedTensor: return "moe-binding: byte resolver returned no data for '" + name + "'";
    case BadRank:
      return "moe-binding: tensor '" + name + "' has rank " + std::to_string(rank) +
             ", expected 2-D [rows, cols]";
    case ShapeInconsistency: return "moe-binding: shape inconsistency: " + detail;
    case DataLengthMismatch:
      return "moe-binding: tensor '" + name + "' data length " + std::to_string(actual) +
             " != shape product " + std::to_string(expected);
    case MissingPackedTensor:
      return "moe-binding: layer " + L + " missing packed expert tensor '" + which + "'";
    case PackedBadRank:
      return "moe-binding: packed tensor '" + name + "' has rank " + std::to_string(rank) + ", expected 3-D";
    case Dense: return "moe-binding: " + dense.to_string();
  }
  return "moe-binding";
}

std::string V3RouterError::to_string() const {
  const std::string A = std::to_string(a), B = std::to_string(b);
  switch (kind) {  // src/moe/v3_router.rs:96-122
    case UnsupportedScoringFunc:
      return "v3-router: unsupported scoring_func '" + got + "' (only 'sigmoid')";
    case ExpertsNotDivisibleByGroups:
      return "v3-router: n_routed_experts (" + A + ") not divisible by n_group (" + B + ")";
    case GroupTooSmall:
      return "v3-router: experts_per_group (" + A + ") < 2 (HF takes top-2 per group)";
    case TopkGroupExceedsGroups: return "v3-router: topk_group (" + A + ") > n_group (" + B + ")";
    case TopKExceedsSelectable:
      return "v3-router: top_k (" + A + ") exceeds experts in selected groups (" + B + ")";
    case ZeroParameter: return std::string("v3-router: ") + what + " must be > 0";
    case LengthMismatch:
      return std::string("v3-router: ") + what + " length " + B + " != n_routed_experts " + A;
    case NonFinite: return std::string("v3-router: ") + what + " at " + A + " is non-finite";
    case TopKMismatch:
      return "v3-router: top_k (" + A + ") differs from the layer's experts_per_token (" + B + ")";
  }
  return "v3-router";
}

Result<ScoringFunc, V3RouterError> parse_scoring_func(const std::string& s) {
  typedef Result<ScoringFunc, V3RouterError> R;
  if (s == "sigmoid") return R::Ok(ScoringFunc::Sigmoid);
  V3RouterError e{V3RouterError::UnsupportedScoringFunc};
  e.got = s;
  return R::Err(e);
}

std::optional<V3RouterError> V3RouterConfig::validate() const {
  auto err = [](V3RouterError::Kind k, size_t a = 0, size_t b = 0, const char* what = "") {
    V3RouterError e{k};
    e.a = a;
    e.b = b;
    e.what = what;
    return e;
  };
  if (top_k == 0) return err(V3RouterError::ZeroParameter, 0, 0, "top_k");
  if (n_group == 0) return err(V3RouterError::ZeroParameter, 0, 0, "n_group");
  if (topk_group == 0) return err(V3RouterError::ZeroParameter, 0, 0, "topk_group");
  if (n_routed_experts % n_group != 0)
    return err(V3RouterError::ExpertsNotDivisibleByGroups, n_routed_experts, n_group);
  const size_t per_group = n_routed_experts / n_group;
  if (per_group < 2) return err(V3RouterError::GroupTooSmall, per_group);
  if (topk_group > n_group) return err(V3RouterError::TopkGroupExceedsGroups, topk_group, n_group);
  if (top_k > topk_group * per_group)
    return err(V3RouterError::TopKExceedsSelectable, top_k, topk_group * per_group);
  return std::nullopt;
}

std::string MoeLayerError::to_string() const {
  switch (kind) {
    case Config: return "moe-layer: " + config.to_string();
    case Binding: return "moe-layer: " + binding.to_string();
    case Sparse: return "moe-layer: " + sparse.to_string();
    case ConfigMismatch: return "moe-layer: config mismatch: " + detail;
    case SharedExpertMissing:
      return "moe-layer: layer " + std::to_string(layer_id) + " has no shared-expert tensors";
    case SharedExpertIncomplete:
      return "moe-layer: layer " + std::to_string(layer_id) + " shared expert is missing gate/up/down";
    case MixedExpertFormat:
      return "moe-layer: layer " + std::to_string(layer_id) +
             " has both classic and packed expert tensors";
    case Device: return "moe-layer: device path failed (rc " + std::to_string(rc) + "): " + detail;
  }
  return "moe-layer";
}

namespace {
MoeLayerError dense_dim_error(const char* what, size_t expected, size_t actual) {
  MoeLayerError e{MoeLayerError::Sparse};
  e.sparse.kind = MoeSparseError::Dense;
  e.sparse.dense = MoeDenseError{MoeDenseError::DimMismatch, what, expected, actual};
  return e;
}
MoeLayerError device_error(int rc) {
  MoeLayerError e{MoeLayerError::Device};
  e.rc = rc;
  e.detail = atenia_moe_hip_last_error_string();
  return e;
}
}  // namespace

// ---- config / parts -----------------------------------------------------------------------
std::optional<MoeConfigError> MoeLayerConfig::validate() const {
  if (num_experts == 0) return MoeConfigError{MoeConfigError::ZeroExperts};
  if (experts_per_token == 0) return MoeConfigError{MoeConfigError::ZeroExpertsPerToken};
  if (experts_per_token > num_experts)
    return MoeConfigError{MoeConfigError::ExpertsPerTokenExceedsCount, experts_per_token, num_experts};
  if (d_model == 0) return MoeConfigError{MoeConfigError::ZeroDModel};
  if (d_ff == 0) return MoeConfigError{MoeConfigError::ZeroDFf};
  return std::nullopt;
}

Result<MoeLayerConfig, MoeConfigError> MoeLayerConfig::make(size_t num_experts,
                                                            size_t experts_per_token,
                                                            bool has_shared_expert, size_t d_model,
                                                            size_t d_ff) {
  MoeLayerConfig c{num_experts, experts_per_token, has_shared_expert, d_model, d_ff};
  if (auto e = c.validate()) return Result<MoeLayerConfig, MoeConfigError>::Err(*e);
  return Result<MoeLayerConfig, MoeConfigError>::Ok(c);
}

Result<MoeDenseExpert, MoeDenseError> MoeDenseExpert::make(size_t d_model, size_t d_ff,
                                                           std::vector<float> w_gate,
                                                           std::vector<float> w_up,
                                                           std::vector<float> w_down) {
  typedef Result<MoeDenseExpert, MoeDenseError> R;
  if (w_gate.size() != d_ff * d_model)
    return R::Err({MoeDenseError::WeightShapeMismatch, "w_gate", d_ff * d_model, w_gate.size()});
  if (w_up.size() != d_ff * d_model)
    return R::Err({MoeDenseError::WeightShapeMismatch, "w_up", d_ff * d_model, w_up.size()});
  if (w_down.size() != d_model * d_ff)
    return R::Err({MoeDenseError::WeightShapeMismatch, "w_down", d_model * d_ff, w_down.size()});
  MoeDenseExpert e;
  e.d_model = d_model;
  e.d_ff = d_ff;
  e.w_gate = std::move(w_gate);
  e.w_up = std::move(w_up);
  e.w_down = std::move(w_down);
  return R::Ok(std::move(e));
}

std::vector<float> QInt8Tensor::dequantize() const {
  std::vector<float> out(rows * cols);
  for (size_t r = 0; r < rows; ++r) {
    const float sc = scales[r];
    for (size_t c = 0; c < cols; ++c) out[r * cols + c] = (float)q[r * cols + c] * sc;
  }
  return out;
}

Result<MoeDenseExpert, MoeDenseError> MoeDenseExpert::from_qint8(size_t d_model, size_t d_ff,
                                                                 QInt8Tensor gate, QInt8Tensor up,
                                                                 QInt8Tensor down) {
  typedef Result<MoeDenseExpert, MoeDenseError> R;
  auto bad = [&](const QInt8Tensor& t, size_t rows, size_t cols) {
    return t.rows != rows || t.cols != cols || t.q.size() != rows * cols || t.scales.size() != rows;
  };
  if (bad(gate, d_ff, d_model))
    return R::Err(MoeDenseError{MoeDenseError::WeightShapeMismatch, "w_gate", d_ff * d_model, gate.q.size()});
  if (bad(up, d_ff, d_model))
    return R::Err(MoeDenseError{MoeDenseError::WeightShapeMismatch, "w_up", d_ff * d_model, up.q.size()});
  if (bad(down, d_model, d_ff))
    return R::Err(MoeDenseError{MoeDenseError::WeightShapeMismatch, "w_down", d_model * d_ff, down.q.size()});
  auto ex = make(d_model, d_ff, gate.dequantize(), up.dequantize(), down.dequantize());
  if (ex.is_err()) return ex;
  auto payload = std::make_shared<QInt8Projections>();
  payload->gate = std::move(gate);
  payload->up = std::move(up);
  payload->down = std::move(down);
  ex.value().q8 = std::move(payload);
  return ex;
}

Result<MoeDenseLayer, MoeDenseError> MoeDenseLayer::make(size_t d_model, size_t d_ff,
                                                         std::vector<float> w_router,
                                                         std::vector<MoeDenseExpert> experts,
                                                         size_t conceptual_top_k) {
  typedef Result<MoeDenseLayer, MoeDenseError> R;  // src/moe/dense.rs:289-322
  if (experts.empty()) return R::Err({MoeDenseError::NoExperts});
  const size_t n = experts.size();
  if (w_router.size() != n * d_model)
    return R::Err({MoeDenseError::RouterExpertCountMismatch, "", d_model ? w_router.size() / d_model : 0, n});
  for (const auto& e : experts) {
    if (e.d_model != d_model)
      return R::Err({MoeDenseError::DimMismatch, "expert d_model", d_model, e.d_model});
    if (e.d_ff != d_ff) return R::Err({MoeDenseError::DimMismatch, "expert d_ff", d_ff, e.d_ff});
  }
  MoeDenseLayer l;
  l.d_model = d_model;
  l.d_ff = d_ff;
  l.w_router = std::move(w_router);
  l.experts = std::move(experts);
  l.conceptual_top_k = conceptual_top_k;
  return R::Ok(std::move(l));
}

// ---- RealMoeLayer ---------------------------------------------------------------------------
struct RealMoeLayer::Device {
  std::mutex mu;
  // key: convention * 2 + with_shared
  std::map<int, AteniaMoeLayer*> handles;
  ~Device() {
    for (auto& kv : handles) atenia_moe_hip_layer_destroy(kv.second);
  }
};

RealMoeLayer::RealMoeLayer() : dev_(new Device()) {}
RealMoeLayer::RealMoeLayer(const RealMoeLayer& o)
    : config(o.config), routed(o.routed), shared(o.shared), shared_gate(o.shared_gate),
      storage(o.storage), v3_router(o.v3_router),
      e_score_correction_bias(o.e_score_correction_bias), dev_(new Device()) {}
RealMoeLayer& RealMoeLayer::operator=(const RealMoeLayer& o) {
  if (this != &o) {
    config = o.config;
    routed = o.routed;
    shared = o.shared;
    shared_gate = o.shared_gate;
    storage = o.storage;
    v3_router = o.v3_router;
    e_score_correction_bias = o.e_score_correction_bias;
    dev_.reset(new Device());
  }
  return *this;
}
RealMoeLayer::RealMoeLayer(RealMoeLayer&& o) noexcept
    : config(o.config), routed(std::move(o.routed)), shared(std::move(o.shared)),
      shared_gate(std::move(o.shared_gate)), storage(o.storage), v3_router(o.v3_router),
      e_score_correction_bias(std::move(o.e_score_correction_bias)), dev_(std::move(o.dev_)) {
  o.dev_.reset(new Device());
}
RealMoeLayer& RealMoeLayer::operator=(RealMoeLayer&& o) noexcept {
  if (this != &o) {
    config = o.config;
    routed = std::move(o.routed);
    shared = std::move(o.shared);
    shared_gate = std::move(o.shared_gate);
    storage = o.storage;
    v3_router = o.v3_router;
    e_score_correction_bias = std::move(o.e_score_correction_bias);
    dev_ = std::move(o.dev_);
    o.dev_.reset(new Device());
  }
  return *this;
}
RealMoeLayer::~RealMoeLayer() = default;

Result<RealMoeLayer, MoeLayerError> RealMoeLayer::assemble(
    MoeLayerConfig config, MoeDenseLayer routed, std::optional<MoeDenseExpert> shared,
    std::optional<std::vector<float>> shared_gate, MoeWeightStorage storage) {
  typedef Result<RealMoeLayer, MoeLayerError> R;
  if (auto e = config.validate()) {
    MoeLayerError le{MoeLayerError::Config};
    le.config = *e;
    return R::Err(le);
  }
  auto mismatch = [](std::string d) {
    MoeLayerError le{MoeLayerError::ConfigMismatch};
    le.detail = std::move(d);
    return le;
  };
  if (routed.num_experts() != config.num_experts)
    return R::Err(mismatch("resolved " + std::to_string(routed.num_experts()) +
                           " experts but config.num_experts = " + std::to_string(config.num_experts)));
  if (routed.d_model != config.d_model || routed.d_ff != config.d_ff)
    return R::Err(mismatch("resolved (d_model=" + std::to_string(routed.d_model) + ", d_ff=" +
                           std::to_string(routed.d_ff) + ") but config (d_model=" +
                           std::to_string(config.d_model) + ", d_ff=" + std::to_string(config.d_ff) + ")"));
  if (config.has_shared_expert != shared.has_value())
    return R::Err(mismatch(config.has_shared_expert ? "config asks for a shared expert, none given"
                                                    : "shared expert given but config has none"));
  if (shared && shared->d_model != config.d_model)
    return R::Err(mismatch("shared expert d_model=" + std::to_string(shared->d_model) +
                           " != config d_model=" + std::to_string(config.d_model)));
  if (shared_gate && !shared) shared_gate.reset();  // captured only next to a shared expert
  RealMoeLayer l;
  l.config = config;
  l.routed = std::move(routed);
  l.routed.conceptual_top_k = config.experts_per_token;
  l.shared = std::move(shared);
  l.shared_gate = std::move(shared_gate);
  l.storage = storage;
  return R::Ok(std::move(l));
}

namespace {
// Expert weights in the storage form the descriptor asks for.
struct Packed {
  std::vector<float> f32;
  std::vector<uint16_t> b16;
  std::vector<int8_t> i8;
  std::vector<float> scale;
  const void* data(MoeWeightStorage s) const {
    return s == MoeWeightStorage::F32 ? (const void*)f32.data()
           : s == MoeWeightStorage::Bf16 ? (const void*)b16.data() : (const void*)i8.data();
  }
};

// `pre` (optional, one per matrix or empty): int8 tier data to upload as it is.
int pack(const std::vector<const std::vector<float>*>& mats, size_t rows, size_t cols,
         MoeWeightStorage s, Packed& out, const std::vector<const QInt8Tensor*>& pre = {}) {
  const size_t per = rows * cols, n = mats.size();
  if (s == MoeWeightStorage::F32) {
    out.f32.resize(n * per);
    for (size_t i = 0; i < n; ++i) std::memcpy(&out.f32[i * per], mats[i]->data(), per * 4);
    return 0;
  }
  if (s == MoeWeightStorage::Bf16) {  // truncation, as the reference stores bf16 (tensor.rs:306-308)
    out.b16.resize(n * per);
    for (size_t i = 0; i < n; ++i) {
      int rc = atenia_moe_f32_to_bf16_trunc(mats[i]->data(), per, &out.b16[i * per]);
      if (rc) return rc;
    }
    return 0;
  }
  if (s == MoeWeightStorage::Int8PerGroup) {  // quantizer.rs:175-248 along each row
    const size_t ng = (cols + kInt8GroupSize - 1) / kInt8GroupSize;
    out.i8.resize(n * per);
    out.scale.resize(n * rows * ng);
    for (size_t i = 0; i < n; ++i) {
      int rc = atenia_moe_quantize_per_group_i8(mats[i]->data(), rows, cols, kInt8GroupSize,
                                                &out.i8[i * per], &out.scale[i * rows * ng]);
      if (rc) return rc;
    }
    return 0;
  }
  out.i8.resize(n * per);  // per output row (disk_tier.rs:231-248)
  out.scale.resize(n * rows);
  bool have_pre = pre.size() == n && s == MoeWeightStorage::Int8W8A16;
  for (size_t i = 0; have_pre && i < n; ++i)
    have_pre = pre[i] && pre[i]->rows == rows && pre[i]->cols == cols;
  for (size_t i = 0; i < n; ++i) {
    if (have_pre) {
      std::memcpy(&out.i8[i * per], pre[i]->q.data(), per);
      std::memcpy(&out.scale[i * rows], pre[i]->scales.data(), rows * 4);
      continue;
    }
    int rc = atenia_moe_quantize_per_row_i8(mats[i]->data(), rows, cols, &out.i8[i * per],
                                            &out.scale[i * rows]);
    if (rc) return rc;
  }
  return 0;
}
}  // namespace

// The C-ABI handle for (convention, with shared expert), created and uploaded on first use.
// Caller holds dev_->mu.
// ---- unit-level forwards of MoeDenseExpert / MoeDenseLayer ---------------------------------------
namespace {
// The routed experts as a RealMoeLayer with k experts per token; `renormalize` picks the
// convention (there is no shared expert, so the conventions differ in nothing else).
Result<std::vector<float>, MoeSparseError> run_routed(const MoeDenseLayer& layer,
                                                       const std::vector<float>& x, size_t k,
                                                       bool renormalize,
                                                       std::vector<int32_t>* indices,
                                                       std::vector<float>* weights) {
  typedef Result<std::vector<float>, MoeSparseError> R;
  MoeSparseError e{MoeSparseError::Dense};
  if (x.size() != layer.d_model) {
    e.dense = MoeDenseError{MoeDenseError::DimMismatch, "router input", layer.d_model, x.size()};
    return R::Err(e);
  }
  if (k == 0) return R::Err(MoeSparseError{MoeSparseError::ZeroK});
  if (k > layer.num_experts()) {
    MoeSparseError ke{MoeSparseError::KExceedsExperts};
    ke.k = k;
    ke.num_experts = layer.num_experts();
    return R::Err(ke);
  }
  auto cfg = MoeLayerConfig::make(layer.num_experts(), k, false, layer.d_model, layer.d_ff);
  auto fail_device = [&](const std::string& text) {
    // no counterpart in the reference (it computes on the CPU): reported as a shape error text
    static thread_local std::string keep;
    keep = text;
    e.dense = MoeDenseError{MoeDenseError::DimMismatch, keep.c_str(), 0, 0};
    return R::Err(e);
  };
  if (cfg.is_err()) return fail_device(cfg.error().to_string());
  auto real = RealMoeLayer::assemble(cfg.value(), layer, std::nullopt, std::nullopt);
  if (real.is_err()) return fail_device(real.error().to_string());
  const MoeExecutionConvention conv =
      renormalize ? MoeExecutionConvention::Atenia : MoeExecutionConvention::HuggingFaceQwen;
  auto out = real.value().forward_with(x, conv);
  if (out.is_err()) {
    if (out.error().kind == MoeLayerError::Sparse) return R::Err(out.error().sparse);
    return fail_device(out.error().to_string());
  }
  if (indices || weights) {
    std::vector<int32_t> idx;
    auto w = real.value().route(x, conv, &idx);
    if (w.is_err()) return fail_device(w.error().to_string());
    if (indices) *indices = idx;
    if (weights) *weights = w.value();
  }
  return R::Ok(out.value());
}
}  // namespace

Result<MoeSparseForwardOutput, MoeSparseError> MoeDenseLayer::forward_sparse_with(
    const std::vector<float>& x, size_t k, bool renormalize) const {
  typedef Result<MoeSparseForwardOutput, MoeSparseError> R;
  std::vector<int32_t> idx;
  auto out = run_routed(*this, x, k, renormalize, &idx, nullptr);
  if (out.is_err()) return R::Err(out.error());
  MoeSparseForwardOutput r;
  r.output = out.value();
  r.selected_experts.assign(idx.begin(), idx.end());
  return R::Ok(std::move(r));
}

Result<MoeSparseForwardOutput, MoeSparseError> MoeDenseLayer::forward_sparse(
    const std::vector<float>& x, size_t k) const {
  return forward_sparse_with(x, k, true);
}

Result<MoeRouterOutput, MoeDenseError> MoeDenseLayer::route(const std::vector<float>& x) const {
  typedef Result<MoeRouterOutput, MoeDenseError> R;
  if (x.size() != d_model)
    return R::Err(MoeDenseError{MoeDenseError::DimMismatch, "router input", d_model, x.size()});
  // all experts, raw weights: the selection lists them in ascending order
  std::vector<float> w;
  auto out = run_routed(*this, x, num_experts(), false, nullptr, &w);
  if (out.is_err()) {
    if (out.error().kind == MoeSparseError::NonFiniteWeight)  // softmax of non-finite logits
      return R::Ok(MoeRouterOutput{std::vector<float>(num_experts(), std::nanf(""))});
    return R::Err(out.error().dense);
  }
  return R::Ok(MoeRouterOutput{std::move(w)});
}

Result<std::vector<float>, MoeDenseError> MoeDenseLayer::forward(const std::vector<float>& x) const {
  typedef Result<std::vector<float>, MoeDenseError> R;
  if (x.size() != d_model)
    return R::Err(MoeDenseError{MoeDenseError::DimMismatch, "router input", d_model, x.size()});
  auto out = run_routed(*this, x, num_experts(), false, nullptr, nullptr);
  if (out.is_err()) {
    if (out.error().kind == MoeSparseError::NonFiniteWeight)
      return R::Ok(std::vector<float>(d_model, std::nanf("")));
    return R::Err(out.error().dense);
  }
  return R::Ok(out.value());
}

Result<std::vector<float>, MoeDenseError> MoeDenseExpert::forward(const std::vector<float>& x) const {
  typedef Result<std::vector<float>, MoeDenseError> R;
  if (x.size() != d_model)
    return R::Err(MoeDenseError{MoeDenseError::DimMismatch, "expert input", d_model, x.size()});
  // a one-expert layer with a zero router: its single routing weight is exactly 1
  auto layer = MoeDenseLayer::make(d_model, d_ff, std::vector<float>(d_model, 0.f), {*this}, 1);
  if (layer.is_err()) return R::Err(layer.error());
  auto out = run_routed(layer.value(), x, 1, true, nullptr, nullptr);
  if (out.is_err()) return R::Err(out.error().dense);
  return R::Ok(out.value());
}

// ---- MoeDenseLayer registry and the decomposed graph ops -----------------------------------------
namespace {
std::mutex& dense_registry_mutex() {
  static std::mutex m;
  return m;
}
std::vector<std::shared_ptr<const MoeDenseLayer>>& dense_registry() {
  static std::vector<std::shared_ptr<const MoeDenseLayer>> r;
  return r;
}
MoeSparseError no_such_layer() {
  MoeSparseError e{MoeSparseError::Dense};
  e.dense = MoeDenseError{MoeDenseError::NoExperts};
  return e;
}
MoeSparseError from_dense(const MoeDenseError& d) {
  MoeSparseError e{MoeSparseError::Dense};
  e.dense = d;
  return e;
}
}  // namespace

uint32_t register_layer(MoeDenseLayer layer) {
  std::lock_guard<std::mutex> lock(dense_registry_mutex());
  dense_registry().push_back(std::make_shared<const MoeDenseLayer>(std::move(layer)));
  return (uint32_t)(dense_registry().size() - 1);
}

std::shared_ptr<const MoeDenseLayer> get_layer(uint32_t layer_id) {
  std::lock_guard<std::mutex> lock(dense_registry_mutex());
  return layer_id < dense_registry().size() ? dense_registry()[layer_id] : nullptr;
}

Result<std::vector<float>, MoeSparseError> execute_sparse_reference(uint32_t layer_id,
                                                                    const std::vector<float>& input,
                                                                    size_t k) {
  typedef Result<std::vector<float>, MoeSparseError> R;
  auto layer = get_layer(layer_id);
  if (!layer) return R::Err(no_such_layer());
  auto out = layer->forward_sparse(input, k);
  if (out.is_err()) return R::Err(out.error());
  return R::Ok(out.value().output);
}

Result<DynamicDispatchOutput, MoeSparseError> execute_dynamic_dispatch(
    uint32_t layer_id, const std::vector<float>& input, const std::vector<float>& selection) {
  typedef Result<DynamicDispatchOutput, MoeSparseError> R;
  auto layer = get_layer(layer_id);
  if (!layer) return R::Err(no_such_layer());
  if (selection.size() % 2 != 0)
    return R::Err(from_dense(MoeDenseError{MoeDenseError::DimMismatch,
                                           "dispatch selection (must be [idx, w, ...])", 0,
                                           selection.size() % 2}));
  const size_t pairs = selection.size() / 2, d = layer->d_model, E = layer->num_experts();
  DynamicDispatchOutput r;
  r.output.assign(d, 0.0f);
  for (size_t p = 0; p < pairs; ++p) {
    const float idx_f = selection[2 * p], weight = selection[2 * p + 1];
    if (!std::isfinite(idx_f) || idx_f < 0.0f) {
      MoeSparseError e{MoeSparseError::NegativeWeight};
      e.index = 2 * p;
      return R::Err(e);
    }
    const size_t idx = (size_t)idx_f;
    if (idx >= E) {
      MoeSparseError e{MoeSparseError::KExceedsExperts};
      e.k = idx + 1;
      e.num_experts = E;
      return R::Err(e);
    }
    auto y = layer->experts[idx].forward(input);  // only the listed experts run
    if (y.is_err()) return R::Err(from_dense(y.error()));
    volatile float prod;  // product and sum rounded separately, as the reference's f32 loop
    for (size_t c = 0; c < d; ++c) {
      prod = weight * y.value()[c];
      r.output[c] = r.output[c] + prod;
    }
    r.executed_experts.push_back(idx);
  }
  return R::Ok(std::move(r));
}

std::optional<float> expert_weight_in_selection(const std::vector<float>& selection,
                                                uint32_t expert_id) {
  for (size_t p = 0; p + 1 < selection.size(); p += 2)
    if ((uint32_t)selection[p] == expert_id) return selection[p + 1];
  return std::nullopt;
}

Result<std::pair<std::vector<float>, bool>, MoeSparseError> execute_conditional_expert(
    uint32_t layer_id, uint32_t expert_id, const std::vector<float>& input,
    const std::vector<float>& selection) {
  typedef Result<std::pair<std::vector<float>, bool>, MoeSparseError> R;
  auto layer = get_layer(layer_id);
  if (!layer) return R::Err(no_such_layer());
  if (expert_id >= layer->num_experts()) {
    MoeSparseError e{MoeSparseError::KExceedsExperts};
    e.k = (size_t)expert_id + 1;
    e.num_experts = layer->num_experts();
    return R::Err(e);
  }
  auto w = expert_weight_in_selection(selection, expert_id);
  if (!w) return R::Ok(std::make_pair(std::vector<float>(layer->d_model, 0.0f), false));
  auto y = layer->experts[expert_id].forward(input);
  if (y.is_err()) return R::Err(from_dense(y.error()));
  std::vector<float> scaled = y.value();
  for (auto& v : scaled) v = v * *w;
  return R::Ok(std::make_pair(std::move(scaled), true));
}

// ---- numeric policy -----------------------------------------------------------------------------
const char* as_str(NumericPolicy p) {
  switch (p) {
    case NumericPolicy::Strict: return "strict";
    case NumericPolicy::Fast: return "fast";
    default: return "certified";
  }
}

std::optional<NumericPolicy> numeric_policy_from_str(const std::string& s) {
  size_t b = 0, e = s.size();
  while (b < e && std::isspace((unsigned char)s[b])) ++b;
  while (e > b && std::isspace((unsigned char)s[e - 1])) --e;
  std::string t = s.substr(b, e - b);
  for (auto& c : t) c = (char)std::tolower((unsigned char)c);
  if (t == "certified" || t == "f64") return NumericPolicy::Certified;
  if (t == "strict" || t == "f32") return NumericPolicy::Strict;
  if (t == "fast") return NumericPolicy::Fast;
  return std::nullopt;
}

namespace {
constexpr int kPolicyUnset = 255;
std::atomic<int> g_policy_override{kPolicyUnset};
NumericPolicy policy_from_env() {  // read once (src/moe/numeric_policy.rs:99-116)
  static const NumericPolicy p = [] {
    const char* e = std::getenv("ATENIA_NUMERIC_POLICY");
    auto v = e ? numeric_policy_from_str(e) : std::nullopt;
    return v ? *v : NumericPolicy::Certified;
  }();
  return p;
}
}  // namespace

NumericPolicy numeric_policy() {
  const int o = g_policy_override.load(std::memory_order_relaxed);
  if (o != kPolicyUnset) return o == 1 ? NumericPolicy::Strict : o == 2 ? NumericPolicy::Fast : NumericPolicy::Certified;
  return policy_from_env();
}
void set_numeric_policy(NumericPolicy p) { g_policy_override.store((int)p, std::memory_order_relaxed); }
void clear_numeric_policy_override() { g_policy_override.store(kPolicyUnset, std::memory_order_relaxed); }

std::optional<NumericalMetrics> NumericalMetrics::compute(const std::vector<float>& atenia,
                                                          const std::vector<float>& reference) {
  if (atenia.empty() || atenia.size() != reference.size()) return std::nullopt;
  auto argmax = [](const std::vector<float>& v) {
    size_t best = 0;
    double bv = (double)v[0];
    for (size_t i = 1; i < v.size(); ++i)
      if ((double)v[i] > bv) {
        bv = (double)v[i];
        best = i;
      }
    return best;
  };
  NumericalMetrics m;
  m.len = atenia.size();
  double sum_abs = 0.0, sum_sq = 0.0;
  for (size_t i = 0; i < m.len; ++i) {
    const double dd = (double)atenia[i] - (double)reference[i];
    const double ad = std::fabs(dd);
    if (ad > m.max_abs_diff) m.max_abs_diff = ad;
    sum_abs += ad;
    sum_sq += dd * dd;
  }
  m.mean_abs_diff = sum_abs / (double)m.len;
  m.rmse = std::sqrt(sum_sq / (double)m.len);
  m.argmax_match = argmax(atenia) == argmax(reference);
  return m;
}

PolicyCertificate PolicyCertificate::compare(NumericPolicy policy,
                                             const std::vector<std::vector<float>>& reference_rows,
                                             const std::vector<std::vector<float>>& candidate_rows,
                                             const std::vector<uint32_t>& reference_tokens,
                                             const std::vector<uint32_t>& candidate_tokens) {
  const size_t rows = std::min(reference_rows.size(), candidate_rows.size());
  double max_abs = 0.0, sum_abs = 0.0, sum_sq = 0.0;
  size_t argmax_ok = 0, counted = 0;
  for (size_t i = 0; i < rows; ++i) {
    auto m = NumericalMetrics::compute(candidate_rows[i], reference_rows[i]);
    if (!m) continue;
    max_abs = std::max(max_abs, m->max_abs_diff);
    sum_abs += m->mean_abs_diff;
    sum_sq += m->rmse * m->rmse;
    if (m->argmax_match) ++argmax_ok;
    ++counted;
  }
  const double denom = (double)std::max<size_t>(counted, 1);
  PolicyCertificate c;
  c.policy = policy;
  c.rows = counted;
  c.max_abs_diff = max_abs;
  c.mean_abs_diff = sum_abs / denom;
  c.rmse = std::sqrt(sum_sq / denom);
  c.argmax_match_rate = (double)argmax_ok / denom;
  c.tokens_match = reference_tokens == candidate_tokens;
  return c;
}

Result<void*, MoeLayerError> RealMoeLayer::handle_for(MoeExecutionConvention convention,
                                                      bool with_shared) const {
  typedef Result<void*, MoeLayerError> R;
  const size_t d = config.d_model;
  const bool use_shared = with_shared && shared.has_value();
  const int key = (int)convention * 2 + (use_shared ? 1 : 0);
  auto it = dev_->handles.find(key);
  if (it != dev_->handles.end()) return R::Ok(it->second);
  const size_t E = routed.num_experts(), f = config.d_ff;
  std::vector<const std::vector<float>*> g, u, dn;
  for (const auto& e : routed.experts) {
    g.push_back(&e.w_gate);
    u.push_back(&e.w_up);
    dn.push_back(&e.w_down);
  }
  std::vector<const QInt8Tensor*> qg, qu, qd;  // tier data, when every expert carries it
  for (const auto& e : routed.experts) {
    if (!e.q8) break;
    qg.push_back(&e.q8->gate);
    qu.push_back(&e.q8->up);
    qd.push_back(&e.q8->down);
  }
  Packed pg, pu, pd, sg, su, sd;
  int rc = pack(g, f, d, storage, pg, qg);
  if (!rc) rc = pack(u, f, d, storage, pu, qu);
  if (!rc) rc = pack(dn, d, f, storage, pd, qd);
  AteniaMoeLayerDesc desc;
  std::memset(&desc, 0, sizeof(desc));
  desc.num_experts = (int32_t)E;
  desc.top_k = (int32_t)config.experts_per_token;
  desc.d_model = (int32_t)d;
  desc.d_ff = (int32_t)f;
  desc.convention = (int32_t)convention;
  desc.weight_dtype = (int32_t)storage;
  desc.w_router = routed.w_router.data();
  desc.w_gate = pg.data(storage);
  desc.w_up = pu.data(storage);
  desc.w_down = pd.data(storage);
  const bool int8 = storage == MoeWeightStorage::Int8W8A16 || storage == MoeWeightStorage::Int8PerGroup;
  if (storage == MoeWeightStorage::Int8PerGroup) desc.group_size = (int32_t)kInt8GroupSize;
  if (int8) {
    desc.scale_gate = pg.scale.data();
    desc.scale_up = pu.scale.data();
    desc.scale_down = pd.scale.data();
  }
  if (use_shared) {
    const size_t fs = shared->d_ff;
    desc.d_ff_shared = (int32_t)fs;
    const QInt8Projections* sq = shared->q8.get();
    if (!rc) rc = pack({&shared->w_gate}, fs, d, storage, sg, sq ? std::vector<const QInt8Tensor*>{&sq->gate} : std::vector<const QInt8Tensor*>{});
    if (!rc) rc = pack({&shared->w_up}, fs, d, storage, su, sq ? std::vector<const QInt8Tensor*>{&sq->up} : std::vector<const QInt8Tensor*>{});
    if (!rc) rc = pack({&shared->w_down}, d, fs, storage, sd, sq ? std::vector<const QInt8Tensor*>{&sq->down} : std::vector<const QInt8Tensor*>{});
    desc.s_gate = sg.data(storage);
    desc.s_up = su.data(storage);
    desc.s_down = sd.data(storage);
    if (int8) {
      desc.s_scale_gate = sg.scale.data();
      desc.s_scale_up = su.scale.data();
      desc.s_scale_down = sd.scale.data();
    }
    if (shared_gate) desc.shared_gate = shared_gate->data();
  }
  if (rc) return R::Err(device_error(rc));
  AteniaMoeLayer* h = nullptr;
  rc = atenia_moe_hip_layer_create(&desc, &h);
  if (rc == ATENIA_MOE_ERR_K) {
    MoeLayerError e{MoeLayerError::Sparse};
    if (config.experts_per_token == 0) {
      e.sparse.kind = MoeSparseError::ZeroK;
    } else {
      e.sparse.kind = MoeSparseError::KExceedsExperts;
      e.sparse.k = config.experts_per_token;
      e.sparse.num_experts = E;
    }
    return R::Err(e);
  }
  if (rc) return R::Err(device_error(rc));
  if (v3_router) {  // validated by set_v3_router; the device repeats the checks
    rc = atenia_moe_hip_layer_set_v3_router(h, (int)v3_router->n_group, (int)v3_router->topk_group,
                                            v3_router->routed_scaling_factor,
                                            v3_router->norm_topk_prob ? 1 : 0,
                                            e_score_correction_bias.data());
    if (rc) {
      MoeLayerError e = device_error(rc);
      atenia_moe_hip_layer_destroy(h);
      return R::Err(e);
    }
  }
  dev_->handles[key] = h;
  return R::Ok(h);
}

std::optional<V3RouterError> RealMoeLayer::set_v3_router(const V3RouterConfig& cfg,
                                                         std::vector<float> bias) {
  if (auto e = cfg.validate()) return e;
  auto err = [](V3RouterError::Kind k, const char* what, size_t a, size_t b) {
    V3RouterError e{k};
    e.what = what;
    e.a = a;
    e.b = b;
    return e;
  };
  if (cfg.n_routed_experts != num_experts())
    return err(V3RouterError::LengthMismatch, "router_logits", cfg.n_routed_experts, num_experts());
  if (bias.size() != cfg.n_routed_experts)
    return err(V3RouterError::LengthMismatch, "e_score_correction_bias", cfg.n_routed_experts,
               bias.size());
  for (size_t i = 0; i < bias.size(); ++i)
    if (!std::isfinite(bias[i])) return err(V3RouterError::NonFinite, "e_score_correction_bias", i, 0);
  if (cfg.top_k != config.experts_per_token)
    return err(V3RouterError::TopKMismatch, "", cfg.top_k, config.experts_per_token);
  std::lock_guard<std::mutex> lock(dev_->mu);
  for (auto& kv : dev_->handles) atenia_moe_hip_layer_destroy(kv.second);  // rebuilt on next use
  dev_->handles.clear();
  v3_router = cfg;
  e_score_correction_bias = std::move(bias);
  return std::nullopt;
}

namespace {
MoeLayerError non_finite_error(AteniaMoeLayer* h) {
  int32_t token = 0, expert = 0;
  atenia_moe_hip_layer_last_non_finite(h, &token, &expert);
  MoeLayerError e{MoeLayerError::Sparse};
  e.sparse.kind = MoeSparseError::NonFiniteWeight;
  e.sparse.index = (size_t)expert;
  e.sparse.token = (size_t)token;
  return e;
}
}  // namespace

Result<std::vector<float>, MoeLayerError> RealMoeLayer::run(const std::vector<float>& x,
                                                            MoeExecutionConvention convention,
                                                            bool with_shared) const {
  typedef Result<std::vector<float>, MoeLayerError> R;
  const size_t d = config.d_model;
  // One token or a flat batch; anything else is the dimension error the row forward raises
  // (src/moe/dense.rs:325-331 via graph_op.rs:340-343).
  if (d == 0 || x.empty() || x.size() % d != 0) return R::Err(dense_dim_error("x", d, x.size()));
  std::lock_guard<std::mutex> lock(dev_->mu);
  auto hr = handle_for(convention, with_shared);
  if (hr.is_err()) return R::Err(hr.error());
  AteniaMoeLayer* h = (AteniaMoeLayer*)hr.value();
  std::vector<float> out(x.size());
  (void)atenia_moe_hip_layer_set_numeric_policy(h, (int)numeric_policy());
  const int rc = atenia_moe_hip_layer_forward(h, x.data(), (int)(x.size() / d), out.data());
  if (rc == ATENIA_MOE_ERR_NON_FINITE) return R::Err(non_finite_error(h));
  if (rc == ATENIA_MOE_ERR_DIM) return R::Err(dense_dim_error("x", d, x.size()));
  if (rc) return R::Err(device_error(rc));
  return R::Ok(std::move(out));
}

Result<std::vector<float>, MoeLayerError> RealMoeLayer::forward(const std::vector<float>& x) const {
  return forward_with(x, MoeExecutionConvention::Atenia);
}
Result<std::vector<float>, MoeLayerError> RealMoeLayer::forward_auto(const std::vector<float>& x) const {
  return forward_with(x, resolve_convention());
}
Result<std::vector<float>, MoeLayerError> RealMoeLayer::forward_with(
    const std::vector<float>& x, MoeExecutionConvention convention) const {
  return run(x, convention, true);
}
Result<std::vector<float>, MoeLayerError> RealMoeLayer::forward_routed(const std::vector<float>& x) const {
  return run(x, MoeExecutionConvention::Atenia, false);
}

Result<std::vector<float>, MoeLayerError> RealMoeLayer::ffn_block(
    const std::vector<float>& x1, const std::vector<float>& gamma, float eps, NormPolicy norm_policy,
    MoeExecutionConvention convention) const {
  typedef Result<std::vector<float>, MoeLayerError> R;
  const size_t d = config.d_model;
  if (d == 0 || x1.empty() || x1.size() % d != 0) return R::Err(dense_dim_error("x", d, x1.size()));
  if (gamma.size() != d) return R::Err(dense_dim_error("gamma", d, gamma.size()));
  std::lock_guard<std::mutex> lock(dev_->mu);
  auto hr = handle_for(convention, true);
  if (hr.is_err()) return R::Err(hr.error());
  AteniaMoeLayer* h = (AteniaMoeLayer*)hr.value();
  std::vector<float> out(x1.size());
  (void)atenia_moe_hip_layer_set_numeric_policy(h, (int)numeric_policy());
  const int rc = atenia_moe_hip_layer_block_forward(h, x1.data(), (int)(x1.size() / d), gamma.data(),
                                                    eps, (int)norm_policy, out.data());
  if (rc == ATENIA_MOE_ERR_NON_FINITE) return R::Err(non_finite_error(h));
  if (rc) return R::Err(device_error(rc));
  return R::Ok(std::move(out));
}

Result<std::vector<float>, MoeLayerError> RealMoeLayer::route(const std::vector<float>& x,
                                                              MoeExecutionConvention convention,
                                                              std::vector<int32_t>* indices) const {
  typedef Result<std::vector<float>, MoeLayerError> R;
  const size_t d = config.d_model;
  if (d == 0 || x.empty() || x.size() % d != 0) return R::Err(dense_dim_error("x", d, x.size()));
  std::lock_guard<std::mutex> lock(dev_->mu);
  auto hr = handle_for(convention, true);
  if (hr.is_err()) return R::Err(hr.error());
  AteniaMoeLayer* h = (AteniaMoeLayer*)hr.value();
  const int T = (int)(x.size() / d);
  const size_t k = config.experts_per_token;
  std::vector<int32_t> idx((size_t)T * k);
  std::vector<float> w((size_t)T * k);
  const int rc = atenia_moe_hip_layer_route(h, x.data(), T, idx.data(), w.data());
  if (rc == ATENIA_MOE_ERR_NON_FINITE) return R::Err(non_finite_error(h));
  if (rc) return R::Err(device_error(rc));
  if (indices) *indices = std::move(idx);
  return R::Ok(std::move(w));
}

// ---- ResidentExpertLayer ----------------------------------------------------------------------
ResidentExpertLayer ResidentExpertLayer::from_real_layer(const RealMoeLayer& layer, ExpertTier tier) {
  ResidentExpertLayer r;
  r.config = layer.config;
  r.convention = layer.resolve_convention();
  r.tier = tier;
  r.layer_ = std::make_shared<RealMoeLayer>(layer);
  return r;
}

namespace {
size_t stored_bytes(MoeWeightStorage st, size_t d, size_t f) {
  switch (st) {
    case MoeWeightStorage::F32: return 3 * d * f * 4;
    case MoeWeightStorage::Bf16: return 3 * d * f * 2;
    case MoeWeightStorage::Int8W8A16: return 3 * d * f + (2 * f + d) * 4;
    case MoeWeightStorage::Int8PerGroup:
      return 3 * d * f + (2 * f * ((d + 127) / 128) + d * ((f + 127) / 128)) * 4;
  }
  return 0;
}
}  // namespace

size_t ResidentExpertLayer::expert_bytes() const {
  return stored_bytes(layer_->storage, config.d_model, config.d_ff);
}
size_t ResidentExpertLayer::shared_bytes() const {
  if (!layer_->shared) return 0;
  return stored_bytes(layer_->storage, config.d_model, layer_->shared->d_ff);
}

Result<std::vector<float>, MoeLayerError> ResidentExpertLayer::forward_batch(
    const std::vector<float>& x, std::vector<ResidencyInfo>* infos) const {
  using R = Result<std::vector<float>, MoeLayerError>;
  auto out = layer_->forward_with(x, convention);
  if (!out.is_ok() || !infos) return out;
  std::vector<int32_t> idx;
  auto w = layer_->route(x, convention, &idx);
  if (!w.is_ok()) return R::Err(w.error());
  const size_t k = config.experts_per_token, n = k ? idx.size() / k : 0;
  infos->assign(n, ResidencyInfo{});
  for (size_t t = 0; t < n; ++t) {
    for (size_t s = 0; s < k; ++s) (*infos)[t].materialized_experts.push_back((size_t)idx[t * k + s]);
    (*infos)[t].materialized_bytes = k * expert_bytes() + shared_bytes();
  }
  return out;
}

Result<std::pair<std::vector<float>, ResidencyInfo>, MoeLayerError> ResidentExpertLayer::forward(
    const std::vector<float>& x) const {
  using R = Result<std::pair<std::vector<float>, ResidencyInfo>, MoeLayerError>;
  if (x.size() != config.d_model) {  // the reference's forward takes one row
    MoeLayerError e{MoeLayerError::Binding};
    e.binding.kind = MoeBindingError::Dense;
    e.binding.dense.kind = MoeDenseError::DimMismatch;
    e.binding.dense.what = "x";
    e.binding.dense.expected = config.d_model;
    e.binding.dense.actual = x.size();
    return R::Err(e);
  }
  std::vector<ResidencyInfo> infos;
  auto out = forward_batch(x, &infos);
  if (!out.is_ok()) return R::Err(out.error());
  return R::Ok({out.value(), infos.empty() ? ResidencyInfo{} : infos[0]});
}

// ---- registry -------------------------------------------------------------------------------
namespace {
// RegisteredMoe (src/moe/graph_op.rs:207-216): a RAM layer or a resident one, one id space.
struct RegisteredMoe {
  std::shared_ptr<RealMoeLayer> real;
  std::shared_ptr<ResidentExpertLayer> resident;
};
std::mutex& registry_mutex() {
  static std::mutex m;
  return m;
}
std::vector<RegisteredMoe>& registry() {
  static std::vector<RegisteredMoe> r;
  return r;
}
MoeLayerError layer_not_found(uint32_t id) {
  MoeLayerError e{MoeLayerError::Binding};
  e.binding.kind = MoeBindingError::LayerNotFound;
  e.binding.layer_id = id;
  return e;
}
bool lookup(uint32_t layer_id, RegisteredMoe* out) {
  std::lock_guard<std::mutex> lock(registry_mutex());
  if (layer_id >= registry().size()) return false;
  *out = registry()[layer_id];
  return true;
}
}  // namespace

uint32_t register_real_moe_layer(RealMoeLayer layer) {
  std::lock_guard<std::mutex> lock(registry_mutex());
  registry().push_back({std::make_shared<RealMoeLayer>(std::move(layer)), nullptr});
  return (uint32_t)(registry().size() - 1);
}

uint32_t register_resident_moe_layer(std::shared_ptr<ResidentExpertLayer> layer, size_t) {
  std::lock_guard<std::mutex> lock(registry_mutex());
  registry().push_back({nullptr, std::move(layer)});
  return (uint32_t)(registry().size() - 1);
}

// A resident id answers None here, as in the reference (graph_op.rs:294-299).
std::shared_ptr<const RealMoeLayer> get_real_moe_layer(uint32_t layer_id) {
  RegisteredMoe m;
  if (!lookup(layer_id, &m)) return nullptr;
  return m.real;
}

Result<std::vector<float>, MoeLayerError> execute_real_moe_layer(uint32_t layer_id,
                                                                 const std::vector<float>& input) {
  RegisteredMoe m;
  if (!lookup(layer_id, &m)) return Result<std::vector<float>, MoeLayerError>::Err(layer_not_found(layer_id));
  // whole batch, one call into the device library; a resident layer drops its evidence here
  // as the reference's execute_moe_row does (graph_op.rs:304-316)
  if (m.resident) return m.resident->forward_batch(input);
  return m.real->forward_auto(input);
}

Result<std::vector<float>, MoeLayerError> execute_real_moe_layer_with(
    uint32_t layer_id, const std::vector<float>& input, MoeExecutionConvention convention) {
  auto layer = get_real_moe_layer(layer_id);
  if (!layer) return Result<std::vector<float>, MoeLayerError>::Err(layer_not_found(layer_id));
  return layer->forward_with(input, convention);
}

std::vector<float> moe_real_layer_reference_node(uint32_t layer_id, const std::vector<float>& input) {
  return execute_real_moe_layer(layer_id, input)
      .expect("MoeRealLayerReference: forward failed (unknown layer_id or bad input dim)");
}

}  // namespace moe
}  // namespace atenia
