// Host-side mirror of the reference's MoE operator interface, over the C ABI of
// libatenia_moe_hip.so.  The reference is Rust; these are the same types, names, argument
// meanings and error behaviour in C++, so a test written against the reference reads the same
// here:
//
//   MoeLayerConfig, MoeConfigError            src/moe/layer.rs:37-117
//   MoeExecutionConvention                    src/moe/layer.rs:185-195
//   MoeDenseExpert, MoeDenseLayer             src/moe/dense.rs:203-250, 276-322
//   RealMoeLayer::{forward, forward_auto, forward_with, forward_routed, resolve_convention}
//                                             src/moe/layer.rs:200-431
//   MoeDenseError / MoeSparseError / MoeBindingError / MoeLayerError
//                                             dense.rs:31-49, sparse.rs:35-50, binding.rs:41-70,
//                                             layer.rs:119-136
//   V3RouterConfig, ScoringFunc, V3RouterError (DeepSeek-V3 routing)
//                                             src/moe/v3_router.rs:36-123, 148-181
//   register_real_moe_layer, get_real_moe_layer, execute_real_moe_layer[_with]
//                                             src/moe/graph_op.rs:228-232, 294-299, 327-364
//   moe_real_layer_reference_node             the executor arm, src/amg/graph.rs:5572-5589
//
// What differs on purpose: a forward runs on the GPU through one C-ABI call for the whole
// [T * d_model] batch (the reference loops over rows on the CPU), and a layer carries the
// storage type its weights are uploaded as (f32 keeps the reference's certified arithmetic;
// bf16 and int8 are the throughput forms).  There is no CPU fallback: without the device
// every forward returns MoeLayerError::Device.
#pragma once

#include <cstddef>
#include <cstdint>
#include <memory>
#include <mutex>
#include <optional>
#include <string>
#include <vector>

namespace atenia {
namespace moe {

// ---- errors ---------------------------------------------------------------------------------
struct MoeConfigError {
  enum Kind { ZeroExperts, ZeroExpertsPerToken, ExpertsPerTokenExceedsCount, ZeroDModel, ZeroDFf };
  Kind kind;
  size_t per_token = 0, total = 0;
  std::string to_string() const;
  bool operator==(const MoeConfigError& o) const {
    return kind == o.kind && per_token == o.per_token && total == o.total;
  }
};

struct MoeDenseError {
  enum Kind { DimMismatch, WeightShapeMismatch, NoExperts, RouterExpertCountMismatch };
  Kind kind;
  const char* what = "";
  size_t expected = 0, actual = 0;  // RouterExpertCountMismatch: router, experts
  std::string to_string() const;
};

struct MoeSparseError {
  enum Kind { ZeroK, KExceedsExperts, NonFiniteWeight, NegativeWeight, SelectedSumNonPositive, Dense };
  Kind kind;
  size_t k = 0, num_experts = 0;  // KExceedsExperts
  size_t index = 0;               // NonFiniteWeight / NegativeWeight: expert index
  size_t token = 0;               // row of the batch the weight belongs to (extension)
  MoeDenseError dense{MoeDenseError::NoExperts};
  std::string to_string() const;
};

struct MoeBindingError {  // src/moe/binding.rs:41-70
  enum Kind {
    LayerNotFound, NoExperts, IncompleteExpert, MissingRouter, UnresolvedTensor, BadRank,
    ShapeInconsistency, DataLengthMismatch, MissingPackedTensor, PackedBadRank, Dense
  };
  Kind kind;
  size_t layer_id = 0, expert_id = 0;
  std::string name;               // UnresolvedTensor / BadRank / DataLengthMismatch / PackedBadRank
  size_t rank = 0;                // BadRank / PackedBadRank
  size_t expected = 0, actual = 0;  // DataLengthMismatch
  std::string detail;             // ShapeInconsistency
  const char* which = "";         // MissingPackedTensor: "gate_up_proj" or "down_proj"
  MoeDenseError dense{MoeDenseError::NoExperts};
  std::string to_string() const;
};

struct MoeLayerError {
  // Config / Binding / Sparse / ConfigMismatch as in the reference; Device = the HIP library
  // reported a failure that has no counterpart there (no device, out of memory, launch failed).
  enum Kind {
    Config, Binding, Sparse, ConfigMismatch, SharedExpertMissing, SharedExpertIncomplete,
    MixedExpertFormat, Device
  };
  Kind kind;
  size_t layer_id = 0;  // SharedExpertMissing / SharedExpertIncomplete / MixedExpertFormat
  MoeConfigError config{MoeConfigError::ZeroExperts};
  MoeBindingError binding{MoeBindingError::LayerNotFound};
  MoeSparseError sparse{MoeSparseError::ZeroK};
  std::string detail;  // ConfigMismatch / Device
  int rc = 0;          // Device: return code of the C ABI
  std::string to_string() const;
};

// DeepSeek-V3 routing (src/moe/v3_router.rs).  Display texts as in the reference.
struct V3RouterError {
  enum Kind {
    UnsupportedScoringFunc, ExpertsNotDivisibleByGroups, GroupTooSmall, TopkGroupExceedsGroups,
    TopKExceedsSelectable, ZeroParameter, LengthMismatch, NonFinite,
    TopKMismatch  // extension: the configuration's top_k is not the layer's experts_per_token
  };
  Kind kind;
  std::string got;          // UnsupportedScoringFunc
  const char* what = "";    // ZeroParameter / LengthMismatch / NonFinite
  size_t a = 0, b = 0;      // (n_routed, n_group) | experts_per_group | (topk_group, n_group) |
                            // (top_k, selectable) | (expected, actual) | index
  std::string to_string() const;
};
enum class ScoringFunc { Sigmoid };

// Result<T, E> of the reference, reduced to what the mirror needs.
template <typename T, typename E>
class Result {
 public:
  static Result Ok(T v) { Result r; r.v_ = std::move(v); return r; }
  static Result Err(E e) { Result r; r.e_ = std::move(e); return r; }
  bool is_ok() const { return v_.has_value(); }
  bool is_err() const { return !is_ok(); }
  const T& value() const { return *v_; }
  T& value() { return *v_; }
  const E& error() const { return *e_; }
  // `.unwrap()` / `.expect(msg)`: the value, or std::runtime_error carrying the error text.
  T unwrap() const;
  T expect(const char* msg) const;

 private:
  std::optional<T> v_;
  std::optional<E> e_;
};

// ---- types ----------------------------------------------------------------------------------
struct MoeLayerConfig {
  size_t num_experts = 0, experts_per_token = 0;
  bool has_shared_expert = false;
  size_t d_model = 0, d_ff = 0;
  // src/moe/layer.rs:86-116 (new + validate)
  static Result<MoeLayerConfig, MoeConfigError> make(size_t num_experts, size_t experts_per_token,
                                                     bool has_shared_expert, size_t d_model,
                                                     size_t d_ff);
  std::optional<MoeConfigError> validate() const;
};

enum class MoeExecutionConvention { Atenia = 0, HuggingFaceQwen = 1 };

// "sigmoid" only; anything else (also "softmax", which has its own path) is refused
// (src/moe/v3_router.rs:44-57).
Result<ScoringFunc, V3RouterError> parse_scoring_func(const std::string& s);

struct V3RouterConfig {  // src/moe/v3_router.rs:59-72
  size_t n_routed_experts = 0, top_k = 0, n_group = 0, topk_group = 0;
  double routed_scaling_factor = 1.0;
  bool norm_topk_prob = true;
  ScoringFunc scoring_func = ScoringFunc::Sigmoid;
  std::optional<V3RouterError> validate() const;  // src/moe/v3_router.rs:148-181
};

// How the layer's expert weights are stored in HBM.
// Int8PerGroup: one scale per output row and group of kInt8GroupSize input elements (the
// reference's per-group scheme, src/tensor/quantizer.rs:175-248).
enum class MoeWeightStorage { F32 = 0, Bf16 = 1, Int8W8A16 = 2, Int8PerGroup = 3 };

// ---- numeric policy (src/moe/numeric_policy.rs) -----------------------------------------------
// Arithmetic of the expert projections of f32 layers: Certified = f64 accumulation (default and
// fallback), Strict = f32 accumulation, Fast = f32 on the GPU (here: the Strict arithmetic, which
// is what the reference's Fast falls back to).  The router is f64 under every policy.  Process
// global like the reference's: resolved once from ATENIA_NUMERIC_POLICY={certified,strict,fast}
// (also f64 / f32), overridable in-process; anything unknown means Certified.
enum class NumericPolicy { Certified = 0, Strict = 1, Fast = 2 };
const char* as_str(NumericPolicy p);
std::optional<NumericPolicy> numeric_policy_from_str(const std::string& s);
inline bool ffn_uses_f32(NumericPolicy p) { return p != NumericPolicy::Certified; }
inline bool ffn_uses_cuda(NumericPolicy p) { return p == NumericPolicy::Fast; }  // "on the GPU"
NumericPolicy numeric_policy();
void set_numeric_policy(NumericPolicy p);
void clear_numeric_policy_override();

// Comparison of an output with a reference in f64 (src/moe/numerical.rs:22-88): nullopt when
// the lengths differ or are zero; argmax = first index of the largest value.
struct NumericalMetrics {
  size_t len = 0;
  double max_abs_diff = 0.0, mean_abs_diff = 0.0, rmse = 0.0;
  bool argmax_match = false;
  static std::optional<NumericalMetrics> compute(const std::vector<float>& atenia,
                                                 const std::vector<float>& reference);
  bool passes(double tolerance) const { return max_abs_diff < tolerance && argmax_match; }
};

// By-tolerance certificate of a non-Certified policy against Certified rows
// (src/moe/numeric_policy.rs:132-196): worst max |diff| over the rows, means of the per-row mean
// |diff| and of the squared rmse (root taken at the end), share of rows whose argmax agrees, and
// whether the token sequences are identical.  Rows that are empty or differ in length are
// skipped, as NumericalMetrics::compute returns None for them.
struct PolicyCertificate {
  NumericPolicy policy = NumericPolicy::Certified;
  size_t rows = 0;
  double max_abs_diff = 0.0, mean_abs_diff = 0.0, rmse = 0.0, argmax_match_rate = 0.0;
  bool tokens_match = false;
  static PolicyCertificate compare(NumericPolicy policy,
                                   const std::vector<std::vector<float>>& reference_rows,
                                   const std::vector<std::vector<float>>& candidate_rows,
                                   const std::vector<uint32_t>& reference_tokens,
                                   const std::vector<uint32_t>& candidate_tokens);
  bool passes(double tolerance) const {
    return argmax_match_rate >= 1.0 && tokens_match && max_abs_diff <= tolerance;
  }
};
constexpr double STRICT_LOGIT_TOLERANCE = 0.5;
constexpr size_t kInt8GroupSize = 128;

// A per-output-row symmetric int8 weight [rows, cols]: w[r, c] = q[r, c] * scales[r]
// (src/tensor/disk_tier.rs:225-262; the payload of the reference's qint8 tier files).
struct QInt8Tensor {
  size_t rows = 0, cols = 0;
  std::vector<int8_t> q;      // [rows * cols]
  std::vector<float> scales;  // [rows]
  std::vector<float> dequantize() const;  // disk_tier.rs:251-262
};
struct QInt8Projections {
  QInt8Tensor gate, up, down;
};

struct MoeDenseExpert {
  size_t d_model = 0, d_ff = 0;
  std::vector<float> w_gate, w_up, w_down;  // [d_ff,d_model], [d_ff,d_model], [d_model,d_ff]
  // Set when the expert came from int8 tier data (from_qint8): w_* hold the dequantised values
  // the reference computes with, and a layer stored as Int8W8A16 uploads q / scales as they
  // are instead of quantising w_* again.
  std::shared_ptr<const QInt8Projections> q8;
  static Result<MoeDenseExpert, MoeDenseError> from_qint8(size_t d_model, size_t d_ff,
                                                          QInt8Tensor gate, QInt8Tensor up,
                                                          QInt8Tensor down);
  static Result<MoeDenseExpert, MoeDenseError> make(size_t d_model, size_t d_ff,
                                                    std::vector<float> w_gate,
                                                    std::vector<float> w_up,
                                                    std::vector<float> w_down);
  // y = W_down (silu(W_gate x) * (W_up x)) for one token (src/moe/dense.rs:253-270), on the
  // device under the active numeric policy.  Unit-level entry: it uploads the expert for the
  // call; layers that run many tokens go through RealMoeLayer / the registry.
  Result<std::vector<float>, MoeDenseError> forward(const std::vector<float>& x) const;
};

// src/moe/dense.rs:189-201 and src/moe/sparse.rs:195-201
struct MoeRouterOutput {
  std::vector<float> weights;  // one per expert, softmax of the router logits
  float weight_sum() const {
    float s = 0.f;
    for (float w : weights) s += w;
    return s;
  }
};
struct MoeSparseForwardOutput {
  std::vector<float> output;
  std::vector<size_t> selected_experts;  // ascending
};

struct MoeDenseLayer {
  size_t d_model = 0, d_ff = 0;
  std::vector<float> w_router;  // [num_experts, d_model]
  std::vector<MoeDenseExpert> experts;
  size_t conceptual_top_k = 0;
  static Result<MoeDenseLayer, MoeDenseError> make(size_t d_model, size_t d_ff,
                                                   std::vector<float> w_router,
                                                   std::vector<MoeDenseExpert> experts,
                                                   size_t conceptual_top_k);
  size_t num_experts() const { return experts.size(); }
  // One token through the routed experts, on the device (unit-level entries like
  // MoeDenseExpert::forward: the layer is uploaded for the call).
  //   route                softmax(W_router x)                      src/moe/dense.rs:325-337
  //   forward              every expert, weighted by its softmax weight   :341-359
  //   forward_sparse[_with] top-k experts, renormalised or raw weights     src/moe/sparse.rs:206-238
  // A non-finite router weight makes forward() return NaNs, as the reference's arithmetic does,
  // and forward_sparse an error, as its validation does.
  Result<MoeRouterOutput, MoeDenseError> route(const std::vector<float>& x) const;
  Result<std::vector<float>, MoeDenseError> forward(const std::vector<float>& x) const;
  Result<MoeSparseForwardOutput, MoeSparseError> forward_sparse(const std::vector<float>& x,
                                                                size_t k) const;
  Result<MoeSparseForwardOutput, MoeSparseError> forward_sparse_with(const std::vector<float>& x,
                                                                     size_t k,
                                                                     bool renormalize) const;
};

class RealMoeLayer {
 public:
  MoeLayerConfig config;
  MoeDenseLayer routed;
  std::optional<MoeDenseExpert> shared;
  std::optional<std::vector<float>> shared_gate;
  MoeWeightStorage storage = MoeWeightStorage::F32;
  // DeepSeek-V3 routing in front of this layer's experts (unset = softmax routing).
  std::optional<V3RouterConfig> v3_router;
  std::vector<float> e_score_correction_bias;

  // Routes every later forward the DeepSeek-V3 way (sigmoid scores, bias-corrected and
  // group-limited selection, scaled weights; src/moe/v3_router.rs:206-309).  The shared expert,
  // if any, is then added ungated.  Fails like v3_route does on a bad configuration or bias;
  // cfg.n_routed_experts / cfg.top_k must be this layer's.
  std::optional<V3RouterError> set_v3_router(const V3RouterConfig& cfg, std::vector<float> bias);

  // Cross-checks the parts against the config the way RealMoeLayer::assemble does
  // (src/moe/layer.rs:282-343): expert count, dimensions, shared expert present iff asked for.
  static Result<RealMoeLayer, MoeLayerError> assemble(MoeLayerConfig config, MoeDenseLayer routed,
                                                      std::optional<MoeDenseExpert> shared,
                                                      std::optional<std::vector<float>> shared_gate,
                                                      MoeWeightStorage storage = MoeWeightStorage::F32);

  size_t num_experts() const { return routed.num_experts(); }
  bool has_shared_expert() const { return shared.has_value(); }
  MoeExecutionConvention resolve_convention() const {
    return shared_gate ? MoeExecutionConvention::HuggingFaceQwen : MoeExecutionConvention::Atenia;
  }

  // x: one token [d_model] or a flat batch [n * d_model]; the layer is position-wise.
  Result<std::vector<float>, MoeLayerError> forward(const std::vector<float>& x) const;
  Result<std::vector<float>, MoeLayerError> forward_auto(const std::vector<float>& x) const;
  Result<std::vector<float>, MoeLayerError> forward_with(const std::vector<float>& x,
                                                         MoeExecutionConvention convention) const;
  // Routed experts only, renormalised combine (src/moe/layer.rs:366-369).
  Result<std::vector<float>, MoeLayerError> forward_routed(const std::vector<float>& x) const;
  // The FFN half of a decoder layer: x1 + MoE(RMSNorm(x1) * gamma) for each row of x1, the
  // layer run under `convention`.  Steps 13-15 of the layer loop in
  // src/moe/full_forward.rs:239-252 (norm_policy GraphF32: RmsNorm + BroadcastMul nodes in
  // f32), and the second half of src/moe/mla.rs:442-453 / decoder_layer_reference
  // (norm_policy F64: src/moe/decoder_layer.rs:97-107).  One C-ABI call for the whole batch.
  enum class NormPolicy { GraphF32 = 0, F64 = 1 };
  Result<std::vector<float>, MoeLayerError> ffn_block(const std::vector<float>& x1,
                                                      const std::vector<float>& gamma, float eps,
                                                      NormPolicy norm_policy,
                                                      MoeExecutionConvention convention) const;
  // Routing of each row: indices [n * k] (ascending per row) and weights, under `convention`.
  Result<std::vector<float>, MoeLayerError> route(const std::vector<float>& x,
                                                  MoeExecutionConvention convention,
                                                  std::vector<int32_t>* indices) const;

  RealMoeLayer();
  RealMoeLayer(const RealMoeLayer& o);             // copies the host weights, not device state
  RealMoeLayer& operator=(const RealMoeLayer& o);
  RealMoeLayer(RealMoeLayer&&) noexcept;
  RealMoeLayer& operator=(RealMoeLayer&&) noexcept;
  ~RealMoeLayer();

 private:
  struct Device;  // lazily created C-ABI handles, one per (convention, with shared)
  mutable std::unique_ptr<Device> dev_;
  Result<std::vector<float>, MoeLayerError> run(const std::vector<float>& x,
                                                MoeExecutionConvention convention,
                                                bool with_shared) const;
  Result<void*, MoeLayerError> handle_for(MoeExecutionConvention convention, bool with_shared) const;
};

// ---- registry of MoeDenseLayer and the decomposed graph ops (src/moe/graph_op.rs:28-205) -------
// Behind NodeType::MoeSparseReference / MoeDynamicDispatch / ConditionalExpert: the selection
// arrives as data, a flat [idx0, w0, idx1, w1, ...] f32 tensor (what MoeTopK emits), and only the
// listed experts run -- here on the device, one MoeDenseExpert::forward per listed expert; the
// weighted sum over the handful of listed experts is formed on the host in the listed order, as
// the reference forms it.
uint32_t register_layer(MoeDenseLayer layer);
std::shared_ptr<const MoeDenseLayer> get_layer(uint32_t layer_id);
// forward_sparse(input, k).output of a registered layer; an unknown id is Dense(NoExperts).
Result<std::vector<float>, MoeSparseError> execute_sparse_reference(uint32_t layer_id,
                                                                    const std::vector<float>& input,
                                                                    size_t k);
struct DynamicDispatchOutput {
  std::vector<float> output;
  std::vector<size_t> executed_experts;  // in the order of the selection
};
Result<DynamicDispatchOutput, MoeSparseError> execute_dynamic_dispatch(
    uint32_t layer_id, const std::vector<float>& input, const std::vector<float>& selection);
std::optional<float> expert_weight_in_selection(const std::vector<float>& selection,
                                                uint32_t expert_id);
// (weight * expert(input), true) when expert_id is in the selection, else (zeros, false) without
// running the expert.
Result<std::pair<std::vector<float>, bool>, MoeSparseError> execute_conditional_expert(
    uint32_t layer_id, uint32_t expert_id, const std::vector<float>& input,
    const std::vector<float>& selection);

// ---- ResidentExpertLayer (src/moe/residency.rs:66-109, 586-614, 706-791) -------------------------
// The reference keeps a layer's experts in a residency tier (RAM f32, bf16 RAM, NVMe) and
// resolves the selected ones per token; its DeepSeek decoders call ResidentExpertLayer::forward
// directly and its registry holds such layers next to the RAM ones (graph_op.rs:234-247).  With
// every expert resident in HBM the tiers collapse to one, `Hbm`: nothing is materialised per
// token, so the evidence the reference returns with each forward is what the kernels read --
// the selected experts and their stored bytes.
enum class ExpertTier { Hbm };
struct ResidencyInfo {
  std::vector<size_t> materialized_experts;  // routed experts the token used, ascending
  size_t materialized_bytes = 0;             // their stored bytes, plus the shared expert's
};
class ResidentExpertLayer {
 public:
  MoeLayerConfig config;
  MoeExecutionConvention convention = MoeExecutionConvention::Atenia;
  ExpertTier tier = ExpertTier::Hbm;

  // The layer's weights go to the device in the layer's own storage type on first use;
  // convention = layer.resolve_convention(), as the reference's constructor takes it.
  static ResidentExpertLayer from_real_layer(const RealMoeLayer& layer, ExpertTier tier = ExpertTier::Hbm);
  size_t num_experts() const { return config.num_experts; }
  // Bytes of one routed expert / of the shared expert as stored in HBM.
  size_t expert_bytes() const;
  size_t shared_bytes() const;
  // One token [d_model]: output and evidence; equal to RealMoeLayer::forward_with under
  // `convention` (src/moe/residency.rs:732-791).
  Result<std::pair<std::vector<float>, ResidencyInfo>, MoeLayerError> forward(
      const std::vector<float>& x) const;
  // A flat batch [n * d_model] in one device call; infos (optional) receives one entry per row.
  Result<std::vector<float>, MoeLayerError> forward_batch(const std::vector<float>& x,
                                                          std::vector<ResidencyInfo>* infos = nullptr) const;

 private:
  std::shared_ptr<RealMoeLayer> layer_;
};

// ---- registry and graph op --------------------------------------------------------------------
// Process-global, grow-only, ids stable per process (src/moe/graph_op.rs:221-232).
// Resident layers share the id space with the RAM ones (graph_op.rs:207-216, 234-247);
// cache_capacity is accepted for signature parity: with one HBM tier there is no expert cache.
uint32_t register_resident_moe_layer(std::shared_ptr<ResidentExpertLayer> layer,
                                     size_t cache_capacity = 0);
uint32_t register_real_moe_layer(RealMoeLayer layer);
std::shared_ptr<const RealMoeLayer> get_real_moe_layer(uint32_t layer_id);
Result<std::vector<float>, MoeLayerError> execute_real_moe_layer(uint32_t layer_id,
                                                                 const std::vector<float>& input);
Result<std::vector<float>, MoeLayerError> execute_real_moe_layer_with(
    uint32_t layer_id, const std::vector<float>& input, MoeExecutionConvention convention);
// The executor arm of NodeType::MoeRealLayerReference{layer_id}: returns the output tensor's data
// or throws std::runtime_error("MoeRealLayerReference: forward failed (unknown layer_id or bad
// input dim)") as the reference panics.
std::vector<float> moe_real_layer_reference_node(uint32_t layer_id, const std::vector<float>& input);

// ---- template members -------------------------------------------------------------------------
}  // namespace moe
}  // namespace atenia

#include <stdexcept>
namespace atenia {
namespace moe {
inline std::string error_text(const std::string& e) { return e; }
template <typename E>
std::string error_text(const E& e) { return e.to_string(); }
template <typename T, typename E>
T Result<T, E>::unwrap() const {
  if (!is_ok()) throw std::runtime_error("called `Result::unwrap()` on an `Err` value: " + error_text(*e_));
  return *v_;
}
template <typename T, typename E>
T Result<T, E>::expect(const char* msg) const {
  if (!is_ok()) throw std::runtime_error(std::string(msg) + ": " + error_text(*e_));
  return *v_;
}
}  // namespace moe
}  // namespace atenia
