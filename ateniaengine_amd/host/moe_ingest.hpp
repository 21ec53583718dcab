// Weight ingestion for the host mirror: from a checkpoint file to a runnable RealMoeLayer.
// Follows the reference's data plane (names and behaviour), in C++:
//
//   SafetensorsReader                      src/v17/loader/safetensors_reader.rs (open / iter / get /
//                                          to_vec_f32; header = 8-byte LE length + JSON)
//   TensorRole, classify_tensor_name, is_moe_expert_tensor, is_moe_router_tensor,
//   MoeDetection, detect_moe, unsupported_message       src/moe/detect.rs:42-262
//   MoeTensorEntry, ExpertTensors, MoeLayerMap, MoeWeightMap::from_tensors
//                                                       src/moe/data_plane.rs:30-190
//   build_real_layer (classic per-expert tensors), packed_dims, build_packed_layer
//   (gate_up_proj [E, 2f, d] with gate = rows 0..f, down_proj [E, d, f])
//                                                       src/moe/binding.rs:246-470
//   assemble_real_moe_layer = RealMoeLayer::assemble    src/moe/layer.rs:212-343
//   MoeConventionResolver                               src/moe/convention.rs
//   MoeConfig (config.json keys of the MoE families)    src/nn/llama/moe_config.rs:52-150
//   qint8 tier files: quantize_per_row_i8, qint8_disk_bytes, write_qint8_tensor_named,
//   read_qint8_tensor / read_qint8_to_f32               src/tensor/disk_tier.rs:168-262
#pragma once

#include <functional>
#include <map>
#include <optional>
#include <string>
#include <utility>
#include <vector>

#include "atenia_moe.hpp"

namespace atenia {
namespace moe {

// ---- safetensors ------------------------------------------------------------------------------
struct SafetensorsEntry {
  std::string name;
  std::string dtype;  // "F32", "BF16", "F16", ...
  std::vector<size_t> shape;
  size_t begin = 0, end = 0;  // byte range inside the data section
  size_t numel() const;
};

class SafetensorsReader {
 public:
  // Reads and validates the header; the tensor data is read on demand.
  static Result<SafetensorsReader, std::string> open(const std::string& path);
  const std::vector<SafetensorsEntry>& entries() const { return entries_; }
  const SafetensorsEntry* get(const std::string& name) const;
  // The tensor as f32 (F32 copied, BF16 / F16 widened exactly); nullopt for an unknown name,
  // an unsupported dtype or a short file.
  std::optional<std::vector<float>> to_vec_f32(const std::string& name) const;
  // (name, shape) of every tensor: what MoeWeightMap::from_tensors consumes.
  std::vector<std::pair<std::string, std::vector<size_t>>> names_and_shapes() const;

 private:
  std::string path_;
  size_t data_start_ = 0, file_size_ = 0;
  std::vector<SafetensorsEntry> entries_;
};

// ---- tensor names -----------------------------------------------------------------------------
enum class TensorRole {
  AttentionQ, AttentionK, AttentionV, AttentionO, MlpGate, MlpUp, MlpDown, MoeRouter,
  MoeExpertGate, MoeExpertUp, MoeExpertDown, MoeSharedExpert, MoePackedGateUp, MoePackedDown,
  Unknown
};
bool role_is_moe(TensorRole r);
bool role_is_moe_expert(TensorRole r);
bool role_is_moe_packed(TensorRole r);

struct TensorNameInfo {
  TensorRole role = TensorRole::Unknown;
  std::optional<size_t> layer_id, expert_id;
};
bool is_moe_expert_tensor(const std::string& name);
bool is_moe_router_tensor(const std::string& name);
TensorNameInfo classify_tensor_name(const std::string& name);

struct MoeDetection {
  bool is_moe = false;
  size_t expert_tensor_count = 0, router_tensor_count = 0, shared_expert_tensor_count = 0;
  std::optional<size_t> max_expert_id;
  std::optional<size_t> implied_expert_count() const;
};
MoeDetection detect_moe(const std::vector<std::string>& names);
std::string unsupported_message(const MoeDetection& det);

// ---- weight map -------------------------------------------------------------------------------
struct MoeTensorEntry {
  std::string name;
  std::optional<size_t> layer_id, expert_id;
  TensorRole role = TensorRole::Unknown;
  std::vector<size_t> shape;
};
struct ExpertTensors {
  std::optional<MoeTensorEntry> gate, up, down;
  bool is_complete() const { return gate && up && down; }
};
struct MoeLayerMap {
  std::optional<MoeTensorEntry> router;
  std::map<size_t, ExpertTensors> experts;  // ascending expert id
  std::vector<MoeTensorEntry> shared;
  std::optional<MoeTensorEntry> packed_gate_up, packed_down;
  size_t num_experts() const { return experts.size(); }
  bool has_classic_experts() const { return !experts.empty(); }
  bool has_packed_experts() const { return packed_gate_up && packed_down; }
};
struct MoeWeightMap {
  std::map<size_t, MoeLayerMap> layers;  // ascending layer id
  static MoeWeightMap from_tensors(
      const std::vector<std::pair<std::string, std::vector<size_t>>>& tensors);
  bool is_empty() const { return layers.empty(); }
  const MoeLayerMap* layer(size_t layer_id) const;
  const MoeTensorEntry* router_weight(size_t layer_id) const;
  const ExpertTensors* expert(size_t layer_id, size_t expert_id) const;
  size_t num_experts(size_t layer_id) const;
  size_t total_expert_tensors() const;
  bool all_experts_complete() const;
};

struct MoeConventionResolver {
  static MoeExecutionConvention from_weight_map(const MoeWeightMap& map);
  static MoeExecutionConvention from_shared_gate_present(bool present) {
    return present ? MoeExecutionConvention::HuggingFaceQwen : MoeExecutionConvention::Atenia;
  }
  // DeepSeek-MoE: its shared expert has no gate tensor, so the combine convention comes from
  // config.json's norm_topk_prob instead (unset or true = renormalise = Atenia; false = raw top-k
  // weights = HuggingFaceQwen with an ungated shared expert).  src/moe/runtime.rs:894-907.
  static MoeExecutionConvention from_norm_topk_prob(std::optional<bool> norm_topk_prob) {
    return norm_topk_prob.value_or(true) ? MoeExecutionConvention::Atenia
                                         : MoeExecutionConvention::HuggingFaceQwen;
  }
};

// ---- config.json ------------------------------------------------------------------------------
// The MoE block of a HuggingFace config.json.  Families name the same thing differently:
// expert count = num_experts | num_local_experts | n_routed_experts, top-k = num_experts_per_tok |
// num_experts_per_token, expert width = moe_intermediate_size | expert_intermediate_size (the
// first key present wins, in that order).  A dense config leaves everything unset.
struct MoeConfig {
  std::optional<size_t> num_experts, experts_per_token, num_shared_experts;
  bool has_shared_experts = false;  // n_shared_experts > 0 or shared_expert_intermediate_size set
  std::optional<bool> norm_topk_prob;
  std::optional<float> router_aux_loss_coef;
  std::optional<size_t> expert_intermediate_size, shared_expert_intermediate_size;

  static Result<MoeConfig, std::string> from_json_str(const std::string& json);
  bool is_moe() const { return num_experts.has_value(); }
  // top-k, at least 1 and at most the expert count when that is known and positive.
  size_t experts_per_token_or(size_t fallback) const;
  bool renormalize_topk_or(bool fallback) const { return norm_topk_prob.value_or(fallback); }
  bool operator==(const MoeConfig& o) const;
};

// ---- qint8 tier files -------------------------------------------------------------------------
// One tensor per file: [rows x f32 scale, little endian][rows * cols x i8], the layout the
// reference's residency tier writes for expert weights (src/moe/residency.rs:344-355).  Read
// back, q and scales go to HBM as they are (MoeDenseExpert::from_qint8 + Int8W8A16 storage).
QInt8Tensor quantize_per_row_i8(const std::vector<float>& data, size_t rows, size_t cols);
inline size_t qint8_disk_bytes(size_t numel, size_t rows) { return rows * 4 + numel; }
// nullopt on success, else what failed.
std::optional<std::string> write_qint8_tensor_named(const std::string& path,
                                                    const std::vector<float>& data, size_t rows,
                                                    size_t cols);
// `rows` is the quantisation axis (the tensor's first dimension), cols = numel / rows.  A file
// whose size is not rows * 4 + numel is refused (the reference's InvalidData).
Result<QInt8Tensor, std::string> read_qint8_tensor(const std::string& path, size_t numel,
                                                   size_t rows);
Result<std::vector<float>, std::string> read_qint8_to_f32(const std::string& path, size_t numel,
                                                          size_t rows);

// ---- binding ----------------------------------------------------------------------------------
// name -> f32 data, or nullopt (the reference's `resolve: &Fn(&str) -> Option<Vec<f32>>`).
typedef std::function<std::optional<std::vector<float>>(const std::string&)> TensorResolver;

struct PackedExpertDims { size_t num_experts = 0, d_model = 0, d_ff = 0; };
Result<PackedExpertDims, MoeBindingError> packed_dims(const MoeTensorEntry& gate_up,
                                                      const MoeTensorEntry& down);
Result<MoeDenseLayer, MoeBindingError> build_real_layer(const MoeWeightMap& map, size_t layer_id,
                                                        size_t conceptual_top_k,
                                                        const TensorResolver& resolve);
Result<MoeDenseLayer, MoeBindingError> build_packed_layer(const MoeWeightMap& map, size_t layer_id,
                                                          size_t conceptual_top_k,
                                                          const TensorResolver& resolve);
// The whole layer for `layer_id`, cross-checked against `config`: classic or packed experts
// (both present = MixedExpertFormat), router, shared expert and its sigmoid gate when
// config.has_shared_expert.
Result<RealMoeLayer, MoeLayerError> assemble_real_moe_layer(
    const MoeWeightMap& map, size_t layer_id, MoeLayerConfig config, const TensorResolver& resolve,
    MoeWeightStorage storage = MoeWeightStorage::F32);

}  // namespace moe
}  // namespace atenia
