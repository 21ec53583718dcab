// Weight ingestion for the host mirror (see moe_ingest.hpp for the reference map).
#include "moe_ingest.hpp"

#include <cstdio>
#include <cstring>
#include <initializer_list>

#include "../../include/atenia_moe_hip.h"
#include "json_mini.hpp"

namespace atenia {
namespace moe {

namespace {
bool has(const std::string& s, const char* needle) { return s.find(needle) != std::string::npos; }

// The decimal id right after the first `marker` in `name` (src/moe/detect.rs:107-116).
std::optional<size_t> id_after(const std::string& name, const char* marker) {
  const size_t at = name.find(marker);
  if (at == std::string::npos) return std::nullopt;
  size_t i = at + std::strlen(marker), v = 0, n = 0;
  for (; i < name.size() && name[i] >= '0' && name[i] <= '9'; ++i, ++n) {
    if (v > (SIZE_MAX - 9) / 10) return std::nullopt;  // would not fit: not an id
    v = v * 10 + (size_t)(name[i] - '0');
  }
  if (n == 0) return std::nullopt;
  return v;
}

// Rust's `{:?}` of a Vec<usize>: "[a, b, c]".
std::string fmt_shape(const std::vector<size_t>& s) {
  std::string o = "[";
  for (size_t i = 0; i < s.size(); ++i) {
    if (i) o += ", ";
    o += std::to_string(s[i]);
  }
  return o + "]";
}

size_t product(const std::vector<size_t>& s) {
  size_t p = 1;
  for (size_t v : s) p *= v;
  return p;
}

float f16_to_f32(uint16_t h) {
  const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1f, man = h & 0x3ffu, bits;
  if (exp == 0) {
    if (man == 0) {
      bits = sign;
    } else {  // subnormal: renormalise
      int e = -1;
      do {
        man <<= 1;
        ++e;
      } while (!(man & 0x400u));
      bits = sign | (uint32_t)(127 - 15 - e) << 23 | (man & 0x3ffu) << 13;
    }
  } else if (exp == 31) {
    bits = sign | 0x7f800000u | man << 13;
  } else {
    bits = sign | (exp + 127 - 15) << 23 | man << 13;
  }
  float f;
  std::memcpy(&f, &bits, 4);
  return f;
}
}  // namespace

// ---- safetensors ------------------------------------------------------------------------------
size_t SafetensorsEntry::numel() const { return product(shape); }

Result<SafetensorsReader, std::string> SafetensorsReader::open(const std::string& path) {
  typedef Result<SafetensorsReader, std::string> R;
  FILE* f = std::fopen(path.c_str(), "rb");
  if (!f) return R::Err("safetensors: cannot open '" + path + "'");
  SafetensorsReader r;
  r.path_ = path;
  std::fseek(f, 0, SEEK_END);
  const long sz = std::ftell(f);
  std::fseek(f, 0, SEEK_SET);
  r.file_size_ = sz < 0 ? 0 : (size_t)sz;
  unsigned char len8[8];
  if (r.file_size_ < 8 || std::fread(len8, 1, 8, f) != 8) {
    std::fclose(f);
    return R::Err("safetensors: '" + path + "' is shorter than its 8-byte header length");
  }
  uint64_t hlen = 0;
  for (int i = 7; i >= 0; --i) hlen = hlen << 8 | len8[i];
  if (hlen > r.file_size_ - 8) {
    std::fclose(f);
    return R::Err("safetensors: header length " + std::to_string(hlen) + " exceeds the file");
  }
  std::string header((size_t)hlen, '\0');
  const size_t got = std::fread(&header[0], 1, (size_t)hlen, f);
  std::fclose(f);
  if (got != hlen) return R::Err("safetensors: short read of the header");
  r.data_start_ = 8 + (size_t)hlen;
  json::Value root;
  if (!json::parse(header, root) || !root.is(json::Value::Object))
    return R::Err("safetensors: header is not a JSON object");
  const size_t data_size = r.file_size_ - r.data_start_;
  for (const auto& kv : root.obj) {
    if (kv.first == "__metadata__") continue;
    const json::Value& t = kv.second;
    const json::Value* dt = t.get("dtype");
    const json::Value* sh = t.get("shape");
    const json::Value* off = t.get("data_offsets");
    if (!dt || !sh || !off || !dt->is(json::Value::String) || !sh->is(json::Value::Array) ||
        !off->is(json::Value::Array) || off->arr.size() != 2)
      return R::Err("safetensors: malformed entry '" + kv.first + "'");
    SafetensorsEntry e;
    e.name = kv.first;
    e.dtype = dt->str;
    for (const auto& d : sh->arr) e.shape.push_back((size_t)d.num);
    e.begin = (size_t)off->arr[0].num;
    e.end = (size_t)off->arr[1].num;
    if (e.begin > e.end || e.end > data_size)
      return R::Err("safetensors: entry '" + kv.first + "' lies outside the data section");
    r.entries_.push_back(std::move(e));
  }
  return R::Ok(std::move(r));
}

const SafetensorsEntry* SafetensorsReader::get(const std::string& name) const {
  for (const auto& e : entries_)
    if (e.name == name) return &e;
  return nullptr;
}

std::vector<std::pair<std::string, std::vector<size_t>>> SafetensorsReader::names_and_shapes() const {
  std::vector<std::pair<std::string, std::vector<size_t>>> v;
  v.reserve(entries_.size());
  for (const auto& e : entries_) v.emplace_back(e.name, e.shape);
  return v;
}

std::optional<std::vector<float>> SafetensorsReader::to_vec_f32(const std::string& name) const {
  const SafetensorsEntry* e = get(name);
  if (!e) return std::nullopt;
  size_t width = 0;
  if (e->dtype == "F32") width = 4;
  else if (e->dtype == "BF16" || e->dtype == "F16") width = 2;
  else return std::nullopt;
  const size_t n = e->numel();
  if (e->end - e->begin != n * width) return std::nullopt;
  FILE* f = std::fopen(path_.c_str(), "rb");
  if (!f) return std::nullopt;
  std::vector<float> out(n);
  bool ok = std::fseek(f, (long)(data_start_ + e->begin), SEEK_SET) == 0;
  if (ok && width == 4) {
    ok = std::fread(out.data(), 4, n, f) == n;
  } else if (ok) {
    std::vector<uint16_t> raw(n);
    ok = std::fread(raw.data(), 2, n, f) == n;
    if (ok && e->dtype == "BF16") {
      for (size_t i = 0; i < n; ++i) {
        const uint32_t b = (uint32_t)raw[i] << 16;
        std::memcpy(&out[i], &b, 4);
      }
    } else if (ok) {
      for (size_t i = 0; i < n; ++i) out[i] = f16_to_f32(raw[i]);
    }
  }
  std::fclose(f);
  if (!ok) return std::nullopt;
  return out;
}

// ---- tensor names -----------------------------------------------------------------------------
bool role_is_moe(TensorRole r) { return r == TensorRole::MoeRouter || role_is_moe_expert(r); }
bool role_is_moe_expert(TensorRole r) {
  return r == TensorRole::MoeExpertGate || r == TensorRole::MoeExpertUp ||
         r == TensorRole::MoeExpertDown || r == TensorRole::MoeSharedExpert || role_is_moe_packed(r);
}
bool role_is_moe_packed(TensorRole r) {
  return r == TensorRole::MoePackedGateUp || r == TensorRole::MoePackedDown;
}

bool is_moe_expert_tensor(const std::string& name) {
  return has(name, ".experts.") || has(name, "shared_expert");
}

bool is_moe_router_tensor(const std::string& name) {
  return has(name, "block_sparse_moe.gate.") ||
         (has(name, ".mlp.gate.") && !has(name, "gate_proj")) || has(name, ".mlp.router.");
}

TensorNameInfo classify_tensor_name(const std::string& name) {
  TensorNameInfo info;
  info.layer_id = id_after(name, ".layers.");
  info.expert_id = id_after(name, ".experts.");
  TensorRole r = TensorRole::Unknown;
  if (has(name, "shared_expert")) {
    r = TensorRole::MoeSharedExpert;
  } else if (has(name, "experts.gate_up_proj")) {
    r = TensorRole::MoePackedGateUp;
  } else if (has(name, "experts.") && !info.expert_id && has(name, "down_proj")) {
    r = TensorRole::MoePackedDown;
  } else if (has(name, ".experts.")) {
    if (has(name, ".w1.") || has(name, ".gate_proj.")) r = TensorRole::MoeExpertGate;
    else if (has(name, ".w3.") || has(name, ".up_proj.")) r = TensorRole::MoeExpertUp;
    else if (has(name, ".w2.") || has(name, ".down_proj.")) r = TensorRole::MoeExpertDown;
  } else if (is_moe_router_tensor(name)) {
    r = TensorRole::MoeRouter;
  } else if (has(name, "q_proj")) {
    r = TensorRole::AttentionQ;
  } else if (has(name, "k_proj")) {
    r = TensorRole::AttentionK;
  } else if (has(name, "v_proj")) {
    r = TensorRole::AttentionV;
  } else if (has(name, "o_proj")) {
    r = TensorRole::AttentionO;
  } else if (has(name, "gate_proj")) {
    r = TensorRole::MlpGate;
  } else if (has(name, "up_proj")) {
    r = TensorRole::MlpUp;
  } else if (has(name, "down_proj")) {
    r = TensorRole::MlpDown;
  }
  info.role = r;
  return info;
}

std::optional<size_t> MoeDetection::implied_expert_count() const {
  if (!max_expert_id) return std::nullopt;
  return *max_expert_id + 1;
}

MoeDetection detect_moe(const std::vector<std::string>& names) {
  MoeDetection det;
  for (const auto& name : names) {
    const TensorNameInfo info = classify_tensor_name(name);
    if (info.role == TensorRole::MoeRouter) {
      ++det.router_tensor_count;
    } else if (info.role == TensorRole::MoeSharedExpert) {
      ++det.shared_expert_tensor_count;
      det.is_moe = true;
    } else if (role_is_moe_expert(info.role)) {
      ++det.expert_tensor_count;
      det.is_moe = true;
    }
    if (info.expert_id && (!det.max_expert_id || *info.expert_id > *det.max_expert_id))
      det.max_expert_id = info.expert_id;
  }
  return det;
}

std::string unsupported_message(const MoeDetection& det) {
  // The sentence a dense loader fails with, worded as the reference words it
  // (src/moe/detect.rs:251-264; its own tests look for "MoE checkpoint detected", "not implemented
  // yet" and the counted fields, detect.rs:425-428, tests/moe_loader_failloud_test.rs:47), followed
  // by this library's advice: such a checkpoint goes through assemble_real_moe_layer instead.
  const auto n = det.implied_expert_count();
  return "MoE checkpoint detected, but MoE execution is not implemented yet (experts=" +
         (n ? std::to_string(*n) : std::string("unknown")) +
         ", expert_tensors=" + std::to_string(det.expert_tensor_count) +
         ", router_tensors=" + std::to_string(det.router_tensor_count) +
         ", shared_expert_tensors=" + std::to_string(det.shared_expert_tensor_count) +
         "). Atenia can load and run dense models only; loading this checkpoint as dense would "
         "silently drop the expert weights and produce a broken model. On the MI355X path bind it "
         "with MoeWeightMap::from_tensors and assemble_real_moe_layer instead.";
}

// ---- weight map -------------------------------------------------------------------------------
MoeWeightMap MoeWeightMap::from_tensors(
    const std::vector<std::pair<std::string, std::vector<size_t>>>& tensors) {
  MoeWeightMap map;
  for (const auto& ns : tensors) {
    const TensorNameInfo info = classify_tensor_name(ns.first);
    if (!role_is_moe(info.role) || !info.layer_id) continue;
    MoeTensorEntry entry{ns.first, info.layer_id, info.expert_id, info.role, ns.second};
    MoeLayerMap& layer = map.layers[*info.layer_id];
    switch (info.role) {
      case TensorRole::MoeRouter: layer.router = std::move(entry); break;
      case TensorRole::MoeSharedExpert: layer.shared.push_back(std::move(entry)); break;
      case TensorRole::MoePackedGateUp: layer.packed_gate_up = std::move(entry); break;
      case TensorRole::MoePackedDown: layer.packed_down = std::move(entry); break;
      default:
        if (info.expert_id) {
          ExpertTensors& ex = layer.experts[*info.expert_id];
          if (info.role == TensorRole::MoeExpertGate) ex.gate = std::move(entry);
          else if (info.role == TensorRole::MoeExpertUp) ex.up = std::move(entry);
          else ex.down = std::move(entry);
        }
    }
  }
  return map;
}

const MoeLayerMap* MoeWeightMap::layer(size_t layer_id) const {
  auto it = layers.find(layer_id);
  return it == layers.end() ? nullptr : &it->second;
}
const MoeTensorEntry* MoeWeightMap::router_weight(size_t layer_id) const {
  const MoeLayerMap* l = layer(layer_id);
  return l && l->router ? &*l->router : nullptr;
}
const ExpertTensors* MoeWeightMap::expert(size_t layer_id, size_t expert_id) const {
  const MoeLayerMap* l = layer(layer_id);
  if (!l) return nullptr;
  auto it = l->experts.find(expert_id);
  return it == l->experts.end() ? nullptr : &it->second;
}
size_t MoeWeightMap::num_experts(size_t layer_id) const {
  const MoeLayerMap* l = layer(layer_id);
  return l ? l->num_experts() : 0;
}
size_t MoeWeightMap::total_expert_tensors() const {
  size_t n = 0;
  for (const auto& l : layers)
    for (const auto& e : l.second.experts)
      n += (size_t)e.second.gate.has_value() + e.second.up.has_value() + e.second.down.has_value();
  return n;
}
bool MoeWeightMap::all_experts_complete() const {
  for (const auto& l : layers)
    for (const auto& e : l.second.experts)
      if (!e.second.is_complete()) return false;
  return true;
}

MoeExecutionConvention MoeConventionResolver::from_weight_map(const MoeWeightMap& map) {
  for (const auto& l : map.layers)
    for (const auto& e : l.second.shared)
      if (has(e.name, "shared_expert_gate")) return MoeExecutionConvention::HuggingFaceQwen;
  return MoeExecutionConvention::Atenia;
}

// ---- config.json ------------------------------------------------------------------------------
namespace {
// The first of `keys` that holds a non-negative integer literal (serde_json's as_u64).
std::optional<size_t> first_usize(const json::Value& v, std::initializer_list<const char*> keys) {
  for (const char* k : keys) {
    const json::Value* x = v.get(k);
    if (x && x->is(json::Value::Number) && x->is_int && x->num >= 0) return (size_t)x->num;
  }
  return std::nullopt;
}
}  // namespace

Result<MoeConfig, std::string> MoeConfig::from_json_str(const std::string& text) {
  typedef Result<MoeConfig, std::string> R;
  json::Value v;
  if (!json::parse(text, v)) return R::Err("moe-config: not valid JSON");
  MoeConfig c;  // a JSON value that is no object has no keys: everything stays unset
  c.num_experts = first_usize(v, {"num_experts", "num_local_experts", "n_routed_experts"});
  c.experts_per_token = first_usize(v, {"num_experts_per_tok", "num_experts_per_token"});
  c.num_shared_experts = first_usize(v, {"n_shared_experts"});
  c.shared_expert_intermediate_size = first_usize(v, {"shared_expert_intermediate_size"});
  c.expert_intermediate_size = first_usize(v, {"moe_intermediate_size", "expert_intermediate_size"});
  c.has_shared_experts = (c.num_shared_experts && *c.num_shared_experts > 0) ||
                         c.shared_expert_intermediate_size.has_value();
  if (const json::Value* b = v.get("norm_topk_prob"))
    if (b->is(json::Value::Bool)) c.norm_topk_prob = b->b;
  if (const json::Value* a = v.get("router_aux_loss_coef"))
    if (a->is(json::Value::Number)) c.router_aux_loss_coef = (float)a->num;
  return R::Ok(c);
}

size_t MoeConfig::experts_per_token_or(size_t fallback) const {
  size_t k = experts_per_token.value_or(fallback);
  if (k < 1) k = 1;
  if (num_experts && *num_experts > 0 && k > *num_experts) k = *num_experts;
  return k;
}

bool MoeConfig::operator==(const MoeConfig& o) const {
  return num_experts == o.num_experts && experts_per_token == o.experts_per_token &&
         num_shared_experts == o.num_shared_experts && has_shared_experts == o.has_shared_experts &&
         norm_topk_prob == o.norm_topk_prob && router_aux_loss_coef == o.router_aux_loss_coef &&
         expert_intermediate_size == o.expert_intermediate_size &&
         shared_expert_intermediate_size == o.shared_expert_intermediate_size;
}

// ---- qint8 tier files -------------------------------------------------------------------------
QInt8Tensor quantize_per_row_i8(const std::vector<float>& data, size_t rows, size_t cols) {
  QInt8Tensor t;
  t.rows = rows;
  t.cols = cols;
  t.q.resize(rows * cols);
  t.scales.resize(rows);
  if (data.size() == rows * cols && rows * cols > 0)
    atenia_moe_quantize_per_row_i8(data.data(), rows, cols, t.q.data(), t.scales.data());
  return t;
}

std::optional<std::string> write_qint8_tensor_named(const std::string& path,
                                                    const std::vector<float>& data, size_t rows,
                                                    size_t cols) {
  if (data.size() != rows * cols) return "qint8: data length does not match rows * cols";
  const QInt8Tensor t = quantize_per_row_i8(data, rows, cols);
  FILE* f = std::fopen(path.c_str(), "wb");
  if (!f) return "qint8: cannot create '" + path + "'";
  bool ok = true;
  for (size_t r = 0; r < rows && ok; ++r) {  // little-endian f32, whatever the host order
    uint32_t b;
    std::memcpy(&b, &t.scales[r], 4);
    const unsigned char le[4] = {(unsigned char)b, (unsigned char)(b >> 8), (unsigned char)(b >> 16),
                                 (unsigned char)(b >> 24)};
    ok = std::fwrite(le, 1, 4, f) == 4;
  }
  ok = ok && std::fwrite(t.q.data(), 1, t.q.size(), f) == t.q.size();
  ok = (std::fclose(f) == 0) && ok;
  if (!ok) return "qint8: short write to '" + path + "'";
  return std::nullopt;
}

Result<QInt8Tensor, std::string> read_qint8_tensor(const std::string& path, size_t numel,
                                                   size_t rows) {
  typedef Result<QInt8Tensor, std::string> R;
  if (rows == 0 || numel % rows != 0) return R::Err("qint8: bad rows for numel");
  FILE* f = std::fopen(path.c_str(), "rb");
  if (!f) return R::Err("qint8: cannot open '" + path + "'");
  std::fseek(f, 0, SEEK_END);
  const long sz = std::ftell(f);
  std::fseek(f, 0, SEEK_SET);
  const size_t expected = qint8_disk_bytes(numel, rows);
  if (sz < 0 || (size_t)sz != expected) {
    std::fclose(f);
    return R::Err("qint8 file '" + path + "': " + std::to_string(sz < 0 ? 0 : sz) +
                  " bytes, expected " + std::to_string(expected));
  }
  QInt8Tensor t;
  t.rows = rows;
  t.cols = numel / rows;
  t.scales.resize(rows);
  t.q.resize(numel);
  std::vector<unsigned char> raw(rows * 4);
  bool ok = std::fread(raw.data(), 1, raw.size(), f) == raw.size();
  ok = ok && std::fread(t.q.data(), 1, numel, f) == numel;
  std::fclose(f);
  if (!ok) return R::Err("qint8: short read of '" + path + "'");
  for (size_t r = 0; r < rows; ++r) {
    const uint32_t b = (uint32_t)raw[4 * r] | (uint32_t)raw[4 * r + 1] << 8 |
                       (uint32_t)raw[4 * r + 2] << 16 | (uint32_t)raw[4 * r + 3] << 24;
    std::memcpy(&t.scales[r], &b, 4);
  }
  return R::Ok(std::move(t));
}

Result<std::vector<float>, std::string> read_qint8_to_f32(const std::string& path, size_t numel,
                                                          size_t rows) {
  typedef Result<std::vector<float>, std::string> R;
  auto t = read_qint8_tensor(path, numel, rows);
  if (t.is_err()) return R::Err(t.error());
  return R::Ok(t.value().dequantize());
}

// ---- binding ----------------------------------------------------------------------------------
namespace {
typedef Result<std::vector<float>, MoeBindingError> DataResult;

MoeBindingError shape_inconsistency(std::string detail) {
  MoeBindingError e{MoeBindingError::ShapeInconsistency};
  e.detail = std::move(detail);
  return e;
}
MoeBindingError from_dense(const MoeDenseError& d) {
  MoeBindingError e{MoeBindingError::Dense};
  e.dense = d;
  return e;
}

// (rows, cols) of a 2-D entry, or BadRank (src/moe/binding.rs:147-155).
std::optional<MoeBindingError> rows_cols(const MoeTensorEntry& t, size_t* rows, size_t* cols) {
  if (t.shape.size() != 2) {
    MoeBindingError e{MoeBindingError::BadRank};
    e.name = t.name;
    e.rank = t.shape.size();
    return e;
  }
  *rows = t.shape[0];
  *cols = t.shape[1];
  return std::nullopt;
}

// The tensor's data, its length checked against the declared shape (binding.rs:158-178).
DataResult resolve_checked(const MoeTensorEntry& t, const TensorResolver& resolve) {
  std::optional<std::vector<float>> data = resolve(t.name);
  if (!data) {
    MoeBindingError e{MoeBindingError::UnresolvedTensor};
    e.name = t.name;
    return DataResult::Err(e);
  }
  const size_t expected = product(t.shape);
  if (data->size() != expected) {
    MoeBindingError e{MoeBindingError::DataLengthMismatch};
    e.name = t.name;
    e.expected = expected;
    e.actual = data->size();
    return DataResult::Err(e);
  }
  return DataResult::Ok(std::move(*data));
}

// One expert from its three entries (RealExpertTensorBinding::resolve, binding.rs:189-236).
Result<MoeDenseExpert, MoeBindingError> bind_expert(size_t layer_id, size_t expert_id,
                                                    const ExpertTensors& t,
                                                    const TensorResolver& resolve) {
  typedef Result<MoeDenseExpert, MoeBindingError> R;
  if (!t.is_complete()) {
    MoeBindingError e{MoeBindingError::IncompleteExpert};
    e.layer_id = layer_id;
    e.expert_id = expert_id;
    return R::Err(e);
  }
  size_t gate_ff, gate_dm, up_ff, up_dm, down_dm, down_ff;
  if (auto e = rows_cols(*t.gate, &gate_ff, &gate_dm)) return R::Err(*e);
  if (auto e = rows_cols(*t.up, &up_ff, &up_dm)) return R::Err(*e);
  if (auto e = rows_cols(*t.down, &down_dm, &down_ff)) return R::Err(*e);
  if (gate_ff != up_ff || gate_dm != up_dm)
    return R::Err(shape_inconsistency("gate " + fmt_shape(t.gate->shape) + " and up " +
                                      fmt_shape(t.up->shape) + " must share shape"));
  if (down_dm != gate_dm || down_ff != gate_ff)
    return R::Err(shape_inconsistency("down " + fmt_shape(t.down->shape) +
                                      " inconsistent with gate/up (d_model=" + std::to_string(gate_dm) +
                                      ", d_ff=" + std::to_string(gate_ff) + ")"));
  DataResult g = resolve_checked(*t.gate, resolve);
  if (g.is_err()) return R::Err(g.error());
  DataResult u = resolve_checked(*t.up, resolve);
  if (u.is_err()) return R::Err(u.error());
  DataResult d = resolve_checked(*t.down, resolve);
  if (d.is_err()) return R::Err(d.error());
  auto ex = MoeDenseExpert::make(gate_dm, gate_ff, std::move(g.value()), std::move(u.value()),
                                 std::move(d.value()));
  if (ex.is_err()) return R::Err(from_dense(ex.error()));
  return R::Ok(std::move(ex.value()));
}

MoeBindingError at_layer(MoeBindingError::Kind k, size_t layer_id) {
  MoeBindingError e{k};
  e.layer_id = layer_id;
  return e;
}
}  // namespace

Result<MoeDenseLayer, MoeBindingError> build_real_layer(const MoeWeightMap& map, size_t layer_id,
                                                        size_t conceptual_top_k,
                                                        const TensorResolver& resolve) {
  typedef Result<MoeDenseLayer, MoeBindingError> R;
  const MoeLayerMap* layer = map.layer(layer_id);
  if (!layer) return R::Err(at_layer(MoeBindingError::LayerNotFound, layer_id));
  if (layer->experts.empty()) return R::Err(at_layer(MoeBindingError::NoExperts, layer_id));
  std::vector<MoeDenseExpert> experts;
  experts.reserve(layer->experts.size());
  size_t d_model = 0, d_ff = 0;
  for (const auto& kv : layer->experts) {  // ascending expert id = router row order
    auto ex = bind_expert(layer_id, kv.first, kv.second, resolve);
    if (ex.is_err()) return R::Err(ex.error());
    const MoeDenseExpert& b = ex.value();
    if (experts.empty()) {
      d_model = b.d_model;
      d_ff = b.d_ff;
    } else if (b.d_model != d_model || b.d_ff != d_ff) {
      return R::Err(shape_inconsistency(
          "expert " + std::to_string(kv.first) + " shape (d_model=" + std::to_string(b.d_model) +
          ", d_ff=" + std::to_string(b.d_ff) + ") differs from layer (d_model=" +
          std::to_string(d_model) + ", d_ff=" + std::to_string(d_ff) + ")"));
    }
    experts.push_back(std::move(ex.value()));
  }
  if (!layer->router) return R::Err(at_layer(MoeBindingError::MissingRouter, layer_id));
  size_t rows, cols;
  if (auto e = rows_cols(*layer->router, &rows, &cols)) return R::Err(*e);
  if (cols != d_model)
    return R::Err(shape_inconsistency("router cols " + std::to_string(cols) + " != d_model " +
                                      std::to_string(d_model) + " (shape " +
                                      fmt_shape(layer->router->shape) + ")"));
  if (rows != experts.size())
    return R::Err(shape_inconsistency("router rows " + std::to_string(rows) + " != expert count " +
                                      std::to_string(experts.size())));
  DataResult w = resolve_checked(*layer->router, resolve);
  if (w.is_err()) return R::Err(w.error());
  auto l = MoeDenseLayer::make(d_model, d_ff, std::move(w.value()), std::move(experts), conceptual_top_k);
  if (l.is_err()) return R::Err(from_dense(l.error()));
  return R::Ok(std::move(l.value()));
}

Result<PackedExpertDims, MoeBindingError> packed_dims(const MoeTensorEntry& gate_up,
                                                      const MoeTensorEntry& down) {
  typedef Result<PackedExpertDims, MoeBindingError> R;
  for (const MoeTensorEntry* t : {&gate_up, &down})
    if (t->shape.size() != 3) {
      MoeBindingError e{MoeBindingError::PackedBadRank};
      e.name = t->name;
      e.rank = t->shape.size();
      return R::Err(e);
    }
  const size_t ne = gate_up.shape[0], two_dff = gate_up.shape[1], d_model = gate_up.shape[2];
  if (two_dff % 2 != 0)
    return R::Err(shape_inconsistency("gate_up_proj dim1 (" + std::to_string(two_dff) +
                                      ") is not 2*d_ff (must be even); shape " +
                                      fmt_shape(gate_up.shape)));
  const size_t d_ff = two_dff / 2;
  if (down.shape[0] != ne || down.shape[1] != d_model || down.shape[2] != d_ff)
    return R::Err(shape_inconsistency("down_proj " + fmt_shape(down.shape) +
                                      " inconsistent with gate_up_proj " + fmt_shape(gate_up.shape) +
                                      " (expected [" + std::to_string(ne) + ", " +
                                      std::to_string(d_model) + ", " + std::to_string(d_ff) + "])"));
  return R::Ok(PackedExpertDims{ne, d_model, d_ff});
}

Result<MoeDenseLayer, MoeBindingError> build_packed_layer(const MoeWeightMap& map, size_t layer_id,
                                                          size_t conceptual_top_k,
                                                          const TensorResolver& resolve) {
  typedef Result<MoeDenseLayer, MoeBindingError> R;
  const MoeLayerMap* layer = map.layer(layer_id);
  if (!layer) return R::Err(at_layer(MoeBindingError::LayerNotFound, layer_id));
  for (int which = 0; which < 2; ++which)
    if (!(which ? layer->packed_down : layer->packed_gate_up)) {
      MoeBindingError e = at_layer(MoeBindingError::MissingPackedTensor, layer_id);
      e.which = which ? "down_proj" : "gate_up_proj";
      return R::Err(e);
    }
  auto dims = packed_dims(*layer->packed_gate_up, *layer->packed_down);
  if (dims.is_err()) return R::Err(dims.error());
  const size_t ne = dims.value().num_experts, d_model = dims.value().d_model, d_ff = dims.value().d_ff;
  DataResult gu = resolve_checked(*layer->packed_gate_up, resolve);
  if (gu.is_err()) return R::Err(gu.error());
  DataResult dn = resolve_checked(*layer->packed_down, resolve);
  if (dn.is_err()) return R::Err(dn.error());
  // Expert e of the fused tensor: gate = rows [0, d_ff), up = rows [d_ff, 2 d_ff) of its
  // [2 d_ff, d_model] block; down = its [d_model, d_ff] block (binding.rs:371-396).
  const size_t half = d_ff * d_model;
  std::vector<MoeDenseExpert> experts;
  experts.reserve(ne);
  for (size_t e = 0; e < ne; ++e) {
    const float* g = gu.value().data() + e * 2 * half;
    const float* d = dn.value().data() + e * half;
    auto ex = MoeDenseExpert::make(d_model, d_ff, std::vector<float>(g, g + half),
                                   std::vector<float>(g + half, g + 2 * half),
                                   std::vector<float>(d, d + half));
    if (ex.is_err()) return R::Err(from_dense(ex.error()));
    experts.push_back(std::move(ex.value()));
  }
  if (!layer->router) return R::Err(at_layer(MoeBindingError::MissingRouter, layer_id));
  size_t rows, cols;
  if (auto e = rows_cols(*layer->router, &rows, &cols)) return R::Err(*e);
  if (cols != d_model || rows != ne)
    return R::Err(shape_inconsistency("router shape " + fmt_shape(layer->router->shape) +
                                      " != [num_experts=" + std::to_string(ne) +
                                      ", d_model=" + std::to_string(d_model) + "]"));
  DataResult w = resolve_checked(*layer->router, resolve);
  if (w.is_err()) return R::Err(w.error());
  auto l = MoeDenseLayer::make(d_model, d_ff, std::move(w.value()), std::move(experts), conceptual_top_k);
  if (l.is_err()) return R::Err(from_dense(l.error()));
  return R::Ok(std::move(l.value()));
}

namespace {
MoeLayerError layer_err(MoeLayerError::Kind k, size_t layer_id) {
  MoeLayerError e{k};
  e.layer_id = layer_id;
  return e;
}
MoeLayerError from_binding(const MoeBindingError& b) {
  MoeLayerError e{MoeLayerError::Binding};
  e.binding = b;
  return e;
}

// The shared expert: the three projections found by name among the layer's shared tensors;
// other shared tensors (the sigmoid gate) are ignored here (src/moe/layer.rs:235-268).
Result<MoeDenseExpert, MoeLayerError> build_shared_expert(const MoeWeightMap& map, size_t layer_id,
                                                          const TensorResolver& resolve) {
  typedef Result<MoeDenseExpert, MoeLayerError> R;
  const MoeLayerMap* layer = map.layer(layer_id);
  if (!layer || layer->shared.empty())
    return R::Err(layer_err(MoeLayerError::SharedExpertMissing, layer_id));
  auto find = [&](const char* needle) -> const MoeTensorEntry* {
    for (const auto& e : layer->shared)
      if (has(e.name, needle)) return &e;
    return nullptr;
  };
  const MoeTensorEntry *g = find(".gate_proj."), *u = find(".up_proj."), *d = find(".down_proj.");
  if (!g || !u || !d) return R::Err(layer_err(MoeLayerError::SharedExpertIncomplete, layer_id));
  ExpertTensors t;
  t.gate = *g;
  t.up = *u;
  t.down = *d;
  auto ex = bind_expert(layer_id, SIZE_MAX, t, resolve);
  if (ex.is_err()) return R::Err(from_binding(ex.error()));
  return R::Ok(std::move(ex.value()));
}
}  // namespace

Result<RealMoeLayer, MoeLayerError> assemble_real_moe_layer(const MoeWeightMap& map, size_t layer_id,
                                                            MoeLayerConfig config,
                                                            const TensorResolver& resolve,
                                                            MoeWeightStorage storage) {
  typedef Result<RealMoeLayer, MoeLayerError> R;
  if (auto e = config.validate()) {
    MoeLayerError le{MoeLayerError::Config};
    le.config = *e;
    return R::Err(le);
  }
  const MoeLayerMap* meta = map.layer(layer_id);
  if (!meta) return R::Err(from_binding(at_layer(MoeBindingError::LayerNotFound, layer_id)));
  const bool classic = meta->has_classic_experts(), packed = meta->has_packed_experts();
  if (classic && packed) return R::Err(layer_err(MoeLayerError::MixedExpertFormat, layer_id));
  // Classic is taken when present, packed otherwise; neither = the classic NoExperts error.
  auto routed = (!classic && packed)
                    ? build_packed_layer(map, layer_id, config.experts_per_token, resolve)
                    : build_real_layer(map, layer_id, config.experts_per_token, resolve);
  if (routed.is_err()) return R::Err(from_binding(routed.error()));
  // The topology checks come before the shared expert is touched, as in the reference; the
  // in-memory assemble repeats them (cheaply) and adds nothing new for a map-built layer.
  auto mismatch = [](std::string d) {
    MoeLayerError le{MoeLayerError::ConfigMismatch};
    le.detail = std::move(d);
    return le;
  };
  const MoeDenseLayer& r = routed.value();
  if (r.num_experts() != config.num_experts)
    return R::Err(mismatch("resolved " + std::to_string(r.num_experts()) +
                           " experts but config.num_experts = " + std::to_string(config.num_experts)));
  if (r.d_model != config.d_model || r.d_ff != config.d_ff)
    return R::Err(mismatch("resolved (d_model=" + std::to_string(r.d_model) + ", d_ff=" +
                           std::to_string(r.d_ff) + ") but config (d_model=" +
                           std::to_string(config.d_model) + ", d_ff=" + std::to_string(config.d_ff) + ")"));
  std::optional<MoeDenseExpert> shared;
  std::optional<std::vector<float>> shared_gate;
  if (config.has_shared_expert) {
    auto se = build_shared_expert(map, layer_id, resolve);
    if (se.is_err()) return R::Err(se.error());
    if (se.value().d_model != config.d_model)
      return R::Err(mismatch("shared expert d_model=" + std::to_string(se.value().d_model) +
                             " != config d_model=" + std::to_string(config.d_model)));
    shared = std::move(se.value());
    // The sigmoid gate, flat [d_model] (stored as [1, d_model]); absent = Atenia convention.
    for (const auto& e : meta->shared)
      if (has(e.name, "shared_expert_gate")) {
        shared_gate = resolve(e.name);
        break;
      }
  }
  return RealMoeLayer::assemble(config, std::move(routed.value()), std::move(shared),
                                std::move(shared_gate), storage);
}

}  // namespace moe
}  // namespace atenia
