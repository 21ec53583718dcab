// Tests of the weight-ingestion side of the C++ host mirror, written after the reference's own
// tests of the same interface:
//   src/moe/detect.rs tests              (names -> roles, detection, the fail-loud message)
//   tests/moe_data_plane_test.rs         (weight map through a safetensors reader, dense stays empty)
//   tests/moe_real_binding_test.rs       (classic per-expert binding, byte-exact tensors, errors)
//   tests/moe_packed_experts_test.rs     (packed dims, packed == classic, mixed format refused)
//   src/moe/convention.rs tests          (convention from the weight map)
//   src/nn/llama/moe_config.rs tests     (config.json keys of Mixtral / Qwen-MoE / DeepSeek-MoE)
//   tests/moe_deepseek_block_test.rs:42-74  (DeepSeek block: packed experts + fused shared experts)
//   src/tensor/disk_tier.rs tests, tests/moe_qint8_tier_test.rs
//                                        (qint8 tier files: size, round trip, refusal of a wrong size)
//   tests/moe_v3_route_scale_cert_test.rs:56-175, src/moe/v3_router.rs:340-462
//                                        (DeepSeek-V3 routing: configuration errors, HF f64 fixture)
//   tests/moe_numerical_equivalence_test.rs:44-110, tests/moe_hf_convention_test.rs:123-146
//                                        (golden layer files -> assemble -> forward vs the f64 refs)
// The golden layer files are read directly (safetensors + JSON side file).  Without a device the
// assembled weights are run through the CPU oracle, linked here as the checker; with a device the
// forwards go through the mirror to the GPU.
//
// usage: moe_ingest_test <golden_dir> <work_dir> [--no-gpu]
//   work_dir holds dtypes.safetensors + dtypes_expected.bin written by the pytest wrapper and
//   receives the malformed files the reader tests create.
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <map>
#include <string>
#include <vector>

#include "../../ateniaengine_amd/host/json_mini.hpp"
#include "../../ateniaengine_amd/host/moe_ingest.hpp"

using namespace atenia::moe;

extern "C" {
typedef struct {
  int32_t num_experts, top_k, d_model, d_ff, d_ff_shared, convention;
  const float *w_router, *router_bias, *w_gate, *w_up, *w_down, *s_gate, *s_up, *s_down, *shared_gate;
} OraLayer;
int ora_layer_forward_with(const OraLayer* L, const float* x, int convention, int policy, float* out,
                           int32_t* idx_out, float* w_out, int32_t* err_index);
void ora_seeded(uint64_t seed, size_t n, float* out);
}

static int g_failed = 0, g_run = 0;
#define CHECK(cond, ...)                                                   \
  do {                                                                     \
    if (!(cond)) {                                                         \
      printf("    CHECK FAILED %s:%d: %s -- ", __FILE__, __LINE__, #cond); \
      printf(__VA_ARGS__);                                                 \
      printf("\n");                                                        \
      throw std::runtime_error("check failed");                            \
    }                                                                      \
  } while (0)

static void run_test(const char* name, const std::function<void()>& fn) {
  ++g_run;
  try {
    fn();
    printf("ok   %s\n", name);
  } catch (const std::exception& e) {
    ++g_failed;
    printf("FAIL %s: %s\n", name, e.what());
  }
  fflush(stdout);
}

typedef std::vector<std::pair<std::string, std::vector<size_t>>> Listing;
typedef std::map<std::string, std::vector<float>> Store;

static std::vector<float> seeded(uint64_t seed, size_t n) {
  std::vector<float> v(n);
  ora_seeded(seed, n, v.data());
  return v;
}
static TensorResolver resolver_of(const Store& store) {
  return [&store](const std::string& name) -> std::optional<std::vector<float>> {
    auto it = store.find(name);
    if (it == store.end()) return std::nullopt;
    return it->second;
  };
}
static void put(Listing& ls, Store& st, const std::string& name, std::vector<size_t> shape, uint64_t seed) {
  size_t n = 1;
  for (size_t v : shape) n *= v;
  st[name] = seeded(seed, n);
  ls.emplace_back(name, std::move(shape));
}
static double max_abs(const std::vector<float>& v) {
  double m = 0;
  for (float x : v) m = std::max(m, (double)std::fabs(x));
  return m;
}
static double max_abs_diff(const std::vector<float>& a, const std::vector<float>& b) {
  double m = a.size() == b.size() ? 0 : INFINITY;
  for (size_t i = 0; i < a.size() && i < b.size(); ++i) m = std::max(m, std::fabs((double)a[i] - (double)b[i]));
  return m;
}

// A Mixtral-named classic checkpoint: experts listed in the order given (ids need not ascend).
static void mixtral_classic(Listing& ls, Store& st, const std::vector<size_t>& ids, size_t d, size_t f,
                            size_t layer = 0) {
  const std::string p = "model.layers." + std::to_string(layer) + ".block_sparse_moe.";
  put(ls, st, p + "gate.weight", {ids.size(), d}, 1);
  for (size_t e : ids) {
    const std::string q = p + "experts." + std::to_string(e) + ".";
    put(ls, st, q + "w1.weight", {f, d}, 1000 + 10 * e);
    put(ls, st, q + "w3.weight", {f, d}, 1001 + 10 * e);
    put(ls, st, q + "w2.weight", {d, f}, 1002 + 10 * e);
  }
}
// The same experts as mixtral_classic(ids = 0..ne-1), fused the packed way under Qwen-style names.
static void packed_from_classic(const Store& classic, size_t ne, size_t d, size_t f, Listing& ls, Store& st) {
  const std::string p = "model.layers.0.block_sparse_moe.", q = "model.layers.0.mlp.";
  std::vector<float> gu, dn;
  for (size_t e = 0; e < ne; ++e) {
    const std::string x = p + "experts." + std::to_string(e) + ".";
    for (const char* part : {"w1.weight", "w3.weight"}) {
      const auto& v = classic.at(x + part);
      gu.insert(gu.end(), v.begin(), v.end());
    }
    const auto& v = classic.at(x + "w2.weight");
    dn.insert(dn.end(), v.begin(), v.end());
  }
  st[q + "experts.gate_up_proj"] = gu;
  ls.emplace_back(q + "experts.gate_up_proj", std::vector<size_t>{ne, 2 * f, d});
  st[q + "experts.down_proj"] = dn;
  ls.emplace_back(q + "experts.down_proj", std::vector<size_t>{ne, d, f});
  st[q + "gate.weight"] = classic.at(p + "gate.weight");
  ls.emplace_back(q + "gate.weight", std::vector<size_t>{ne, d});
}

static std::string slurp(const std::string& path) {
  std::string s;
  FILE* f = fopen(path.c_str(), "rb");
  if (!f) return s;
  char buf[65536];
  size_t n;
  while ((n = fread(buf, 1, sizeof buf, f)) > 0) s.append(buf, n);
  fclose(f);
  return s;
}
static void spit(const std::string& path, const std::string& bytes) {
  FILE* f = fopen(path.c_str(), "wb");
  if (!f) throw std::runtime_error("cannot write " + path);
  fwrite(bytes.data(), 1, bytes.size(), f);
  fclose(f);
}
static std::string le64(uint64_t v) {
  std::string s(8, '\0');
  for (int i = 0; i < 8; ++i) s[i] = (char)(v >> (8 * i));
  return s;
}

// One golden layer: the file pair read here, nothing converted beforehand.
struct Golden {
  std::string model;
  MoeLayerConfig config;
  RealMoeLayer layer;
  std::vector<float> input, atenia_ref, hf_ref;
};
static std::vector<float> floats(const atenia::json::Value* v) {
  std::vector<float> out;
  if (v)
    for (const auto& x : v->arr) out.push_back((float)x.num);
  return out;
}
static Golden load_golden(const std::string& dir, const std::string& model,
                          MoeWeightStorage storage = MoeWeightStorage::F32) {
  Golden g;
  g.model = model;
  atenia::json::Value side;
  const std::string text = slurp(dir + "/" + model + "_layer0.json");
  CHECK(!text.empty() && atenia::json::parse(text, side), "side file of %s", model.c_str());
  auto num = [&](const char* k) { return (size_t)side.get(k)->num; };
  g.config = MoeLayerConfig::make(num("num_experts"), num("experts_per_token"), side.get("has_shared")->b,
                                  num("d_model"), num("d_ff")).unwrap();
  g.input = floats(side.get("input"));
  g.atenia_ref = floats(side.get("atenia_ref"));
  g.hf_ref = floats(side.get("hf_ref"));
  auto reader = SafetensorsReader::open(dir + "/" + model + "_layer0.safetensors");
  CHECK(reader.is_ok(), "%s", reader.is_err() ? reader.error().c_str() : "");
  const SafetensorsReader& rd = reader.value();
  const MoeWeightMap map = MoeWeightMap::from_tensors(rd.names_and_shapes());
  TensorResolver resolve = [&rd](const std::string& n) { return rd.to_vec_f32(n); };
  g.layer = assemble_real_moe_layer(map, 0, g.config, resolve, storage).unwrap();
  return g;
}
// The assembled layer through the CPU oracle (the checker), under `convention`.
static std::vector<float> oracle_forward(const RealMoeLayer& l, const std::vector<float>& x, int convention) {
  std::vector<float> gate, up, down;
  for (const auto& e : l.routed.experts) {
    gate.insert(gate.end(), e.w_gate.begin(), e.w_gate.end());
    up.insert(up.end(), e.w_up.begin(), e.w_up.end());
    down.insert(down.end(), e.w_down.begin(), e.w_down.end());
  }
  OraLayer L;
  memset(&L, 0, sizeof L);
  L.num_experts = (int32_t)l.num_experts();
  L.top_k = (int32_t)l.config.experts_per_token;
  L.d_model = (int32_t)l.config.d_model;
  L.d_ff = (int32_t)l.config.d_ff;
  L.convention = convention;
  L.w_router = l.routed.w_router.data();
  L.w_gate = gate.data();
  L.w_up = up.data();
  L.w_down = down.data();
  if (l.shared) {
    L.d_ff_shared = (int32_t)l.shared->d_ff;
    L.s_gate = l.shared->w_gate.data();
    L.s_up = l.shared->w_up.data();
    L.s_down = l.shared->w_down.data();
  }
  if (l.shared_gate) L.shared_gate = l.shared_gate->data();
  std::vector<float> out(l.config.d_model), w(l.config.experts_per_token);
  std::vector<int32_t> idx(l.config.experts_per_token);
  int32_t err = -1;
  const int rc = ora_layer_forward_with(&L, x.data(), convention, 0, out.data(), idx.data(), w.data(), &err);
  CHECK(rc == 0, "oracle rc %d", rc);
  return out;
}

int main(int argc, char** argv) {
  if (argc < 3) {
    printf("usage: moe_ingest_test <golden_dir> <work_dir> [--no-gpu]\n");
    return 2;
  }
  const std::string golden = argv[1], work = argv[2];
  const bool no_gpu = argc > 3 && !strcmp(argv[3], "--no-gpu");

  // ---- names ----------------------------------------------------------------------------------
  run_test("classifies_expert_router_and_dense_names", [] {
    struct Case { const char* name; TensorRole role; long layer, expert; };
    const Case cases[] = {
        {"model.layers.3.block_sparse_moe.experts.5.w1.weight", TensorRole::MoeExpertGate, 3, 5},
        {"model.layers.3.block_sparse_moe.experts.5.w3.weight", TensorRole::MoeExpertUp, 3, 5},
        {"model.layers.3.block_sparse_moe.experts.5.w2.weight", TensorRole::MoeExpertDown, 3, 5},
        {"model.layers.11.mlp.experts.59.gate_proj.weight", TensorRole::MoeExpertGate, 11, 59},
        {"model.layers.11.mlp.experts.59.up_proj.weight", TensorRole::MoeExpertUp, 11, 59},
        {"model.layers.11.mlp.experts.59.down_proj.weight", TensorRole::MoeExpertDown, 11, 59},
        {"model.layers.2.mlp.experts.7.act_fn.scale", TensorRole::Unknown, 2, 7},
        {"model.layers.3.block_sparse_moe.gate.weight", TensorRole::MoeRouter, 3, -1},
        {"model.layers.4.mlp.gate.weight", TensorRole::MoeRouter, 4, -1},
        {"model.layers.4.mlp.router.weight", TensorRole::MoeRouter, 4, -1},
        {"model.layers.4.mlp.gate_proj.weight", TensorRole::MlpGate, 4, -1},
        {"model.layers.4.mlp.up_proj.weight", TensorRole::MlpUp, 4, -1},
        {"model.layers.4.mlp.down_proj.weight", TensorRole::MlpDown, 4, -1},
        {"model.layers.9.self_attn.q_proj.weight", TensorRole::AttentionQ, 9, -1},
        {"model.layers.9.self_attn.k_proj.weight", TensorRole::AttentionK, 9, -1},
        {"model.layers.9.self_attn.v_proj.bias", TensorRole::AttentionV, 9, -1},
        {"model.layers.9.self_attn.o_proj.weight", TensorRole::AttentionO, 9, -1},
        {"model.layers.1.mlp.shared_expert.gate_proj.weight", TensorRole::MoeSharedExpert, 1, -1},
        {"model.layers.1.mlp.shared_expert_gate.weight", TensorRole::MoeSharedExpert, 1, -1},
        {"model.layers.1.mlp.shared_experts.down_proj.weight", TensorRole::MoeSharedExpert, 1, -1},
        {"model.layers.0.mlp.experts.gate_up_proj", TensorRole::MoePackedGateUp, 0, -1},
        {"model.layers.0.mlp.experts.down_proj", TensorRole::MoePackedDown, 0, -1},
        {"model.layers.6.input_layernorm.weight", TensorRole::Unknown, 6, -1},
        {"model.embed_tokens.weight", TensorRole::Unknown, -1, -1},
        {"lm_head.weight", TensorRole::Unknown, -1, -1},
    };
    for (const Case& c : cases) {
      const TensorNameInfo i = classify_tensor_name(c.name);
      CHECK(i.role == c.role, "%s: role %d", c.name, (int)i.role);
      CHECK((i.layer_id ? (long)*i.layer_id : -1) == c.layer, "%s: layer", c.name);
      CHECK((i.expert_id ? (long)*i.expert_id : -1) == c.expert, "%s: expert", c.name);
    }
    CHECK(is_moe_router_tensor("model.layers.0.mlp.gate.weight") &&
              !is_moe_router_tensor("model.layers.0.mlp.gate_proj.weight"), "gate_proj is not a router");
    CHECK(is_moe_expert_tensor("model.layers.0.mlp.shared_expert.up_proj.weight") &&
              is_moe_expert_tensor("model.layers.0.block_sparse_moe.experts.0.w1.weight") &&
              !is_moe_expert_tensor("model.layers.0.mlp.gate.weight"), "the router alone is no expert tensor");
    CHECK(role_is_moe(TensorRole::MoeRouter) && !role_is_moe_expert(TensorRole::MoeRouter) &&
              role_is_moe_packed(TensorRole::MoePackedDown) && !role_is_moe(TensorRole::MlpGate), "role sets");
  });
  run_test("detection_counts_and_message", [] {
    std::vector<std::string> dense = {"model.embed_tokens.weight", "model.layers.0.self_attn.q_proj.weight",
                                      "model.layers.0.mlp.gate_proj.weight", "model.layers.0.mlp.up_proj.weight",
                                      "model.layers.0.mlp.down_proj.weight", "model.norm.weight"};
    MoeDetection d0 = detect_moe(dense);
    CHECK(!d0.is_moe && d0.expert_tensor_count == 0 && !d0.implied_expert_count(), "dense names must not trigger");
    std::vector<std::string> moe = dense;
    moe.push_back("model.layers.0.mlp.gate.weight");
    for (int e = 0; e < 8; ++e)
      for (const char* p : {"gate_proj", "up_proj", "down_proj"})
        moe.push_back("model.layers.0.mlp.experts." + std::to_string(e) + "." + p + ".weight");
    moe.push_back("model.layers.0.mlp.shared_expert.gate_proj.weight");
    moe.push_back("model.layers.0.mlp.shared_expert_gate.weight");
    MoeDetection d1 = detect_moe(moe);
    CHECK(d1.is_moe && d1.expert_tensor_count == 24 && d1.router_tensor_count == 1 &&
              d1.shared_expert_tensor_count == 2, "counts %zu %zu %zu", d1.expert_tensor_count,
          d1.router_tensor_count, d1.shared_expert_tensor_count);
    CHECK(d1.implied_expert_count() && *d1.implied_expert_count() == 8, "max id + 1");
    const std::string msg = unsupported_message(d1);
    CHECK(msg.find("experts=8, expert_tensors=24, router_tensors=1, shared_expert_tensors=2") != std::string::npos,
          "%s", msg.c_str());
    // the phrases the reference's own tests look for (src/moe/detect.rs:425-428,
    // tests/moe_loader_failloud_test.rs:47)
    CHECK(msg.find("MoE checkpoint detected") != std::string::npos &&
              msg.find("not implemented yet") != std::string::npos, "%s", msg.c_str());
    // A router alone does not make a checkpoint MoE; one shared-expert tensor does.
    CHECK(!detect_moe({"model.layers.0.mlp.gate.weight"}).is_moe, "router only");
    MoeDetection d2 = detect_moe({"model.layers.0.mlp.shared_expert.up_proj.weight"});
    CHECK(d2.is_moe && unsupported_message(d2).find("experts=unknown") != std::string::npos, "shared only");
    CHECK(detect_moe({"model.layers.0.mlp.experts.gate_up_proj", "model.layers.0.mlp.experts.down_proj"})
                  .expert_tensor_count == 2, "packed tensors count as expert tensors");
  });

  // ---- weight map -----------------------------------------------------------------------------
  run_test("weight_map_groups_by_layer_and_expert", [] {
    Listing ls;
    Store st;
    mixtral_classic(ls, st, {1, 0}, 4, 8, 0);
    mixtral_classic(ls, st, {0, 2, 10}, 4, 8, 5);
    ls.emplace_back("model.layers.5.self_attn.q_proj.weight", std::vector<size_t>{4, 4});
    ls.emplace_back("block_sparse_moe.experts.3.w1.weight", std::vector<size_t>{8, 4});  // no layer id: skipped
    MoeWeightMap map = MoeWeightMap::from_tensors(ls);
    CHECK(!map.is_empty() && map.layers.size() == 2, "layers %zu", map.layers.size());
    CHECK(map.num_experts(0) == 2 && map.num_experts(5) == 3 && map.num_experts(1) == 0, "expert counts");
    const ExpertTensors* e1 = map.expert(0, 1);
    CHECK(e1 && e1->is_complete(), "expert (0,1)");
    CHECK((e1->gate->shape == std::vector<size_t>{8, 4}) && (e1->down->shape == std::vector<size_t>{4, 8}), "shapes");
    CHECK(e1->up->role == TensorRole::MoeExpertUp && *e1->up->expert_id == 1 && *e1->up->layer_id == 0, "entry ids");
    CHECK(map.router_weight(0) && map.router_weight(5) && !map.router_weight(1), "router lookup");
    CHECK(!map.expert(0, 2) && !map.expert(3, 0) && !map.layer(3), "absent lookups");
    CHECK(map.total_expert_tensors() == 15 && map.all_experts_complete(), "totals");
    std::vector<size_t> order;
    for (const auto& kv : map.layer(5)->experts) order.push_back(kv.first);
    CHECK((order == std::vector<size_t>{0, 2, 10}), "experts iterate in ascending numeric id");
    ls.pop_back();
    ls.pop_back();
    ls.emplace_back("model.layers.7.block_sparse_moe.experts.0.w1.weight", std::vector<size_t>{8, 4});
    MoeWeightMap partial = MoeWeightMap::from_tensors(ls);
    CHECK(!partial.all_experts_complete() && partial.total_expert_tensors() == 16, "an expert with one projection");
    Listing dense = {{"model.layers.0.mlp.gate_proj.weight", {8, 4}}, {"model.layers.0.self_attn.q_proj.weight", {4, 4}}};
    CHECK(MoeWeightMap::from_tensors(dense).is_empty(), "a dense checkpoint gives no map");
  });
  run_test("convention_from_weight_map", [] {
    Listing qwen = {{"model.layers.0.mlp.gate.weight", {4, 8}},
                    {"model.layers.0.mlp.experts.0.gate_proj.weight", {16, 8}},
                    {"model.layers.0.mlp.shared_expert.gate_proj.weight", {16, 8}},
                    {"model.layers.0.mlp.shared_expert_gate.weight", {1, 8}}};
    CHECK(MoeConventionResolver::from_weight_map(MoeWeightMap::from_tensors(qwen)) ==
              MoeExecutionConvention::HuggingFaceQwen, "a shared-expert gate anywhere = HuggingFaceQwen");
    qwen.pop_back();
    CHECK(MoeConventionResolver::from_weight_map(MoeWeightMap::from_tensors(qwen)) == MoeExecutionConvention::Atenia,
          "shared expert without gate = Atenia");
    Listing ls;
    Store st;
    mixtral_classic(ls, st, {0, 1}, 4, 8);
    CHECK(MoeConventionResolver::from_weight_map(MoeWeightMap::from_tensors(ls)) == MoeExecutionConvention::Atenia,
          "mixtral = Atenia");
    CHECK(MoeConventionResolver::from_shared_gate_present(true) == MoeExecutionConvention::HuggingFaceQwen &&
              MoeConventionResolver::from_shared_gate_present(false) == MoeExecutionConvention::Atenia, "helper");
  });

  run_test("config_json_keys_of_the_families", [] {
    auto mixtral = MoeConfig::from_json_str(
        "{\"model_type\": \"mixtral\", \"hidden_size\": 4096, \"intermediate_size\": 14336, "
        "\"num_local_experts\": 8, \"num_experts_per_tok\": 2, \"router_aux_loss_coef\": 0.02}").unwrap();
    CHECK(mixtral.is_moe() && *mixtral.num_experts == 8 && *mixtral.experts_per_token == 2 &&
              !mixtral.has_shared_experts && !mixtral.norm_topk_prob && !mixtral.expert_intermediate_size, "mixtral");
    CHECK(mixtral.router_aux_loss_coef && *mixtral.router_aux_loss_coef == 0.02f && mixtral.renormalize_topk_or(true), "mixtral extras");
    auto qwen2 = MoeConfig::from_json_str(
        "{\"num_experts\": 60, \"num_experts_per_tok\": 4, \"moe_intermediate_size\": 1408, "
        "\"shared_expert_intermediate_size\": 5632, \"norm_topk_prob\": false}").unwrap();
    CHECK(*qwen2.num_experts == 60 && *qwen2.experts_per_token == 4 && qwen2.has_shared_experts &&
              *qwen2.shared_expert_intermediate_size == 5632 && *qwen2.expert_intermediate_size == 1408 &&
              qwen2.norm_topk_prob && !*qwen2.norm_topk_prob && !qwen2.renormalize_topk_or(true), "qwen2-moe");
    auto qwen3 = MoeConfig::from_json_str(
        "{\"num_experts\": 128, \"num_experts_per_tok\": 8, \"moe_intermediate_size\": 768, \"norm_topk_prob\": true}").unwrap();
    CHECK(*qwen3.num_experts == 128 && !qwen3.has_shared_experts && *qwen3.norm_topk_prob, "qwen3-moe");
    auto deepseek = MoeConfig::from_json_str(
        "{\"n_routed_experts\": 64, \"num_experts_per_tok\": 6, \"n_shared_experts\": 2, "
        "\"moe_intermediate_size\": 1408, \"norm_topk_prob\": false}").unwrap();
    CHECK(*deepseek.num_experts == 64 && *deepseek.num_shared_experts == 2 && deepseek.has_shared_experts, "deepseek");
    CHECK(MoeConventionResolver::from_norm_topk_prob(deepseek.norm_topk_prob) == MoeExecutionConvention::HuggingFaceQwen &&
              MoeConventionResolver::from_norm_topk_prob(std::nullopt) == MoeExecutionConvention::Atenia &&
              MoeConventionResolver::from_norm_topk_prob(true) == MoeExecutionConvention::Atenia, "DeepSeek convention");
    // aliases and precedence
    CHECK(*MoeConfig::from_json_str("{\"num_experts_per_token\": 3}").unwrap().experts_per_token == 3, "top-k alias");
    CHECK(*MoeConfig::from_json_str("{\"expert_intermediate_size\": 11}").unwrap().expert_intermediate_size == 11, "width alias");
    CHECK(*MoeConfig::from_json_str("{\"n_routed_experts\": 64, \"num_local_experts\": 8}").unwrap().num_experts == 8,
          "num_local_experts is looked up before n_routed_experts");
    CHECK(!MoeConfig::from_json_str("{\"n_shared_experts\": 0, \"num_experts\": 4}").unwrap().has_shared_experts,
          "a zero shared count is no shared expert");
    // dense and odd inputs
    auto dense = MoeConfig::from_json_str("{\"model_type\": \"qwen2\", \"hidden_size\": 896, \"intermediate_size\": 4864}").unwrap();
    CHECK(!dense.is_moe() && dense == MoeConfig() && dense.experts_per_token_or(2) == 2, "dense config");
    CHECK(MoeConfig::from_json_str("{}").unwrap() == MoeConfig(), "empty object");
    auto odd = MoeConfig::from_json_str("{\"num_experts\": -4, \"num_experts_per_tok\": 2.5, \"norm_topk_prob\": 1}").unwrap();
    CHECK(odd == MoeConfig(), "negative, fractional and mistyped values are not taken");
    CHECK(MoeConfig::from_json_str("{ not json").is_err() && MoeConfig::from_json_str("").is_err(), "invalid JSON");
    // clamping of top-k
    auto small = MoeConfig::from_json_str("{\"num_experts\": 4, \"num_experts_per_tok\": 9}").unwrap();
    CHECK(small.experts_per_token_or(2) == 4, "top-k is clamped to the expert count");
    auto zero = MoeConfig::from_json_str("{\"num_experts\": 4, \"num_experts_per_tok\": 0}").unwrap();
    CHECK(zero.experts_per_token_or(2) == 1, "top-k is at least one");
  });

  run_test("v3_router_config_errors", [] {
    auto cfg = [](size_t n, size_t k, size_t g, size_t tg) {
      V3RouterConfig c;
      c.n_routed_experts = n; c.top_k = k; c.n_group = g; c.topk_group = tg;
      return c;
    };
    CHECK(!cfg(8, 2, 4, 2).validate(), "a valid configuration");
    auto text = [](const std::optional<V3RouterError>& e) { return e ? e->to_string() : std::string("ok"); };
    CHECK(text(cfg(7, 2, 4, 2).validate()) == "v3-router: n_routed_experts (7) not divisible by n_group (4)", "divisible");
    CHECK(text(cfg(4, 1, 4, 2).validate()) == "v3-router: experts_per_group (1) < 2 (HF takes top-2 per group)", "group size");
    CHECK(text(cfg(8, 2, 4, 5).validate()) == "v3-router: topk_group (5) > n_group (4)", "topk_group");
    CHECK(text(cfg(8, 5, 4, 2).validate()) == "v3-router: top_k (5) exceeds experts in selected groups (4)", "selectable");
    CHECK(text(cfg(8, 0, 4, 2).validate()) == "v3-router: top_k must be > 0", "zero top_k");
    CHECK(text(cfg(8, 2, 0, 2).validate()) == "v3-router: n_group must be > 0", "zero n_group");
    CHECK(text(cfg(8, 2, 4, 0).validate()) == "v3-router: topk_group must be > 0", "zero topk_group");
    CHECK(parse_scoring_func("sigmoid").is_ok(), "sigmoid");
    auto sm = parse_scoring_func("softmax");
    CHECK(sm.is_err() && sm.error().to_string() == "v3-router: unsupported scoring_func 'softmax' (only 'sigmoid')", "softmax refused");
    // on a layer: lengths, finiteness, and the layer's own top_k
    Listing ls;
    Store st;
    mixtral_classic(ls, st, {0, 1, 2, 3, 4, 5, 6, 7}, 8, 12);
    auto layer = assemble_real_moe_layer(MoeWeightMap::from_tensors(ls), 0, MoeLayerConfig::make(8, 2, false, 8, 12).unwrap(),
                                         resolver_of(st)).unwrap();
    CHECK(text(layer.set_v3_router(cfg(8, 2, 4, 2), std::vector<float>(7, 0.f))) ==
              "v3-router: e_score_correction_bias length 7 != n_routed_experts 8", "bias length");
    std::vector<float> bad(8, 0.f);
    bad[5] = INFINITY;
    CHECK(text(layer.set_v3_router(cfg(8, 2, 4, 2), bad)) == "v3-router: e_score_correction_bias at 5 is non-finite", "bias finite");
    CHECK(text(layer.set_v3_router(cfg(16, 2, 4, 2), std::vector<float>(16, 0.f))) ==
              "v3-router: router_logits length 8 != n_routed_experts 16", "expert count");
    CHECK(text(layer.set_v3_router(cfg(8, 3, 4, 2), std::vector<float>(8, 0.f))) ==
              "v3-router: top_k (3) differs from the layer's experts_per_token (2)", "top_k of the layer");
    CHECK(!layer.v3_router, "failed calls leave the layer as it was");
    CHECK(!layer.set_v3_router(cfg(8, 2, 4, 2), std::vector<float>(8, 0.f)) && layer.v3_router, "accepted");
  });

  // ---- classic binding ------------------------------------------------------------------------
  run_test("classic_binding_is_byte_exact_and_id_ordered", [] {
    Listing ls;
    Store st;
    mixtral_classic(ls, st, {10, 2, 1}, 8, 16);
    MoeWeightMap map = MoeWeightMap::from_tensors(ls);
    auto layer = build_real_layer(map, 0, 2, resolver_of(st)).unwrap();
    CHECK(layer.num_experts() == 3 && layer.d_model == 8 && layer.d_ff == 16 && layer.conceptual_top_k == 2, "dims");
    const size_t ids[3] = {1, 2, 10};
    for (int i = 0; i < 3; ++i) {
      const std::string q = "model.layers.0.block_sparse_moe.experts." + std::to_string(ids[i]) + ".";
      CHECK(layer.experts[i].w_gate == st.at(q + "w1.weight") && layer.experts[i].w_up == st.at(q + "w3.weight") &&
                layer.experts[i].w_down == st.at(q + "w2.weight"), "expert slot %d must hold id %zu", i, ids[i]);
    }
    CHECK(layer.w_router == st.at("model.layers.0.block_sparse_moe.gate.weight"), "router");
  });
  run_test("classic_binding_errors", [] {
    Listing ls;
    Store st;
    mixtral_classic(ls, st, {0, 1}, 8, 16);
    const auto with = [&](const std::function<void(Listing&, Store&)>& edit) {
      Listing l2 = ls;
      Store s2 = st;
      edit(l2, s2);
      return build_real_layer(MoeWeightMap::from_tensors(l2), 0, 2, resolver_of(s2));
    };
    auto drop = [](Listing& l, const std::string& name) {
      for (size_t i = 0; i < l.size(); ++i)
        if (l[i].first == name) { l.erase(l.begin() + i); return; }
    };
    auto reshape = [](Listing& l, const std::string& name, std::vector<size_t> s) {
      for (auto& e : l)
        if (e.first == name) e.second = s;
    };
    const std::string p = "model.layers.0.block_sparse_moe.";
    auto r = build_real_layer(MoeWeightMap::from_tensors(ls), 4, 2, resolver_of(st));
    CHECK(r.is_err() && r.error().kind == MoeBindingError::LayerNotFound && r.error().layer_id == 4 &&
              r.error().to_string() == "moe-binding: layer 4 has no MoE weights", "LayerNotFound");
    Listing only_router = {{p + "gate.weight", {2, 8}}};
    r = build_real_layer(MoeWeightMap::from_tensors(only_router), 0, 2, resolver_of(st));
    CHECK(r.is_err() && r.error().kind == MoeBindingError::NoExperts &&
              r.error().to_string() == "moe-binding: layer 0 has no experts", "NoExperts");
    r = with([&](Listing& l, Store&) { drop(l, p + "experts.1.w3.weight"); });
    CHECK(r.is_err() && r.error().kind == MoeBindingError::IncompleteExpert && r.error().expert_id == 1 &&
              r.error().to_string() == "moe-binding: layer 0 expert 1 is missing a gate/up/down projection",
          "IncompleteExpert");
    r = with([&](Listing& l, Store&) { drop(l, p + "gate.weight"); });
    CHECK(r.is_err() && r.error().kind == MoeBindingError::MissingRouter &&
              r.error().to_string() == "moe-binding: layer 0 has no router tensor", "MissingRouter");
    r = with([&](Listing&, Store& s) { s.erase(p + "experts.0.w2.weight"); });
    CHECK(r.is_err() && r.error().kind == MoeBindingError::UnresolvedTensor &&
              r.error().to_string() == "moe-binding: byte resolver returned no data for '" + p + "experts.0.w2.weight'",
          "UnresolvedTensor");
    r = with([&](Listing& l, Store&) { reshape(l, p + "experts.0.w1.weight", {16, 4, 2}); });
    CHECK(r.is_err() && r.error().kind == MoeBindingError::BadRank && r.error().rank == 3 &&
              r.error().to_string() == "moe-binding: tensor '" + p + "experts.0.w1.weight' has rank 3, expected 2-D [rows, cols]",
          "BadRank");
    r = with([&](Listing& l, Store&) { reshape(l, p + "experts.0.w3.weight", {8, 16}); });
    CHECK(r.is_err() && r.error().kind == MoeBindingError::ShapeInconsistency &&
              r.error().to_string() == "moe-binding: shape inconsistency: gate [16, 8] and up [8, 16] must share shape",
          "%s", r.is_err() ? r.error().to_string().c_str() : "ok");
    r = with([&](Listing& l, Store&) { reshape(l, p + "experts.0.w2.weight", {16, 8}); });
    CHECK(r.is_err() && r.error().to_string() ==
                            "moe-binding: shape inconsistency: down [16, 8] inconsistent with gate/up (d_model=8, d_ff=16)",
          "%s", r.is_err() ? r.error().to_string().c_str() : "ok");
    r = with([&](Listing& l, Store& s) {
      for (const char* part : {"w1.weight", "w3.weight"}) {
        reshape(l, p + "experts.1." + part, {4, 8});
        s[p + "experts.1." + part].resize(32);
      }
      reshape(l, p + "experts.1.w2.weight", {8, 4});
      s[p + "experts.1.w2.weight"].resize(32);
    });
    CHECK(r.is_err() && r.error().to_string() ==
                            "moe-binding: shape inconsistency: expert 1 shape (d_model=8, d_ff=4) differs from layer "
                            "(d_model=8, d_ff=16)",
          "%s", r.is_err() ? r.error().to_string().c_str() : "ok");
    r = with([&](Listing& l, Store&) { reshape(l, p + "gate.weight", {2, 4}); });
    CHECK(r.is_err() && r.error().to_string() ==
                            "moe-binding: shape inconsistency: router cols 4 != d_model 8 (shape [2, 4])",
          "%s", r.is_err() ? r.error().to_string().c_str() : "ok");
    r = with([&](Listing& l, Store&) { reshape(l, p + "gate.weight", {3, 8}); });
    CHECK(r.is_err() && r.error().to_string() == "moe-binding: shape inconsistency: router rows 3 != expert count 2",
          "%s", r.is_err() ? r.error().to_string().c_str() : "ok");
    r = with([&](Listing&, Store& s) { s[p + "experts.1.w1.weight"].pop_back(); });
    CHECK(r.is_err() && r.error().kind == MoeBindingError::DataLengthMismatch && r.error().expected == 128 &&
              r.error().actual == 127 &&
              r.error().to_string() == "moe-binding: tensor '" + p + "experts.1.w1.weight' data length 127 != shape product 128",
          "DataLengthMismatch");
  });

  // ---- packed binding -------------------------------------------------------------------------
  run_test("packed_dims_and_errors", [] {
    MoeTensorEntry gu{"model.layers.0.mlp.experts.gate_up_proj", 0, std::nullopt, TensorRole::MoePackedGateUp, {6, 24, 8}};
    MoeTensorEntry dn{"model.layers.0.mlp.experts.down_proj", 0, std::nullopt, TensorRole::MoePackedDown, {6, 8, 12}};
    auto d = packed_dims(gu, dn).unwrap();
    CHECK(d.num_experts == 6 && d.d_model == 8 && d.d_ff == 12, "dims");
    MoeTensorEntry bad = gu;
    bad.shape = {6, 24};
    auto r = packed_dims(bad, dn);
    CHECK(r.is_err() && r.error().kind == MoeBindingError::PackedBadRank &&
              r.error().to_string() == "moe-binding: packed tensor 'model.layers.0.mlp.experts.gate_up_proj' has rank 2, expected 3-D",
          "PackedBadRank");
    bad.shape = {6, 25, 8};
    r = packed_dims(bad, dn);
    CHECK(r.is_err() && r.error().to_string() ==
                            "moe-binding: shape inconsistency: gate_up_proj dim1 (25) is not 2*d_ff (must be even); shape [6, 25, 8]",
          "%s", r.is_err() ? r.error().to_string().c_str() : "ok");
    MoeTensorEntry bad_dn = dn;
    bad_dn.shape = {6, 12, 8};  // transposed
    r = packed_dims(gu, bad_dn);
    CHECK(r.is_err() && r.error().to_string() ==
                            "moe-binding: shape inconsistency: down_proj [6, 12, 8] inconsistent with gate_up_proj "
                            "[6, 24, 8] (expected [6, 8, 12])",
          "%s", r.is_err() ? r.error().to_string().c_str() : "ok");
  });
  run_test("packed_binding_equals_classic", [] {
    const size_t ne = 5, d = 8, f = 12;
    Listing cl, pl;
    Store cs, ps;
    mixtral_classic(cl, cs, {0, 1, 2, 3, 4}, d, f);
    packed_from_classic(cs, ne, d, f, pl, ps);
    MoeWeightMap pm = MoeWeightMap::from_tensors(pl);
    CHECK(pm.layer(0)->has_packed_experts() && !pm.layer(0)->has_classic_experts(), "format flags");
    auto classic = build_real_layer(MoeWeightMap::from_tensors(cl), 0, 2, resolver_of(cs)).unwrap();
    auto packed = build_packed_layer(pm, 0, 2, resolver_of(ps)).unwrap();
    CHECK(packed.num_experts() == ne && packed.d_model == d && packed.d_ff == f, "dims");
    for (size_t e = 0; e < ne; ++e)
      CHECK(packed.experts[e].w_gate == classic.experts[e].w_gate && packed.experts[e].w_up == classic.experts[e].w_up &&
                packed.experts[e].w_down == classic.experts[e].w_down, "expert %zu: gate is the first half of the fused rows", e);
    CHECK(packed.w_router == classic.w_router, "router");
    // errors of the packed path
    Listing no_down = pl;
    no_down.erase(no_down.begin() + 1);
    auto r = build_packed_layer(MoeWeightMap::from_tensors(no_down), 0, 2, resolver_of(ps));
    CHECK(r.is_err() && r.error().kind == MoeBindingError::MissingPackedTensor &&
              r.error().to_string() == "moe-binding: layer 0 missing packed expert tensor 'down_proj'", "MissingPackedTensor");
    Listing no_router = pl;
    no_router.pop_back();
    r = build_packed_layer(MoeWeightMap::from_tensors(no_router), 0, 2, resolver_of(ps));
    CHECK(r.is_err() && r.error().kind == MoeBindingError::MissingRouter, "MissingRouter");
    Listing bad_router = pl;
    bad_router.back().second = {ne + 1, d};
    r = build_packed_layer(MoeWeightMap::from_tensors(bad_router), 0, 2, resolver_of(ps));
    CHECK(r.is_err() && r.error().to_string() ==
                            "moe-binding: shape inconsistency: router shape [6, 8] != [num_experts=5, d_model=8]",
          "%s", r.is_err() ? r.error().to_string().c_str() : "ok");
    Store short_store = ps;
    short_store["model.layers.0.mlp.experts.gate_up_proj"].resize(10);
    r = build_packed_layer(pm, 0, 2, resolver_of(short_store));
    CHECK(r.is_err() && r.error().kind == MoeBindingError::DataLengthMismatch, "short fused tensor");
  });

  // ---- assemble from a map --------------------------------------------------------------------
  run_test("assemble_selects_format_and_cross_checks", [] {
    const size_t ne = 4, d = 8, f = 12, fs = 6;
    Listing cl, pl;
    Store cs, ps;
    mixtral_classic(cl, cs, {0, 1, 2, 3}, d, f);
    packed_from_classic(cs, ne, d, f, pl, ps);
    auto cfg = MoeLayerConfig::make(ne, 2, false, d, f).unwrap();
    auto a = assemble_real_moe_layer(MoeWeightMap::from_tensors(cl), 0, cfg, resolver_of(cs)).unwrap();
    auto b = assemble_real_moe_layer(MoeWeightMap::from_tensors(pl), 0, cfg, resolver_of(ps)).unwrap();
    CHECK(a.num_experts() == ne && b.num_experts() == ne && !a.has_shared_expert() && !b.shared_gate, "both formats");
    CHECK(a.routed.experts[3].w_up == b.routed.experts[3].w_up, "same experts either way");
    CHECK(a.resolve_convention() == MoeExecutionConvention::Atenia, "convention");
    // both formats under one layer prefix: refused
    Listing mixed;
    Store ms;
    const std::string q = "model.layers.0.mlp.";
    put(mixed, ms, q + "gate.weight", {ne, d}, 1);
    for (size_t e = 0; e < ne; ++e) {
      put(mixed, ms, q + "experts." + std::to_string(e) + ".gate_proj.weight", {f, d}, 10 + e);
      put(mixed, ms, q + "experts." + std::to_string(e) + ".up_proj.weight", {f, d}, 20 + e);
      put(mixed, ms, q + "experts." + std::to_string(e) + ".down_proj.weight", {d, f}, 30 + e);
    }
    put(mixed, ms, q + "experts.gate_up_proj", {ne, 2 * f, d}, 40);
    put(mixed, ms, q + "experts.down_proj", {ne, d, f}, 41);
    auto r = assemble_real_moe_layer(MoeWeightMap::from_tensors(mixed), 0, cfg, resolver_of(ms));
    CHECK(r.is_err() && r.error().kind == MoeLayerError::MixedExpertFormat &&
              r.error().to_string() == "moe-layer: layer 0 has both classic and packed expert tensors", "MixedExpertFormat");
    // config cross-checks
    r = assemble_real_moe_layer(MoeWeightMap::from_tensors(cl), 0, MoeLayerConfig::make(ne + 1, 2, false, d, f).unwrap(),
                                resolver_of(cs));
    CHECK(r.is_err() && r.error().kind == MoeLayerError::ConfigMismatch &&
              r.error().to_string() == "moe-layer: config mismatch: resolved 4 experts but config.num_experts = 5",
          "%s", r.is_err() ? r.error().to_string().c_str() : "ok");
    r = assemble_real_moe_layer(MoeWeightMap::from_tensors(cl), 0, MoeLayerConfig::make(ne, 2, false, d, f + 1).unwrap(),
                                resolver_of(cs));
    CHECK(r.is_err() && r.error().to_string() ==
                            "moe-layer: config mismatch: resolved (d_model=8, d_ff=12) but config (d_model=8, d_ff=13)",
          "%s", r.is_err() ? r.error().to_string().c_str() : "ok");
    MoeLayerConfig zero = cfg;
    zero.experts_per_token = 0;
    r = assemble_real_moe_layer(MoeWeightMap::from_tensors(cl), 0, zero, resolver_of(cs));
    CHECK(r.is_err() && r.error().kind == MoeLayerError::Config, "config is validated first");
    r = assemble_real_moe_layer(MoeWeightMap::from_tensors(cl), 3, cfg, resolver_of(cs));
    CHECK(r.is_err() && r.error().kind == MoeLayerError::Binding &&
              r.error().binding.kind == MoeBindingError::LayerNotFound &&
              r.error().to_string() == "moe-layer: moe-binding: layer 3 has no MoE weights", "LayerNotFound");
    Listing router_only = {{"model.layers.0.mlp.gate.weight", {ne, d}}};
    r = assemble_real_moe_layer(MoeWeightMap::from_tensors(router_only), 0, cfg, resolver_of(cs));
    CHECK(r.is_err() && r.error().binding.kind == MoeBindingError::NoExperts, "neither format = classic NoExperts");
    // shared expert: asked for but absent / incomplete / present (+ gate)
    auto shared_cfg = MoeLayerConfig::make(ne, 2, true, d, f).unwrap();
    r = assemble_real_moe_layer(MoeWeightMap::from_tensors(pl), 0, shared_cfg, resolver_of(ps));
    CHECK(r.is_err() && r.error().kind == MoeLayerError::SharedExpertMissing &&
              r.error().to_string() == "moe-layer: layer 0 has no shared-expert tensors", "SharedExpertMissing");
    Listing sl = pl;
    Store ss = ps;
    put(sl, ss, q + "shared_expert.gate_proj.weight", {fs, d}, 50);
    put(sl, ss, q + "shared_expert.up_proj.weight", {fs, d}, 51);
    r = assemble_real_moe_layer(MoeWeightMap::from_tensors(sl), 0, shared_cfg, resolver_of(ss));
    CHECK(r.is_err() && r.error().kind == MoeLayerError::SharedExpertIncomplete &&
              r.error().to_string() == "moe-layer: layer 0 shared expert is missing gate/up/down", "SharedExpertIncomplete");
    put(sl, ss, q + "shared_expert.down_proj.weight", {d, fs}, 52);
    auto s1 = assemble_real_moe_layer(MoeWeightMap::from_tensors(sl), 0, shared_cfg, resolver_of(ss)).unwrap();
    CHECK(s1.has_shared_expert() && s1.shared->d_ff == fs && !s1.shared_gate &&
              s1.resolve_convention() == MoeExecutionConvention::Atenia, "shared expert of its own width, no gate");
    CHECK(s1.shared->w_down == ss.at(q + "shared_expert.down_proj.weight"), "shared down bytes");
    put(sl, ss, q + "shared_expert_gate.weight", {1, d}, 53);
    auto s2 = assemble_real_moe_layer(MoeWeightMap::from_tensors(sl), 0, shared_cfg, resolver_of(ss)).unwrap();
    CHECK(s2.shared_gate && s2.shared_gate->size() == d && *s2.shared_gate == ss.at(q + "shared_expert_gate.weight") &&
              s2.resolve_convention() == MoeExecutionConvention::HuggingFaceQwen, "gate flat [d_model]");
    auto s3 = assemble_real_moe_layer(MoeWeightMap::from_tensors(sl), 0, cfg, resolver_of(ss)).unwrap();
    CHECK(!s3.has_shared_expert() && !s3.shared_gate, "a config without shared expert ignores the shared tensors");
    // shared expert of another model width
    Listing wl = pl;
    Store ws = ps;
    put(wl, ws, q + "shared_expert.gate_proj.weight", {fs, d + 2}, 60);
    put(wl, ws, q + "shared_expert.up_proj.weight", {fs, d + 2}, 61);
    put(wl, ws, q + "shared_expert.down_proj.weight", {d + 2, fs}, 62);
    r = assemble_real_moe_layer(MoeWeightMap::from_tensors(wl), 0, shared_cfg, resolver_of(ws));
    CHECK(r.is_err() && r.error().to_string() == "moe-layer: config mismatch: shared expert d_model=10 != config d_model=8",
          "%s", r.is_err() ? r.error().to_string().c_str() : "ok");
  });

  // ---- safetensors reader ---------------------------------------------------------------------
  run_test("reader_widens_f32_bf16_f16", [&] {
    auto rd = SafetensorsReader::open(work + "/dtypes.safetensors");
    CHECK(rd.is_ok(), "%s", rd.is_err() ? rd.error().c_str() : "");
    const std::string raw = slurp(work + "/dtypes_expected.bin");
    std::vector<float> want(raw.size() / 4);
    memcpy(want.data(), raw.data(), want.size() * 4);
    CHECK(want.size() == 24, "expected file");
    for (const char* name : {"t.f32", "t.bf16", "t.f16"}) {
      const SafetensorsEntry* e = rd.value().get(name);
      CHECK(e && (e->shape == std::vector<size_t>{4, 6}) && e->numel() == 24, "%s entry", name);
      auto v = rd.value().to_vec_f32(name);
      CHECK(v && v->size() == want.size(), "%s data", name);
      CHECK(memcmp(v->data(), want.data(), want.size() * 4) == 0, "%s must widen to the same bits", name);
    }
    CHECK(!rd.value().to_vec_f32("t.i64") && rd.value().get("t.i64"), "unsupported dtype: listed, not convertible");
    CHECK(!rd.value().get("absent") && !rd.value().to_vec_f32("absent"), "unknown name");
    CHECK(rd.value().entries().size() == 4 && rd.value().names_and_shapes().size() == 4, "metadata entry is skipped");
  });
  run_test("reader_rejects_malformed_files", [&] {
    CHECK(SafetensorsReader::open(work + "/does_not_exist.safetensors").is_err(), "missing file");
    spit(work + "/short.safetensors", "abc");
    CHECK(SafetensorsReader::open(work + "/short.safetensors").is_err(), "shorter than the length field");
    spit(work + "/long_header.safetensors", le64(1000) + "{}");
    CHECK(SafetensorsReader::open(work + "/long_header.safetensors").is_err(), "header length beyond the file");
    const std::string not_json = "[1, 2";
    spit(work + "/not_json.safetensors", le64(not_json.size()) + not_json);
    CHECK(SafetensorsReader::open(work + "/not_json.safetensors").is_err(), "header not an object");
    const std::string outside = "{\"a\":{\"dtype\":\"F32\",\"shape\":[4],\"data_offsets\":[0,16]}}";
    spit(work + "/outside.safetensors", le64(outside.size()) + outside + std::string(8, '\0'));
    CHECK(SafetensorsReader::open(work + "/outside.safetensors").is_err(), "entry beyond the data section");
    const std::string wrong_len = "{\"a\":{\"dtype\":\"F32\",\"shape\":[4],\"data_offsets\":[0,8]}}";
    spit(work + "/wrong_len.safetensors", le64(wrong_len.size()) + wrong_len + std::string(8, '\0'));
    auto rd = SafetensorsReader::open(work + "/wrong_len.safetensors");
    CHECK(rd.is_ok() && !rd.value().to_vec_f32("a"), "byte range that disagrees with shape x dtype");
    // nesting far beyond any real header must be refused, not followed down the stack
    const std::string deep = "{\"a\":" + std::string(200000, '[') + "}";
    spit(work + "/deep.safetensors", le64(deep.size()) + deep);
    CHECK(SafetensorsReader::open(work + "/deep.safetensors").is_err(), "deeply nested header");
    CHECK(MoeConfig::from_json_str(std::string(200000, '[')).is_err(), "deeply nested config");
    CHECK(MoeConfig::from_json_str("{\"num_local_experts\": " + std::string(100, '[') + "8" + std::string(100, ']') + "}").is_err() ||
              true, "moderate nesting either parses or is refused");
    const std::string empty = "{}";
    spit(work + "/empty.safetensors", le64(empty.size()) + empty);
    auto e = SafetensorsReader::open(work + "/empty.safetensors");
    CHECK(e.is_ok() && e.value().entries().empty(), "empty checkpoint");
  });

  // ---- qint8 tier files -----------------------------------------------------------------------
  run_test("qint8_tier_file_round_trip", [&] {
    const size_t rows = 6, cols = 40;
    std::vector<float> w = seeded(31, rows * cols);
    for (size_t c = 0; c < cols; ++c) w[2 * cols + c] = 0.f;  // an all-zero row: scale 1, q 0
    w[4 * cols + 7] = 3.5f;                                   // an outlier sets its row's scale
    const std::string path = work + "/gate.qint8";
    auto werr = write_qint8_tensor_named(path, w, rows, cols);
    CHECK(!werr, "%s", werr ? werr->c_str() : "");
    CHECK(slurp(path).size() == qint8_disk_bytes(rows * cols, rows) && qint8_disk_bytes(rows * cols, rows) == 264,
          "rows * 4 + numel bytes: about one byte per element");
    auto t = read_qint8_tensor(path, rows * cols, rows).unwrap();
    const QInt8Tensor direct = quantize_per_row_i8(w, rows, cols);
    CHECK(t.q == direct.q && t.scales == direct.scales && t.rows == rows && t.cols == cols, "file == quantiser");
    CHECK(t.scales[2] == 1.0f && t.scales[4] == 3.5f / 127.0f && t.q[4 * cols + 7] == 127, "scales");
    const std::vector<float> back = read_qint8_to_f32(path, rows * cols, rows).unwrap();
    CHECK(back == t.dequantize(), "read_qint8_to_f32 is q * scale");
    for (size_t r = 0; r < rows; ++r)
      for (size_t c = 0; c < cols; ++c)
        CHECK(std::fabs(back[r * cols + c] - w[r * cols + c]) <= 0.5f * t.scales[r] * 1.0001f,
              "round trip within half a step at (%zu, %zu)", r, c);
    // the quantisation axis must divide the element count, and the size must match
    CHECK(read_qint8_tensor(path, rows * cols, 7).is_err(), "rows that do not divide numel");
    CHECK(read_qint8_tensor(path, rows * cols, 3).is_err(), "a file of another size");
    CHECK(read_qint8_tensor(work + "/absent.qint8", 8, 2).is_err(), "missing file");
    CHECK(write_qint8_tensor_named(path, w, rows, cols + 1).has_value(), "length mismatch on write");
  });
  run_test("expert_from_qint8_keeps_the_tier_data", [&] {
    const size_t d = 16, f = 24;
    auto g = quantize_per_row_i8(seeded(1, f * d), f, d), u = quantize_per_row_i8(seeded(2, f * d), f, d),
         dn = quantize_per_row_i8(seeded(3, d * f), d, f);
    auto ex = MoeDenseExpert::from_qint8(d, f, g, u, dn).unwrap();
    CHECK(ex.q8 && ex.q8->gate.q == g.q && ex.q8->down.scales == dn.scales, "payload kept");
    CHECK(ex.w_gate == g.dequantize() && ex.w_up == u.dequantize() && ex.w_down == dn.dequantize(),
          "w_* are the dequantised values");
    auto bad = MoeDenseExpert::from_qint8(d, f, g, u, g);
    CHECK(bad.is_err() && bad.error().kind == MoeDenseError::WeightShapeMismatch, "down of the wrong shape");
  });

  // ---- golden layer files ---------------------------------------------------------------------
  const char* models[] = {"mixtral", "qwen15_moe", "qwen2_moe", "qwen3_moe"};
  run_test("golden_layers_assemble_with_sidecar_config", [&] {
    for (const char* m : models) {
      Golden g = load_golden(golden, m);
      CHECK(g.layer.num_experts() == g.config.num_experts && g.input.size() == g.config.d_model &&
                g.atenia_ref.size() == g.config.d_model && g.hf_ref.size() == g.config.d_model, "%s sizes", m);
      const bool qwen_shared = !strcmp(m, "qwen15_moe") || !strcmp(m, "qwen2_moe");
      CHECK(g.layer.has_shared_expert() == qwen_shared && g.layer.shared_gate.has_value() == qwen_shared, "%s shared", m);
      CHECK(g.layer.resolve_convention() ==
                (qwen_shared ? MoeExecutionConvention::HuggingFaceQwen : MoeExecutionConvention::Atenia), "%s convention", m);
    }
    Golden q = load_golden(golden, "qwen15_moe");
    CHECK(q.layer.shared->d_ff == 22 && q.config.d_ff == 44, "Qwen1.5 shared expert has its own width");
  });
  run_test("golden_layers_through_the_oracle_match_f64_refs", [&] {
    for (const char* m : models) {
      Golden g = load_golden(golden, m);
      const double tol = 1e-5 * max_abs(g.atenia_ref);
      const double da = max_abs_diff(oracle_forward(g.layer, g.input, 0), g.atenia_ref);
      CHECK(da <= tol, "%s atenia_ref: %g > %g", m, da, tol);
      if (g.layer.shared_gate) {
        const double dh = max_abs_diff(oracle_forward(g.layer, g.input, 1), g.hf_ref);
        CHECK(dh <= 1e-5 * max_abs(g.hf_ref), "%s hf_ref: %g", m, dh);
      }
    }
  });
  // The DeepSeek block file: packed routed experts, `shared_experts.*` fused into one expert, no
  // gate tensor; the side file carries the DeepSeek config keys, the probe and the f64 output.
  struct DeepSeekBlock {
    RealMoeLayer layer;
    std::vector<float> probe, want;
    MoeExecutionConvention convention;
  };
  auto load_deepseek = [&]() {
    DeepSeekBlock b;
    const std::string text = slurp(golden + "/deepseek_block.json");
    atenia::json::Value side;
    CHECK(!text.empty() && atenia::json::parse(text, side), "side file");
    MoeConfig mc = MoeConfig::from_json_str(text).unwrap();
    CHECK(mc.is_moe() && *mc.num_experts == 4 && mc.experts_per_token_or(1) == 2 && mc.has_shared_experts &&
              *mc.expert_intermediate_size == 16, "config keys of the side file");
    auto cfg = MoeLayerConfig::make(*mc.num_experts, mc.experts_per_token_or(1), mc.has_shared_experts,
                                    (size_t)side.get("hidden")->num, *mc.expert_intermediate_size).unwrap();
    auto rd = SafetensorsReader::open(golden + "/deepseek_block.safetensors");
    CHECK(rd.is_ok(), "reader");
    const SafetensorsReader& reader = rd.value();
    const MoeWeightMap map = MoeWeightMap::from_tensors(reader.names_and_shapes());
    CHECK(MoeConventionResolver::from_weight_map(map) == MoeExecutionConvention::Atenia,
          "no gate tensor: the weight map alone would say Atenia");
    b.layer = assemble_real_moe_layer(map, 0, cfg, [&reader](const std::string& n) { return reader.to_vec_f32(n); }).unwrap();
    CHECK(b.layer.has_shared_expert() && !b.layer.shared_gate, "fused shared experts, ungated");
    b.probe = floats(side.get("probe"));
    b.want = floats(side.get("mlp_output"));
    b.convention = MoeConventionResolver::from_norm_topk_prob(false);  // the block's "simple routing": no renormalisation
    return b;
  };
  run_test("deepseek_block_through_the_oracle", [&] {
    DeepSeekBlock b = load_deepseek();
    const double d = max_abs_diff(oracle_forward(b.layer, b.probe, (int)b.convention), b.want);
    CHECK(d <= 1e-5 * max_abs(b.want), "%g", d);
  });
  if (no_gpu) {
    run_test("ingested_layer_without_device_fails_loudly", [&] {
      Golden g = load_golden(golden, "mixtral");
      auto r = g.layer.forward(g.input);
      CHECK(r.is_err() && r.error().kind == MoeLayerError::Device, "a forward without a device must fail, not fall back");
    });
    printf("%d tests, %d failed\n", g_run, g_failed);
    return g_failed ? 1 : 0;
  }

  // ---- device ---------------------------------------------------------------------------------
  run_test("atenia_mode_matches_atenia_ref", [&] {
    for (const char* m : models) {
      Golden g = load_golden(golden, m);
      auto out = g.layer.forward(g.input).unwrap();
      const double d = max_abs_diff(out, g.atenia_ref);
      CHECK(d <= 1e-5 * max_abs(g.atenia_ref), "%s: %g", m, d);
      CHECK(max_abs_diff(out, oracle_forward(g.layer, g.input, 0)) <= 1e-6 * max_abs(g.atenia_ref), "%s vs oracle", m);
    }
  });
  run_test("hf_qwen_mode_matches_hf_ref", [&] {
    for (const char* m : {"qwen15_moe", "qwen2_moe"}) {
      Golden g = load_golden(golden, m);
      auto out = g.layer.forward_with(g.input, MoeExecutionConvention::HuggingFaceQwen).unwrap();
      const double d = max_abs_diff(out, g.hf_ref);
      CHECK(d <= 1e-5 * max_abs(g.hf_ref), "%s: %g", m, d);
      auto automatic = g.layer.forward_auto(g.input).unwrap();
      CHECK(automatic == out, "%s: forward_auto resolves to HuggingFaceQwen", m);
      CHECK(max_abs_diff(out, g.layer.forward(g.input).unwrap()) > 1e-5, "%s: the conventions differ", m);
    }
  });
  run_test("mixtral_also_matches_hf_block", [&] {
    // Mixtral's own block renormalises the top-k weights, which is the Atenia convention.
    Golden g = load_golden(golden, "mixtral");
    auto out = g.layer.forward_auto(g.input).unwrap();
    CHECK(max_abs_diff(out, g.hf_ref) <= 1e-5 * max_abs(g.hf_ref), "%g", max_abs_diff(out, g.hf_ref));
  });
  run_test("deepseek_block_on_device", [&] {
    DeepSeekBlock b = load_deepseek();
    auto out = b.layer.forward_with(b.probe, b.convention).unwrap();
    CHECK(max_abs_diff(out, b.want) <= 1e-5 * max_abs(b.want), "%g", max_abs_diff(out, b.want));
  });
  run_test("deepseek_v3_routing_fixture_on_device", [&] {
    // tests/moe_v3_route_scale_cert_test.rs: 8 experts in 4 groups, 2 groups kept, top-2, weights
    // normalised and scaled by 2.5, one ungated shared expert; HuggingFace f64 block output.
    atenia::json::Value side;
    const std::string text = slurp(golden + "/v3_route_ref.json");
    CHECK(!text.empty() && atenia::json::parse(text, side), "side file");
    auto num = [&](const char* k) { return (size_t)side.get(k)->num; };
    auto rd = SafetensorsReader::open(golden + "/v3_route_ref.safetensors");
    CHECK(rd.is_ok(), "reader");
    const SafetensorsReader& reader = rd.value();
    const size_t n = num("n_routed_experts"), d = num("hidden_size"), f = num("moe_intermediate_size");
    std::vector<MoeDenseExpert> experts;
    for (size_t e = 0; e < n; ++e) {
      const std::string p = "expert." + std::to_string(e) + ".";
      experts.push_back(MoeDenseExpert::make(d, f, *reader.to_vec_f32(p + "w_gate"), *reader.to_vec_f32(p + "w_up"),
                                             *reader.to_vec_f32(p + "w_down")).unwrap());
    }
    auto routed = MoeDenseLayer::make(d, f, *reader.to_vec_f32("router.weight"), std::move(experts), num("top_k")).unwrap();
    auto shared = MoeDenseExpert::make(d, num("shared_intermediate_size"), *reader.to_vec_f32("shared.w_gate"),
                                       *reader.to_vec_f32("shared.w_up"), *reader.to_vec_f32("shared.w_down")).unwrap();
    auto layer = RealMoeLayer::assemble(MoeLayerConfig::make(n, num("top_k"), true, d, f).unwrap(), std::move(routed),
                                        std::move(shared), std::nullopt).unwrap();
    V3RouterConfig cfg;
    cfg.n_routed_experts = n; cfg.top_k = num("top_k"); cfg.n_group = num("n_group"); cfg.topk_group = num("topk_group");
    cfg.routed_scaling_factor = side.get("routed_scaling_factor")->num;
    cfg.norm_topk_prob = side.get("norm_topk_prob")->b;
    cfg.scoring_func = parse_scoring_func(side.get("scoring_func")->str).unwrap();
    auto err = layer.set_v3_router(cfg, *reader.to_vec_f32("router.bias"));
    CHECK(!err, "%s", err ? err->to_string().c_str() : "");
    const std::vector<float> hidden = *reader.to_vec_f32("hidden");
    std::vector<int32_t> idx;
    auto w = layer.route(hidden, MoeExecutionConvention::HuggingFaceQwen, &idx).unwrap();
    const auto& want_sets = side.get("selected_experts")->arr;
    const std::vector<float> dense = floats(side.get("dense_combine_weights"));
    for (size_t t = 0; t < num("tokens"); ++t)
      for (size_t s_ = 0; s_ < cfg.top_k; ++s_) {
        CHECK((size_t)idx[t * cfg.top_k + s_] == (size_t)want_sets[t].arr[s_].num, "token %zu slot %zu", t, s_);
        CHECK(std::fabs(w[t * cfg.top_k + s_] - dense[t * n + idx[t * cfg.top_k + s_]]) < 1e-6, "weight of token %zu", t);
      }
    auto out = layer.forward_with(hidden, MoeExecutionConvention::HuggingFaceQwen).unwrap();
    const std::vector<float> want = floats(side.get("block_out"));
    CHECK(max_abs_diff(out, want) < 1e-6, "block output: %g", max_abs_diff(out, want));
  });
  run_test("qint8_tier_files_to_device_without_requantising", [&] {
    // The Mixtral golden layer written as qint8 tier files, read back, and run as an Int8W8A16
    // layer: the tier data reaches the device as it is, so the result equals the layer that
    // quantises the same f32 weights itself, bit for bit; and it stays within the int8 bar of
    // the oracle run on the dequantised weights (the values the reference computes with).
    Golden g = load_golden(golden, "mixtral", MoeWeightStorage::Int8W8A16);
    const size_t E = g.layer.num_experts(), d = g.config.d_model, f = g.config.d_ff;
    std::vector<MoeDenseExpert> experts;
    for (size_t e = 0; e < E; ++e) {
      const MoeDenseExpert& src = g.layer.routed.experts[e];
      const std::string base = work + "/expert" + std::to_string(e);
      CHECK(!write_qint8_tensor_named(base + ".gate", src.w_gate, f, d) &&
                !write_qint8_tensor_named(base + ".up", src.w_up, f, d) &&
                !write_qint8_tensor_named(base + ".down", src.w_down, d, f), "write tier files");
      experts.push_back(MoeDenseExpert::from_qint8(d, f, read_qint8_tensor(base + ".gate", f * d, f).unwrap(),
                                                   read_qint8_tensor(base + ".up", f * d, f).unwrap(),
                                                   read_qint8_tensor(base + ".down", d * f, d).unwrap()).unwrap());
    }
    auto routed = MoeDenseLayer::make(d, f, g.layer.routed.w_router, std::move(experts), g.config.experts_per_token).unwrap();
    auto tier = RealMoeLayer::assemble(g.config, std::move(routed), std::nullopt, std::nullopt,
                                       MoeWeightStorage::Int8W8A16).unwrap();
    const std::vector<float> from_tier = tier.forward_auto(g.input).unwrap();
    const std::vector<float> from_f32 = g.layer.forward_auto(g.input).unwrap();
    CHECK(from_tier == from_f32, "tier data must reach the device unchanged: %g", max_abs_diff(from_tier, from_f32));
    const std::vector<float> want = oracle_forward(tier, g.input, 0);  // tier.routed holds the dequantised weights
    CHECK(max_abs_diff(from_tier, want) <= 1e-2 * max_abs(want), "%g of %g", max_abs_diff(from_tier, want), max_abs(want));
  });
  run_test("ingested_layer_through_the_registry", [&] {
    Golden g = load_golden(golden, "qwen2_moe");
    const std::vector<float> direct = g.layer.forward_auto(g.input).unwrap();
    const uint32_t id = register_real_moe_layer(std::move(g.layer));
    CHECK(execute_real_moe_layer(id, g.input).unwrap() == direct, "graph op == forward_auto");
    CHECK(moe_real_layer_reference_node(id, g.input) == direct, "executor arm");
  });
  run_test("ingested_layer_in_bf16_and_int8_storage", [&] {
    for (const char* m : models) {
      Golden f32 = load_golden(golden, m);
      const std::vector<float> want = f32.layer.forward_auto(f32.input).unwrap();
      const double scale = max_abs(want);
      for (MoeWeightStorage st : {MoeWeightStorage::Bf16, MoeWeightStorage::Int8W8A16}) {
        Golden g = load_golden(golden, m, st);
        const double d = max_abs_diff(g.layer.forward_auto(g.input).unwrap(), want);
        CHECK(d <= 3e-2 * scale, "%s storage %d: %g of %g", m, (int)st, d, scale);
      }
    }
  });
  printf("%d tests, %d failed\n", g_run, g_failed);
  return g_failed ? 1 : 0;
}
