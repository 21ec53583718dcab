// Tests of the C++ host mirror, written after the reference's own tests of the same interface:
//   tests/moe_real_layer_graph_op_test.rs  (graph op == forward_auto, determinism, unknown id,
//                                            bad input dim, explicit convention)
//   src/moe/layer.rs tests                 (config validation, convention resolution)
//   src/moe/binding.rs:611-640             (identical experts reproduce a single expert)
// The expected values come from the committed golden fixtures (written to a flat file by the
// pytest wrapper) and from the CPU oracle, which this test links as the checker.
//
// usage: host_mirror_test <fixtures.bin> [--no-gpu]
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <string>
#include <vector>

#include "../../ateniaengine_amd/host/atenia_moe.hpp"

using namespace atenia::moe;

// ---- the oracle's C interface (oracle/moe_oracle.c) -------------------------------------------
extern "C" {
typedef struct {
  int32_t num_experts, top_k, d_model, d_ff, d_ff_shared, convention;
  const float *w_router, *router_bias, *w_gate, *w_up, *w_down, *s_gate, *s_up, *s_down, *shared_gate;
} OraLayer;
int ora_layer_forward_with(const OraLayer* L, const float* x, int convention, int policy, float* out,
                           int32_t* idx_out, float* w_out, int32_t* err_index);
int ora_block_forward(const OraLayer* L, const float* x1, size_t n_tokens, const float* gamma, float eps,
                      int norm_policy, int policy, float* out, float* h2_out, int32_t* idx_out, float* w_out,
                      int32_t* err_token, int32_t* err_index);
void ora_expert_forward(const float* w_gate, const float* w_up, const float* w_down, size_t d, size_t f,
                        const float* x, float* out, int policy);
void ora_seeded(uint64_t seed, size_t n, float* out);
void ora_matvec(const float* w, size_t rows, size_t cols, const float* x, float* y);
void ora_softmax(const float* logits, size_t n, float* out);
}

static int g_failed = 0, g_run = 0;
#define CHECK(cond, ...)                                         \
  do {                                                           \
    if (!(cond)) {                                               \
      printf("    CHECK FAILED %s:%d: %s -- ", __FILE__, __LINE__, #cond); \
      printf(__VA_ARGS__);                                       \
      printf("\n");                                              \
      throw std::runtime_error("check failed");                  \
    }                                                            \
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

struct Metrics {  // src/moe/numerical.rs:58-88
  double max_abs_diff = 0, mean_abs_diff = 0, rmse = 0;
  bool argmax_match = false;
};
static Metrics metrics(const std::vector<float>& a, const std::vector<float>& r) {
  Metrics m;
  size_t ia = 0, ir = 0;
  double sum = 0, sq = 0;
  for (size_t i = 0; i < a.size(); ++i) {
    double d = std::fabs((double)a[i] - (double)r[i]);
    m.max_abs_diff = std::max(m.max_abs_diff, d);
    sum += d;
    sq += d * d;
    if ((double)a[i] > (double)a[ia]) ia = i;
    if ((double)r[i] > (double)r[ir]) ir = i;
  }
  m.mean_abs_diff = sum / a.size();
  m.rmse = std::sqrt(sq / a.size());
  m.argmax_match = ia == ir;
  return m;
}

// ---- fixtures ---------------------------------------------------------------------------------
struct Fixture {
  std::string name;
  int E, k, d, f, fs, gated;
  std::vector<float> w_router, gate, up, down, s_gate, s_up, s_down, shared_gate, input, atenia_ref, hf_ref;
};

static std::vector<Fixture> load_fixtures(const char* path) {
  std::vector<Fixture> out;
  FILE* fp = fopen(path, "rb");
  if (!fp) return out;
  int32_t n = 0;
  if (fread(&n, 4, 1, fp) != 1) n = 0;
  for (int i = 0; i < n; ++i) {
    Fixture fx;
    char nm[32];
    int32_t h[6];
    if (fread(nm, 1, 32, fp) != 32 || fread(h, 4, 6, fp) != 6) break;
    fx.name = nm;
    fx.E = h[0]; fx.k = h[1]; fx.d = h[2]; fx.f = h[3]; fx.fs = h[4]; fx.gated = h[5];
    auto rd = [&](std::vector<float>& v, size_t cnt) {
      v.resize(cnt);
      if (cnt && fread(v.data(), 4, cnt, fp) != cnt) v.clear();
    };
    const size_t E = fx.E, d = fx.d, f = fx.f, fs = fx.fs;
    rd(fx.w_router, E * d); rd(fx.gate, E * f * d); rd(fx.up, E * f * d); rd(fx.down, E * d * f);
    rd(fx.s_gate, fs * d); rd(fx.s_up, fs * d); rd(fx.s_down, d * fs);
    rd(fx.shared_gate, fx.gated ? d : 0);
    rd(fx.input, d); rd(fx.atenia_ref, d); rd(fx.hf_ref, d);
    out.push_back(std::move(fx));
  }
  fclose(fp);
  return out;
}

static RealMoeLayer layer_from(const Fixture& fx, MoeWeightStorage st = MoeWeightStorage::F32) {
  const size_t E = fx.E, d = fx.d, f = fx.f, fs = fx.fs;
  auto cfg = MoeLayerConfig::make(E, fx.k, fs > 0, d, f).unwrap();
  std::vector<MoeDenseExpert> ex;
  for (size_t e = 0; e < E; ++e) {
    auto sl = [&](const std::vector<float>& v, size_t per) {
      return std::vector<float>(v.begin() + e * per, v.begin() + (e + 1) * per);
    };
    ex.push_back(MoeDenseExpert::make(d, f, sl(fx.gate, f * d), sl(fx.up, f * d), sl(fx.down, d * f)).unwrap());
  }
  auto routed = MoeDenseLayer::make(d, f, fx.w_router, std::move(ex), fx.k).unwrap();
  std::optional<MoeDenseExpert> shared;
  if (fs) shared = MoeDenseExpert::make(d, fs, fx.s_gate, fx.s_up, fx.s_down).unwrap();
  std::optional<std::vector<float>> sg;
  if (fx.gated) sg = fx.shared_gate;
  return RealMoeLayer::assemble(cfg, std::move(routed), std::move(shared), std::move(sg), st).unwrap();
}

// The reference's synthetic fixture generator (dense.rs:368-379) through the oracle's restatement.
static std::vector<float> seeded(uint64_t seed, size_t n) {
  std::vector<float> v(n);
  ora_seeded(seed, n, v.data());
  return v;
}
static Fixture synthetic(int E, int k, int d, int f, bool identical = false) {
  Fixture fx;
  fx.name = "synthetic";
  fx.E = E; fx.k = k; fx.d = d; fx.f = f; fx.fs = 0; fx.gated = 0;
  fx.w_router = seeded(1, (size_t)E * d);
  for (int e = 0; e < E; ++e) {
    const uint64_t s = identical ? 100 : 100 + 10 * e;
    auto g = seeded(s, (size_t)f * d), u = seeded(s + 1, (size_t)f * d), dn = seeded(s + 2, (size_t)d * f);
    fx.gate.insert(fx.gate.end(), g.begin(), g.end());
    fx.up.insert(fx.up.end(), u.begin(), u.end());
    fx.down.insert(fx.down.end(), dn.begin(), dn.end());
  }
  fx.input = seeded(7, d);
  return fx;
}
static OraLayer ora_of(const Fixture& fx, int conv) {
  OraLayer L;
  memset(&L, 0, sizeof(L));
  L.num_experts = fx.E; L.top_k = fx.k; L.d_model = fx.d; L.d_ff = fx.f; L.d_ff_shared = fx.fs;
  L.convention = conv;
  L.w_router = fx.w_router.data(); L.w_gate = fx.gate.data(); L.w_up = fx.up.data(); L.w_down = fx.down.data();
  if (fx.fs) { L.s_gate = fx.s_gate.data(); L.s_up = fx.s_up.data(); L.s_down = fx.s_down.data(); }
  if (fx.gated) L.shared_gate = fx.shared_gate.data();
  return L;
}

int main(int argc, char** argv) {
  const bool no_gpu = argc > 2 && !strcmp(argv[2], "--no-gpu");
  std::vector<Fixture> fixtures = argc > 1 ? load_fixtures(argv[1]) : std::vector<Fixture>();
  auto find = [&](const char* n) -> const Fixture* {
    for (auto& f : fixtures) if (f.name == n) return &f;
    return nullptr;
  };

  // ---- host logic (no device needed) --------------------------------------------------------
  run_test("config_validation_errors", [] {
    CHECK(MoeLayerConfig::make(0, 1, false, 4, 4).error().kind == MoeConfigError::ZeroExperts, "kind");
    CHECK(MoeLayerConfig::make(4, 0, false, 4, 4).error().kind == MoeConfigError::ZeroExpertsPerToken, "kind");
    auto e = MoeLayerConfig::make(2, 3, false, 4, 4).error();
    CHECK(e.kind == MoeConfigError::ExpertsPerTokenExceedsCount && e.per_token == 3 && e.total == 2, "payload");
    CHECK(MoeLayerConfig::make(2, 1, false, 0, 4).error().kind == MoeConfigError::ZeroDModel, "kind");
    CHECK(MoeLayerConfig::make(2, 1, false, 4, 0).error().kind == MoeConfigError::ZeroDFf, "kind");
    CHECK(MoeLayerConfig::make(8, 2, true, 64, 128).is_ok(), "valid config rejected");
  });
  run_test("expert_and_layer_shape_errors", [] {
    auto e = MoeDenseExpert::make(4, 8, std::vector<float>(31), std::vector<float>(32), std::vector<float>(32));
    CHECK(e.is_err() && e.error().kind == MoeDenseError::WeightShapeMismatch, "kind");
    CHECK(e.error().to_string() == "moe-dense: w_gate weight shape mismatch: expected 32 elems, got 31", "%s",
          e.error().to_string().c_str());
    auto l = MoeDenseLayer::make(4, 8, std::vector<float>(8), {}, 1);
    CHECK(l.is_err() && l.error().kind == MoeDenseError::NoExperts, "kind");
    auto ex = MoeDenseExpert::make(4, 8, std::vector<float>(32), std::vector<float>(32), std::vector<float>(32)).unwrap();
    auto l2 = MoeDenseLayer::make(4, 8, std::vector<float>(12), {ex, ex}, 1);
    CHECK(l2.is_err() && l2.error().kind == MoeDenseError::RouterExpertCountMismatch, "kind");
  });
  run_test("assemble_cross_checks_config", [] {
    Fixture fx = synthetic(4, 2, 8, 16);
    RealMoeLayer ok = layer_from(fx);
    CHECK(ok.num_experts() == 4 && !ok.has_shared_expert(), "topology");
    CHECK(ok.resolve_convention() == MoeExecutionConvention::Atenia, "no gate => Atenia");
    auto cfg = MoeLayerConfig::make(5, 2, false, 8, 16).unwrap();
    auto bad = RealMoeLayer::assemble(cfg, ok.routed, std::nullopt, std::nullopt);
    CHECK(bad.is_err() && bad.error().kind == MoeLayerError::ConfigMismatch, "kind");
    CHECK(bad.error().detail == "resolved 4 experts but config.num_experts = 5", "%s", bad.error().detail.c_str());
    auto cfg2 = MoeLayerConfig::make(4, 2, true, 8, 16).unwrap();
    CHECK(RealMoeLayer::assemble(cfg2, ok.routed, std::nullopt, std::nullopt).is_err(), "missing shared accepted");
  });
  run_test("graph_real_moe_layer_rejects_unknown_layer", [] {
    auto r = execute_real_moe_layer(0xffffffffu, std::vector<float>(64, 0.f));
    CHECK(r.is_err() && r.error().kind == MoeLayerError::Binding &&
              r.error().binding.kind == MoeBindingError::LayerNotFound, "kind");
    CHECK(r.error().binding.layer_id == 0xffffffffu, "layer id");
    bool thrown = false;
    try {
      moe_real_layer_reference_node(0xffffffffu, std::vector<float>(64, 0.f));
    } catch (const std::runtime_error& e) {
      thrown = strstr(e.what(), "unknown layer_id") != nullptr;
    }
    CHECK(thrown, "node did not fail loudly with the reference's message");
  });
  run_test("graph_real_moe_layer_rejects_bad_input_dim", [] {
    uint32_t id = register_real_moe_layer(layer_from(synthetic(4, 2, 8, 16)));
    auto r = execute_real_moe_layer(id, std::vector<float>(5, 0.f));
    CHECK(r.is_err() && r.error().kind == MoeLayerError::Sparse &&
              r.error().sparse.kind == MoeSparseError::Dense &&
              r.error().sparse.dense.kind == MoeDenseError::DimMismatch, "kind");
    CHECK(r.error().sparse.dense.expected == 8 && r.error().sparse.dense.actual == 5, "payload");
    bool thrown = false;
    try { moe_real_layer_reference_node(id, std::vector<float>(5, 0.f)); } catch (const std::runtime_error&) { thrown = true; }
    CHECK(thrown, "node accepted a bad input dim");
    CHECK(get_real_moe_layer(id) != nullptr && get_real_moe_layer(id + 1000) == nullptr, "registry lookup");
  });
  // src/moe/numeric_policy.rs:208-251 and tests/numeric_policy_test.rs, same cases
  run_test("policy_classification_is_correct", [] {
    CHECK(!ffn_uses_f32(NumericPolicy::Certified) && !ffn_uses_cuda(NumericPolicy::Certified), "certified");
    CHECK(ffn_uses_f32(NumericPolicy::Strict) && !ffn_uses_cuda(NumericPolicy::Strict), "strict");
    CHECK(ffn_uses_f32(NumericPolicy::Fast) && ffn_uses_cuda(NumericPolicy::Fast), "fast");
    CHECK(std::string(as_str(NumericPolicy::Strict)) == "strict" && std::string(as_str(NumericPolicy::Fast)) == "fast" &&
              std::string(as_str(NumericPolicy::Certified)) == "certified", "as_str");
  });
  run_test("policy_from_str_unknown_is_none_known_ok", [] {
    CHECK(numeric_policy_from_str("certified") == NumericPolicy::Certified, "certified");
    CHECK(numeric_policy_from_str("STRICT") == NumericPolicy::Strict, "case");
    CHECK(numeric_policy_from_str(" fast \n") == NumericPolicy::Fast, "trim");
    CHECK(numeric_policy_from_str("f64") == NumericPolicy::Certified && numeric_policy_from_str("f32") == NumericPolicy::Strict, "aliases");
    CHECK(!numeric_policy_from_str("garbage").has_value() && !numeric_policy_from_str("").has_value(), "unknown");
  });
  run_test("policy_override_selects_and_clears", [] {
    clear_numeric_policy_override();
    const NumericPolicy from_env = numeric_policy();  // Certified unless ATENIA_NUMERIC_POLICY says otherwise
    const char* env = getenv("ATENIA_NUMERIC_POLICY");
    CHECK(env || from_env == NumericPolicy::Certified, "no override and no env must mean Certified");
    set_numeric_policy(NumericPolicy::Strict);
    CHECK(numeric_policy() == NumericPolicy::Strict, "strict");
    set_numeric_policy(NumericPolicy::Fast);
    CHECK(numeric_policy() == NumericPolicy::Fast, "fast");
    set_numeric_policy(NumericPolicy::Certified);
    CHECK(numeric_policy() == NumericPolicy::Certified, "certified");
    clear_numeric_policy_override();
    CHECK(numeric_policy() == from_env, "cleared");
  });
  run_test("policy_certificate_passes_on_identical_and_fails_on_token_mismatch", [] {
    std::vector<std::vector<float>> r = {{1.0f, 2.0f, 0.5f}, {0.1f, 0.2f, 9.0f}};
    std::vector<uint32_t> toks = {1, 2};
    auto c = PolicyCertificate::compare(NumericPolicy::Strict, r, r, toks, toks);
    CHECK(c.passes(STRICT_LOGIT_TOLERANCE) && c.argmax_match_rate == 1.0 && c.max_abs_diff == 0.0 && c.rows == 2, "identical");
    std::vector<std::vector<float>> cand = {{1.0001f, 2.0f, 0.5f}, {0.1f, 0.2f, 9.0001f}};
    auto c2 = PolicyCertificate::compare(NumericPolicy::Strict, r, cand, toks, toks);
    CHECK(c2.passes(STRICT_LOGIT_TOLERANCE) && c2.max_abs_diff > 9e-5 && c2.max_abs_diff < 1.1e-4, "tiny drift: %g", c2.max_abs_diff);
    // mean of the per-row means, root of the mean of the per-row squared rmse
    const double d0 = (double)1.0001f - 1.0, d1 = (double)9.0001f - 9.0;
    CHECK(std::fabs(c2.mean_abs_diff - (d0 / 3 + d1 / 3) / 2) < 1e-12, "mean_abs_diff %g", c2.mean_abs_diff);
    CHECK(std::fabs(c2.rmse - std::sqrt((d0 * d0 / 3 + d1 * d1 / 3) / 2)) < 1e-12, "rmse %g", c2.rmse);
    auto c3 = PolicyCertificate::compare(NumericPolicy::Strict, r, r, toks, {1, 3});
    CHECK(!c3.passes(STRICT_LOGIT_TOLERANCE), "token mismatch");
    std::vector<std::vector<float>> flip = {{2.0f, 1.0f, 0.5f}, {0.1f, 0.2f, 9.0f}};
    auto c4 = PolicyCertificate::compare(NumericPolicy::Strict, r, flip, toks, toks);
    CHECK(!c4.passes(STRICT_LOGIT_TOLERANCE) && c4.argmax_match_rate == 0.5, "argmax flip");
    // rows of different length are skipped, as NumericalMetrics::compute returns None
    std::vector<std::vector<float>> ragged = {{1.0f, 2.0f}, {0.1f, 0.2f, 9.0f}};
    auto c5 = PolicyCertificate::compare(NumericPolicy::Fast, r, ragged, toks, toks);
    CHECK(c5.rows == 1 && c5.policy == NumericPolicy::Fast, "skipped rows");
    CHECK(!NumericalMetrics::compute({}, {}).has_value() && !NumericalMetrics::compute({1.f}, {1.f, 2.f}).has_value(), "None cases");
    auto m = NumericalMetrics::compute({1.f, 5.f, 5.f}, {1.f, 5.f, 4.f}).value();
    CHECK(m.argmax_match && m.max_abs_diff == 1.0 && m.passes(1.5) && !m.passes(1.0), "first maximum wins; gate is strict");
  });
  if (no_gpu) {
    run_test("forward_without_device_fails_loudly", [] {
      RealMoeLayer l = layer_from(synthetic(4, 2, 8, 16));
      auto r = l.forward_auto(seeded(3, 8));
      CHECK(r.is_err() && r.error().kind == MoeLayerError::Device, "a forward without a GPU must be a Device error");
    });
    printf("%d tests, %d failed\n", g_run, g_failed);
    return g_failed ? 1 : 0;
  }

  // ---- device path ----------------------------------------------------------------------------
  const Fixture* mix = find("mixtral_layer0");
  const Fixture* q15 = find("qwen15_moe_layer0");
  run_test("fixtures_present", [&] { CHECK(mix && q15, "fixture file missing or truncated"); });
  if (!mix || !q15) return 1;

  run_test("graph_real_moe_layer_matches_reference", [&] {
    RealMoeLayer layer = layer_from(*mix);
    auto reference = layer.forward_auto(mix->input).unwrap();
    uint32_t id = register_real_moe_layer(layer);
    auto got = moe_real_layer_reference_node(id, mix->input);
    Metrics m = metrics(got, reference);
    CHECK(m.max_abs_diff < 1e-5, "graph vs forward_auto: %g", m.max_abs_diff);
    Metrics mhf = metrics(got, mix->hf_ref);
    CHECK(mhf.argmax_match && mhf.max_abs_diff < 0.5, "graph vs HF: %g", mhf.max_abs_diff);
    Metrics ma = metrics(got, mix->atenia_ref);  // the fixture's f64 reference, much tighter
    CHECK(ma.max_abs_diff < 1e-5, "graph vs f64 reference: %g", ma.max_abs_diff);
  });
  run_test("graph_real_moe_layer_is_deterministic", [&] {
    uint32_t id = register_real_moe_layer(layer_from(*mix));
    auto a = moe_real_layer_reference_node(id, mix->input), b = moe_real_layer_reference_node(id, mix->input);
    CHECK(a == b, "two runs differ");
    for (float v : a) CHECK(std::isfinite(v), "non-finite output");
  });
  run_test("graph_real_moe_layer_with_explicit_convention", [&] {
    RealMoeLayer layer = layer_from(*mix);
    auto direct = layer.forward_auto(mix->input).unwrap();
    uint32_t id = register_real_moe_layer(layer);
    auto via = execute_real_moe_layer_with(id, mix->input, MoeExecutionConvention::Atenia).unwrap();
    CHECK(via == direct, "explicit Atenia convention differs from forward_auto on a layer without gate");
  });
  run_test("qwen_convention_auto_resolved", [&] {
    RealMoeLayer layer = layer_from(*q15);
    CHECK(layer.has_shared_expert() && layer.resolve_convention() == MoeExecutionConvention::HuggingFaceQwen,
          "gate present => HuggingFaceQwen");
    auto hf = layer.forward_auto(q15->input).unwrap();
    CHECK(metrics(hf, q15->hf_ref).max_abs_diff < 1e-5, "HuggingFaceQwen vs hf_ref: %g",
          metrics(hf, q15->hf_ref).max_abs_diff);
    auto at = layer.forward(q15->input).unwrap();
    CHECK(metrics(at, q15->atenia_ref).max_abs_diff < 1e-5, "Atenia vs atenia_ref: %g",
          metrics(at, q15->atenia_ref).max_abs_diff);
    CHECK(metrics(at, hf).max_abs_diff > 1e-7, "the two conventions must differ on this layer");
  });
  run_test("batch_equals_rows_and_oracle", [&] {
    Fixture fx = synthetic(4, 2, 8, 16);
    RealMoeLayer layer = layer_from(fx);
    uint32_t id = register_real_moe_layer(layer);
    const int T = 5, d = fx.d;
    std::vector<float> x = seeded(11, (size_t)T * d);
    auto batch = execute_real_moe_layer(id, x).unwrap();
    std::vector<int32_t> idx;
    auto w = layer.route(x, MoeExecutionConvention::Atenia, &idx).unwrap();
    OraLayer ol = ora_of(fx, 0);
    for (int t = 0; t < T; ++t) {
      std::vector<float> row(x.begin() + t * d, x.begin() + (t + 1) * d), want(d), ow(fx.k);
      std::vector<int32_t> oi(fx.k);
      int32_t err = 0;
      CHECK(ora_layer_forward_with(&ol, row.data(), 0, 0, want.data(), oi.data(), ow.data(), &err) == 0, "oracle");
      auto one = execute_real_moe_layer(id, row).unwrap();
      std::vector<float> brow(batch.begin() + t * d, batch.begin() + (t + 1) * d);
      CHECK(metrics(one, want).max_abs_diff < 1e-5, "row %d vs oracle: %g", t, metrics(one, want).max_abs_diff);
      CHECK(metrics(brow, one).max_abs_diff < 1e-6, "row %d of the batch vs the row alone", t);
      for (int s = 0; s < fx.k; ++s) {
        CHECK(idx[t * fx.k + s] == oi[s], "row %d slot %d routed to %d, oracle %d", t, s, idx[t * fx.k + s], oi[s]);
        CHECK(std::fabs(w[t * fx.k + s] - ow[s]) <= 1.2e-7f * std::fabs(ow[s]), "routing weight");
      }
    }
  });
  run_test("strict_policy_accumulates_in_f32_like_the_reference", [&] {
    // f32 layer under Strict / Fast: the oracle's f32-accumulating expert (dense.rs:120-140);
    // routing must not move; Certified afterwards is the f64 result again.
    Fixture fx = synthetic(4, 2, 64, 96);
    RealMoeLayer layer = layer_from(fx);
    const int T = 6, d = fx.d;
    std::vector<float> x = seeded(21, (size_t)T * d);
    OraLayer ol = ora_of(fx, 0);
    auto oracle_rows = [&](int policy) {
      std::vector<float> out((size_t)T * d);
      for (int t = 0; t < T; ++t) {
        std::vector<float> ow(fx.k);
        std::vector<int32_t> oi(fx.k);
        int32_t err = 0;
        CHECK(ora_layer_forward_with(&ol, x.data() + (size_t)t * d, 0, policy, out.data() + (size_t)t * d,
                                     oi.data(), ow.data(), &err) == 0, "oracle");
      }
      return out;
    };
    const std::vector<float> want_cert = oracle_rows(0), want_strict = oracle_rows(1);
    CHECK(metrics(want_cert, want_strict).max_abs_diff > 0.0, "the two arithmetics should differ somewhere");
    std::vector<int32_t> idx_cert, idx_strict;
    clear_numeric_policy_override();
    auto cert = layer.forward(x).unwrap();
    layer.route(x, MoeExecutionConvention::Atenia, &idx_cert).unwrap();
    for (NumericPolicy p : {NumericPolicy::Strict, NumericPolicy::Fast}) {
      set_numeric_policy(p);
      auto got = layer.forward(x).unwrap();
      layer.route(x, MoeExecutionConvention::Atenia, &idx_strict).unwrap();
      size_t differ = 0;
      for (size_t i = 0; i < got.size(); ++i) differ += memcmp(&got[i], &want_strict[i], 4) != 0;
      // bit for bit, up to the last ulp of the device's f64 exp inside silu
      CHECK(differ * 1000 <= got.size(), "%zu of %zu elements differ from the f32-accumulating oracle", differ, got.size());
      CHECK(metrics(got, want_strict).max_abs_diff <= 1e-6 * (1.0 + metrics(want_strict, std::vector<float>(got.size(), 0.f)).max_abs_diff), "drift");
      CHECK(idx_strict == idx_cert, "routing moved under %s", as_str(p));
    }
    set_numeric_policy(NumericPolicy::Certified);
    auto again = layer.forward(x).unwrap();
    CHECK(memcmp(again.data(), cert.data(), cert.size() * 4) == 0, "Certified after Strict differs from Certified before");
    CHECK(metrics(cert, want_cert).max_abs_diff < 1e-5, "certified vs oracle");
    clear_numeric_policy_override();
    // the certificate the reference's harness would form
    std::vector<std::vector<float>> ref_rows, cand_rows;
    for (int t = 0; t < T; ++t) {
      ref_rows.emplace_back(want_cert.begin() + (size_t)t * d, want_cert.begin() + (size_t)(t + 1) * d);
      cand_rows.emplace_back(want_strict.begin() + (size_t)t * d, want_strict.begin() + (size_t)(t + 1) * d);
    }
    auto cert_c = PolicyCertificate::compare(NumericPolicy::Strict, ref_rows, cand_rows, {1, 2}, {1, 2});
    CHECK(cert_c.passes(STRICT_LOGIT_TOLERANCE), "strict certificate: max %g argmax %g", cert_c.max_abs_diff, cert_c.argmax_match_rate);
  });
  run_test("dense_layer_unit_forwards_match_the_oracle", [&] {
    // MoeDenseExpert::forward, MoeDenseLayer::{route, forward, forward_sparse[_with]} as the
    // reference's in-module tests use them (src/moe/dense.rs:405-470, src/moe/sparse.rs:341-397)
    Fixture fx = synthetic(6, 2, 16, 24);
    RealMoeLayer rl = layer_from(fx);
    const MoeDenseLayer& layer = rl.routed;
    const std::vector<float> x = seeded(5, fx.d);
    OraLayer ol = ora_of(fx, 0);
    // one expert
    for (int e : {0, 5}) {
      std::vector<float> want(fx.d);
      ora_expert_forward(fx.gate.data() + (size_t)e * fx.f * fx.d, fx.up.data() + (size_t)e * fx.f * fx.d,
                         fx.down.data() + (size_t)e * fx.d * fx.f, fx.d, fx.f, x.data(), want.data(), 0);
      auto got = layer.experts[e].forward(x).unwrap();
      CHECK(metrics(got, want).max_abs_diff <= 1e-6, "expert %d: %g", e, metrics(got, want).max_abs_diff);
    }
    // router weights
    std::vector<float> lg(fx.E), sm(fx.E);
    ora_matvec(fx.w_router.data(), fx.E, fx.d, x.data(), lg.data());
    ora_softmax(lg.data(), fx.E, sm.data());
    auto ro = layer.route(x).unwrap();
    CHECK(ro.weights.size() == (size_t)fx.E, "one weight per expert");
    for (int e = 0; e < fx.E; ++e)
      CHECK(std::fabs(ro.weights[e] - sm[e]) <= 1.2e-7f * sm[e], "weight %d: %g vs %g", e, ro.weights[e], sm[e]);
    CHECK(std::fabs(ro.weight_sum() - 1.0f) < 1e-5f, "weights sum to one");
    // sparse, both conventions, against the oracle; selected experts ascending
    for (int conv = 0; conv < 2; ++conv) {
      std::vector<float> want(fx.d), ow(fx.k);
      std::vector<int32_t> oi(fx.k);
      int32_t err = 0;
      CHECK(ora_layer_forward_with(&ol, x.data(), conv, 0, want.data(), oi.data(), ow.data(), &err) == 0, "oracle");
      auto sp = layer.forward_sparse_with(x, fx.k, conv == 0).unwrap();
      CHECK(metrics(sp.output, want).max_abs_diff <= 1e-6, "sparse conv %d: %g", conv, metrics(sp.output, want).max_abs_diff);
      CHECK(sp.selected_experts.size() == (size_t)fx.k, "k experts");
      for (int s = 0; s < fx.k; ++s) CHECK((int32_t)sp.selected_experts[s] == oi[s], "selected expert %d", s);
    }
    auto sp_default = layer.forward_sparse(x, fx.k).unwrap();
    auto sp_renorm = layer.forward_sparse_with(x, fx.k, true).unwrap();
    CHECK(sp_default.output == sp_renorm.output, "forward_sparse renormalises");
    // k = E with raw weights is the dense forward (sparse.rs "k_equals_num_experts" test)
    auto dense = layer.forward(x).unwrap();
    auto all = layer.forward_sparse_with(x, fx.E, false).unwrap();
    CHECK(dense == all.output, "dense forward == sparse with every expert and raw weights");
    std::vector<float> manual(fx.d, 0.f);
    for (int e = 0; e < fx.E; ++e) {
      auto y = layer.experts[e].forward(x).unwrap();
      for (int c = 0; c < fx.d; ++c) manual[c] += ro.weights[e] * y[c];
    }
    CHECK(metrics(dense, manual).max_abs_diff <= 1e-6, "dense forward vs manual weighted sum");
    // errors: dimension first, then k (the order of route() and top_k_routing_with())
    auto e1 = layer.forward_sparse(std::vector<float>(3, 0.f), 0);
    CHECK(e1.is_err() && e1.error().kind == MoeSparseError::Dense && e1.error().dense.kind == MoeDenseError::DimMismatch &&
              e1.error().dense.expected == (size_t)fx.d && e1.error().dense.actual == 3, "dim before k");
    CHECK(layer.forward_sparse(x, 0).error().kind == MoeSparseError::ZeroK, "zero k");
    auto e3 = layer.forward_sparse(x, fx.E + 1).error();
    CHECK(e3.kind == MoeSparseError::KExceedsExperts && e3.k == (size_t)fx.E + 1 && e3.num_experts == (size_t)fx.E, "k > E");
    CHECK(e3.to_string() == "moe-sparse: k (7) exceeds num_experts (6)", "%s", e3.to_string().c_str());
    auto e4 = layer.experts[0].forward(std::vector<float>(2, 0.f)).error();
    CHECK(e4.kind == MoeDenseError::DimMismatch && std::string(e4.what) == "expert input", "expert input dim");
  });
  run_test("decomposed_graph_ops_match_the_sparse_reference", [&] {
    // tests/moe_dynamic_dispatch_test.rs and tests/moe_conditional_expert_test.rs, same checks
    Fixture fx = synthetic(6, 2, 16, 24);
    RealMoeLayer rl = layer_from(fx);
    const uint32_t id = register_layer(rl.routed);
    auto layer = get_layer(id);
    CHECK(layer && layer->num_experts() == 6 && !get_layer(id + 1000), "registry");
    const std::vector<float> x = seeded(9, fx.d);
    const size_t k = 2;
    auto reference = execute_sparse_reference(id, x, k).unwrap();
    auto sp = layer->forward_sparse(x, k).unwrap();
    CHECK(reference == sp.output, "graph op == forward_sparse");
    // the selection as MoeTopK emits it: [idx0, w0, idx1, w1], renormalised weights
    auto ro = layer->route(x).unwrap();
    double sum = 0;
    for (size_t e : sp.selected_experts) sum += (double)ro.weights[e];
    std::vector<float> selection;
    for (size_t e : sp.selected_experts) {
      selection.push_back((float)e);
      selection.push_back((float)((double)ro.weights[e] * (1.0 / sum)));
    }
    auto dd = execute_dynamic_dispatch(id, x, selection).unwrap();
    CHECK(metrics(dd.output, reference).max_abs_diff < 1e-5, "dispatch vs sparse reference: %g",
          metrics(dd.output, reference).max_abs_diff);
    CHECK(dd.executed_experts == sp.selected_experts && dd.executed_experts.size() < layer->num_experts(),
          "only the selected experts run");
    auto dd2 = execute_dynamic_dispatch(id, x, selection).unwrap();
    CHECK(dd.output == dd2.output, "deterministic");
    // conditional experts: one node per expert, contributions summed
    std::vector<float> conditional(fx.d, 0.f);
    size_t executed = 0, skipped = 0;
    for (uint32_t e = 0; e < 6; ++e) {
      auto ce = execute_conditional_expert(id, e, x, selection).unwrap();
      CHECK(ce.first.size() == (size_t)fx.d, "contribution length");
      if (ce.second) {
        ++executed;
        for (int c = 0; c < fx.d; ++c) conditional[c] += ce.first[c];
      } else {
        ++skipped;
        for (float v : ce.first) CHECK(v == 0.0f, "a skipped expert contributes zeros");
      }
    }
    CHECK(executed == k && skipped == 6 - k, "exactly k experts execute");
    CHECK(metrics(conditional, dd.output).max_abs_diff < 1e-6, "conditional pipeline == dynamic dispatch");
    CHECK(metrics(conditional, reference).max_abs_diff < 1e-5, "conditional pipeline == sparse reference");
    auto one = execute_conditional_expert(id, (uint32_t)sp.selected_experts[0], x, {(float)sp.selected_experts[0], 0.6f}).unwrap();
    auto y0 = layer->experts[sp.selected_experts[0]].forward(x).unwrap();
    for (int c = 0; c < fx.d; ++c) CHECK(std::fabs(one.first[c] - 0.6f * y0[c]) < 1e-6, "weight * expert output");
    CHECK(expert_weight_in_selection(selection, (uint32_t)sp.selected_experts[1]).value() == selection[3] &&
              !expert_weight_in_selection(selection, 99).has_value(), "weight lookup");
    // errors (dispatch_rejects_bad_selection / unknown layer / expert out of range)
    CHECK(execute_dynamic_dispatch(id, x, {0.0f, 0.5f, 1.0f}).is_err(), "odd selection length");
    auto bad = execute_dynamic_dispatch(id, x, {99.0f, 1.0f}).error();
    CHECK(bad.kind == MoeSparseError::KExceedsExperts && bad.k == 100 && bad.num_experts == 6, "index out of range");
    CHECK(execute_dynamic_dispatch(id, x, {-1.0f, 1.0f}).error().kind == MoeSparseError::NegativeWeight, "negative index");
    auto unk = execute_dynamic_dispatch(0xffffffffu, x, {0.0f, 1.0f});
    CHECK(unk.is_err() && unk.error().kind == MoeSparseError::Dense && unk.error().dense.kind == MoeDenseError::NoExperts, "unknown layer");
    CHECK(execute_conditional_expert(0xffffffffu, 0, x, {0.0f, 1.0f}).is_err(), "unknown layer");
    CHECK(execute_conditional_expert(id, 6, x, {0.0f, 1.0f}).error().kind == MoeSparseError::KExceedsExperts, "expert out of range");
    CHECK(execute_sparse_reference(0xffffffffu, x, 2).is_err(), "unknown layer");
  });
  run_test("identical_experts_reproduce_single_expert", [&] {
    Fixture fx = synthetic(4, 2, 8, 16, true);
    RealMoeLayer layer = layer_from(fx);
    auto out = layer.forward_routed(fx.input).unwrap();
    std::vector<float> want(fx.d);
    ora_expert_forward(fx.gate.data(), fx.up.data(), fx.down.data(), fx.d, fx.f, fx.input.data(), want.data(), 0);
    CHECK(metrics(out, want).max_abs_diff < 1e-5, "renormalised combine of identical experts: %g",
          metrics(out, want).max_abs_diff);
  });
  run_test("ffn_block_is_residual_plus_layer_of_normed_rows", [&] {
    // src/moe/full_forward.rs:239-252 on the Qwen fixture's weights (gated shared expert), three
    // rows, both norm arithmetics; the oracle's block is the checker.
    RealMoeLayer layer = layer_from(*q15);
    const size_t d = q15->d;
    std::vector<float> x1 = seeded(21, 3 * d), gamma = seeded(22, d);
    for (auto& g : gamma) g = 1.0f + 0.25f * g;
    const MoeExecutionConvention conv = layer.resolve_convention();
    OraLayer L = ora_of(*q15, (int)conv);
    for (int pol = 0; pol < 2; ++pol) {
      auto got = layer.ffn_block(x1, gamma, 1e-6f, (RealMoeLayer::NormPolicy)pol, conv).unwrap();
      std::vector<float> want(x1.size());
      int32_t et = -1, ei = -1;
      CHECK(ora_block_forward(&L, x1.data(), 3, gamma.data(), 1e-6f, pol, 0, want.data(), nullptr, nullptr,
                              nullptr, &et, &ei) == 0, "oracle block");
      double scale = 0;
      for (float v : want) scale = std::max(scale, (double)std::fabs(v));
      CHECK(metrics(got, want).max_abs_diff <= 1e-5 * scale, "policy %d: %g of %g", pol,
            metrics(got, want).max_abs_diff, scale);
    }
    auto bad = layer.ffn_block(x1, std::vector<float>(d - 1, 1.0f), 1e-6f, RealMoeLayer::NormPolicy::GraphF32, conv);
    CHECK(bad.is_err() && bad.error().kind == MoeLayerError::Sparse, "gamma of the wrong length");
  });
  run_test("non_finite_input_surfaces_as_sparse_error", [&] {
    Fixture fx = synthetic(4, 2, 8, 16);
    RealMoeLayer layer = layer_from(fx);
    std::vector<float> x = seeded(5, 3 * 8);
    x[8 + 2] = NAN;  // token 1
    auto r = layer.forward_auto(x);
    CHECK(r.is_err() && r.error().kind == MoeLayerError::Sparse &&
              r.error().sparse.kind == MoeSparseError::NonFiniteWeight, "kind");
    CHECK(r.error().sparse.token == 1 && r.error().sparse.index == 0, "token %zu index %zu", r.error().sparse.token,
          r.error().sparse.index);
    CHECK(r.error().to_string() == "moe-layer: moe-sparse: routing weight at 0 is non-finite", "%s",
          r.error().to_string().c_str());
    CHECK(layer.forward_auto(seeded(5, 8)).is_ok(), "the handle must stay usable after an error");
  });
  // ResidentExpertLayer::forward == RealMoeLayer::forward_with under the resolved convention, with
  // the evidence the reference returns (src/moe/residency.rs:732-791); a resident layer shares the
  // registry with the RAM ones and is invisible to get_real_moe_layer (graph_op.rs:234-247, 294-299).
  run_test("resident_expert_layer_equals_real_layer_and_registers", [&] {
    RealMoeLayer real = layer_from(*q15);  // shared expert + sigmoid gate => HuggingFaceQwen
    auto res = std::make_shared<ResidentExpertLayer>(ResidentExpertLayer::from_real_layer(real));
    CHECK(res->convention == MoeExecutionConvention::HuggingFaceQwen && res->tier == ExpertTier::Hbm, "resolved");
    CHECK(res->num_experts() == real.num_experts(), "experts");
    auto want = real.forward_with(q15->input, real.resolve_convention()).unwrap();
    auto got = res->forward(q15->input).unwrap();
    CHECK(got.first == want, "resident forward differs from the RAM layer's");
    std::vector<int32_t> idx;
    real.route(q15->input, real.resolve_convention(), &idx).unwrap();
    CHECK(got.second.materialized_experts.size() == idx.size(), "k experts reported");
    for (size_t i = 0; i < idx.size(); ++i) {
      CHECK(got.second.materialized_experts[i] == (size_t)idx[i], "expert %zu", i);
      CHECK(i == 0 || idx[i] > idx[i - 1], "ascending");
    }
    const size_t d = real.config.d_model, f = real.config.d_ff, fs = real.shared->d_ff;
    CHECK(got.second.materialized_bytes == idx.size() * 3 * d * f * 4 + 3 * d * fs * 4, "bytes %zu",
          got.second.materialized_bytes);
    // hf_ref of the fixture through the resident layer as well
    CHECK(metrics(got.first, q15->hf_ref).max_abs_diff <= 1e-5, "hf_ref: %g",
          metrics(got.first, q15->hf_ref).max_abs_diff);
    // a row of the wrong length is the dense DimMismatch of the reference's forward
    auto bad = res->forward(std::vector<float>(d + 1, 0.f));
    CHECK(bad.is_err() && bad.error().kind == MoeLayerError::Binding, "wrong length refused");
    // batch of rows == row by row, infos per row
    std::vector<float> xb = q15->input;
    auto x2 = seeded(91, d);
    xb.insert(xb.end(), x2.begin(), x2.end());
    std::vector<ResidencyInfo> infos;
    auto yb = res->forward_batch(xb, &infos).unwrap();
    auto y2 = res->forward(x2).unwrap();
    CHECK(infos.size() == 2 && std::equal(y2.first.begin(), y2.first.end(), yb.begin() + d), "batch rows");
    CHECK(infos[1].materialized_experts == y2.second.materialized_experts, "row evidence");
    const uint32_t id = register_resident_moe_layer(res, 4);
    CHECK(execute_real_moe_layer(id, q15->input).unwrap() == want, "graph op on a resident id");
    CHECK(get_real_moe_layer(id) == nullptr, "a resident id is not a RealMoeLayer");
    CHECK(moe_real_layer_reference_node(id, xb) == yb, "executor arm, flat batch");
  });
  run_test("bf16_and_int8_storage_track_f32", [&] {
    auto f32 = layer_from(*mix).forward_auto(mix->input).unwrap();
    double scale = 0;
    for (float v : mix->atenia_ref) scale = std::max(scale, (double)std::fabs(v));
    auto b16 = layer_from(*mix, MoeWeightStorage::Bf16).forward_auto(mix->input).unwrap();
    auto i8 = layer_from(*mix, MoeWeightStorage::Int8W8A16).forward_auto(mix->input).unwrap();
    CHECK(metrics(b16, f32).max_abs_diff <= 3e-2 * scale, "bf16 storage: %g of %g", metrics(b16, f32).max_abs_diff, scale);
    CHECK(metrics(i8, f32).max_abs_diff <= 3e-2 * scale, "int8 storage: %g of %g", metrics(i8, f32).max_abs_diff, scale);
    auto i8g = layer_from(*mix, MoeWeightStorage::Int8PerGroup).forward_auto(mix->input).unwrap();
    CHECK(metrics(i8g, f32).max_abs_diff <= 3e-2 * scale, "per-group int8 storage: %g of %g",
          metrics(i8g, f32).max_abs_diff, scale);
  });
  printf("%d tests, %d failed\n", g_run, g_failed);
  return g_failed ? 1 : 0;
}
