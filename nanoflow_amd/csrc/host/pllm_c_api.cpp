// Flat C ABI over the C++ control plane (include/nanoflow_pllm.h).
#include "nanoflow_pllm.h"

#include <cstdarg>
#include <cstring>

#include "computeBound.h"

static thread_local char g_err[512] = "";
static int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  std::vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

static int g_nranks = 1, g_vnranks = 1;
static bool g_config_loaded = false, g_inited = false, g_configured = false, g_updated = false;
static bool g_running = false;
static std::vector<vortexInitData> g_init(1);
static std::vector<vortexOutputData> g_out(1);
static std::vector<vortexConfigData> g_cfg(1);
static std::vector<vortexUpdateData> g_upd(1);

static vortexWeight to_cpp(const nf_vortex_weight& w) {
  vortexWeight r;
  r.ptr = w.ptr;
  r.N = w.N;
  r.K = w.K;
  return r;
}
static nf_vortex_weight to_c(const vortexWeight& w) { return nf_vortex_weight{w.ptr, w.N, w.K}; }

static vortexModelWeight to_cpp(const nf_vortex_model_weight& m) {
  vortexModelWeight r;
  r.lm_head = to_cpp(m.lm_head);
  r.embedding = to_cpp(m.embedding);
  r.model_layernorm = to_cpp(m.model_layernorm);
  r.layer_weight.resize(m.num_layers);
  for (int i = 0; i < m.num_layers; ++i) {
    const auto& s = m.layer_weight[i];
    auto& t = r.layer_weight[i];
    t.W_O1 = to_cpp(s.W_O1); t.W_O2 = to_cpp(s.W_O2); t.W_U = to_cpp(s.W_U); t.W_G = to_cpp(s.W_G);
    t.W_D = to_cpp(s.W_D); t.W_KQV = to_cpp(s.W_KQV); t.B_KQV = to_cpp(s.B_KQV);
    t.W_LN_Attention = to_cpp(s.W_LN_Attention); t.W_LN_FFN = to_cpp(s.W_LN_FFN);
    t.W_ROT = to_cpp(s.W_ROT);
  }
  return r;
}

extern "C" {

const char* pllm_last_error(void) { return g_err; }

int pllm_set_model_config(const char* json_path) {
  if (!json_path) return fail(NF_PLLM_ERR_INVALID_ARGUMENT, "pllm_set_model_config: null path");
  if (g_inited) return fail(NF_PLLM_ERR_STATE, "pllm_set_model_config: pipeline already initialised");
  if (!updateVortexModelConfig(json_path))
    return fail(NF_PLLM_ERR_INVALID_ARGUMENT, "pllm_set_model_config: cannot load %s", json_path);
  const auto& c = ModelConfig;
  if (c.gpu_num != 1)
    return fail(NF_PLLM_ERR_UNSUPPORTED, "model_configs.gpu_num=%d: this build runs one GPU", c.gpu_num);
  if (c.model_head_dim != 128 || c.frame_page_size != 16)
    return fail(NF_PLLM_ERR_UNSUPPORTED, "head_dim=%d page_size=%d: kernels are built for 128 / 16",
                c.model_head_dim, c.frame_page_size);
  if (c.model_hidden_dim % 8 || c.model_ff_dim % 8 || c.vocab_size % 8 || c.run_layer < 1 ||
      c.model_layer < 1)
    return fail(NF_PLLM_ERR_INVALID_ARGUMENT, "hidden/ffn/vocab must be multiples of 8, layers >= 1");
  g_config_loaded = true;
  return NF_PLLM_OK;
}

int pllm_set_rank(int nranks, int vnranks) {
  if (nranks != 1 || vnranks != 1)
    return fail(NF_PLLM_ERR_UNSUPPORTED, "pllm_set_rank(%d, %d): this build runs exactly one rank",
                nranks, vnranks);
  g_nranks = nranks;
  g_vnranks = vnranks;
  return NF_PLLM_OK;
}

size_t pllm_tmp_buffer_halves(void) { return ModelConfig.k_temp_size; }
size_t pllm_max_page_num(void) { return ModelConfig.max_page_num; }

int pllm_init(const nf_vortex_init_data* input, int pipeline_type) {
  if (!g_config_loaded) return fail(NF_PLLM_ERR_STATE, "pllm_init: call pllm_set_model_config first");
  if (g_inited) return fail(NF_PLLM_ERR_STATE, "pllm_init: already initialised");
  if (!input || !input->kv_data || !input->tmp_buffer || !input->weight.layer_weight)
    return fail(NF_PLLM_ERR_INVALID_ARGUMENT, "pllm_init: null pointer in init data");
  if (pipeline_type < 0 || pipeline_type > NF_PIPE_NANOBATCH_LOCAL)
    return fail(NF_PLLM_ERR_INVALID_ARGUMENT, "pllm_init: unknown pipeline type %d", pipeline_type);
  auto ty = static_cast<Worker::PipelineType>(pipeline_type);
  if (!Worker::isSupported(ty)) return fail(NF_PLLM_ERR_UNSUPPORTED, "pllm_init: unknown pipeline type %d", pipeline_type);
  if (getWeightFormat() == WeightFormat::E4M3 && Worker::hasKQVBias(ty))
    return fail(NF_PLLM_ERR_UNSUPPORTED, "pllm_init: the QKV bias pipelines take fp16 weights only");
  if (input->weight.num_layers < ModelConfig.model_layer)
    return fail(NF_PLLM_ERR_INVALID_ARGUMENT, "pllm_init: %d layers of weights, model has %d",
                input->weight.num_layers, ModelConfig.model_layer);
  if (Worker::hasKQVBias(ty))
    for (int i = 0; i < ModelConfig.model_layer; ++i) {
      const nf_vortex_weight& b = input->weight.layer_weight[i].B_KQV;
      if (!b.ptr || (size_t)b.N * (size_t)b.K != (size_t)ModelConfig.kqv_n)
        return fail(NF_PLLM_ERR_INVALID_ARGUMENT,
                    "pllm_init: pipeline type %d adds a QKV bias; layer %d has B_KQV %d x %d, wants %d elements",
                    pipeline_type, i, b.N, b.K, ModelConfig.kqv_n);
    }
  vortexInitData d;
  d.kv_data = new half*[ModelConfig.model_layer];
  for (int i = 0; i < ModelConfig.model_layer; ++i) {
    if (!input->kv_data[i]) return fail(NF_PLLM_ERR_INVALID_ARGUMENT, "pllm_init: kv_data[%d] is null", i);
    d.kv_data[i] = input->kv_data[i];
  }
  d.weight = to_cpp(input->weight);
  d.weight_size = input->weight_size;
  d.tmp_buffer = input->tmp_buffer;
  d.tmp_buffer_size = input->tmp_buffer_size;
  g_init[0] = d;
  g_out[0] = vortexOutputData();
  HIP_CHECK(hipSetDevice(0));
  TensorManager::getInstance().init(g_nranks, g_vnranks);
  init(g_nranks, g_vnranks, g_init, g_out, ty);
  g_inited = true;
  g_configured = g_updated = g_running = false;
  return NF_PLLM_OK;
}

static void layers_to_c(const vortexModelWeight& d, nf_vortex_model_weight* out, nf_vortex_layer_weight* layers) {
  out->lm_head = to_c(d.lm_head);
  out->embedding = to_c(d.embedding);
  out->model_layernorm = to_c(d.model_layernorm);
  out->num_layers = (int)d.layer_weight.size();
  out->layer_weight = layers;
  for (size_t i = 0; i < d.layer_weight.size(); ++i) {
    const auto& s = d.layer_weight[i];
    layers[i] = nf_vortex_layer_weight{to_c(s.W_O1), to_c(s.W_O2), to_c(s.W_U), to_c(s.W_G),
                                       to_c(s.W_D), to_c(s.W_KQV), to_c(s.B_KQV),
                                       to_c(s.W_LN_Attention), to_c(s.W_LN_FFN), to_c(s.W_ROT)};
  }
}

int pllm_create_model_weight(nf_vortex_model_weight* weight, nf_vortex_layer_weight* layers,
                             int layers_capacity) {
  if (!g_config_loaded) return fail(NF_PLLM_ERR_STATE, "pllm_create_model_weight: call pllm_set_model_config first");
  if (!weight || !layers || layers_capacity < ModelConfig.model_layer)
    return fail(NF_PLLM_ERR_INVALID_ARGUMENT, "pllm_create_model_weight: room for %d layers needed",
                ModelConfig.model_layer);
  vortexModelWeight d;
  createModelWeight(d, 0);
  layers_to_c(d, weight, layers);
  return NF_PLLM_OK;
}

int pllm_create_model_weight_host(nf_vortex_model_weight* weight, nf_vortex_layer_weight* layers,
                                  int layers_capacity) {
  if (!g_config_loaded)
    return fail(NF_PLLM_ERR_STATE, "pllm_create_model_weight_host: call pllm_set_model_config first");
  if (!weight || !layers || layers_capacity < ModelConfig.model_layer)
    return fail(NF_PLLM_ERR_INVALID_ARGUMENT, "pllm_create_model_weight_host: room for %d layers needed",
                ModelConfig.model_layer);
  vortexModelWeight h;
  createModelWeightCPU(h, 0);
  layers_to_c(h, weight, layers);
  return NF_PLLM_OK;
}

int pllm_num_layers(void) { return g_config_loaded ? ModelConfig.model_layer : 0; }

int pllm_create_init_data(nf_vortex_init_data* data, uint16_t** kv_data, int layers_capacity,
                          const nf_vortex_model_weight* weight) {
  if (!g_config_loaded) return fail(NF_PLLM_ERR_STATE, "pllm_create_init_data: call pllm_set_model_config first");
  if (!data || !kv_data || !weight || layers_capacity < ModelConfig.model_layer)
    return fail(NF_PLLM_ERR_INVALID_ARGUMENT, "pllm_create_init_data: room for %d layers needed",
                ModelConfig.model_layer);
  vortexInitData d;
  vortexModelWeight w = to_cpp(*weight);
  createInitData(d, w, 0);
  for (int i = 0; i < ModelConfig.model_layer; ++i) kv_data[i] = reinterpret_cast<uint16_t*>(d.kv_data[i]);
  delete[] d.kv_data;
  data->kv_data = kv_data;
  data->weight = *weight;
  data->weight_size = d.weight_size;
  data->tmp_buffer = reinterpret_cast<uint16_t*>(d.tmp_buffer);
  data->tmp_buffer_size = d.tmp_buffer_size;
  return NF_PLLM_OK;
}

int pllm_model_weight_to_gpu(const nf_vortex_model_weight* host_weight,
                             nf_vortex_model_weight* device_weight,
                             nf_vortex_layer_weight* device_layers) {
  if (!host_weight || !device_weight || !device_layers)
    return fail(NF_PLLM_ERR_INVALID_ARGUMENT, "pllm_model_weight_to_gpu: null pointer");
  vortexModelWeight h = to_cpp(*host_weight);
  vortexModelWeight d = modelWeightToGPU(h, 0);
  layers_to_c(d, device_weight, device_layers);
  return NF_PLLM_OK;
}

static bool four_way(int pipeline_type) {
  const auto t = static_cast<Worker::PipelineType>(pipeline_type);
  return Worker::isSupported(t) && Worker::isFourWay(t);
}

int pllm_check_nanobatch_split(int pipeline_type, int max_batch_size, int global_batch_size, int nanobatch_1_size,
                               int kqv1_size, int kqv3_size) {
  const auto t = static_cast<Worker::PipelineType>(pipeline_type);
  if (!Worker::isSupported(t)) return fail(NF_PLLM_ERR_INVALID_ARGUMENT, "pipeline type %d unknown", pipeline_type);
  if (global_batch_size <= 0 || global_batch_size > max_batch_size)
    return fail(NF_PLLM_ERR_INVALID_ARGUMENT, "pllm_config: global_batch_size %d not in (0, %d]", global_batch_size,
                max_batch_size);
  if (!Worker::isSequential(t) && (nanobatch_1_size <= 0 || nanobatch_1_size >= global_batch_size))
    return fail(NF_PLLM_ERR_INVALID_ARGUMENT, "pllm_config: nanobatch_1_size %d not in (0, %d)", nanobatch_1_size,
                global_batch_size);
  // the four-way schedule cuts each nano-batch once more for the QKV projection and attention
  if (four_way(pipeline_type)) {
    if (kqv1_size < 0 || kqv1_size > nanobatch_1_size)
      return fail(NF_PLLM_ERR_INVALID_ARGUMENT, "pllm_config: kqv1_size %d not in [0, nanobatch_1_size = %d]",
                  kqv1_size, nanobatch_1_size);
    if (kqv3_size < 0 || kqv3_size > global_batch_size - nanobatch_1_size)
      return fail(NF_PLLM_ERR_INVALID_ARGUMENT, "pllm_config: kqv3_size %d not in [0, %d] (nano-batch 2)", kqv3_size,
                  global_batch_size - nanobatch_1_size);
  }
  return NF_PLLM_OK;
}

int pllm_check_gemv_split(int pipeline_type, int nanobatch_1_size, int kqv1_size, int kqv3_size, int decode_rows,
                          const int32_t* g) {
  const auto t = static_cast<Worker::PipelineType>(pipeline_type);
  if (!Worker::isSupported(t)) return fail(NF_PLLM_ERR_INVALID_ARGUMENT, "pipeline type %d unknown", pipeline_type);
  if (!g) return fail(NF_PLLM_ERR_INVALID_ARGUMENT, "pllm_update: null gemv_batch_size");
  if (g[0] < 0 || g[1] < 0 || g[2] < 0 || g[3] < 0)
    return fail(NF_PLLM_ERR_INVALID_ARGUMENT, "pllm_update: negative gemv_batch_size");
  const long long gsum = (long long)g[0] + g[1] + g[2] + g[3];
  if (gsum != decode_rows)
    return fail(NF_PLLM_ERR_INVALID_ARGUMENT, "pllm_update: gemv_batch_size sums to %lld, decode requests %d", gsum,
                decode_rows);
  if (Worker::isSequential(t)) return NF_PLLM_OK;
  // decode groups 0 and 1 are the decode rows of nano-batch 1, groups 2 and 3 those of
  // nano-batch 2 (the O projection of nano-batch 1 waits for groups 0/1 only)
  const int want = std::min(decode_rows, nanobatch_1_size);
  if (g[0] + g[1] != want)
    return fail(NF_PLLM_ERR_INVALID_ARGUMENT,
                "pllm_update: decode groups 0+1 hold %d requests, nano-batch 1 has %d decode rows", g[0] + g[1], want);
  if (four_way(pipeline_type)) {
    // decode attention of group i starts once QKV piece i and its RoPE-append are done: the rows of
    // groups 0..i must lie inside QKV pieces 0..i, or the launch reads Q and KV rows not yet written
    if (g[0] > kqv1_size)
      return fail(NF_PLLM_ERR_INVALID_ARGUMENT, "pllm_update: decode group 0 holds %d requests, QKV piece 1 has %d rows",
                  g[0], kqv1_size);
    if (g[0] + g[1] + g[2] > nanobatch_1_size + kqv3_size)
      return fail(NF_PLLM_ERR_INVALID_ARGUMENT,
                  "pllm_update: decode groups 0..2 hold %d requests, QKV pieces 1..3 have %d rows", g[0] + g[1] + g[2],
                  nanobatch_1_size + kqv3_size);
  }
  return NF_PLLM_OK;
}

int pllm_config(const nf_vortex_config_data* c) {
  if (!g_inited) return fail(NF_PLLM_ERR_STATE, "pllm_config: call pllm_init first");
  if (g_configured) return fail(NF_PLLM_ERR_STATE, "pllm_config: already configured");
  if (!c) return fail(NF_PLLM_ERR_INVALID_ARGUMENT, "pllm_config: null config");
  if (int rc = pllm_check_nanobatch_split(static_cast<int>(Worker::PipeTy), ModelConfig.max_batch_size,
                                          c->global_batch_size, c->nanobatch_1_size, c->kqv1_size, c->kqv3_size))
    return rc;
  vortexConfigData d;
  for (int i = 0; i < c->num_gemm_op_tag; ++i) {
    GemmTag t;
    if (!c->gemm_op_tag[i] || !parseGemmTag(c->gemm_op_tag[i], t) ||
        t.layout_a != PllmLayout::ROW_MAJOR || t.layout_out != PllmLayout::ROW_MAJOR)
      return fail(NF_PLLM_ERR_INVALID_ARGUMENT, "pllm_config: bad GEMM tag %d: \"%s\"", i,
                  c->gemm_op_tag[i] ? c->gemm_op_tag[i] : "(null)");
    d.gemm_op_tag.push_back(c->gemm_op_tag[i]);
  }
  d.global_batch_size = c->global_batch_size;
  d.nanobatch_1_size = c->nanobatch_1_size;
  d.kqv1_size = c->kqv1_size;
  d.kqv3_size = c->kqv3_size;
  // tmp buffer must hold the schedule's intermediates (upper bound of the buffer plan)
  const size_t T = d.global_batch_size, H = ModelConfig.model_hidden_dim;
  const size_t need = T * ((size_t)ModelConfig.kqv_n + 8 * H + 2 * (size_t)ModelConfig.model_ff_dim +
                           ModelConfig.vocab_size + 8);
  if (g_init[0].tmp_buffer_size < need)
    return fail(NF_PLLM_ERR_INVALID_ARGUMENT, "pllm_config: tmp buffer has %zu halves, schedule needs %zu",
                g_init[0].tmp_buffer_size, need);
  g_cfg[0] = d;
  config(g_nranks, g_cfg);
  if (PipelineBase* p = currentPipeline(); p && !p->configError().empty())
    return fail(NF_PLLM_ERR_INVALID_ARGUMENT, "pllm_config: %s", p->configError().c_str());
  g_configured = true;
  return NF_PLLM_OK;
}

int pllm_update(const nf_vortex_update_data* u) {
  if (!g_configured) return fail(NF_PLLM_ERR_STATE, "pllm_update: call pllm_config first");
  if (g_running) return fail(NF_PLLM_ERR_STATE, "pllm_update: a run is in flight; call pllm_run_async_wait");
  if (!u || !u->input_indptr || !u->rev_input_indptr || !u->kv_indptr || !u->kv_indices ||
      !u->kv_last_page_len || !u->per_token_offset || !u->gemv_batch_size || !u->gemv_num_blocks ||
      (u->prefillTokensNum > 0 && !u->input_tokens) || (u->keepTokenListLength > 0 && !u->keep_token_list))
    return fail(NF_PLLM_ERR_INVALID_ARGUMENT, "pllm_update: null pointer in update data");
  const int T = g_cfg[0].global_batch_size;
  const int req = u->decodePrefillBorder + u->prefillNum;
  const int tok = u->decodePrefillBorder + u->prefillTokensNum;
  if (u->decodePrefillBorder < 0 || u->prefillNum < 0 || u->prefillTokensNum < 0 || tok > T || req > T ||
      tok < 1)
    return fail(NF_PLLM_ERR_INVALID_ARGUMENT, "pllm_update: %d requests / %d tokens do not fit batch %d",
                req, tok, T);
  if (u->input_indptr[req] != tok)
    return fail(NF_PLLM_ERR_INVALID_ARGUMENT, "pllm_update: input_indptr[%d]=%d but the batch has %d tokens",
                req, u->input_indptr[req], tok);
  if ((size_t)u->kv_indptr[req] > ModelConfig.max_page_num)
    return fail(NF_PLLM_ERR_INVALID_ARGUMENT, "pllm_update: %d pages in use, pool has %zu",
                u->kv_indptr[req], ModelConfig.max_page_num);
  if (int rc = pllm_check_gemv_split(static_cast<int>(Worker::PipeTy), g_cfg[0].nanobatch_1_size, g_cfg[0].kqv1_size,
                                     g_cfg[0].kqv3_size, u->decodePrefillBorder, u->gemv_batch_size))
    return rc;
  vortexUpdateData d;
  d.decodePrefillBorder = u->decodePrefillBorder;
  d.prefillNum = u->prefillNum;
  d.prefillTokensNum = u->prefillTokensNum;
  d.keepTokenListLength = u->keepTokenListLength;
  d.input_tokens = u->input_tokens;
  d.input_indptr = u->input_indptr;
  d.rev_input_indptr = u->rev_input_indptr;
  d.keep_token_list = u->keep_token_list;
  d.kv_indptr = u->kv_indptr;
  d.kv_indices = u->kv_indices;
  d.kv_last_page_len = u->kv_last_page_len;
  d.per_token_offset = u->per_token_offset;
  d.gemv_batch_size = u->gemv_batch_size;
  d.gemv_num_blocks = u->gemv_num_blocks;
  // kept slots + prefill tokens must add up to the batch rows
  int kept = 0;
  for (int i = 0; i < u->keepTokenListLength; ++i) kept += u->keep_token_list[i] == 1;
  if (kept != u->decodePrefillBorder)
    return fail(NF_PLLM_ERR_INVALID_ARGUMENT, "pllm_update: keep_token_list keeps %d slots, decode rows %d",
                kept, u->decodePrefillBorder);
  if (!aggregated_output.empty() && u->keepTokenListLength > (int)aggregated_output.size())
    return fail(NF_PLLM_ERR_INVALID_ARGUMENT, "pllm_update: keep list of %d over %zu previous outputs",
                u->keepTokenListLength, aggregated_output.size());
  g_upd[0] = d;
  update(g_nranks, g_upd);
  g_updated = true;
  return NF_PLLM_OK;
}

int pllm_run_async(void) {
  if (!g_updated) return fail(NF_PLLM_ERR_STATE, "pllm_run_async: call pllm_update first");
  if (g_running) return fail(NF_PLLM_ERR_STATE, "pllm_run_async: a run is already in flight");
  run_async();
  g_running = true;
  return NF_PLLM_OK;
}

int pllm_run_async_wait(void) {
  if (!g_running) return fail(NF_PLLM_ERR_STATE, "pllm_run_async_wait: no run in flight");
  run_async_wait();
  g_running = false;
  return NF_PLLM_OK;
}

int pllm_run(void) {
  int rc = pllm_run_async();
  return rc ? rc : pllm_run_async_wait();
}

int pllm_get_pipeline_output(const int32_t** tokens, int* count) {
  if (!tokens || !count) return fail(NF_PLLM_ERR_INVALID_ARGUMENT, "pllm_get_pipeline_output: null pointer");
  *tokens = aggregated_output.data();
  *count = (int)aggregated_output.size();
  return NF_PLLM_OK;
}

int pllm_finalize(void) {
  if (g_running) pllm_run_async_wait();
  if (g_inited) finalize();
  g_inited = g_configured = g_updated = g_running = false;
  delete[] g_init[0].kv_data;
  g_init[0] = vortexInitData();
  return NF_PLLM_OK;
}

int pllm_build_input_tokens(const int32_t* prev_output, int prev_count, const int32_t* keep_token_list,
                            int keep_token_list_length, const int32_t* prefill_tokens,
                            int prefill_tokens_num, int32_t* out) {
  if ((keep_token_list_length > 0 && !keep_token_list) || (prefill_tokens_num > 0 && !prefill_tokens) || !out)
    return fail(NF_PLLM_ERR_INVALID_ARGUMENT, "pllm_build_input_tokens: null pointer");
  return buildInputTokens(prev_output, prev_count, keep_token_list, keep_token_list_length, prefill_tokens,
                          prefill_tokens_num, out);
}

int pllm_set_weight_format(int format) {
  if (g_inited) return fail(NF_PLLM_ERR_STATE, "pllm_set_weight_format: call it before pllm_init");
  if (format != NF_WEIGHTS_F16 && format != NF_WEIGHTS_E4M3)
    return fail(NF_PLLM_ERR_INVALID_ARGUMENT, "pllm_set_weight_format: unknown format %d", format);
  setWeightFormat(format == NF_WEIGHTS_E4M3 ? WeightFormat::E4M3 : WeightFormat::F16);
  return NF_PLLM_OK;
}

int pllm_get_weight_format(void) { return getWeightFormat() == WeightFormat::E4M3 ? NF_WEIGHTS_E4M3 : NF_WEIGHTS_F16; }

size_t pllm_e4m3_weight_bytes(int N, int K) {
  return N > 0 && K > 0 ? e4m3WeightBytes((size_t)N, (size_t)K) : 0;
}

size_t pllm_e4m3_weight_scale_offset(int N, int K) {
  return N > 0 && K > 0 ? e4m3WeightScaleOffset((size_t)N, (size_t)K) : 0;
}

int pllm_quantize_weight_e4m3(const uint16_t* w_f16, void* out, int N, int K, void* stream) {
  if (!w_f16 || !out || N <= 0 || K <= 0)
    return fail(NF_PLLM_ERR_INVALID_ARGUMENT, "pllm_quantize_weight_e4m3: bad argument");
  uint8_t* q = static_cast<uint8_t*>(out);
  if (nf_quantize_weight_e4m3(w_f16, q, reinterpret_cast<float*>(q + e4m3WeightScaleOffset((size_t)N, (size_t)K)), K, N,
                              stream) != 0)
    return fail(NF_PLLM_ERR_INVALID_ARGUMENT, "pllm_quantize_weight_e4m3: %s", nf_last_error());
  return NF_PLLM_OK;
}

int pllm_set_profiling_stride(int stride) {
  if (stride < 0) return fail(NF_PLLM_ERR_INVALID_ARGUMENT, "pllm_set_profiling_stride: %d", stride);
  PipelineBase::profile_stride_override = stride;
  return NF_PLLM_OK;
}

int pllm_set_profiling(int on) {
  setPipelineProfiling(on < 0 ? 0 : on > 2 ? 2 : on);
  return NF_PLLM_OK;
}

int pllm_set_graph_mode(int on) {
  if (g_running) return fail(NF_PLLM_ERR_STATE, "pllm_set_graph_mode: a run is in flight");
  setPipelineGraphMode(on != 0);
  return NF_PLLM_OK;
}

int pllm_get_graph_counters(long counters[3]) {
  PipelineBase* p = currentPipeline();
  if (!p || !counters) return fail(NF_PLLM_ERR_STATE, "pllm_get_graph_counters: no pipeline");
  p->graphCounters(counters);
  return NF_PLLM_OK;
}

int pllm_get_timings(nf_pipeline_timings* out) {
  PipelineBase* p = currentPipeline();
  if (!p || !out) return fail(NF_PLLM_ERR_STATE, "pllm_get_timings: no pipeline");
  const PipelineTimings& t = p->getTimings();
  out->iter_ms = t.iter_ms;
  out->decode_attn_ms = t.decode_attn_ms;
  out->decode_attn_launches = t.decode_attn_launches;
  out->prefill_attn_ms = t.prefill_attn_ms;
  out->prefill_attn_launches = t.prefill_attn_launches;
  out->gemm_ms = t.gemm_ms;
  out->gemm_launches = t.gemm_launches;
  out->gemm_flop = t.gemm_flop;
  out->layer_stride = t.layer_stride;
  return NF_PLLM_OK;
}

int pllm_reset_timings(void) {
  PipelineBase* p = currentPipeline();
  if (!p) return fail(NF_PLLM_ERR_STATE, "pllm_reset_timings: no pipeline");
  p->resetTimings();
  return NF_PLLM_OK;
}

int pllm_debug_buffer(const char* name, uint16_t** ptr, int* rows, int* cols) {
  PipelineBase* p = currentPipeline();
  if (!p || !g_configured || !name || !ptr || !rows || !cols)
    return fail(NF_PLLM_ERR_STATE, "pllm_debug_buffer: no configured pipeline");
  pllmTensor<half> t;
  if (auto* lp = dynamic_cast<LocalPipeline*>(p)) {
    if (!std::strcmp(name, "hidden")) t = lp->keepToken.input;
    else if (!std::strcmp(name, "logits")) t = lp->maxSampler.d_matrix;
  } else if (auto* pp = dynamic_cast<Pipeline*>(p)) {
    if (!std::strcmp(name, "hidden")) t = pp->keepToken.input;
    else if (!std::strcmp(name, "logits")) t = pp->maxSampler.d_matrix;
    // whole-iteration buffers (the nano-batch pieces are consecutive rows of them); they hold the
    // LAST layer's values once an iteration has run
    else if (!std::strcmp(name, "kqv")) t = pp->KQV_output;
    else if (!std::strcmp(name, "attn_out")) t = pp->gemvAggregateOutput;
    else if (!std::strcmp(name, "ln_attn") || !std::strcmp(name, "o_out") || !std::strcmp(name, "ln_ffn") ||
             !std::strcmp(name, "act")) {
      const pllmTensor<half> first = !std::strcmp(name, "ln_attn") ? pp->layerNormAttention1.getOutput()
                                     : !std::strcmp(name, "o_out") ? pp->O1->getD()
                                     : !std::strcmp(name, "ln_ffn") ? pp->dual1.getA()
                                                                    : pp->D1->getA();
      t = pllmTensor<half>(first.ptr, pp->KQV_output.dim1, first.dim2, PllmLayout::ROW_MAJOR);
    }
    else if (!std::strcmp(name, "offload_host") && pp->offloadKVCache)  // pinned host memory: what the last layer's round trip left
      t = pllmTensor<half>(pp->offloadKVCache, pp->offload_pages, ModelConfig.page_mem_size / sizeof(half), PllmLayout::ROW_MAJOR);
  } else if (auto* np = dynamic_cast<NonOverlapLocalPipeline*>(p)) {
    // the intermediates hold the LAST layer's values once an iteration has run
    if (!std::strcmp(name, "hidden")) t = np->keepToken.input;
    else if (!std::strcmp(name, "logits")) t = np->maxSampler.d_matrix;
    else if (!std::strcmp(name, "ln_attn")) t = np->KQV->getA();
    else if (!std::strcmp(name, "kqv")) t = np->KQV->getD();
    else if (!std::strcmp(name, "attn_out")) t = np->O->getA();
    else if (!std::strcmp(name, "o_out")) t = np->O->getD();
    else if (!std::strcmp(name, "ln_ffn")) t = np->dual.getA();
    else if (!std::strcmp(name, "act")) t = np->D->getA();
  }
  if (!t.ptr) return fail(NF_PLLM_ERR_INVALID_ARGUMENT, "pllm_debug_buffer: unknown buffer \"%s\"", name);
  *ptr = t.ptr;
  *rows = (int)t.dim1;
  *cols = (int)t.dim2;
  return NF_PLLM_OK;
}

}  // extern "C"

// ---------------------------------------------------------------- batch former / serve loop
#include "batchFormer.h"

struct nf_batch_former {
  BatchFormer former;
  FormedBatch batch;
  std::vector<FlyPtr> retired;
  int avg_prefill, avg_decode;
  nf_batch_former(int pages, int page, int gb, int n1, int k1, int k3, int ap, int ad)
      : former(pages, page, gb, n1, k1, k3, ap, ad), avg_prefill(ap), avg_decode(ad) {}
};

extern "C" {

nf_batch_former* pllm_sched_create(int kv_pages, int page_size, int global_batch_size,
                                   int nanobatch_1_size, int kqv1_size, int kqv3_size,
                                   int average_prefill_length, int average_decode_length) {
  if (kv_pages <= 0 || page_size <= 0 || global_batch_size <= 0 || nanobatch_1_size < 0 ||
      kqv1_size < 0 || kqv1_size > nanobatch_1_size || kqv3_size < 0 || average_prefill_length < 0 ||
      average_decode_length < 0) {
    fail(NF_PLLM_ERR_INVALID_ARGUMENT, "pllm_sched_create: bad sizes");
    return nullptr;
  }
  return new nf_batch_former(kv_pages, page_size, global_batch_size, nanobatch_1_size, kqv1_size,
                             kqv3_size, average_prefill_length, average_decode_length);
}

void pllm_sched_destroy(nf_batch_former* f) { delete f; }

int pllm_sched_add_request(nf_batch_former* f, int req_idx, const int32_t* prompt, int prompt_len,
                           int output_len, double start_time) {
  if (!f || !prompt || prompt_len <= 0 || output_len <= 0)
    return fail(NF_PLLM_ERR_INVALID_ARGUMENT, "pllm_sched_add_request: bad request");
  SchedRequest r;
  r.req_idx = req_idx;
  r.prompt.assign(prompt, prompt + prompt_len);
  r.output_len = output_len;
  r.start_time = start_time;
  f->former.add_request(std::move(r));
  return NF_PLLM_OK;
}

int pllm_sched_schedule(nf_batch_former* f) {
  if (!f) return fail(NF_PLLM_ERR_INVALID_ARGUMENT, "pllm_sched_schedule: null");
  try {
    f->former.schedule();
  } catch (const std::exception& e) {
    return fail(NF_PLLM_ERR_STATE, "pllm_sched_schedule: %s", e.what());
  }
  return NF_PLLM_OK;
}

int pllm_sched_form(nf_batch_former* f, nf_vortex_update_data* out) {
  if (!f || !out) return fail(NF_PLLM_ERR_INVALID_ARGUMENT, "pllm_sched_form: null");
  try {
    f->former.form(f->batch);
  } catch (const std::exception& e) {
    return fail(NF_PLLM_ERR_STATE, "pllm_sched_form: %s", e.what());
  }
  FormedBatch& b = f->batch;
  out->decodePrefillBorder = b.decodePrefillBorder;
  out->prefillNum = b.prefillNum;
  out->prefillTokensNum = b.prefillTokensNum;
  out->keepTokenListLength = b.keepTokenListLength;
  out->input_tokens = b.input_tokens.data();
  out->input_indptr = b.input_indptr.data();
  out->rev_input_indptr = b.rev_input_indptr.data();
  out->keep_token_list = b.keep_token_list.data();
  out->kv_indptr = b.kv_indptr.data();
  out->kv_indices = b.kv_indices.data();
  out->kv_last_page_len = b.kv_last_page_len.data();
  out->per_token_offset = b.per_token_offset.data();
  out->gemv_batch_size = b.gemv_batch_size;
  out->gemv_num_blocks = b.gemv_num_blocks;
  return NF_PLLM_OK;
}

int pllm_sched_harvest(nf_batch_former* f, const int32_t* ids, int n) {
  if (!f || (n > 0 && !ids)) return fail(NF_PLLM_ERR_INVALID_ARGUMENT, "pllm_sched_harvest: null");
  f->former.harvest(ids, n);
  return NF_PLLM_OK;
}

int pllm_sched_advance(nf_batch_former* f, double now, int placeholder_zero, int* n_retired) {
  if (!f) return fail(NF_PLLM_ERR_INVALID_ARGUMENT, "pllm_sched_advance: null");
  const size_t before = f->retired.size();
  f->former.advance(now, f->retired, placeholder_zero != 0);
  if (n_retired) *n_retired = (int)(f->retired.size() - before);
  return NF_PLLM_OK;
}

int pllm_sched_state(nf_batch_former* f, int counts[5]) {
  if (!f || !counts) return fail(NF_PLLM_ERR_INVALID_ARGUMENT, "pllm_sched_state: null");
  counts[0] = (int)f->former.queued();
  counts[1] = (int)f->former.decoding();
  counts[2] = (int)f->former.prefilling();
  counts[3] = f->former.pool().num_free_pages();
  counts[4] = (int)f->retired.size();
  return NF_PLLM_OK;
}

int pllm_sched_retired_output(nf_batch_former* f, int which, int* req_idx, int32_t* out, int cap) {
  if (!f || which < 0 || which >= (int)f->retired.size() || (cap > 0 && !out))
    return fail(NF_PLLM_ERR_INVALID_ARGUMENT, "pllm_sched_retired_output: bad index %d", which);
  const FlyRequest& r = *f->retired[which];
  if (req_idx) *req_idx = r.req_idx;
  const int n = std::min<int>(cap, (int)r.output.size());
  for (int i = 0; i < n; ++i) out[i] = r.output[i];
  return n;
}

int pllm_sched_retired_info(nf_batch_former* f, int which, int* req_idx, int* input_len, int* output_len,
                            double times[4]) {
  if (!f || which < 0 || which >= (int)f->retired.size())
    return fail(NF_PLLM_ERR_INVALID_ARGUMENT, "pllm_sched_retired_info: bad index %d", which);
  const FlyRequest& r = *f->retired[which];
  if (req_idx) *req_idx = r.req_idx;
  if (input_len) *input_len = r.input_len;
  if (output_len) *output_len = r.output_len;
  if (times) {
    times[0] = r.request_comein_time;
    times[1] = r.encode_latency;
    times[2] = r.decode_start_at;
    times[3] = r.decode_latency;
  }
  return NF_PLLM_OK;
}

int pllm_sched_future_page_usage(nf_batch_former* f, int64_t* out, int cap) {
  if (!f || (cap > 0 && !out)) return fail(NF_PLLM_ERR_INVALID_ARGUMENT, "pllm_sched_future_page_usage: null");
  std::vector<long long> u = f->former.future_page_usage();
  for (int i = 0; i < cap && i < (int)u.size(); ++i) out[i] = u[i];
  return (int)u.size();
}

int pllm_serve(nf_batch_former* f, int skip_cycles, int warmup_cycles, int run_cycles, nf_serve_stats* stats) {
  if (!f || !stats) return fail(NF_PLLM_ERR_INVALID_ARGUMENT, "pllm_serve: null");
  if (!g_configured) return fail(NF_PLLM_ERR_STATE, "pllm_serve: call pllm_init and pllm_config first");
  if (g_running) return fail(NF_PLLM_ERR_STATE, "pllm_serve: a run is in flight");
  ServeStats s;
  try {
    s = serveLoop(f->former, skip_cycles, warmup_cycles, run_cycles, &f->retired);
  } catch (const std::exception& e) {
    g_updated = false;
    return fail(NF_PLLM_ERR_STATE, "pllm_serve: %s", e.what());
  }
  stats->cycles = s.cycles;
  stats->retired = s.retired;
  stats->wall_s = s.wall_s;
  stats->tokens_per_s = s.wall_s > 0 ? s.retired * double(f->avg_prefill + f->avg_decode) / s.wall_s : 0;
  stats->cycle_ms = s.cycle_ms;
  stats->form_ms = s.form_ms;
  stats->wait_ms = s.wait_ms;
  stats->update_ms = s.update_ms;
  stats->gpu_iter_ms = s.gpu_iter_ms;
  stats->tokens_processed = s.tokens_processed;
  g_updated = false;
  return NF_PLLM_OK;
}

}  // extern "C"
