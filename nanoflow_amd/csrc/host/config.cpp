#include "config.h"

#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <iostream>

#include "helper.h"
#include "mini_json.h"

vortexModelConfig ModelConfig;

namespace nflog {
int level() {
  static int lvl = [] {
    const char* v = std::getenv("NANOFLOW_LOG");
    if (!v) return (int)WARN;
    if (!std::strcmp(v, "trace")) return (int)TRACE;
    if (!std::strcmp(v, "info")) return (int)INFO;
    if (!std::strcmp(v, "warn")) return (int)WARN;
    if (!std::strcmp(v, "error")) return (int)ERROR;
    if (!std::strcmp(v, "off")) return (int)OFF;
    return (int)WARN;
  }();
  return lvl;
}
void write(Level lvl, const char* fmt, ...) {
  static const char* names[] = {"trace", "info", "warn", "error"};
  char buf[1024];
  va_list ap;
  va_start(ap, fmt);
  std::vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  std::fprintf(stderr, "[nanoflow] [%s] %s\n", names[lvl], buf);
}
}  // namespace nflog

void vortexModelConfig::printConfig() const {
  std::cout << "GPU_NUM: " << gpu_num << "\nMODEL_LAYER: " << model_layer << "\nRUN_LAYER: " << run_layer
            << "\nALLOCATE_KV_DATA_BATCH: " << allocate_kv_data_batch
            << "\nMODEL_HEAD_DIM: " << model_head_dim << "\nMODEL_GQA: " << model_gqa
            << "\nMODEL_KV_HEADS: " << model_kv_heads << "\nMODEL_QO_HEADS: " << model_qo_heads
            << "\nMODEL_FF_DIM: " << model_ff_dim << "\nMODEL_HIDDEN_DIM: " << model_hidden_dim
            << "\nKQV_N: " << kqv_n << "\nFRAME_PAGE_SIZE: " << frame_page_size
            << "\nMAX_BATCH_SIZE: " << max_batch_size << "\nVOCABULARY_SIZE: " << vocab_size
            << "\nPAGE_MEM_SIZE: " << page_mem_size << "\nMAX_PAGE_NUM: " << max_page_num
            << "\nROPE_THETA: " << rope_theta << "\nFACTOR: " << factor
            << "\nRMS_NORM_EPS: " << rms_norm_eps << "\nK_TEMP_SIZE: " << k_temp_size
            << "\nSMOOTH_A: " << smooth_a << "\nSMOOTH_B: " << smooth_b << std::endl;
}

bool updateVortexModelConfig(const std::string& filename) {
  mini_json::Value j;
  try {
    j = mini_json::parse_file(filename);
  } catch (const std::exception& e) {
    std::cerr << e.what() << std::endl;
    return false;
  }
  try {
    const auto& model = j.at("model");
    vortexModelConfig c;
    c.model_hidden_dim = (int)model.at("hidden_size").number();
    c.model_qo_heads = (int)model.at("num_attention_heads").number();
    c.model_kv_heads = (int)model.at("num_key_value_heads").number();
    c.model_ff_dim = (int)model.at("intermediate_size").number();
    c.model_layer = (int)model.at("num_hidden_layers").number();
    c.rms_norm_eps = (float)model.at("rms_norm_eps").number();
    c.vocab_size = (size_t)model.at("vocab_size").number();
    c.rope_theta = model.value<float>("rope_theta", 10000.0f);
    if (model.contains("rope_scaling") && !model.at("rope_scaling").is_null()) {
      const auto& rs = model.at("rope_scaling");
      c.rope_3_1 = true;
      c.factor = (float)rs.at("factor").number();
      c.low_freq_factor = (float)rs.at("low_freq_factor").number();
      c.high_freq_factor = (float)rs.at("high_freq_factor").number();
      c.original_max_position_embeddings = (int)rs.at("original_max_position_embeddings").number();
    } else {
      c.rope_3_1 = false;
      c.factor = 1.0f;
    }
    static const mini_json::Value empty_obj = [] {
      mini_json::Value v;
      v.kind = mini_json::Value::Object;
      return v;
    }();
    const auto& mc = j.contains("model_configs") ? j.at("model_configs") : empty_obj;
    c.gpu_num = mc.value<int>("gpu_num", 1);
    c.run_layer = mc.value<int>("run_layer", c.model_layer);
    c.allocate_kv_data_batch = mc.value<int>("allocate_kv_data_batch", 400);
    c.frame_page_size = mc.value<int>("frame_page_size", 16);
    c.max_batch_size = mc.value<int>("max_batch_size", 2048);
    c.model_head_dim = c.model_hidden_dim / c.model_qo_heads;
    c.model_gqa = c.model_qo_heads / c.model_kv_heads;
    c.calculateConfig();
    ModelConfig = c;
  } catch (const std::exception& e) {
    std::cerr << "config " << filename << ": " << e.what() << std::endl;
    return false;
  }
  if (nflog::level() <= nflog::INFO) ModelConfig.printConfig();
  return true;
}
