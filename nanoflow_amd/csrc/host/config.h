// Global model configuration, filled from the pipeline JSON file.
// Field names and derivations follow the reference's vortexModelConfig
// (pipeline/include/config.h:10-142, pipeline/src/load_config.cu:11-112).  One difference on
// purpose: max_page_num is the size of the KV pool that is actually allocated per layer
// (allocate_kv_data_batch requests x 1024 tokens), not a figure derived from a fixed
// 64 GiB as at config.h:97-99, so it scales with the 288 GB of an MI355X.
#pragma once
#include <algorithm>
#include <cmath>
#include <cstddef>
#include <string>

struct vortexModelConfig {
  int gpu_num = 1;
  int model_layer = 32;
  int run_layer = 32;
  int allocate_kv_data_batch = 400;  // requests of 1024 tokens the KV pool is sized for

  int model_head_dim = 128;
  int model_gqa = 4;
  int model_kv_heads = 8;
  int model_qo_heads = 32;
  int model_kv_heads_gpu = 8;
  int model_qo_heads_gpu = 32;
  int model_ff_dim = 14336;
  int model_ff_dim_gpu = 14336;
  int ug_n = 28672;
  int model_hidden_dim = 4096;
  int model_hidden_dim_pergpu = 4096;
  int kqv_n = 6144;
  int frame_page_size = 16;
  int max_batch_size = 2048;
  float rms_norm_eps = 1e-5f;

  float rope_theta = 1e4f;
  float factor = 1.0f;
  float low_freq_factor = 1.0f;
  float high_freq_factor = 4.0f;
  int original_max_position_embeddings = 8192;
  float smooth_a = 0;
  float smooth_b = 0;
  bool rope_3_1 = false;

  size_t vocab_size = 32000;

  size_t page_mem_size = 0;  // bytes of one page (K and V)
  size_t max_page_num = 0;   // pages per layer pool
  size_t k_temp_size = 0;    // halves in the tmp buffer

  void calculateConfig() {
    model_kv_heads_gpu = model_kv_heads / gpu_num;
    model_qo_heads_gpu = model_qo_heads / gpu_num;
    model_ff_dim_gpu = model_ff_dim / gpu_num;
    ug_n = model_ff_dim_gpu * 2;
    model_hidden_dim_pergpu = model_hidden_dim / gpu_num;
    kqv_n = model_hidden_dim_pergpu + 2 * model_hidden_dim_pergpu / model_gqa;
    page_mem_size = (size_t)frame_page_size * model_kv_heads_gpu * model_head_dim * 2 * 2;
    max_page_num = (size_t)allocate_kv_data_batch * ((1024 + frame_page_size - 1) / frame_page_size);
    // the reference's figure (config.h:100) plus room for the FFN activation rows, which it only
    // covers when the vocabulary term is large
    k_temp_size = (size_t)max_batch_size * model_hidden_dim * 16 + (size_t)max_batch_size * vocab_size * 2 +
                  (size_t)max_batch_size * model_ff_dim + 65536;
    // quantised activations of the fp8-weight GEMMs (one byte per element of the QKV, O, gate/up
    // and down inputs, a scale per row, 256-byte alignment of up to 8 wrappers)
    k_temp_size += (size_t)max_batch_size * (3 * model_hidden_dim + model_ff_dim + 32) / 2 + 8 * 256;
    // the same form of the two RMSNorm outputs, written by the RMSNorms themselves (a byte per
    // element, a scale per row, per nano-batch piece)
    k_temp_size += (size_t)max_batch_size * (2 * model_hidden_dim + 8) / 2 + 12 * 256;
    // fp32 partial sums of GEMM launches split over K: shares x M x N is at most CUs x the largest
    // split tile (256 x 256 x 256 elements = 67 MB) per wrapper, up to 7 wrappers, 256-byte
    // alignment (the fused gate/up pair keeps two sets of sums of 128 x 128 tiles, 34 MB together,
    // for up to 2 of its wrappers)
    k_temp_size += (size_t)(7 + 2) * ((size_t)256 * 65536 * 2 + 128);
    // ... and 84 MB for each of the pair's wrappers from 257 to 320 rows (two sets of sums of
    // 320 x 128 tiles)
    k_temp_size += (size_t)2 * ((size_t)256 * 320 * 128 * 2 * 2 - (size_t)256 * 65536 * 2);
    if (!rope_3_1) {
      smooth_a = 0;
      smooth_b = 0;
    } else {
      smooth_a = original_max_position_embeddings /
                 (2 * M_PI * high_freq_factor - 2 * M_PI * low_freq_factor);
      smooth_b = -1.0f / (high_freq_factor / low_freq_factor - 1.0f);
    }
  }
  void printConfig() const;
};

extern vortexModelConfig ModelConfig;
// Reads the "model" and "model_configs" blocks of a pipeline JSON into ModelConfig.
// Returns false (and leaves ModelConfig untouched) when the file cannot be read or parsed.
bool updateVortexModelConfig(const std::string& filename);
