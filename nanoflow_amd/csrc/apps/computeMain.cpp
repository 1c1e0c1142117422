// test_compute: the C++ end-to-end entry of the pipeline, same command line and call sequence as
// the reference's pipeline/src/computeMain.cu (./test_compute [config_path] [runs]):
// model config -> weights (device memory, contents as allocated) -> init data (tmp buffer, KV
// pools) -> config data -> synthetic update data for an average prompt of 1024 and an average
// output of 512 tokens -> init, config, update, run x N, finalize.  Prints the wall time of each
// run and the number of sampled tokens, and exits non-zero when anything fails.
// An optional serve_configs.weight_format of "e4m3" in the config (not in the reference's schema)
// makes the weights and the pipeline use the fp8 form of the per-layer GEMM weights.
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <string>
#include <vector>

#include "computeBound.h"
#include "mini_json.h"

static bool pipeline_type_of(const std::string& name, Worker::PipelineType& out) {
  static const std::pair<const char*, Worker::PipelineType> table[] = {
      {"LOCAL", Worker::PipelineType::LOCAL},
      {"PLLM", Worker::PipelineType::PLLM},
      {"NON_OVERLAP", Worker::PipelineType::NONOVERLAP},
      {"NANOBATCH", Worker::PipelineType::NANOBATCH},
      {"PLLM_OFFLOAD", Worker::PipelineType::PLLMOFFLOAD},
      {"NON_OVERLAP_LOCAL", Worker::PipelineType::NON_OVERLAP_LOCAL},
      {"NANOBATCH_LOCAL", Worker::PipelineType::NANOBATCH_LOCAL},
      {"KQVBIAS", Worker::PipelineType::KQVBIAS},
      {"NONOVERLAP_KQVBIAS", Worker::PipelineType::NONOVERLAP_KQVBIAS},
      {"NANOBATCH_KQVBIAS", Worker::PipelineType::NANOBATCH_KQVBIAS},
  };
  for (const auto& e : table)
    if (name == e.first) {
      out = e.second;
      return true;
    }
  return false;
}

int main(int argc, char** argv) {
  if (argc < 2) {
    std::fprintf(stderr, "usage: %s config_path [runs]\n", argv[0]);
    return 2;
  }
  const std::string config_path = argv[1];
  const int runs = argc >= 3 ? std::atoi(argv[2]) : 5;
  int nranks = 1, vnranks = 1, global_batch_size = 0;
  std::string pipe_name;
  try {
    const mini_json::Value j = mini_json::parse_file(config_path);
    nranks = j.at("serve_configs").value<int>("actual_gpu_num", 1);
    vnranks = j.at("model_configs").value<int>("gpu_num", 1);
    global_batch_size = j.at("pipeline_configs").value<int>("global_batch_size", 0);
    pipe_name = j.at("serve_configs").at("pipeline_type").str;
    const auto& sc = j.at("serve_configs");
    const std::string fmt = sc.contains("weight_format") ? sc.at("weight_format").str : std::string("f16");
    if (fmt != "f16" && fmt != "e4m3") {
      std::fprintf(stderr, "unknown weight_format %s\n", fmt.c_str());
      return 2;
    }
    setWeightFormat(fmt == "e4m3" ? WeightFormat::E4M3 : WeightFormat::F16);
  } catch (const std::exception& e) {
    std::fprintf(stderr, "%s: %s\n", config_path.c_str(), e.what());
    return 2;
  }
  Worker::PipelineType pipe;
  if (!pipeline_type_of(pipe_name, pipe)) {
    std::fprintf(stderr, "unknown pipeline type %s\n", pipe_name.c_str());
    return 2;
  }
  if (nranks != 1 || vnranks != 1 || !Worker::isSupported(pipe)) {
    std::fprintf(stderr, "this build runs every pipeline type on ONE GPU (got %s, %d ranks, gpu_num %d)\n",
                 pipe_name.c_str(), nranks, vnranks);
    return 2;
  }

  TensorManager::getInstance().init(nranks, vnranks);
  if (!updateVortexModelConfig(config_path)) {
    std::fprintf(stderr, "cannot load the model configuration from %s\n", config_path.c_str());
    return 2;
  }
  std::vector<vortexInitData> input(nranks);
  std::vector<vortexOutputData> output(nranks);
  std::vector<vortexConfigData> config_data(nranks);
  std::vector<vortexUpdateData> update_data(nranks);
  std::vector<vortexModelWeight> weights(nranks);
  for (int rank = 0; rank < nranks; ++rank) {
    createModelWeight(weights[rank], rank);
    createInitData(input[rank], weights[rank], rank);
    if (!readConfigData(config_data[rank], rank, config_path)) return 2;
    createUpdateData(update_data[rank], rank, global_batch_size, 1024, 512);
  }
  std::printf("pipeline %s, %d tokens per iteration (%d decode requests, %d prefill requests with %d tokens)\n",
              pipe_name.c_str(), update_data[0].decodePrefillBorder + update_data[0].prefillTokensNum,
              update_data[0].decodePrefillBorder, update_data[0].prefillNum, update_data[0].prefillTokensNum);

  Worker::PipeTy = pipe;
  init(nranks, vnranks, input, output, pipe);
  config(nranks, config_data);
  update(nranks, update_data);
  for (int i = 0; i < runs; ++i) {
    const auto t0 = std::chrono::steady_clock::now();
    run();
    const double ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
    std::printf("run %d: %.3f ms, %zu sampled tokens\n", i, ms, aggregated_output.size());
  }
  finalize();
  return 0;
}
