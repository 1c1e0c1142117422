#include "computeBound.h"

#include <pthread.h>
#include <sched.h>

#include <cstring>
#include <iostream>

std::vector<std::unique_ptr<Worker>> workers;
std::vector<vortexOutputData> outputs;
std::vector<int> aggregated_output;

struct SharedState {
  WorkerOp op = WorkerOp::STOP;
  std::vector<vortexUpdateData>* updates_ptr = nullptr;
  std::vector<vortexConfigData>* config_ptr = nullptr;
};
static SharedState shared_state;
static std::unique_ptr<SimpleThreadSync> global_sync;  // workers + the caller's thread
static vortexInitData* persistant_input = nullptr;
static std::vector<int> complete_input_tokens;
static int g_profiling = 0;
static WeightFormat g_weight_format = WeightFormat::F16;
void setWeightFormat(WeightFormat format) { g_weight_format = format; }
WeightFormat getWeightFormat() { return g_weight_format; }
static bool g_graph_mode = false;

int buildInputTokens(const int* prev_output, int prev_count, const int32_t* keep_token_list,
                     int keep_token_list_length, const int* prefill_tokens, int prefill_tokens_num,
                     int* out) {
  int n = 0;
  const bool first = prev_output == nullptr || prev_count == 0;
  for (int i = 0; i < keep_token_list_length; ++i)
    if (keep_token_list[i] == 1) out[n++] = first ? 1 : prev_output[i];
  for (int i = 0; i < prefill_tokens_num; ++i) out[n++] = prefill_tokens[i];
  return n;
}

void run_async() {
  shared_state.op = WorkerOp::RUN;
  global_sync->barrier();  // issue the command; the worker runs while the caller continues
}

void run_async_wait() {
  global_sync->barrier();  // wait for the worker to finish the command
  outputs.clear();
  for (auto& worker : workers) outputs.push_back(*worker->getOutput());
  aggregated_output.clear();
  for (auto& output : outputs)
    for (int i = 0; i < output.sampled_tokens; ++i)
      aggregated_output.push_back(output.sampled_token_array[i]);
}

void run() {
  run_async();
  run_async_wait();
}

void init(int nranks, int vnranks, std::vector<vortexInitData>& input,
          std::vector<vortexOutputData>& output, Worker::PipelineType pipeTy) {
  if (nranks != 1 || (int)input.size() != nranks || (int)output.size() != nranks) {
    std::fprintf(stderr, "init: this build runs exactly one rank (nranks=%d, inputs=%zu, outputs=%zu)\n",
                 nranks, input.size(), output.size());
    std::exit(EXIT_FAILURE);
  }
  if (!Worker::isSupported(pipeTy)) {
    std::fprintf(stderr, "init: unknown pipeline type %d\n", static_cast<int>(pipeTy));
    std::exit(EXIT_FAILURE);
  }
  if (!workers.empty()) {
    std::fprintf(stderr, "init: already initialised; call finalize() first\n");
    std::exit(EXIT_FAILURE);
  }
  if (g_weight_format == WeightFormat::E4M3 && Worker::hasKQVBias(pipeTy)) {
    std::fprintf(stderr, "init: the QKV bias pipelines take fp16 weights only\n");
    std::exit(EXIT_FAILURE);
  }
  Worker::PipeTy = pipeTy;
  // the update mirrors are sized from the model configuration: callers that follow the
  // reference's order (mirrors first, configuration second: computeMain.cu:37-38) get them
  // resized here; a no-op when they already fit
  TensorManager::getInstance().init(nranks, vnranks);
  aggregated_output.clear();
  outputs.clear();
  global_sync = std::make_unique<SimpleThreadSync>(nranks + 1);
  persistant_input = new vortexInitData[nranks];
  for (int i = 0; i < nranks; ++i) persistant_input[i] = input[i];
  for (int rank = 0; rank < nranks; ++rank) {
    workers.emplace_back(std::make_unique<Worker>(rank, nranks, vnranks, persistant_input + rank, &output[rank]))
        ->as_thread(-1);
  }
  global_sync->barrier();  // end of worker init
  NF_LOG_INFO("All multi-threading workers are initialized");
}

void update(int nranks, std::vector<vortexUpdateData>& updateData) {
  assert((int)updateData.size() == nranks);
  auto& update_d = updateData[0];
  // Checked before anything is written: the kept slots are the decode rows, and every kept slot
  // must have an output of the previous iteration to take its token from.
  int kept = 0;
  for (int i = 0; i < update_d.keepTokenListLength; ++i) kept += update_d.keep_token_list[i] == 1;
  const bool first = aggregated_output.empty();
  if (kept != update_d.decodePrefillBorder || update_d.prefillTokensNum < 0 ||
      (!first && update_d.keepTokenListLength > (int)aggregated_output.size())) {
    std::fprintf(stderr,
                 "update: keep list of %d entries keeps %d slots, the batch has %d decode rows and the previous "
                 "iteration produced %zu outputs\n",
                 update_d.keepTokenListLength, kept, update_d.decodePrefillBorder, aggregated_output.size());
    std::exit(EXIT_FAILURE);
  }
  complete_input_tokens.resize((size_t)kept + update_d.prefillTokensNum + 1);
  buildInputTokens(aggregated_output.data(), (int)aggregated_output.size(), update_d.keep_token_list,
                   update_d.keepTokenListLength, update_d.input_tokens, update_d.prefillTokensNum,
                   complete_input_tokens.data());
  for (int i = 0; i < nranks; ++i) updateData[i].input_tokens = complete_input_tokens.data();
  shared_state.op = WorkerOp::UPDATE;
  shared_state.updates_ptr = &updateData;
  global_sync->barrier();
  global_sync->barrier();
}

void config(int nranks, std::vector<vortexConfigData>& config) {
  assert((int)config.size() == nranks);
  shared_state.op = WorkerOp::CONFIG;
  shared_state.config_ptr = &config;
  global_sync->barrier();
  global_sync->barrier();
}

void finalize() {
  if (workers.empty()) return;
  shared_state.op = WorkerOp::STOP;
  global_sync->barrier();
  global_sync->barrier();
  workers.clear();
  delete[] persistant_input;
  persistant_input = nullptr;
}

PipelineBase* currentPipeline() { return workers.empty() ? nullptr : workers[0]->getPipeline(); }

void setPipelineGraphMode(bool on) {
  g_graph_mode = on;
  if (auto* p = currentPipeline()) p->setGraphMode(on);
}

void setPipelineProfiling(int level) {
  g_profiling = level;
  if (auto* p = currentPipeline()) p->setProfiling(level);
}

Worker::PipelineType Worker::PipeTy = Worker::PipelineType::LOCAL;

void Worker::as_thread(int core) {
  thread = std::make_unique<std::thread>(&Worker::thread_entry, this);
  if (core >= 0) {  // the reference pins workers to fixed cores; optional here
    cpu_set_t cpuSet;
    CPU_ZERO(&cpuSet);
    CPU_SET(core, &cpuSet);
    int result = pthread_setaffinity_np(thread->native_handle(), sizeof(cpuSet), &cpuSet);
    if (result != 0) std::cerr << "Error setting thread affinity: " << strerror(result) << std::endl;
  }
}

void Worker::init() {
  HIP_CHECK(hipSetDevice(rank));
  // Type -> schedule as the reference maps them (pipeline/src/computeBound.cu:234-247): the five
  // types of its main Pipeline run the four-way nano-batch schedule, without their exchange steps.
  const bool bias = hasKQVBias(PipeTy);
  if (isFourWay(PipeTy))
    pipeline = std::make_unique<Pipeline>(input, rank, nranks, vnranks, PipeTy == PipelineType::PLLMOFFLOAD,
                                          PipeTy == PipelineType::NANOBATCH || PipeTy == PipelineType::NANOBATCH_KQVBIAS,
                                          bias);
  else if (PipeTy == PipelineType::NONOVERLAP || PipeTy == PipelineType::NONOVERLAP_KQVBIAS ||
           PipeTy == PipelineType::NON_OVERLAP_LOCAL)
    pipeline = std::make_unique<NonOverlapLocalPipeline>(input, rank, nranks, vnranks, bias);
  else if (PipeTy == PipelineType::LOCAL || PipeTy == PipelineType::NANOBATCH_LOCAL)
    pipeline = std::make_unique<LocalPipeline>(input, rank, nranks, vnranks, PipeTy == PipelineType::NANOBATCH_LOCAL);
  else
    NF_LOG_ERROR("Unknown pipeline type %d", static_cast<int>(PipeTy));
  if (pipeline && g_profiling) pipeline->setProfiling(g_profiling);
  if (pipeline && g_graph_mode) pipeline->setGraphMode(true);
}

void Worker::run_pipeline() { *output = pipeline->run(); }

void Worker::run_update(vortexUpdateData* update_data) {
  auto& tm = TensorManager::getInstance();
  vortexUpdateData* gpu = tm.update_data_to_gpu(*update_data, rank, pipeline->uploadStream());
  if (!gpu) {
    std::fprintf(stderr, "update: iteration does not fit the configured limits\n");
    std::exit(EXIT_FAILURE);
  }
  pipeline->setHostUpdate(tm.host_data(rank));
  pipeline->update(gpu);
}

void Worker::thread_entry() {
  init();
  global_sync->barrier();  // end of init
  bool stop = false;
  while (!stop) {
    global_sync->barrier();  // wait for a command
    switch (shared_state.op) {
      case WorkerOp::STOP:
        stop = true;
        pipeline.reset();
        break;
      case WorkerOp::RUN:
        run_pipeline();
        break;
      case WorkerOp::UPDATE:
        run_update(&(shared_state.updates_ptr->at(rank)));
        break;
      case WorkerOp::CONFIG:
        run_config(&(shared_state.config_ptr->at(rank)));
        break;
    }
    global_sync->barrier();  // command done
  }
}
