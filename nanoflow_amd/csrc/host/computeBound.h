// Control plane: one worker thread per rank owning a pipeline, driven by
// init / config / update / run / run_async / run_async_wait / finalize.
// Same free functions, Worker class and PipelineType values as the reference's
// pipeline/include/computeBound.cuh:14-87 and pipeline/src/computeBound.cu:23-290.
// This build runs one rank; the tensor-parallel pipeline types are rejected.
#pragma once
#include <condition_variable>
#include <memory>
#include <mutex>
#include <thread>
#include <vector>

#include "config.h"
#include "pipeline.h"
#include "tensorManager.h"
#include "vortexData.h"

extern std::vector<vortexOutputData> outputs;
extern std::vector<int> aggregated_output;

// Barrier between the caller's thread and the worker threads
// (reference: SimpleThreadSync, pipeline/include/networkManager.cuh:8-34).
class SimpleThreadSync {
  std::mutex mtx;
  std::condition_variable cv;
  int count = 0;
  int total;
  unsigned long generation = 0;

public:
  explicit SimpleThreadSync(int total) : total(total) {}
  void barrier() {
    std::unique_lock<std::mutex> lck(mtx);
    const unsigned long gen = generation;
    if (++count == total) {
      count = 0;
      ++generation;
      cv.notify_all();
    } else {
      cv.wait(lck, [&] { return gen != generation; });  // immune to spurious wake-ups
    }
  }
};

enum class WorkerOp { STOP, RUN, UPDATE, CONFIG };

class Worker {
public:
  enum class PipelineType {
    PLLM,
    NONOVERLAP,
    NANOBATCH,
    PLLMOFFLOAD,
    KQVBIAS,
    NONOVERLAP_KQVBIAS,
    NANOBATCH_KQVBIAS,
    LOCAL,
    NON_OVERLAP_LOCAL,
    NANOBATCH_LOCAL,
  };
  static PipelineType PipeTy;
  // Every type runs on the one rank of this build.  PLLM, NANOBATCH, PLLMOFFLOAD and the two
  // nano-batched bias types are the reference's main Pipeline (four QKV / attention nano-batches)
  // without its exchange steps, NONOVERLAP its sequential schedule, so that the reference's multi-GPU
  // pipeline files serve here once their gpu_num is 1.
  static bool isSupported(PipelineType t) { return static_cast<int>(t) >= 0 && static_cast<int>(t) <= 9; }
  // the QKV GEMMs add vortexLayerWeight::B_KQV
  static bool hasKQVBias(PipelineType t) {
    return t == PipelineType::KQVBIAS || t == PipelineType::NONOVERLAP_KQVBIAS ||
           t == PipelineType::NANOBATCH_KQVBIAS;
  }
  // the reference's main schedule: four QKV / attention nano-batches (class Pipeline)
  static bool isFourWay(PipelineType t) {
    return t == PipelineType::PLLM || t == PipelineType::PLLMOFFLOAD || t == PipelineType::NANOBATCH ||
           t == PipelineType::KQVBIAS || t == PipelineType::NANOBATCH_KQVBIAS;
  }
  static bool isSequential(PipelineType t) {
    return t == PipelineType::NON_OVERLAP_LOCAL || t == PipelineType::NONOVERLAP_KQVBIAS ||
           t == PipelineType::NONOVERLAP;
  }

private:
  int rank;
  int nranks;
  int vnranks;
  vortexInitData* input;
  vortexOutputData* output;
  std::unique_ptr<PipelineBase> pipeline;
  std::unique_ptr<std::thread> thread;
  void thread_entry();

public:
  Worker(int rank, int nranks, int vnranks, vortexInitData* input, vortexOutputData* output)
      : rank(rank), nranks(nranks), vnranks(vnranks), input(input), output(output) {}
  void init();
  void as_thread(int core);
  void join() {
    if (thread && thread->joinable()) thread->join();
  }
  void run_pipeline();
  void run_update(vortexUpdateData* update_data);
  void run_config(vortexConfigData* config_data) { pipeline->config(config_data); }
  vortexOutputData* getOutput() { return output; }
  PipelineBase* getPipeline() { return pipeline.get(); }
  ~Worker() { join(); }
};

void run();
void init(int nranks, int vnranks, std::vector<vortexInitData>& input,
          std::vector<vortexOutputData>& output,
          Worker::PipelineType pipeTy = Worker::PipelineType::LOCAL);
inline void init(int nranks, std::vector<vortexInitData>& input, std::vector<vortexOutputData>& output,
                 Worker::PipelineType pipeTy = Worker::PipelineType::LOCAL) {
  init(nranks, nranks, input, output, pipeTy);
}
void update(int nranks, std::vector<vortexUpdateData>& update);
void finalize();
void run_async();
void run_async_wait();
void config(int nranks, std::vector<vortexConfigData>& config);

// Decode-token feed of update(): the tokens of slots that keep decoding are taken from the
// previous iteration's sampled ids, followed by this iteration's prefill tokens
// (pipeline/src/computeBound.cu:121-150).  prev_output == nullptr or prev_count == 0 means
// "first iteration": every kept slot is fed token id 1.  Returns the number written.
int buildInputTokens(const int* prev_output, int prev_count, const int32_t* keep_token_list,
                     int keep_token_list_length, const int* prefill_tokens, int prefill_tokens_num,
                     int* out);

// Access for measurement code: the rank-0 pipeline (nullptr before init()).
PipelineBase* currentPipeline();
void setPipelineProfiling(int level);
// Replay iterations from captured hipGraphs (one per launch signature) instead of enqueueing
// every launch; takes effect for the current and for later pipelines.
void setPipelineGraphMode(bool on);
