// OperatorWrapper: the scheduling vocabulary every pipeline operator inherits -- a stream,
// optional start/end events, run()/skip()/wait()/wait_for_start().
// Same interface as the reference's pipeline/include/operatorWrapper.cuh:14-157 on HIP streams
// and events.  Added: an optional per-launch timing ring (enableProfiling) so that the
// durations of a chosen operator can be read back after an iteration.
#pragma once
#include <memory>
#include <string>
#include <vector>

#include "helper.h"
#include "tensor.h"
#include "tensorLogger.h"

struct OperatorWrapper {
  hipStream_t stream = nullptr;
  hipEvent_t start_event = nullptr, end_event = nullptr;
  std::string name;
  bool streamInited = false;

  // per-launch timing (off by default)
  std::vector<hipEvent_t> prof_events;  // 2 per launch: start, end
  size_t prof_used = 0;
  unsigned prof_stride = 1, prof_seq = 0;

  OperatorWrapper(bool create_start = false, bool create_end = true) {
    if (create_start) HIP_CHECK(hipEventCreate(&start_event));
    if (create_end) HIP_CHECK(hipEventCreate(&end_event));
  }
  OperatorWrapper(const OperatorWrapper&) = delete;
  OperatorWrapper& operator=(const OperatorWrapper&) = delete;

  void updateEventExistance(bool create_start, bool create_end) {
    if (start_event) (void)hipEventDestroy(start_event);
    if (end_event) (void)hipEventDestroy(end_event);
    start_event = end_event = nullptr;
    if (create_start) HIP_CHECK(hipEventCreate(&start_event));
    if (create_end) HIP_CHECK(hipEventCreate(&end_event));
  }

  virtual ~OperatorWrapper() {
    if (start_event) (void)hipEventDestroy(start_event);
    if (end_event) (void)hipEventDestroy(end_event);
    for (auto e : prof_events) (void)hipEventDestroy(e);
  }

  OperatorWrapper& setStream(hipStream_t s) {
    stream = s;
    streamInited = true;
    return *this;
  }
  OperatorWrapper& setName(std::string n) {
    name = n + " ";
    return *this;
  }

  virtual void work() = 0;

  void recordStartEvent() {
    if (start_event) HIP_CHECK(hipEventRecord(start_event, stream));
  }
  void recordEndEvent() {
    if (end_event) HIP_CHECK(hipEventRecord(end_event, stream));
  }

  virtual OperatorWrapper& run() {
    if (!streamInited) {
      NF_LOG_ERROR("%s Stream not inited", name.c_str());
      return *this;
    }
    recordStartEvent();
    const bool prof = prof_used + 2 <= prof_events.size() && (prof_seq++ % prof_stride) == 0;
    if (prof) HIP_CHECK(hipEventRecord(prof_events[prof_used], stream));
    work();
    if (prof) {
      HIP_CHECK(hipEventRecord(prof_events[prof_used + 1], stream));
      prof_used += 2;
    }
    recordEndEvent();
    return *this;
  }

  virtual OperatorWrapper& skip() {
    if (!streamInited) {
      NF_LOG_ERROR("Stream not inited");
      return *this;
    }
    recordStartEvent();
    recordEndEvent();
    return *this;
  }

  virtual OperatorWrapper& wait(const OperatorWrapper& other) {
    if (other.end_event)
      HIP_CHECK(hipStreamWaitEvent(stream, other.end_event, 0));
    else
      NF_LOG_WARN("The other operator does not have an end event");
    return *this;
  }
  virtual OperatorWrapper& wait(const OperatorWrapper* other) { return wait(*other); }

  virtual OperatorWrapper& wait_for_start(const OperatorWrapper& other) {
    if (other.start_event)
      HIP_CHECK(hipStreamWaitEvent(stream, other.start_event, 0));
    else
      NF_LOG_WARN("The other operator does not have a start event");
    return *this;
  }

  // Tensor dumps (operatorWrapper.cuh:146-156): log() after run() prints the operator's operands
  // when NANOFLOW_TENSOR_LOG names a sink; logImpl() is the per-operator part.  Launches that are
  // being captured into a graph are not dumped.
  virtual OperatorWrapper& logImpl() { return *this; }
  OperatorWrapper& log() {
    if (tensorlog::enabled() && streamInited && !tensorlog::capturing(stream)) return logImpl();
    return *this;
  }
  template <typename T>
  void logTensor(const char* tensor_name, const pllmTensor<T>& t, size_t rows = 1, size_t cols = 20) {
    tensorlog::log_tensor(stream, name.empty() || name.back() == ' ' ? name : name + " ", tensor_name, t, rows, cols);
  }

  // Time up to max_launches launches per iteration with event pairs on the op's own stream.
  // Every stride-th launch is timed (event records cost device time, so long schedules sample).
  void enableProfiling(size_t max_launches, unsigned stride = 1) {
    prof_stride = stride ? stride : 1;
    prof_seq = 0;
    for (auto e : prof_events) (void)hipEventDestroy(e);
    prof_events.assign(2 * max_launches, nullptr);
    for (auto& e : prof_events) HIP_CHECK(hipEventCreate(&e));
    prof_used = 0;
  }
  // After the streams are idle: adds the recorded durations, resets the ring.
  void collectProfile(double& total_ms, long& launches) {
    for (size_t i = 0; i + 1 < prof_used; i += 2) {
      float ms = 0.f;
      HIP_CHECK(hipEventElapsedTime(&ms, prof_events[i], prof_events[i + 1]));
      total_ms += ms;
      ++launches;
    }
    prof_used = 0;
  }
};
