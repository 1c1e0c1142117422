// Named HIP events shared by a pipeline (reference: pipeline/include/eventManager.cuh:6-69).
#pragma once
#include <vector>

#include "helper.h"

class EventManager {
public:
  enum EVENT_NAME {
    GEMM_TIMING_START = 0,
    GEMM_TIMING_END,
    CAPTURE_GEMM_START,
    CAPTURE_GEMV_END,
    NUM
  };
  std::vector<hipEvent_t> events;
  EventManager() {
    events.resize(NUM);
    for (auto& e : events) HIP_CHECK(hipEventCreate(&e));
  }
  ~EventManager() {
    for (auto& e : events) (void)hipEventDestroy(e);
  }
  EventManager(const EventManager&) = delete;
  EventManager& operator=(const EventManager&) = delete;
};
