// CPU batch formation and paged-KV bookkeeping for the serving loop.
//
// C++ counterpart of the reference's Python scheduler:
//   KVPool / KVCache        pipeline/utils/kv_cache.py:20-104   (DistKVPool / DistKVCache)
//   batched KV metadata     pipeline/utils/kv_cache.py:106-135  (BatchedDistKVCache)
//   BatchFormer::schedule   pipeline/utils/serve_8B.py:177-346  (check_future_page_usage,
//                                                                schedule_req: admission with the
//                                                                page forecast, chunked prefill)
//   BatchFormer::form       pipeline/utils/serve_8B.py:348-451  (bench_text_gen, first half:
//                                                                page allocation, gemv_batch_size,
//                                                                indptr / rev_indptr / offsets)
//   BatchFormer::harvest    pipeline/utils/serve_8B.py:499-520  (outputs of the iteration that
//                                                                has just completed)
//   BatchFormer::advance    pipeline/utils/serve_8B.py:523-569  (length-only retirement, keep
//                                                                list, next worksets)
// All of it is integer bookkeeping and reproduces the reference's results exactly, with one
// stated freedom: which free page a request receives.  The reference pops from a Python set
// (an implementation detail of CPython); here the pool is a LIFO stack that initially hands out
// 0, 1, 2, ... and re-issues the most recently freed page first.
#pragma once
#include <cstdint>
#include <deque>
#include <memory>
#include <vector>

struct SchedRequest {  // NewRequestInfo (pipeline/utils/request_info.py:2-11)
  int req_idx = 0;
  std::vector<int32_t> prompt;
  int output_len = 0;
  double start_time = 0;
};

class KVPool {
public:
  KVPool(int capacity, int page_size);
  int num_free_pages() const { return (int)free_.size(); }
  int capacity() const { return capacity_; }
  int page_size() const { return page_size_; }
  int alloc_page();          // throws std::runtime_error("... Out of memory") when empty (the reference asserts)
  void free_page(int idx);

private:
  int capacity_, page_size_;
  std::vector<int> free_;  // stack; back() is handed out next
};

class KVCache {
public:
  explicit KVCache(KVPool* pool) : pool_(pool) {}
  int seqlen() const { return seqlen_; }
  const std::vector<int32_t>& indices() const { return indices_; }
  int last_page_offset() const { return (seqlen_ - 1 + pool_->page_size()) % pool_->page_size() + 1; }
  void allocate_tokens(int num_tokens);
  void release();

private:
  KVPool* pool_;
  std::vector<int32_t> indices_;
  int seqlen_ = 0;
};

struct FlyRequest {  // FlyRequestInfo (pipeline/utils/request_info.py:33-57)
  int req_idx = 0;
  std::vector<int32_t> input;   // tokens this request contributes to the next iteration
  std::vector<int32_t> output;  // sampled tokens; the last one may be a placeholder
  std::shared_ptr<const std::vector<int32_t>> prompt;
  bool chunked_prefill = false;
  std::shared_ptr<KVCache> kv_cache;  // shared between the chunks of one request
  int output_len = 0;
  int input_len = 0;
  double request_comein_time = 0, encode_latency = 0, decode_start_at = 0, decode_latency = 0;
};
using FlyPtr = std::shared_ptr<FlyRequest>;

// One iteration's update data, host side (layout of vortexUpdateData).
struct FormedBatch {
  int decodePrefillBorder = 0, prefillNum = 0, prefillTokensNum = 0, keepTokenListLength = 0;
  std::vector<int32_t> input_tokens;  // prefill tokens only
  std::vector<int32_t> input_indptr, rev_input_indptr, per_token_offset;
  std::vector<int32_t> kv_indptr, kv_indices, kv_last_page_len;
  std::vector<int32_t> keep_token_list;  // over the PREVIOUS iteration's requests
  int32_t gemv_batch_size[4] = {0, 0, 0, 0};
  int32_t gemv_num_blocks[4] = {0, 0, 0, 0};
};

class BatchFormer {
public:
  BatchFormer(int kv_capacity_pages, int page_size, int global_bsz, int nanobatch1, int kqv1, int kqv3,
              int average_prefill_length, int average_decode_length);

  void add_request(SchedRequest r) { queue_.push_back(std::move(r)); }
  size_t queued() const { return queue_.size(); }
  size_t decoding() const { return decode_.size(); }
  size_t prefilling() const { return prefill_.size(); }
  const KVPool& pool() const { return pool_; }

  // One scheduling cycle, split the way the serving loop interleaves it with the GPU:
  //   schedule(); form(batch);                    CPU work that overlaps the previous run
  //   [wait for the previous run; update(batch); run_async()]
  //   harvest(outputs of the run that just completed);
  //   advance(now, retired);
  void schedule();
  void form(FormedBatch& out);
  // ids[i] = token sampled for request i of the iteration before the one just formed
  // (decode requests first, then prefill requests).  Pass n == 0 when nothing completed yet.
  void harvest(const int32_t* ids, int n);
  // placeholder_zero: append 0 instead of -1 (the reference's skip-cycle mode).
  void advance(double now, std::vector<FlyPtr>& retired, bool placeholder_zero = false);

  // Forecast of pages in use over the coming iterations (serve_8B.py:177-203).
  std::vector<long long> future_page_usage() const;

  void set_num_blocks(const int32_t nb[4]) {
    for (int i = 0; i < 4; ++i) num_blocks_[i] = nb[i];
  }

private:
  KVPool pool_;
  std::deque<SchedRequest> queue_;
  int global_bsz_, nano1_, kqv1_, kqv3_, avg_prefill_, avg_decode_;
  std::vector<FlyPtr> decode_, prefill_, new_decode_, new_prefill_, old_decode_, old_prefill_;
  std::vector<int32_t> keep_list_;  // built by advance(), consumed by the next form()
  int old_token_length_ = 0;
  int32_t num_blocks_[4] = {0, 0, 0, 0};

  static int effective_bsz(const std::vector<FlyPtr>& set);
};

// Statistics of a serving run (what the reference writes to its .stat file,
// pipeline/utils/serve_8B.py:755-793, plus the CPU-side split of a cycle).
struct ServeStats {
  int cycles = 0;
  int retired = 0;             // requests completed inside the timed cycles
  double wall_s = 0;           // timed cycles only
  double tokens_per_s = 0;     // retired * (avg_prefill + avg_decode) / wall_s
  double cycle_ms = 0;         // wall_s / cycles
  double form_ms = 0;          // mean CPU time per cycle in schedule() + form()
  double wait_ms = 0;          // mean time blocked in run_async_wait()
  double update_ms = 0;        // mean time in update()
  double gpu_iter_ms = 0;      // mean device time of an iteration
  long long tokens_processed = 0;  // dense-batch rows executed in the timed cycles
};

// The asynchronous serving loop (pipeline/utils/serve_8B.py:348-569, 655-700): batch i+1 is
// scheduled and formed on the CPU while the GPU runs batch i; outputs are harvested one
// iteration late.  skip_cycles advance the scheduler without touching the GPU (the reference's
// simulated warm-up), warmup_cycles are executed untimed, run_cycles are executed and timed (the
// timed region starts and ends with the GPU idle; the pipeline's accumulated timings are reset
// at its start).  Requires an initialised and configured pipeline (init() + config()).
ServeStats serveLoop(BatchFormer& former, int skip_cycles, int warmup_cycles, int run_cycles,
                     std::vector<FlyPtr>* retired_out = nullptr);
