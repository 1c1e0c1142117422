#include <chrono>

#include "batchFormer.h"
#include "computeBound.h"

static double now_s() {
  return std::chrono::duration<double>(std::chrono::steady_clock::now().time_since_epoch()).count();
}

static void to_update(FormedBatch& b, vortexUpdateData& u) {
  u.decodePrefillBorder = b.decodePrefillBorder;
  u.prefillNum = b.prefillNum;
  u.prefillTokensNum = b.prefillTokensNum;
  u.keepTokenListLength = b.keepTokenListLength;
  u.input_tokens = b.input_tokens.data();
  u.input_indptr = b.input_indptr.data();
  u.rev_input_indptr = b.rev_input_indptr.data();
  u.keep_token_list = b.keep_token_list.data();
  u.kv_indptr = b.kv_indptr.data();
  u.kv_indices = b.kv_indices.data();
  u.kv_last_page_len = b.kv_last_page_len.data();
  u.per_token_offset = b.per_token_offset.data();
  u.gemv_batch_size = b.gemv_batch_size;
  u.gemv_num_blocks = b.gemv_num_blocks;
}

ServeStats serveLoop(BatchFormer& former, int skip_cycles, int warmup_cycles, int run_cycles,
                     std::vector<FlyPtr>* retired_out) {
  ServeStats st;
  std::vector<FlyPtr> retired_local;
  std::vector<FlyPtr>& retired = retired_out ? *retired_out : retired_local;
  FormedBatch batch;
  std::vector<vortexUpdateData> upd(1);
  auto busy = [&] { return former.queued() + former.decoding() + former.prefilling() > 0; };

  // simulated warm-up: the scheduler advances, the GPU does not run
  for (int c = 0; c < skip_cycles && busy(); ++c) {
    former.schedule();
    former.form(batch);
    former.advance(now_s(), retired, /*placeholder_zero=*/true);
  }

  bool in_flight = false;     // an iteration is running on the worker thread
  bool have_outputs = false;  // aggregated_output holds the samples of the former's previous iteration
  size_t retired_before = retired.size();
  double t_form = 0, t_wait = 0, t_update = 0, t_gpu = 0, t1 = now_s();
  auto wait_iteration = [&] {
    run_async_wait();
    in_flight = false;
    have_outputs = true;
    if (auto* p = currentPipeline()) t_gpu += p->getTimings().iter_ms;
  };
  try {
    for (int c = 0; c < warmup_cycles + run_cycles && busy(); ++c) {
      if (c == warmup_cycles) {  // the timed region starts with the GPU idle
        if (in_flight) wait_iteration();
        if (auto* p = currentPipeline()) p->resetTimings();
        retired_before = retired.size();
        t_form = t_wait = t_update = t_gpu = 0;
        st = ServeStats();
        t1 = now_s();
      }
      const double a = now_s();
      former.schedule();
      former.form(batch);
      const double b = now_s();
      if (batch.decodePrefillBorder + batch.prefillTokensNum == 0) break;  // nothing left to run
      if (in_flight) wait_iteration();  // iteration c-1 is done; its samples feed the decode rows below
      const double w = now_s();
      to_update(batch, upd[0]);
      update(1, upd);
      const double u = now_s();
      run_async();
      in_flight = true;
      if (have_outputs) former.harvest(aggregated_output.data(), (int)aggregated_output.size());
      former.advance(now_s(), retired, false);
      t_form += b - a;
      t_wait += w - b;
      t_update += u - w;
      st.tokens_processed += batch.decodePrefillBorder + batch.prefillTokensNum;
      ++st.cycles;
    }
  } catch (...) {
    if (in_flight) run_async_wait();  // never leave an iteration in flight behind an error
    throw;
  }
  if (in_flight) wait_iteration();
  const double t2 = now_s();
  st.wall_s = t2 - t1;
  st.retired = (int)(retired.size() - retired_before);
  if (st.cycles > 0) {
    st.cycle_ms = st.wall_s * 1e3 / st.cycles;
    st.form_ms = t_form * 1e3 / st.cycles;
    st.wait_ms = t_wait * 1e3 / st.cycles;
    st.update_ms = t_update * 1e3 / st.cycles;
    st.gpu_iter_ms = t_gpu / st.cycles;
  }
  return st;
}
