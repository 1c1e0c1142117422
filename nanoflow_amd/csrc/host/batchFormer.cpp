#include "batchFormer.h"

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <stdexcept>
#include <string>

KVPool::KVPool(int capacity, int page_size) : capacity_(capacity), page_size_(page_size) {
  free_.reserve(capacity);
  for (int i = capacity - 1; i >= 0; --i) free_.push_back(i);  // back() == 0 is handed out first
}

int KVPool::alloc_page() {
  if (free_.empty()) throw std::runtime_error("KVPool: Out of memory");
  int idx = free_.back();
  free_.pop_back();
  return idx;
}

void KVPool::free_page(int idx) { free_.push_back(idx); }

// pages appended = (num_tokens + last_page_offset - 1) / page_size, where an empty cache
// counts as a full last page (kv_cache.py:87-98).
void KVCache::allocate_tokens(int num_tokens) {
  if (num_tokens <= 0 || (long long)num_tokens > (long long)pool_->num_free_pages() * pool_->page_size()) {
    throw std::runtime_error("KVCache: Out of memory (" + std::to_string(num_tokens) + " tokens, " +
                             std::to_string(pool_->num_free_pages()) + " free pages)");
  }
  const int appended = (num_tokens + last_page_offset() - 1) / pool_->page_size();
  for (int i = 0; i < appended; ++i) indices_.push_back(pool_->alloc_page());
  seqlen_ += num_tokens;
}

void KVCache::release() {
  seqlen_ = 0;
  for (int idx : indices_) pool_->free_page(idx);
  indices_.clear();
}

BatchFormer::BatchFormer(int kv_capacity_pages, int page_size, int global_bsz, int nanobatch1, int kqv1,
                         int kqv3, int average_prefill_length, int average_decode_length)
    : pool_(kv_capacity_pages, page_size),
      global_bsz_(global_bsz),
      nano1_(nanobatch1),
      kqv1_(kqv1),
      kqv3_(kqv3),
      avg_prefill_(average_prefill_length),
      avg_decode_(average_decode_length) {}

int BatchFormer::effective_bsz(const std::vector<FlyPtr>& set) {
  int n = 0;
  for (const auto& r : set) n += (int)r->input.size();
  return n;
}

// future[i] = pages the current worksets will hold i iterations from now, assuming every
// request grows by one token per iteration up to prefill + decode + 2 tokens.
std::vector<long long> BatchFormer::future_page_usage() const {
  const int max_seq_len = avg_decode_ + avg_prefill_ + 2;
  const int P = pool_.page_size();
  std::vector<long long> usage(max_seq_len, 0);
  auto add = [&](int current_seq_len) {
    // the reference slices [0 : max_seq_len - current_seq_len]; a negative bound counts from
    // the end (numpy), which only happens for requests longer than the trace average
    int n = max_seq_len - current_seq_len;
    if (n < 0) n = std::max(0, max_seq_len + n);
    for (int i = 0; i < n; ++i) usage[i] += (i + current_seq_len + P - 1) / P;
  };
  for (const auto& r : decode_) add(r->kv_cache->seqlen() + 1);
  for (size_t i = 0; i < prefill_.size(); ++i) add(avg_prefill_ + 1);
  return usage;
}

void BatchFormer::schedule() {
  new_decode_.clear();
  new_prefill_.clear();
  const int P = pool_.page_size();
  const int decode_tokens = effective_bsz(decode_);
  int decode_idle_tokens = global_bsz_ - decode_tokens;
  int prefill_idle_tokens = global_bsz_ - effective_bsz(prefill_) - decode_tokens;
  std::vector<long long> future = future_page_usage();
  auto min_avail = [&] { return (long long)pool_.capacity() - *std::max_element(future.begin(), future.end()); };
  long long new_min_avail_pages = min_avail();
  const int max_seq_len = avg_decode_ + avg_prefill_ + 2;

  while (prefill_idle_tokens > 0 && decode_idle_tokens > 0 && !queue_.empty() &&
         new_min_avail_pages > (avg_prefill_ + avg_decode_ + P) / P) {
    SchedRequest nr = std::move(queue_.front());
    queue_.pop_front();
    auto prompt = std::make_shared<const std::vector<int32_t>>(std::move(nr.prompt));
    auto kv = std::make_shared<KVCache>(&pool_);
    const int plen = (int)prompt->size();
    auto make = [&](int from, int to, bool chunked) {
      auto f = std::make_shared<FlyRequest>();
      f->req_idx = nr.req_idx;
      f->input.assign(prompt->begin() + from, prompt->begin() + to);
      f->prompt = prompt;
      f->request_comein_time = nr.start_time;
      f->chunked_prefill = chunked;
      f->kv_cache = kv;
      f->output_len = nr.output_len;
      f->input_len = plen;
      return f;
    };
    if (plen > prefill_idle_tokens) {
      // chunked prefill: the head goes into this iteration, the tail into the next
      prefill_.push_back(make(0, prefill_idle_tokens, true));
      new_prefill_.push_back(make(prefill_idle_tokens, plen, false));
      prefill_idle_tokens = 0;
      decode_idle_tokens -= 1;
    } else {
      prefill_.push_back(make(0, plen, false));
      prefill_idle_tokens -= plen;
      decode_idle_tokens -= 1;
    }
    const int current_seq_len = avg_prefill_ + 1;
    for (int i = 0; i < max_seq_len - current_seq_len; ++i) future[i] += (i + current_seq_len + P - 1) / P;
    new_min_avail_pages = min_avail();
  }

  if (prefill_idle_tokens < 0) {
    // a continuing prefill alone exceeds the room left by the decode tokens: cut it again
    if (prefill_.size() != 1) {
      throw std::runtime_error("BatchFormer: At most add one large prefill each iteration.");
    }
    const int over = -prefill_idle_tokens;
    FlyPtr head = prefill_[0];
    auto tail = std::make_shared<FlyRequest>(*head);
    tail->input.assign(head->input.end() - over, head->input.end());
    tail->output.clear();
    tail->chunked_prefill = false;
    new_prefill_.push_back(tail);
    head->input.resize(head->input.size() - over);
    head->chunked_prefill = true;
  }
}

void BatchFormer::form(FormedBatch& out) {
  out = FormedBatch();
  for (const auto& r : prefill_) out.input_tokens.insert(out.input_tokens.end(), r->input.begin(), r->input.end());
  for (const auto& r : prefill_) r->kv_cache->allocate_tokens((int)r->input.size());
  for (const auto& r : decode_) r->kv_cache->allocate_tokens((int)r->input.size());

  const int dpb = effective_bsz(decode_);
  out.decodePrefillBorder = dpb;
  out.prefillNum = (int)prefill_.size();
  out.prefillTokensNum = (int)out.input_tokens.size();
  out.gemv_batch_size[0] = std::min(dpb, kqv1_);
  out.gemv_batch_size[1] = std::min(dpb - out.gemv_batch_size[0], nano1_ - kqv1_);
  out.gemv_batch_size[2] = std::min(dpb - out.gemv_batch_size[0] - out.gemv_batch_size[1], kqv3_);
  out.gemv_batch_size[3] = dpb - out.gemv_batch_size[0] - out.gemv_batch_size[1] - out.gemv_batch_size[2];
  for (int i = 0; i < 4; ++i) out.gemv_num_blocks[i] = num_blocks_[i];

  std::vector<int> prev_len;
  out.input_indptr.push_back(0);
  out.kv_indptr.push_back(0);
  auto add_kv = [&](const KVCache& kv) {
    out.kv_indices.insert(out.kv_indices.end(), kv.indices().begin(), kv.indices().end());
    out.kv_last_page_len.push_back(kv.last_page_offset());
    out.kv_indptr.push_back(out.kv_indptr.back() + (int)kv.indices().size());
  };
  for (const auto& r : decode_) {
    out.input_indptr.push_back(out.input_indptr.back() + (int)r->input.size());
    prev_len.push_back(r->kv_cache->seqlen() - 1);  // the new token's slot is already counted
    add_kv(*r->kv_cache);
  }
  for (const auto& r : prefill_) {
    out.input_indptr.push_back(out.input_indptr.back() + (int)r->input.size());
    prev_len.push_back(r->kv_cache->seqlen() - (int)r->input.size());
    add_kv(*r->kv_cache);
  }
  for (size_t i = 0; i + 1 < out.input_indptr.size(); ++i)
    for (int j = out.input_indptr[i]; j < out.input_indptr[i + 1]; ++j) {
      out.rev_input_indptr.push_back((int32_t)i);
      out.per_token_offset.push_back(j - out.input_indptr[i] + prev_len[i]);
    }
  out.keep_token_list = keep_list_;
  out.keepTokenListLength = old_token_length_;
}

void BatchFormer::harvest(const int32_t* ids, int n) {
  if (n <= 0) return;
  for (size_t i = 0; i < old_prefill_.size(); ++i) {
    FlyRequest& r = *old_prefill_[i];
    const size_t slot = i + old_decode_.size();
    if (!r.chunked_prefill && slot < (size_t)n && !r.output.empty()) {
      r.output.back() = ids[slot];
      r.input.assign(1, r.output.back());
    }
  }
  for (size_t i = 0; i < old_decode_.size() && i < (size_t)n; ++i) {
    FlyRequest& r = *old_decode_[i];
    if (!r.output.empty()) {
      r.output.back() = ids[i];
      r.input.assign(1, r.output.back());
    }
  }
}

void BatchFormer::advance(double now, std::vector<FlyPtr>& retired, bool placeholder_zero) {
  old_token_length_ = (int)(decode_.size() + prefill_.size());
  const int32_t append_token_id = placeholder_zero ? 0 : -1;
  keep_list_.assign(global_bsz_, 0);
  for (size_t i = 0; i < decode_.size(); ++i) {
    FlyPtr& r = decode_[i];
    if ((int)r->output.size() >= r->output_len - 1) {  // length-only retirement, EOS ignored
      r->decode_latency = now - r->decode_start_at;
      r->kv_cache->release();
      retired.push_back(r);
    } else {
      keep_list_[i] = 1;
      r->output.push_back(append_token_id);
      r->input.assign(1, 0);
      new_decode_.push_back(r);
    }
  }
  for (size_t i = 0; i < prefill_.size(); ++i) {
    FlyPtr& r = prefill_[i];
    if (!r->chunked_prefill) {  // whole prompt is in the cache: the request starts decoding
      keep_list_[decode_.size() + i] = 1;
      r->decode_start_at = now;
      r->encode_latency = now - r->request_comein_time;
      r->input.assign(1, 0);
      r->output.push_back(append_token_id);
      new_decode_.push_back(r);
    }
  }
  old_decode_ = std::move(decode_);
  old_prefill_ = std::move(prefill_);
  decode_ = std::move(new_decode_);
  prefill_ = std::move(new_prefill_);
  new_decode_.clear();
  new_prefill_.clear();
}
