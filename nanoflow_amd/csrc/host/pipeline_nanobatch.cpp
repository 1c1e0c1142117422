// Pipeline: the reference's main nano-batch schedule (pipeline/src/pipeline.cu) on one device.
//
// Rows of the dense batch are cut at nano1 into two nano-batches for the O projection and the
// FFN, and each of those in two for the QKV projection, RoPE-append and decode attention
// (sizes kqv1, nano1 - kqv1, kqv3, T - nano1 - kqv3: pipeline/include/vortexData.cuh:129-132).
// Dense operators run on stream_gemm, attention on stream_gemv: decode attention of group i starts
// as soon as QKV_i and its RoPE-append are done and runs beside QKV_{i+1..}; the O projection of
// nano-batch 1 only waits for the attention of its own rows (operator order and event edges of
// Pipeline::run, pipeline.cu:599-789; buffer plan :279-470; attention slicing :797-933).
// What the reference exchanges between ranks (AG1_GEMV, AG_O1, AR_O2, AR_D1, AR1_D2 / AR2_D2, and
// the splitTensor / copyTensor steps around them) moves nothing on one rank and is not here; the
// RMSNorm that its last all-reduce fuses (comm.cu:325-361) runs as an operator of its own.
// One prefill launch covers all prefill requests after the fourth RoPE-append, so no request is
// ever cut by a nano-batch border.
#include <cstdlib>
#include <numeric>

#include "pipeline.h"
#include "tensorManager.h"

Pipeline::Pipeline(vortexInitData* input_data, int nrank, int nranks, int vnranks, bool enable_offload_,
                   bool nanobatch_only_, bool kqv_bias_)
    : PipelineBase(input_data, nrank, nranks, vnranks), enable_offload(enable_offload_), nanobatch_only(nanobatch_only_) {
  kqv_bias = kqv_bias_;
  // Optional CU partition, as in LocalPipeline: dense operators on CUs [0, g), attention on [g, g + a)
  // (NANOFLOW_GEMM_CUS / NANOFLOW_GEMV_CUS; 0 = no restriction).  Eager launches only (masked_streams).
  const char* ge = std::getenv("NANOFLOW_GEMM_CUS");
  const char* ve = std::getenv("NANOFLOW_GEMV_CUS");
  const int gemm_cus = ge ? std::atoi(ge) : 0, gemv_cus = ve ? std::atoi(ve) : 0;
  masked_streams = gemm_cus > 0 || gemv_cus > 0;
  stream_gemm = createPipelineStream(0, gemm_cus);
  stream_gemv = createPipelineStream(gemm_cus, gemv_cus);
  stream_cpy = createPipelineStream(0, 0);
  if (enable_offload) {
    // room for two requests of 256 pages each (4096 tokens): the iteration's leading requests are
    // moved as long as their pages fit together; a first request longer than the room moves nothing
    offload_pages_cap = 512;
    const size_t bytes = offload_pages_cap * ModelConfig.page_mem_size;
    HIP_CHECK(hipHostMalloc(&offloadKVCache, bytes, hipHostMallocDefault));
    HIP_CHECK(hipMalloc(&deviceOffloadKVCache, bytes));
    HIP_CHECK(hipMalloc(&deviceLoadKVCache, bytes));
    std::vector<int32_t> idx(ModelConfig.max_batch_size);
    std::iota(idx.begin(), idx.end(), 0);
    HIP_CHECK(hipMalloc(&finished_idx, idx.size() * sizeof(int32_t)));
    HIP_CHECK(hipMalloc(&load_idx, idx.size() * sizeof(int32_t)));
    HIP_CHECK(hipMemcpy(finished_idx, idx.data(), idx.size() * sizeof(int32_t), hipMemcpyHostToDevice));
    HIP_CHECK(hipMemcpy(load_idx, idx.data(), idx.size() * sizeof(int32_t), hipMemcpyHostToDevice));
    HIP_CHECK(hipEventCreateWithFlags(&offload_done, hipEventDisableTiming));
  }
  NF_LOG_INFO("Init pipeline (four QKV / attention nano-batches)%s%s", enable_offload ? ", KV offload round trip" : "",
              nanobatch_only ? ", one stream" : "");
}

Pipeline::~Pipeline() {
  clearGraphs();
  for (auto g : gemms) delete g;
  delete[] output_data.sampled_token_array;
  if (offloadKVCache) (void)hipHostFree(offloadKVCache);
  if (deviceOffloadKVCache) (void)hipFree(deviceOffloadKVCache);
  if (deviceLoadKVCache) (void)hipFree(deviceLoadKVCache);
  if (finished_idx) (void)hipFree(finished_idx);
  if (load_idx) (void)hipFree(load_idx);
  if (offload_done) (void)hipEventDestroy(offload_done);
  if (stream_gemm) (void)hipStreamDestroy(stream_gemm);
  if (stream_gemv) (void)hipStreamDestroy(stream_gemv);
  if (stream_cpy) (void)hipStreamDestroy(stream_cpy);
}

void Pipeline::setName() {
  SET_NAME_PTR(O1);
  SET_NAME_PTR(O2);
  SET_NAME_PTR(D1);
  SET_NAME_PTR(D2);
  SET_NAME_PTR(KQV1);
  SET_NAME_PTR(KQV2);
  SET_NAME_PTR(KQV3);
  SET_NAME_PTR(KQV4);
  SET_NAME_PTR(LOGITS);
  SET_NAME_REF(dual1);
  SET_NAME_REF(dual2);
  SET_NAME_REF(genEmbedding1);
  SET_NAME_REF(genEmbedding2_1);
  SET_NAME_REF(genEmbedding2_2);
  SET_NAME_REF(GEMV1);
  SET_NAME_REF(GEMV2);
  SET_NAME_REF(GEMV3);
  SET_NAME_REF(GEMV4);
  SET_NAME_REF(prefill);
  SET_NAME_REF(layerNormAttention1);
  SET_NAME_REF(layerNormAttention2_1);
  SET_NAME_REF(layerNormAttention2_2);
  SET_NAME_REF(layerNormFFN1);
  SET_NAME_REF(layerNormFFN2);
  SET_NAME_REF(layerNormModel1);
  SET_NAME_REF(pageAgg);
  SET_NAME_REF(pageDisp);
  SET_NAME_REF(maxSampler);
  SET_NAME_REF(keepToken);
}

void Pipeline::setProfiling(int level) {
  profiling = level > 0;
  profile_gemms = level > 1;
  const unsigned stride = profileStride();
  timings.layer_stride = (int)stride;
  const size_t n = profiling ? (size_t)ModelConfig.run_layer : 0;
  for (auto gemv : gemvs) gemv->enableProfiling(n, stride);
  prefill.enableProfiling(n, stride);
  const size_t ng = profile_gemms ? (size_t)ModelConfig.run_layer : 0;
  for (auto g : gemms)
    if (g) g->enableProfiling(ng, stride);
  dual1.enableProfiling(ng, stride);
  dual2.enableProfiling(ng, stride);
}

void Pipeline::setWeight(int layer) {
  auto& lw = input_data->weight.layer_weight[layer];
  bool success = true;
  success &= O1->set_weight(lw.W_O1);
  success &= O2->set_weight(lw.W_O2);
  success &= D1->set_weight(lw.W_D);
  success &= D2->set_weight(lw.W_D);
  for (auto kqv : KQV_ptrs) {
    success &= kqv->set_weight(lw.W_KQV);
    success &= bindKQVBias(kqv, lw.B_KQV);
  }
  success &= layerNormAttention1.setWeight(lw.W_LN_Attention);
  success &= layerNormAttention2_1.setWeight(lw.W_LN_Attention);
  success &= layerNormAttention2_2.setWeight(lw.W_LN_Attention);
  success &= layerNormFFN1.setWeight(lw.W_LN_FFN);
  success &= layerNormFFN2.setWeight(lw.W_LN_FFN);
  success &= dual1.set_weight(lw.W_G, lw.W_U);
  success &= dual2.set_weight(lw.W_G, lw.W_U);
  if (!success) NF_LOG_ERROR("Failed to set weight for layer %d", layer);
  for (auto gemv : gemvs) gemv->setKVData(input_data->kv_data[layer]);
  prefill.setKVData(input_data->kv_data[layer]);
  for (auto& r : roPEAppends) r.setKVData(input_data->kv_data[layer]);
  pageAgg.setKVData(input_data->kv_data[layer]);
  pageDisp.setKVData(input_data->kv_data[layer]);
}

void Pipeline::GEMMOpInit() {
  setWeight(0);
  O1->init(1.f);  // O and D add the residual stream through C (beta = 1)
  O2->init(1.f);
  D1->init(1.f);
  D2->init(1.f);
  for (auto kqv : KQV_ptrs) kqv->init(kqv_bias ? 1.f : 0.f);
  LOGITS->set_weight(input_data->weight.lm_head);
  LOGITS->init();
  for (int i = 0; i < gemmNum; ++i) gemms[i]->setStream(stream_gemm);
  dual1.init();
  dual2.init();
  dual1.setStream(stream_gemm);
  dual2.setStream(stream_gemm);
}

void Pipeline::GEMVOpInit() {
  hipStream_t s = nanobatch_only ? stream_gemm : stream_gemv;
  for (auto gemv : gemvs) gemv->setStream(s);
  prefill.setStream(s);
}

void Pipeline::OtherOpInit() {
  genEmbedding1.setWeight(input_data->weight.embedding);
  genEmbedding2_1.setWeight(input_data->weight.embedding);
  genEmbedding2_2.setWeight(input_data->weight.embedding);
  layerNormModel1.setWeight(input_data->weight.model_layernorm);
  for (OperatorWrapper* op : std::initializer_list<OperatorWrapper*>{
           &genEmbedding1, &genEmbedding2_1, &genEmbedding2_2, &layerNormAttention1, &layerNormAttention2_1,
           &layerNormAttention2_2, &layerNormFFN1, &layerNormFFN2, &layerNormModel1, &maxSampler, &keepToken})
    op->setStream(stream_gemm).updateEventExistance(false, false);
  for (auto& r : roPEAppends) r.setStream(stream_gemm);
  pageAgg.setStream(stream_cpy);
  pageDisp.setStream(stream_cpy);
}

// Carves every intermediate out of tmp_buffer and wires operator inputs and outputs.  The
// residual stream lives in the D-output buffer (embeddings write it, O adds it, D adds O's output).
void Pipeline::ScheduleInit() {
  const int kdim = ModelConfig.model_head_dim * ModelConfig.model_kv_heads_gpu;
  const int qdim = ModelConfig.model_head_dim * ModelConfig.model_qo_heads_gpu;
  const int T = config_data.global_batch_size;
  const int H = ModelConfig.model_hidden_dim;
  const auto ROW = PllmLayout::ROW_MAJOR;
  const auto DR = PllmDimension::ROW;
  const size_t k[4] = {KQV1->M, KQV2->M, KQV3->M, KQV4->M};

  KQV_output = tmpBufferM.allocTensor(T, 2 * kdim + qdim, ROW);
  gemvQ = tmpBufferM.allocTensor(T, qdim, ROW);
  gemvAggregateOutput = tmpBufferM.allocTensor(T, ModelConfig.model_hidden_dim_pergpu, ROW);
  const auto D_output = tmpBufferM.allocTensor(T, H, ROW);
  const auto LNA_output = tmpBufferM.allocTensor(T, H, ROW);
  const auto O_output = tmpBufferM.allocTensor(T, H, ROW);
  const auto LNF_output = tmpBufferM.allocTensor(T, H, ROW);
  const auto act_output = tmpBufferM.allocTensor(T, (int)D1->K, ROW);

  const auto D12 = D_output.splitTensor(DR, O1->M, O2->M);
  const auto O12 = O_output.splitTensor(DR, O1->M, O2->M);
  const auto LNF12 = LNF_output.splitTensor(DR, O1->M, O2->M);
  const auto act12 = act_output.splitTensor(DR, O1->M, O2->M);
  const auto attn12 = gemvAggregateOutput.splitTensor(DR, O1->M, O2->M);
  const auto D4 = D_output.splitTensor(DR, k[0], k[1], k[2], k[3]);
  const auto LNA4 = LNA_output.splitTensor(DR, k[0], k[1], k[2], k[3]);
  const auto LNA12 = LNA_output.splitTensor(DR, O1->M, O2->M);
  const auto KQV4s = KQV_output.splitTensor(DR, k[0], k[1], k[2], k[3]);

  // a QKV cut may sit on a nano-batch border (kqv1 == nano1, kqv3 == T - nano1): that piece is
  // empty, its operators are never bound or run
  genEmbedding1.setOutput(D12[0]);
  layerNormAttention1.setInput(D12[0]).setOutput(LNA12[0]);
  if (k[2] > 0) {
    genEmbedding2_1.setOutput(D4[2]);
    layerNormAttention2_1.setInput(D4[2]).setOutput(LNA4[2]);
  }
  if (k[3] > 0) {
    genEmbedding2_2.setOutput(D4[3]);
    layerNormAttention2_2.setInput(D4[3]).setOutput(LNA4[3]);
  }
  for (int i = 0; i < 4; ++i)
    if (k[i] > 0) KQV_ptrs[i]->setA(LNA4[i]).setOutput(KQV4s[i]);

  O1->setA(attn12[0]);
  O1->setC(D12[0]);
  O1->setD(O12[0]);
  layerNormFFN1.setInput(O12[0]).setOutput(LNF12[0]);
  dual1.setA(LNF12[0]);
  dual1.setD(pllmTensor<half>(), pllmTensor<half>(), act12[0]);
  D1->setA(act12[0]);
  D1->setC(O12[0]);
  D1->setD(D12[0]);

  O2->setA(attn12[1]);
  O2->setC(D12[1]);
  O2->setD(O12[1]);
  layerNormFFN2.setInput(O12[1]).setOutput(LNF12[1]);
  dual2.setA(LNF12[1]);
  dual2.setD(pllmTensor<half>(), pllmTensor<half>(), act12[1]);
  D2->setA(act12[1]);
  D2->setC(O12[1]);
  D2->setD(D12[1]);

  // sampling: last token of each request -> final norm -> LM head -> argmax
  const auto keepTokenOutput = tmpBufferM.allocTensor(T, H, ROW);
  keepToken.setInput(D_output).setOutput(keepTokenOutput);
  const auto layerNormModel_output = tmpBufferM.allocTensor(T, H, ROW);
  layerNormModel1.setInput(keepTokenOutput).setOutput(layerNormModel_output);
  const auto LOGITS_output = tmpBufferM.allocTensor(T, (int)LOGITS->N, ROW);
  LOGITS->setA(layerNormModel_output);
  LOGITS->setOutput(LOGITS_output);
  int* sample_output_alloc = (int*)tmpBufferM.alloc((size_t)T * sizeof(int) / sizeof(half));
  pllmTensor<int> sample_output = {sample_output_alloc, T, 1, ROW};
  const auto maxSampler_maxVals = tmpBufferM.allocTensor(T, 1, ROW);
  maxSampler.init(LOGITS_output, maxSampler_maxVals, sample_output);
  for (int i = 0; i < gemmNum; ++i)
    gemms[i]->setWorkspace(tmpBufferM.allocBytes(gemms[i]->workspaceBytes()), gemms[i]->workspaceBytes());
  dual1.setWorkspace(tmpBufferM.allocBytes(dual1.workspaceBytes()), dual1.workspaceBytes());
  dual2.setWorkspace(tmpBufferM.allocBytes(dual2.workspaceBytes()), dual2.workspaceBytes());
  // e4m3 weights: the RMSNorms hand their consumers quantised rows (one image of all T rows for
  // the attention side: layerNormAttention1 covers the rows of KQV1 and KQV2)
  if (const QuantRows q = allocQuantRows(T)) {
    const size_t row0[4] = {0, k[0], k[0] + k[1], k[0] + k[1] + k[2]};
    bool all = true;
    for (int i = 0; i < 4; ++i)
      if (k[i] > 0) all &= KQV_ptrs[i]->setQuantizedA(q.at(row0[i]).q, q.at(row0[i]).scale);
    if (all) {
      layerNormAttention1.setQuantOutput(q.q, q.scale);
      if (k[2] > 0) layerNormAttention2_1.setQuantOutput(q.at(row0[2]).q, q.at(row0[2]).scale);
      if (k[3] > 0) layerNormAttention2_2.setQuantOutput(q.at(row0[3]).q, q.at(row0[3]).scale);
    } else {
      for (int i = 0; i < 4; ++i) KQV_ptrs[i]->setQuantizedA(nullptr, nullptr);
    }
  }
  if (const QuantRows q = allocQuantRows(dual1.M); q && dual1.setQuantizedA(q.q, q.scale))
    layerNormFFN1.setQuantOutput(q.q, q.scale);
  if (const QuantRows q = allocQuantRows(dual2.M); q && dual2.setQuantizedA(q.q, q.scale))
    layerNormFFN2.setQuantOutput(q.q, q.scale);
  NF_LOG_INFO("allocated num: %zu", tmpBufferM.getAllocation());
}

// One iteration's worth of enqueues (no host synchronisation inside).
void Pipeline::enqueueIteration() {
  HIP_CHECK(hipEventRecord(events[EventManager::CAPTURE_GEMM_START], stream_gemm));
  if (!nanobatch_only) HIP_CHECK(hipStreamWaitEvent(stream_gemv, events[EventManager::CAPTURE_GEMM_START], 0));
  if (enable_offload) HIP_CHECK(hipStreamWaitEvent(stream_cpy, events[EventManager::CAPTURE_GEMM_START], 0));

  genEmbedding1.run().log();
  if (KQV3->M > 0) genEmbedding2_1.run().log();
  if (KQV4->M > 0) genEmbedding2_2.run().log();

  for (int iter = 0; iter < ModelConfig.run_layer; ++iter) {
    setWeight(iter % ModelConfig.model_layer);

    layerNormAttention1.run().log();
    if (KQV3->M > 0) layerNormAttention2_1.run().log();
    if (KQV4->M > 0) layerNormAttention2_2.run().log();

    // the layer's pool must not be appended to while the previous offload round trip (which may
    // have used the same pool when run_layer > model_layer) is still writing its pages back
    if (enable_offload && iter > 0) HIP_CHECK(hipStreamWaitEvent(stream_gemm, offload_done, 0));

    for (int i = 0; i < 4; ++i) {
      if (KQV_ptrs[i]->M > 0) KQV_ptrs[i]->run().log();
      if (roPEAppends[i].dense_batch_size > 0) roPEAppends[i].run().log(); else roPEAppends[i].skip();
      if (gemvs[i]->batch_size > 0) gemvs[i]->wait(roPEAppends[i]).run().log(); else gemvs[i]->wait(roPEAppends[i]).skip();
    }
    if (update_data.prefillNum > 0) prefill.wait(roPEAppends[3]).run().log(); else prefill.wait(roPEAppends[3]).skip();

    // nano-batch 1 holds decode rows only when the first two groups fill it; otherwise some of its
    // rows are prefill rows, and prefill is the last launch on the attention stream
    OperatorWrapper* nano1_attention = &prefill;
    if ((int)config_data.nanobatch_1_size == update_data.gemv_batch_size[0] + update_data.gemv_batch_size[1])
      nano1_attention = &GEMV2;
    O1->wait(*nano1_attention).run().log();
    layerNormFFN1.run().log();
    O2->wait(GEMV4).wait(prefill).run().log();
    layerNormFFN2.run().log();
    dual1.run().log();
    D1->run().log();
    if (enable_offload && offload_pages > 0) {
      // gather -> host -> back -> scatter, beside the second nano-batch's FFN
      const size_t bytes = offload_pages * ModelConfig.page_mem_size;
      pageAgg.wait(dual1).run().log();
      HIP_CHECK(hipMemcpyAsync(offloadKVCache, deviceOffloadKVCache, bytes, hipMemcpyDeviceToHost, stream_cpy));
      HIP_CHECK(hipMemcpyAsync(deviceLoadKVCache, offloadKVCache, bytes, hipMemcpyHostToDevice, stream_cpy));
      pageDisp.run().log();
      HIP_CHECK(hipEventRecord(offload_done, stream_cpy));
    } else if (enable_offload) {
      HIP_CHECK(hipEventRecord(offload_done, stream_cpy));
    }
    dual2.run().log();
    D2->run().log();
  }

  keepToken.run().log();
  layerNormModel1.run().log();
  LOGITS->run().log();
  maxSampler.run().log();
  // the side streams rejoin the dense stream (a capture needs the joins to be explicit)
  if (!nanobatch_only) {
    HIP_CHECK(hipEventRecord(events[EventManager::CAPTURE_GEMV_END], stream_gemv));
    HIP_CHECK(hipStreamWaitEvent(stream_gemm, events[EventManager::CAPTURE_GEMV_END], 0));
  }
  if (enable_offload) HIP_CHECK(hipStreamWaitEvent(stream_gemm, offload_done, 0));
}

vortexOutputData Pipeline::run() {
  setWeight(0);
  HIP_CHECK(hipEventRecord(events[EventManager::GEMM_TIMING_START], stream_gemm));
  std::vector<int> sig = baseSignature();
  sig.push_back((int)offload_pages);
  sig.push_back(offload_reqs);  // baked into the gather / scatter launches
  runIteration(stream_gemm, sig, [this] { enqueueIteration(); });
  HIP_CHECK(hipEventRecord(events[EventManager::GEMM_TIMING_END], stream_gemm));
  HIP_CHECK(hipMemcpyAsync(output_data.sampled_token_array, maxSampler.d_argMax.ptr,
                           output_data.sampled_tokens * sizeof(int), hipMemcpyDeviceToHost, stream_gemm));
  HIP_CHECK(hipStreamSynchronize(stream_gemm));
  HIP_CHECK(hipStreamSynchronize(stream_gemv));
  HIP_CHECK(hipStreamSynchronize(stream_cpy));

  float runtime_ms = 0;
  HIP_CHECK(hipEventElapsedTime(&runtime_ms, events[EventManager::GEMM_TIMING_START],
                                events[EventManager::GEMM_TIMING_END]));
  timings.iter_ms = runtime_ms;
  if (profiling) {
    for (auto gemv : gemvs) gemv->collectProfile(timings.decode_attn_ms, timings.decode_attn_launches);
    prefill.collectProfile(timings.prefill_attn_ms, timings.prefill_attn_launches);
  }
  if (profile_gemms) {
    auto add = [&](OperatorWrapper& op, double flop) {
      const long before = timings.gemm_launches;
      op.collectProfile(timings.gemm_ms, timings.gemm_launches);
      timings.gemm_flop += flop * double(timings.gemm_launches - before);
    };
    for (auto g : gemms)
      if (g) add(*g, g->totalCompute());
    add(dual1, dual1.totalCompute());
    add(dual2, dual2.totalCompute());
  }
  NF_LOG_INFO("Total running cost (ms) of one microbatch is %f", runtime_ms);
  return output_data;
}

// Slices the iteration's request metadata over the four decode-attention launches, the prefill
// launch and the four RoPE-append launches (pipeline.cu:797-933).
void Pipeline::GEMVOpUpdate() {
  const int32_t* gb = update_data.gemv_batch_size;
  const int32_t* nb = update_data.gemv_num_blocks;
  uint32_t arr[] = {uint32_t(gb[0]), uint32_t(gb[1]), uint32_t(gb[2]), uint32_t(gb[3]), uint32_t(update_data.prefillNum)};
  std::span<uint32_t, 5> batch_sizes(arr, 5);
  const size_t total_batch_size = std::accumulate(batch_sizes.begin(), batch_sizes.end(), size_t(0));
  if ((int)total_batch_size != update_data.decodePrefillBorder + update_data.prefillNum) {
    std::fprintf(stderr, "Pipeline::update: attention groups %u+%u+%u+%u do not add up to %d decode requests\n", arr[0],
                 arr[1], arr[2], arr[3], update_data.decodePrefillBorder);
    std::exit(EXIT_FAILURE);
  }
  const auto DR = PllmDimension::ROW;
  const uint32_t T = (uint32_t)config_data.global_batch_size;
  const auto kv_indptr_split = pllmTensor<int32_t>{update_data.kv_indptr, total_batch_size + 1}.splitTensor(DR, batch_sizes, 1U);
  const auto kv_last_page_len_split = pllmTensor<int32_t>{update_data.kv_last_page_len, total_batch_size}.splitTensor(DR, batch_sizes);
  const auto input_ptr_split = pllmTensor<int32_t>{update_data.input_indptr, total_batch_size + 1}.splitTensor(DR, batch_sizes, 1U);
  pllmTensor<int32_t> kv_indices{update_data.kv_indices, ModelConfig.max_page_num};
  pllmTensor<int32_t> kv_indptr{update_data.kv_indptr, total_batch_size + 1};
  pllmTensor<int32_t> kv_last_page_len{update_data.kv_last_page_len, total_batch_size};

  const size_t k[4] = {KQV1->M, KQV2->M, KQV3->M, KQV4->M};
  const auto Q_split = gemvQ.splitTensor(DR, k[0], k[1], k[2], k[3]);
  const auto KQV_split = KQV_output.splitTensor(DR, k[0], k[1], k[2], k[3]);
  const auto rev_split = pllmTensor<int32_t>{update_data.rev_input_indptr, (size_t)T}.splitTensor(DR, k[0], k[1], k[2], k[3]);
  const auto off_split = pllmTensor<int32_t>{update_data.per_token_offset, (size_t)T}.splitTensor(DR, k[0], k[1], k[2], k[3]);

  size_t token_remaining = update_token_num;
  for (int i = 0; i < 4; ++i) {
    const size_t n = std::min(token_remaining, k[i]);
    roPEAppends[i].update((int)n, KQV_split[i], Q_split[i], rev_split[i], off_split[i], kv_indices, kv_indptr,
                          kv_last_page_len);
    token_remaining -= n;
  }
  // q / o are the base of the whole iteration buffers: rows are addressed through the absolute
  // values in the input_indptr slices
  for (int i = 0; i < 4; ++i)
    gemvs[i]->init(batch_sizes[i], nb[i], input_ptr_split[i], kv_indptr_split[i], update_data.kv_indices,
                   kv_last_page_len_split[i], gemvQ, gemvAggregateOutput);
  prefill.init(batch_sizes[4], 0, input_ptr_split[4], kv_indptr_split[4], update_data.kv_indices,
               kv_last_page_len_split[4], gemvQ, gemvAggregateOutput);

  // KV offload round trip: the first requests of the iteration, as many of their pages as the
  // staging buffers hold (planned from the staged host copy of kv_indptr)
  offload_reqs = 0;
  offload_pages = 0;
  if (enable_offload) {
    const int32_t* h_indptr = host_update_data.kv_indptr;
    while (offload_reqs < kOffloadReqs && offload_reqs < (int)total_batch_size &&
           (size_t)h_indptr[offload_reqs + 1] <= offload_pages_cap)
      ++offload_reqs;
    offload_pages = offload_reqs ? (size_t)h_indptr[offload_reqs] : 0;
    pageAgg.init(offload_reqs, finished_idx, update_data.kv_indptr, update_data.kv_indices, deviceOffloadKVCache);
    pageDisp.init(offload_reqs, load_idx, update_data.kv_indptr, update_data.kv_indices, deviceLoadKVCache);
  }
}

void Pipeline::update(vortexUpdateData* update_data_) {
  this->update_data = *update_data_;
  const int T = config_data.global_batch_size;
  const int nano1 = config_data.nanobatch_1_size, k3 = (int)KQV3->M;
  auto input_span = pllmTensor<int>(update_data.input_tokens, T, 1, PllmLayout::ROW_MAJOR);
  genEmbedding1.setInput(input_span.subtensor(0, nano1));
  if (k3 > 0) genEmbedding2_1.setInput(input_span.subtensor(nano1, k3));
  if (T - nano1 - k3 > 0) genEmbedding2_2.setInput(input_span.subtensor(nano1 + k3));

  update_token_num = update_data.decodePrefillBorder + update_data.prefillTokensNum;
  auto live = [&](int start, int len) { return std::clamp(update_token_num - start, 0, len); };
  const int live1 = live(0, nano1), live2 = live(nano1, T - nano1);
  const int starts[4] = {0, (int)KQV1->M, nano1, nano1 + k3};
  for (int i = 0; i < 4; ++i) KQV_ptrs[i]->set_live_rows((size_t)live(starts[i], (int)KQV_ptrs[i]->M));
  for (BaseGEMMWrapper* g : {O1, D1}) g->set_live_rows((size_t)live1);
  for (BaseGEMMWrapper* g : {O2, D2}) g->set_live_rows((size_t)live2);
  dual1.set_live_rows(live1);
  dual2.set_live_rows(live2);
  genEmbedding1.set_live_rows(live1);
  genEmbedding2_1.set_live_rows(live(nano1, k3));
  genEmbedding2_2.set_live_rows(live(nano1 + k3, T - nano1 - k3));
  layerNormAttention1.set_live_rows(live1);
  layerNormAttention2_1.set_live_rows(live(nano1, k3));
  layerNormAttention2_2.set_live_rows(live(nano1 + k3, T - nano1 - k3));
  layerNormFFN1.set_live_rows(live1);
  layerNormFFN2.set_live_rows(live2);

  const int req_num = update_data.decodePrefillBorder + update_data.prefillNum;
  maxSampler.set_batch_size(req_num);
  keepToken.update(req_num, update_data.input_indptr);
  // LM-head rows are padded up to a multiple of 128 as in the reference (pipeline.cu:985-988)
  LOGITS->set_shape(std::min((req_num + 127) / 128 * 128, T), (int)ModelConfig.vocab_size, ModelConfig.model_hidden_dim);
  LOGITS->init();
  layerNormModel1.set_live_rows((int)LOGITS->M);
  output_data.sampled_tokens = req_num;
  GEMVOpUpdate();
  NF_LOG_INFO("prefill: %d, decode: %d; Batch size: %d, %d, %d, %d", update_data.prefillNum,
              update_data.decodePrefillBorder, update_data.gemv_batch_size[0], update_data.gemv_batch_size[1],
              update_data.gemv_batch_size[2], update_data.gemv_batch_size[3]);
}

void Pipeline::config(vortexConfigData* config_data_) {
  NF_LOG_INFO("Config pipeline (four QKV / attention nano-batches)");
  clearGraphs();  // the buffer plan below may move every operand
  config_error.clear();
  for (auto*& g : gemms) {  // a second config() replaces the wrappers of the first
    delete g;
    g = nullptr;
  }
  this->config_data = *config_data_;
  for (int i = 0; i < gemmNum; ++i) {
    const std::string& tag =
        i < (int)config_data.gemm_op_tag.size() ? config_data.gemm_op_tag[i] : std::string(gemmConfig[i]);
    // the LM head stays fp16 in both weight formats
    gemms[i] = generateGEMM(tag, i == static_cast<int>(GEMM_NAME::LOGITS) ? WeightFormat::F16 : weight_format);
    if (!gemms[i]) {
      configFail("Pipeline::config: cannot build GEMM %d from tag \"%s\"", i, tag.c_str());
      return;
    }
  }
  KQV_ptrs[0] = KQV1;
  KQV_ptrs[1] = KQV2;
  KQV_ptrs[2] = KQV3;
  KQV_ptrs[3] = KQV4;
  const int T = config_data.global_batch_size;
  const int nano1 = config_data.nanobatch_1_size, nano2 = T - nano1;
  const int k1 = config_data.kqv1_size, k3 = config_data.kqv3_size;
  if (nano1 <= 0 || nano2 <= 0 || T > ModelConfig.max_batch_size || k1 < 0 || k1 > nano1 || k3 < 0 || k3 > nano2) {
    configFail("Pipeline::config: bad nano-batch split %d + %d with QKV cuts %d, %d (max batch %d)", nano1,
                 nano2, k1, k3, ModelConfig.max_batch_size);
      return;
  }
  const int kqv_n = (2 * ModelConfig.model_kv_heads_gpu + ModelConfig.model_qo_heads_gpu) * ModelConfig.model_head_dim;
  const int H = ModelConfig.model_hidden_dim;
  O1->set_shape(nano1, ModelConfig.model_hidden_dim_pergpu, H);
  O2->set_shape(nano2, ModelConfig.model_hidden_dim_pergpu, H);
  D1->set_shape(nano1, H, ModelConfig.model_ff_dim_gpu);
  D2->set_shape(nano2, H, ModelConfig.model_ff_dim_gpu);
  KQV1->set_shape(k1, kqv_n, H);
  KQV2->set_shape(nano1 - k1, kqv_n, H);
  KQV3->set_shape(k3, kqv_n, H);
  KQV4->set_shape(nano2 - k3, kqv_n, H);
  LOGITS->set_shape(T / nranks, (int)ModelConfig.vocab_size, H);
  dual1.set_shape(nano1, ModelConfig.model_ff_dim_gpu, H);
  dual2.set_shape(nano2, ModelConfig.model_ff_dim_gpu, H);
  dual1.setWeightFormat(weight_format);
  dual1.setWeightLayout(pairWeightLayout(gemms, static_cast<int>(GEMM_NAME::LOGITS)));
  dual2.setWeightFormat(weight_format);
  dual2.setWeightLayout(pairWeightLayout(gemms, static_cast<int>(GEMM_NAME::LOGITS)));

  setName();
  ScheduleInit();
  GEMMOpInit();
  GEMVOpInit();
  OtherOpInit();

  output_data = vortexOutputData();
  output_data.sampled_token_array = new int[T];
  output_data.global_batch_size = T;
  if (profiling) setProfiling(profilingLevel());
}
