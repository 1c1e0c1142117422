// LocalPipeline: the single-GPU nano-batch schedule.
//
// The iteration's dense batch is cut into two nano-batches (rows [0, nano1) and [nano1, T)).
// Dense operators (RMSNorm, QKV / O / gate-up / down GEMMs, RoPE-append) of both nano-batches
// are enqueued on stream_gemm, attention of both on stream_gemv, so the memory-bound attention
// of one nano-batch overlaps the MFMA-bound GEMMs of the other; the only cross-stream edges
// are event waits.  Operator order and dependencies follow the reference's
// LocalPipeline::run (pipeline/src/pipeline_local.cpp counterpart: pipeline_local.cu:319-469),
// buffer plan :198-317, per-iteration attention slicing :514-801, config :846-899.
//
// Differences on purpose (same results):
//  * update() plans from the host copy of the update data and patches the border-straddling
//    prefill request on the host; the reference reads the values back from the device with
//    blocking copies (pipeline_local.cu:670-716,821).
//  * attention planning runs on the device inside the attention launch.
//  * streams may be restricted to disjoint CU sets (NANOFLOW_GEMM_CUS / NANOFLOW_GEMV_CUS).
#include "pipeline.h"

#include <cstdlib>
#include <numeric>

#include "tensorManager.h"

PipelineBase::PipelineBase(vortexInitData* input_data, int nrank, int nranks, int vnranks)
    : input_data(input_data),
      rank(nrank),
      nranks(nranks),
      vnranks(vnranks),
      tmpBufferM(input_data->tmp_buffer, input_data->tmp_buffer_size) {
  tensorlog::configure();  // NANOFLOW_TENSOR_LOG is read when a pipeline is created
}

static int env_int(const char* name, int dflt) {
  const char* v = std::getenv(name);
  return v && *v ? std::atoi(v) : dflt;
}

// CUs first_cu .. first_cu + num_cus - 1 in the numbering of the CU mask, whose bit i is a CU of XCD
// i % 8 on this part: a range of 8 n bits is n CUs of every XCD, so both streams of a split keep
// all eight L2s and memory ports.
hipStream_t createPipelineStream(int first_cu, int num_cus) {
  hipStream_t s = nullptr;
  if (num_cus <= 0) {
    HIP_CHECK(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
    return s;
  }
  hipDeviceProp_t prop;
  int dev = 0;
  HIP_CHECK(hipGetDevice(&dev));
  HIP_CHECK(hipGetDeviceProperties(&prop, dev));
  const int total = prop.multiProcessorCount;
  const int words = (total + 31) / 32;
  std::vector<uint32_t> mask(words, 0u);
  for (int cu = first_cu; cu < first_cu + num_cus && cu < total; ++cu) mask[cu / 32] |= 1u << (cu % 32);
  HIP_CHECK(hipExtStreamCreateWithCUMask(&s, (uint32_t)words, mask.data()));
  return s;
}

LocalPipeline::LocalPipeline(vortexInitData* input_data, int nrank, int nranks, int vnranks,
                             bool nanobatch_only, bool kqv_bias_)
    : PipelineBase(input_data, nrank, nranks, vnranks), nanobatch_only(nanobatch_only) {
  kqv_bias = kqv_bias_;
  init();
}

LocalPipeline::~LocalPipeline() {
  clearGraphs();
  for (auto g : gemms) delete g;
  delete[] output_data.sampled_token_array;
  if (prefill1_update.input_indptr) (void)hipFree(prefill1_update.input_indptr);
  if (prefill1_update.kv_indptr) (void)hipFree(prefill1_update.kv_indptr);
  if (prefill1_update.kv_last_page_len) (void)hipFree(prefill1_update.kv_last_page_len);
  if (prefill1_staging.input_indptr) (void)hipHostFree(prefill1_staging.input_indptr);
  if (prefill1_staging.kv_indptr) (void)hipHostFree(prefill1_staging.kv_indptr);
  if (prefill1_staging.kv_last_page_len) (void)hipHostFree(prefill1_staging.kv_last_page_len);
  if (stream_gemm) (void)hipStreamDestroy(stream_gemm);
  if (stream_gemv) (void)hipStreamDestroy(stream_gemv);
  if (stream_other) (void)hipStreamDestroy(stream_other);
}

void LocalPipeline::init() {
  // Optional CU partition: GEMM stream on CUs [0, g), attention stream on [g, g + a).
  const int gemm_cus = env_int("NANOFLOW_GEMM_CUS", 0);
  const int gemv_cus = env_int("NANOFLOW_GEMV_CUS", 0);
  masked_streams = gemm_cus > 0 || gemv_cus > 0;
  stream_gemm = createPipelineStream(0, gemm_cus);
  stream_gemv = createPipelineStream(gemm_cus, gemv_cus);
  stream_other = createPipelineStream(0, 0);
  NF_LOG_INFO("Init pipeline (local): gemm CUs %d, attention CUs %d (0 = all)", gemm_cus, gemv_cus);
}

void LocalPipeline::setName() {
  SET_NAME_PTR(O1);
  SET_NAME_PTR(O2);
  SET_NAME_PTR(D1);
  SET_NAME_PTR(D2);
  SET_NAME_PTR(KQV1);
  SET_NAME_PTR(KQV2);
  SET_NAME_PTR(LOGITS);
  SET_NAME_REF(dual1);
  SET_NAME_REF(dual2);
  SET_NAME_REF(genEmbedding1);
  SET_NAME_REF(genEmbedding2);
  SET_NAME_REF(GEMV1);
  SET_NAME_REF(GEMV2);
  SET_NAME_REF(GEMV3);
  SET_NAME_REF(GEMV4);
  SET_NAME_REF(prefill1);
  SET_NAME_REF(prefill2);
  SET_NAME_REF(layerNormAttention1);
  SET_NAME_REF(layerNormAttention2);
  SET_NAME_REF(layerNormFFN1);
  SET_NAME_REF(layerNormFFN2);
  SET_NAME_REF(layerNormModel);
  SET_NAME_REF(roPEAppends[0]);
  SET_NAME_REF(roPEAppends[1]);
  SET_NAME_REF(maxSampler);
  SET_NAME_REF(keepToken);
}

void LocalPipeline::assignSameStream() {
  for (auto gemv : gemvs) gemv->setStream(stream_gemm);
  prefill1.setStream(stream_gemm);
  prefill2.setStream(stream_gemm);
}

void LocalPipeline::setProfiling(int level) {
  profiling = level > 0;
  profile_gemms = level > 1;
  const unsigned stride = profileStride();
  timings.layer_stride = (int)stride;
  const size_t n = profiling ? (size_t)ModelConfig.run_layer : 0;
  for (auto gemv : gemvs) gemv->enableProfiling(n, stride);
  prefill1.enableProfiling(n, stride);
  prefill2.enableProfiling(n, stride);
  const size_t ng = profile_gemms ? (size_t)ModelConfig.run_layer : 0;
  for (auto g : gemms)
    if (g) g->enableProfiling(ng, stride);
  dual1.enableProfiling(ng, stride);
  dual2.enableProfiling(ng, stride);
}

void LocalPipeline::setWeight(int layer) {
  auto& lw = input_data->weight.layer_weight[layer];
  bool success = true;
  success &= O1->set_weight(lw.W_O1);
  success &= O2->set_weight(lw.W_O2);
  success &= D1->set_weight(lw.W_D);
  success &= D2->set_weight(lw.W_D);
  success &= KQV1->set_weight(lw.W_KQV);
  success &= KQV2->set_weight(lw.W_KQV);
  success &= bindKQVBias(KQV1, lw.B_KQV);
  success &= bindKQVBias(KQV2, lw.B_KQV);
  success &= layerNormAttention1.setWeight(lw.W_LN_Attention);
  success &= layerNormAttention2.setWeight(lw.W_LN_Attention);
  success &= layerNormFFN1.setWeight(lw.W_LN_FFN);
  success &= layerNormFFN2.setWeight(lw.W_LN_FFN);
  success &= dual1.set_weight(lw.W_G, lw.W_U);
  success &= dual2.set_weight(lw.W_G, lw.W_U);
  if (!success) NF_LOG_ERROR("Failed to set weight for layer %d", layer);
  for (auto gemv : gemvs) gemv->setKVData(input_data->kv_data[layer]);
  prefill1.setKVData(input_data->kv_data[layer]);
  prefill2.setKVData(input_data->kv_data[layer]);
  roPEAppends[0].setKVData(input_data->kv_data[layer]);
  roPEAppends[1].setKVData(input_data->kv_data[layer]);
}

// Weights of the second half of a layer (O, FFN norm, gate/up, down) and the KV pool the
// attention ops read.
void LocalPipeline::setWeight_group_O(int layer) {
  auto& lw = input_data->weight.layer_weight[layer];
  bool success = true;
  success &= O1->set_weight(lw.W_O1);
  success &= O2->set_weight(lw.W_O2);
  success &= layerNormFFN1.setWeight(lw.W_LN_FFN);
  success &= layerNormFFN2.setWeight(lw.W_LN_FFN);
  success &= dual1.set_weight(lw.W_G, lw.W_U);
  success &= dual2.set_weight(lw.W_G, lw.W_U);
  success &= D1->set_weight(lw.W_D);
  success &= D2->set_weight(lw.W_D);
  if (!success) NF_LOG_ERROR("Failed to set weight group 1 for layer %d", layer);
  for (auto gemv : gemvs) gemv->setKVData(input_data->kv_data[layer]);
  prefill1.setKVData(input_data->kv_data[layer]);
  prefill2.setKVData(input_data->kv_data[layer]);
}

// Weights of the first half of a layer (attention norm, QKV) and the KV pool RoPE-append
// writes.
void LocalPipeline::setWeight_group_LN(int layer) {
  auto& lw = input_data->weight.layer_weight[layer];
  bool success = true;
  success &= layerNormAttention1.setWeight(lw.W_LN_Attention);
  success &= layerNormAttention2.setWeight(lw.W_LN_Attention);
  success &= KQV1->set_weight(lw.W_KQV);
  success &= KQV2->set_weight(lw.W_KQV);
  success &= bindKQVBias(KQV1, lw.B_KQV);
  success &= bindKQVBias(KQV2, lw.B_KQV);
  if (!success) NF_LOG_ERROR("Failed to set weight group 2 for layer %d", layer);
  roPEAppends[0].setKVData(input_data->kv_data[layer]);
  roPEAppends[1].setKVData(input_data->kv_data[layer]);
}

void LocalPipeline::GEMMOpInit() {
  setWeight(0);
  O1->init(1.f);  // O and D add the residual stream through C (beta = 1)
  O2->init(1.f);
  D1->init(1.f);
  D2->init(1.f);
  KQV1->init(kqv_bias ? 1.f : 0.f);
  KQV2->init(kqv_bias ? 1.f : 0.f);
  LOGITS->set_weight(input_data->weight.lm_head);
  LOGITS->init();
  for (int i = 0; i < gemmNum; ++i) {
    gemms[i]->setStream(stream_gemm);
    gemms[i]->updateEventExistance(false, false);
  }
  dual1.init();
  dual2.init();
  dual1.setStream(stream_gemm);
  dual2.setStream(stream_gemm);
}

void LocalPipeline::GEMVOpInit() {
  for (auto gemv : gemvs) gemv->setStream(stream_gemv);
  prefill1.setStream(stream_gemv);
  prefill2.setStream(stream_gemv);
}

void LocalPipeline::OtherOpInit() {
  genEmbedding1.setWeight(input_data->weight.embedding);
  genEmbedding2.setWeight(input_data->weight.embedding);
  layerNormModel.setWeight(input_data->weight.model_layernorm);
  genEmbedding1.setStream(stream_gemm).updateEventExistance(false, false);
  genEmbedding2.setStream(stream_gemm).updateEventExistance(false, false);
  layerNormAttention1.setStream(stream_gemm).updateEventExistance(false, false);
  layerNormAttention2.setStream(stream_gemm).updateEventExistance(false, false);
  layerNormFFN1.setStream(stream_gemm).updateEventExistance(false, false);
  layerNormFFN2.setStream(stream_gemm).updateEventExistance(false, false);
  layerNormModel.setStream(stream_gemm);
  roPEAppends[0].setStream(stream_gemm);
  roPEAppends[1].setStream(stream_gemm);
  maxSampler.setStream(stream_gemm);
  keepToken.setStream(stream_gemm);
}

// Carves every intermediate out of tmp_buffer and wires operator inputs/outputs.
// The residual stream lives in the D-output buffer: the embedding writes it, O adds it
// (C = D output), D adds the O output (C = O output).
void LocalPipeline::ScheduleInit() {
  const int kdim = ModelConfig.model_head_dim * ModelConfig.model_kv_heads_gpu;
  const int qdim = ModelConfig.model_head_dim * ModelConfig.model_qo_heads_gpu;
  const int vdim = kdim;
  const int T = config_data.global_batch_size;
  const auto ROW = PllmLayout::ROW_MAJOR;

  const auto KQV_shared_output = tmpBufferM.allocTensor(T, kdim + qdim + vdim, ROW);
  const auto KQV_output12 = KQV_shared_output.splitTensor(PllmDimension::ROW, O1->M, O2->M);
  KQV_output1 = KQV_output12[0];
  KQV_output2 = KQV_output12[1];

  const auto gemvQ = tmpBufferM.allocTensor(T, qdim, ROW);
  const auto gemvQ12 = gemvQ.splitTensor(PllmDimension::ROW, O1->M, O2->M);
  gemvQ1 = gemvQ12[0];
  gemvQ2 = gemvQ12[1];

  const auto GEMV_shared_output = tmpBufferM.allocTensor(T, ModelConfig.model_hidden_dim_pergpu, ROW);
  const auto gemvAggregateOutput12 = GEMV_shared_output.splitTensor(PllmDimension::ROW, O1->M, O2->M);
  gemvAggregateOutput1 = gemvAggregateOutput12[0];
  gemvAggregateOutput2 = gemvAggregateOutput12[1];

  const auto D_shared_output = tmpBufferM.allocTensor(T, (int)D1->N, ROW);
  const auto D_output12 = D_shared_output.splitTensor(PllmDimension::ROW, D1->M, D2->M);

  // nano-batch 1
  const auto D1_output = D_output12[0];
  genEmbedding1.setOutput(D1_output);
  const auto layerNormAttention1_output = tmpBufferM.allocTensor((int)D1->M, (int)D1->N, ROW);
  layerNormAttention1.setInput(D1_output).setOutput(layerNormAttention1_output);
  KQV1->setA(layerNormAttention1_output).setOutput(KQV_output12[0]);
  O1->setA(gemvAggregateOutput12[0]);
  const auto O1_output = tmpBufferM.allocTensor((int)O1->M, (int)O1->N, ROW);
  O1->setC(D1_output);
  O1->setD(O1_output);
  layerNormFFN1.setInput(O1_output);
  const auto LayerNormFFN1_output = tmpBufferM.allocTensor(dual1.M, dual1.K, ROW);
  layerNormFFN1.setOutput(LayerNormFFN1_output);
  const auto activation1_output = tmpBufferM.allocTensor((int)D1->M, (int)D1->K, ROW);
  dual1.setA(LayerNormFFN1_output);
  dual1.setD(pllmTensor<half>(), pllmTensor<half>(), activation1_output);
  D1->setA(activation1_output);
  D1->setC(O1_output);
  D1->setD(D1_output);

  // nano-batch 2
  const auto D2_output = D_output12[1];
  genEmbedding2.setOutput(D2_output);
  const auto layerNormAttention2_output = tmpBufferM.allocTensor((int)D2->M, (int)D2->N, ROW);
  layerNormAttention2.setInput(D2_output).setOutput(layerNormAttention2_output);
  KQV2->setA(layerNormAttention2_output).setOutput(KQV_output12[1]);
  O2->setA(gemvAggregateOutput12[1]);
  const auto O2_output = tmpBufferM.allocTensor((int)O2->M, (int)O2->N, ROW);
  O2->setC(D2_output);
  O2->setD(O2_output);
  layerNormFFN2.setInput(O2_output);
  const auto LayerNormFFN2_output = tmpBufferM.allocTensor(dual2.M, dual2.K, ROW);
  layerNormFFN2.setOutput(LayerNormFFN2_output);
  const auto activation2_output = tmpBufferM.allocTensor((int)D2->M, (int)D2->K, ROW);
  dual2.setA(LayerNormFFN2_output);
  dual2.setD(pllmTensor<half>(), pllmTensor<half>(), activation2_output);
  D2->setA(activation2_output);
  D2->setC(O2_output);
  D2->setD(D2_output);

  // sampling: last token of each request -> final norm -> LM head -> argmax
  const auto keepTokenOutput = tmpBufferM.allocTensor(T, (int)D2->N, ROW);
  keepToken.setInput(D_shared_output).setOutput(keepTokenOutput);
  const auto layerNormModel_output = tmpBufferM.allocTensor(T, (int)D2->N, ROW);
  layerNormModel.setInput(keepTokenOutput).setOutput(layerNormModel_output);
  const auto LOGITS_output = tmpBufferM.allocTensor(T, (int)LOGITS->N, ROW);
  LOGITS->setA(layerNormModel_output);
  LOGITS->setOutput(LOGITS_output);
  int* sample_output_alloc = (int*)tmpBufferM.alloc((size_t)T * sizeof(int) / sizeof(half));
  pllmTensor<int> sample_output = {sample_output_alloc, T, 1, ROW};
  const auto maxSampler_maxVals = tmpBufferM.allocTensor(T, 1, ROW);
  maxSampler.init(LOGITS_output, maxSampler_maxVals, sample_output);
  // scratch of the fp8-weight wrappers (none for fp16 weights)
  for (int i = 0; i < gemmNum; ++i)
    gemms[i]->setWorkspace(tmpBufferM.allocBytes(gemms[i]->workspaceBytes()), gemms[i]->workspaceBytes());
  dual1.setWorkspace(tmpBufferM.allocBytes(dual1.workspaceBytes()), dual1.workspaceBytes());
  dual2.setWorkspace(tmpBufferM.allocBytes(dual2.workspaceBytes()), dual2.workspaceBytes());
  // e4m3 weights: the RMSNorms hand their consumers quantised rows
  if (const QuantRows q = allocQuantRows(KQV1->M); q && KQV1->setQuantizedA(q.q, q.scale))
    layerNormAttention1.setQuantOutput(q.q, q.scale);
  if (const QuantRows q = allocQuantRows(KQV2->M); q && KQV2->setQuantizedA(q.q, q.scale))
    layerNormAttention2.setQuantOutput(q.q, q.scale);
  if (const QuantRows q = allocQuantRows(dual1.M); q && dual1.setQuantizedA(q.q, q.scale))
    layerNormFFN1.setQuantOutput(q.q, q.scale);
  if (const QuantRows q = allocQuantRows(dual2.M); q && dual2.setQuantizedA(q.q, q.scale))
    layerNormFFN2.setQuantOutput(q.q, q.scale);
  NF_LOG_INFO("allocated num: %zu", tmpBufferM.getAllocation());
}

// One iteration's worth of enqueues (no host synchronisation inside).
void LocalPipeline::enqueueIteration() {
  HIP_CHECK(hipEventRecord(events[EventManager::CAPTURE_GEMM_START], stream_gemm));
  HIP_CHECK(hipStreamWaitEvent(stream_gemv, events[EventManager::CAPTURE_GEMM_START], 0));

  genEmbedding1.run().log();
  genEmbedding2.run().log();

  // prologue: first half of layer 0 for both nano-batches
  setWeight_group_LN(0);
  layerNormAttention1.run().log();
  KQV1->run().log();
  if (roPEAppends[0].dense_batch_size > 0) roPEAppends[0].run().log(); else roPEAppends[0].skip();
  layerNormAttention2.run().log();
  KQV2->run().log();
  if (roPEAppends[1].dense_batch_size > 0) roPEAppends[1].run().log(); else roPEAppends[1].skip();

  for (int iter = 0; iter < ModelConfig.run_layer; ++iter) {
    setWeight_group_O(iter % ModelConfig.model_layer);

    // attention of nano-batch 1 (stream_gemv)
    if (GEMV1.batch_size > 0) GEMV1.wait(roPEAppends[0]).run().log(); else GEMV1.skip();
    if (GEMV2.batch_size > 0) GEMV2.wait(roPEAppends[0]).run().log(); else GEMV2.skip();
    if (prefill1.batch_size > 0) prefill1.wait(roPEAppends[0]).run().log(); else prefill1.skip();

    // dense half of nano-batch 1 (stream_gemm)
    O1->wait(prefill1).wait(GEMV2).run().log();
    layerNormFFN1.run().log();
    dual1.run().log();
    D1->run().log();

    // attention of nano-batch 2 overlaps the dense ops above
    if (GEMV3.batch_size > 0) GEMV3.wait(roPEAppends[1]).run().log(); else GEMV3.skip();
    if (GEMV4.batch_size > 0) GEMV4.wait(roPEAppends[1]).run().log(); else GEMV4.skip();
    if (prefill2.batch_size > 0) prefill2.wait(roPEAppends[1]).wait(dual1).run().log(); else prefill2.skip();

    setWeight_group_LN((iter + 1) % ModelConfig.model_layer);

    if (iter != ModelConfig.run_layer - 1) {
      layerNormAttention1.run().log();
      KQV1->run().log();
      if (roPEAppends[0].dense_batch_size > 0) roPEAppends[0].run().log(); else roPEAppends[0].skip();
    }

    O2->wait(prefill2).run().log();
    layerNormFFN2.run().log();
    dual2.run().log();
    D2->run().log();

    if (iter != ModelConfig.run_layer - 1) {
      layerNormAttention2.run().log();
      KQV2->run().log();
      if (roPEAppends[1].dense_batch_size > 0) roPEAppends[1].run().log(); else roPEAppends[1].skip();
    }
  }

  keepToken.run().log();
  layerNormModel.run().log();
  LOGITS->run().log();
  maxSampler.run().log();
  // the attention stream rejoins the dense stream (all of its launches are already ordered
  // before O1/O2; a capture needs the join to be explicit)
  HIP_CHECK(hipEventRecord(events[EventManager::CAPTURE_GEMV_END], stream_gemv));
  HIP_CHECK(hipStreamWaitEvent(stream_gemm, events[EventManager::CAPTURE_GEMV_END], 0));
}

vortexOutputData LocalPipeline::run() {
  setWeight(0);
  HIP_CHECK(hipEventRecord(events[EventManager::GEMM_TIMING_START], stream_gemm));
  // The attention slices also depend on which request straddles the nano-batch border (a
  // function of the individual prefill lengths, not of their total): it is part of the signature.
  std::vector<int> sig = baseSignature();
  sig.push_back(border_request);
  sig.push_back((int)prefill1.batch_size);
  sig.push_back((int)prefill2.batch_size);
  runIteration(stream_gemm, sig, [this] { enqueueIteration(); });
  // the sampler (stream_gemm) depends on every attention launch through O1/O2
  HIP_CHECK(hipEventRecord(events[EventManager::GEMM_TIMING_END], stream_gemm));
  HIP_CHECK(hipMemcpyAsync(output_data.sampled_token_array, maxSampler.d_argMax.ptr,
                           output_data.sampled_tokens * sizeof(int), hipMemcpyDeviceToHost,
                           stream_gemm));
  HIP_CHECK(hipStreamSynchronize(stream_gemm));
  HIP_CHECK(hipStreamSynchronize(stream_gemv));

  float runtime_ms = 0;
  HIP_CHECK(hipEventElapsedTime(&runtime_ms, events[EventManager::GEMM_TIMING_START],
                                events[EventManager::GEMM_TIMING_END]));
  timings.iter_ms = runtime_ms;
  if (profiling) {
    for (auto gemv : gemvs) gemv->collectProfile(timings.decode_attn_ms, timings.decode_attn_launches);
    prefill1.collectProfile(timings.prefill_attn_ms, timings.prefill_attn_launches);
    prefill2.collectProfile(timings.prefill_attn_ms, timings.prefill_attn_launches);
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
  NF_LOG_INFO("Total running cost (ms) of one microbatch is %f (%.1f token/s)", runtime_ms,
              config_data.global_batch_size / (runtime_ms / 1000.0));
  return output_data;
}

// Slices the iteration's request metadata over the six attention launches
// (GEMV1, GEMV2, prefill1 | GEMV3, GEMV4, prefill2) and the two RoPE-append launches.
void LocalPipeline::GEMVOpUpdate() {
  const int nano1 = config_data.nanobatch_1_size;
  const int dpb = update_data.decodePrefillBorder;
  bool need_overlap = true;  // a prefill request straddles the nano-batch border
  border_request = -1;
  if (nano1 >= update_token_num) need_overlap = false;
  else if (dpb >= nano1) need_overlap = false;

  const size_t req_num = dpb + update_data.prefillNum;
  const uint32_t T = (uint32_t)config_data.global_batch_size;

  pllmTensor<int32_t> kv_indptr{update_data.kv_indptr, req_num + 1};
  pllmTensor<int32_t> kv_last_page_len{update_data.kv_last_page_len, req_num};
  pllmTensor<int32_t> kv_indices{update_data.kv_indices, ModelConfig.max_page_num};
  pllmTensor<int32_t> input_ptr{update_data.input_indptr, req_num + 1};
  pllmTensor<int32_t> rev_input_indptr{update_data.rev_input_indptr, (size_t)T};
  pllmTensor<int32_t> per_token_offset{update_data.per_token_offset, (size_t)T};

  const pllmTensor<half> KQV_split[] = {KQV_output1, KQV_output2};
  const pllmTensor<half> Q_split[] = {gemvQ1, gemvQ2};
  const auto rev_input_indptr_split = rev_input_indptr.splitTensor(PllmDimension::ROW, KQV1->M, KQV2->M);
  const auto per_token_offset_split = per_token_offset.splitTensor(PllmDimension::ROW, KQV1->M, KQV2->M);
  const int32_t* nb = update_data.gemv_num_blocks;
  const int32_t* gb = update_data.gemv_batch_size;

  if (!need_overlap) {
    // Either the whole iteration fits nano-batch 1 (all prefill requests go to prefill1) or
    // the decode rows reach the border (all prefill rows lie in nano-batch 2).  When the
    // tokens fill nano-batch 1 exactly the reference sends the prefill requests to prefill2
    // (pipeline_local.cu:551-555), which O1 does not wait for; they belong to prefill1.
    int nano1_prefill_size = update_data.prefillNum;
    int nano2_prefill_size = 0;
    if (nano1 < update_token_num) {
      assert(nano1 <= dpb);
      nano1_prefill_size = 0;
      nano2_prefill_size = update_data.prefillNum;
    }
    uint32_t arr[] = {uint32_t(gb[0]), uint32_t(gb[1]), uint32_t(nano1_prefill_size),
                      uint32_t(gb[2]), uint32_t(gb[3]), uint32_t(nano2_prefill_size)};
    NF_LOG_INFO("GEMVOpUpdate: local, batch_sizes: %u, %u, %u, %u, %u, %u", arr[0], arr[1], arr[2],
                arr[3], arr[4], arr[5]);
    std::span<uint32_t, 6> batch_sizes(arr, 6);
    const auto kv_indptr_split = kv_indptr.splitTensor(PllmDimension::ROW, batch_sizes, 1U);
    const auto kv_last_page_len_split = kv_last_page_len.splitTensor(PllmDimension::ROW, batch_sizes);
    const auto input_ptr_split = input_ptr.splitTensor(PllmDimension::ROW, batch_sizes, 1U);

    // q / o are the base of the whole iteration buffers: rows are addressed through the
    // absolute values in the input_indptr slices.
    GEMV1.init(batch_sizes[0], nb[0], input_ptr_split[0], kv_indptr_split[0], update_data.kv_indices,
               kv_last_page_len_split[0], gemvQ1, gemvAggregateOutput1);
    GEMV2.init(batch_sizes[1], nb[1], input_ptr_split[1], kv_indptr_split[1], update_data.kv_indices,
               kv_last_page_len_split[1], gemvQ1, gemvAggregateOutput1);
    prefill1.init(batch_sizes[2], 0, input_ptr_split[2], kv_indptr_split[2], update_data.kv_indices,
                  kv_last_page_len_split[2], gemvQ1, gemvAggregateOutput1);
    GEMV3.init(batch_sizes[3], nb[2], input_ptr_split[3], kv_indptr_split[3], update_data.kv_indices,
               kv_last_page_len_split[3], gemvQ1, gemvAggregateOutput1);
    GEMV4.init(batch_sizes[4], nb[3], input_ptr_split[4], kv_indptr_split[4], update_data.kv_indices,
               kv_last_page_len_split[4], gemvQ1, gemvAggregateOutput1);
    prefill2.init(batch_sizes[5], 0, input_ptr_split[5], kv_indptr_split[5], update_data.kv_indices,
                  kv_last_page_len_split[5], gemvQ1, gemvAggregateOutput1);
  } else {
    // The request that owns row nano1-1 is cut: prefill1 sees it truncated at the border
    // (patched copies of input_indptr / kv_indptr / kv_last_page_len), prefill2 sees it whole.
    const vortexUpdateData& h = host_update_data;
    const int border_prefill_request = h.rev_input_indptr[nano1 - 1];
    border_request = border_prefill_request;
    assert(border_prefill_request - dpb >= 0);
    assert(update_data.prefillNum + dpb - border_prefill_request >= 0);
    uint32_t arr[] = {uint32_t(gb[0]), uint32_t(gb[1]), uint32_t(border_prefill_request - dpb),
                      0, 0, uint32_t(update_data.prefillNum + dpb - border_prefill_request)};
    std::span<uint32_t, 6> batch_sizes_for_split(arr, 6);
    uint32_t suffix_arr[] = {1, 1, 2, 1, 1, 1};
    std::span<uint32_t, 6> suffix(suffix_arr, 6);
    uint32_t suffix_lpl_arr[] = {0, 0, 1, 0, 0, 0};
    std::span<uint32_t, 6> suffix_for_last_page_len(suffix_lpl_arr, 6);

    const auto kv_indptr_split = kv_indptr.splitTensor(PllmDimension::ROW, batch_sizes_for_split, suffix);
    const auto kv_last_page_len_split =
        kv_last_page_len.splitTensor(PllmDimension::ROW, batch_sizes_for_split, suffix_for_last_page_len);
    const auto input_ptr_split = input_ptr.splitTensor(PllmDimension::ROW, batch_sizes_for_split, suffix);

    const int page = ModelConfig.frame_page_size;
    const int seq_len = h.per_token_offset[nano1 - 1] + 1;  // KV length up to the border row
    const int num_page = (seq_len + page - 1) / page;
    const int last_page_len = (seq_len - 1) % page + 1;

    std::memcpy(prefill1_staging.input_indptr, h.input_indptr, (req_num + 1) * sizeof(int32_t));
    prefill1_staging.input_indptr[border_prefill_request + 1] = nano1;
    std::memcpy(prefill1_staging.kv_indptr, h.kv_indptr, (req_num + 1) * sizeof(int32_t));
    prefill1_staging.kv_indptr[border_prefill_request + 1] =
        prefill1_staging.kv_indptr[border_prefill_request] + num_page;
    std::memcpy(prefill1_staging.kv_last_page_len, h.kv_last_page_len, req_num * sizeof(int32_t));
    prefill1_staging.kv_last_page_len[border_prefill_request] = last_page_len;
    HIP_CHECK(hipMemcpyAsync(prefill1_update.input_indptr, prefill1_staging.input_indptr,
                             (req_num + 1) * sizeof(int32_t), hipMemcpyHostToDevice, stream_gemm));
    HIP_CHECK(hipMemcpyAsync(prefill1_update.kv_indptr, prefill1_staging.kv_indptr,
                             (req_num + 1) * sizeof(int32_t), hipMemcpyHostToDevice, stream_gemm));
    HIP_CHECK(hipMemcpyAsync(prefill1_update.kv_last_page_len, prefill1_staging.kv_last_page_len,
                             req_num * sizeof(int32_t), hipMemcpyHostToDevice, stream_gemm));

    pllmTensor<int32_t> p1_input{prefill1_update.input_indptr, req_num + 1};
    pllmTensor<int32_t> p1_kv_indptr{prefill1_update.kv_indptr, req_num + 1};
    pllmTensor<int32_t> p1_lpl{prefill1_update.kv_last_page_len, req_num};
    const auto p1_input_split = p1_input.splitTensor(PllmDimension::ROW, batch_sizes_for_split, suffix);
    const auto p1_kv_indptr_split = p1_kv_indptr.splitTensor(PllmDimension::ROW, batch_sizes_for_split, suffix);
    const auto p1_lpl_split = p1_lpl.splitTensor(PllmDimension::ROW, batch_sizes_for_split, suffix_for_last_page_len);

    uint32_t actual[6] = {arr[0], arr[1], arr[2] + 1, arr[3], arr[4], arr[5]};
    GEMV1.init(actual[0], nb[0], input_ptr_split[0], kv_indptr_split[0], update_data.kv_indices,
               kv_last_page_len_split[0], gemvQ1, gemvAggregateOutput1);
    GEMV2.init(actual[1], nb[1], input_ptr_split[1], kv_indptr_split[1], update_data.kv_indices,
               kv_last_page_len_split[1], gemvQ1, gemvAggregateOutput1);
    prefill1.init(actual[2], 0, p1_input_split[2], p1_kv_indptr_split[2], update_data.kv_indices,
                  p1_lpl_split[2], gemvQ1, gemvAggregateOutput1);
    GEMV3.init(actual[3], nb[2], input_ptr_split[3], kv_indptr_split[3], update_data.kv_indices,
               kv_last_page_len_split[3], gemvQ1, gemvAggregateOutput1);
    GEMV4.init(actual[4], nb[3], input_ptr_split[4], kv_indptr_split[4], update_data.kv_indices,
               kv_last_page_len_split[4], gemvQ1, gemvAggregateOutput1);
    prefill2.init(actual[5], 0, input_ptr_split[5], kv_indptr_split[5], update_data.kv_indices,
                  kv_last_page_len_split[5], gemvQ1, gemvAggregateOutput1);
  }

  size_t token_remaining = update_token_num;
  for (int i = 0; i < 2; i++) {
    const size_t n = std::min(token_remaining, (size_t)KQV_ptrs[i]->M);
    roPEAppends[i].update((int)n, KQV_split[i], Q_split[i], rev_input_indptr_split[i],
                          per_token_offset_split[i], kv_indices, kv_indptr, kv_last_page_len);
    token_remaining -= n;
  }
  NF_LOG_INFO("RopeAppend Tokens: %d, %d", roPEAppends[0].dense_batch_size,
              roPEAppends[1].dense_batch_size);
}

void LocalPipeline::update(vortexUpdateData* update_data_) {
  this->update_data = *update_data_;
  const int T = config_data.global_batch_size;
  const int nano1 = config_data.nanobatch_1_size;
  auto input_span = pllmTensor<int>(update_data.input_tokens, T, 1, PllmLayout::ROW_MAJOR);
  genEmbedding1.setInput(input_span.subtensor(0, nano1));
  genEmbedding2.setInput(input_span.subtensor(nano1, T - nano1));

  update_token_num = update_data.decodePrefillBorder + update_data.prefillTokensNum;
  const int live1 = std::min(update_token_num, nano1), live2 = std::max(update_token_num - nano1, 0);
  for (BaseGEMMWrapper* g : {O1, D1, KQV1}) g->set_live_rows((size_t)live1);
  for (BaseGEMMWrapper* g : {O2, D2, KQV2}) g->set_live_rows((size_t)live2);
  dual1.set_live_rows(live1);
  dual2.set_live_rows(live2);
  genEmbedding1.set_live_rows(live1);
  genEmbedding2.set_live_rows(live2);
  layerNormAttention1.set_live_rows(live1);
  layerNormFFN1.set_live_rows(live1);
  layerNormAttention2.set_live_rows(live2);
  layerNormFFN2.set_live_rows(live2);
  const int req_num = update_data.decodePrefillBorder + update_data.prefillNum;
  maxSampler.set_batch_size(req_num);
  keepToken.update(req_num, update_data.input_indptr);
  // LM-head rows are padded up to a multiple of 128 as in the reference; the buffers behind
  // them are T rows long.
  LOGITS->set_shape(std::min((req_num + 127) / 128 * 128, T), (int)ModelConfig.vocab_size,
                    ModelConfig.model_hidden_dim);
  LOGITS->init();
  layerNormModel.set_live_rows((int)LOGITS->M);  // the rows the LM head reads (sampled rows padded to 128)
  output_data.sampled_tokens = req_num;
  GEMVOpUpdate();
  NF_LOG_INFO("prefill: %d, decode: %d; Batch size: %d, %d, %d, %d", update_data.prefillNum,
              update_data.decodePrefillBorder, update_data.gemv_batch_size[0],
              update_data.gemv_batch_size[1], update_data.gemv_batch_size[2],
              update_data.gemv_batch_size[3]);
}

double LocalPipeline::totalCompute() {
  double total = 0;
  for (auto gemm : gemms) total += gemm->totalCompute();
  return total;
}

void LocalPipeline::config(vortexConfigData* config_data_) {
  NF_LOG_INFO("Config local pipeline");
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
      configFail("LocalPipeline::config: cannot build GEMM %d from tag \"%s\"", i, tag.c_str());
      return;
    }
  }
  KQV_ptrs[0] = KQV1;
  KQV_ptrs[1] = KQV2;
  const int globalbatch = config_data.global_batch_size;
  const int nano1 = config_data.nanobatch_1_size;
  const int nano2 = globalbatch - nano1;
  if (nano1 <= 0 || nano2 <= 0 || globalbatch > ModelConfig.max_batch_size) {
    configFail("LocalPipeline::config: bad nano-batch split %d + %d (max batch %d)", nano1,
                 nano2, ModelConfig.max_batch_size);
      return;
  }
  const int kqv_n = (2 * ModelConfig.model_kv_heads_gpu + ModelConfig.model_qo_heads_gpu) *
                    ModelConfig.model_head_dim;
  O1->set_shape(nano1, ModelConfig.model_hidden_dim_pergpu, ModelConfig.model_hidden_dim);
  O2->set_shape(nano2, ModelConfig.model_hidden_dim_pergpu, ModelConfig.model_hidden_dim);
  D1->set_shape(nano1, ModelConfig.model_hidden_dim, ModelConfig.model_ff_dim_gpu);
  D2->set_shape(nano2, ModelConfig.model_hidden_dim, ModelConfig.model_ff_dim_gpu);
  KQV1->set_shape(nano1, kqv_n, ModelConfig.model_hidden_dim);
  KQV2->set_shape(nano2, kqv_n, ModelConfig.model_hidden_dim);
  LOGITS->set_shape(globalbatch / nranks, (int)ModelConfig.vocab_size, ModelConfig.model_hidden_dim);
  dual1.set_shape(nano1, ModelConfig.model_ff_dim_gpu, ModelConfig.model_hidden_dim);
  dual2.set_shape(nano2, ModelConfig.model_ff_dim_gpu, ModelConfig.model_hidden_dim);
  dual1.setWeightFormat(weight_format);
  dual1.setWeightLayout(pairWeightLayout(gemms, static_cast<int>(GEMM_NAME::LOGITS)));
  dual2.setWeightFormat(weight_format);
  dual2.setWeightLayout(pairWeightLayout(gemms, static_cast<int>(GEMM_NAME::LOGITS)));

  setName();
  ScheduleInit();
  GEMMOpInit();
  GEMVOpInit();
  OtherOpInit();
  if (nanobatch_only) assignSameStream();

  output_data = vortexOutputData();
  output_data.sampled_token_array = new int[globalbatch];
  output_data.global_batch_size = globalbatch;

  const size_t n = (size_t)globalbatch + 1;
  HIP_CHECK(hipMalloc(&prefill1_update.input_indptr, sizeof(int) * n));
  HIP_CHECK(hipMalloc(&prefill1_update.kv_indptr, sizeof(int) * n));
  HIP_CHECK(hipMalloc(&prefill1_update.kv_last_page_len, sizeof(int) * n));
  HIP_CHECK(hipHostMalloc(&prefill1_staging.input_indptr, sizeof(int) * n, hipHostMallocDefault));
  HIP_CHECK(hipHostMalloc(&prefill1_staging.kv_indptr, sizeof(int) * n, hipHostMallocDefault));
  HIP_CHECK(hipHostMalloc(&prefill1_staging.kv_last_page_len, sizeof(int) * n, hipHostMallocDefault));
  if (profiling) setProfiling(profilingLevel());
}
