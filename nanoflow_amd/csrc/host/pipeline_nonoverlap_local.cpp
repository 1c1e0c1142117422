// NonOverlapLocalPipeline: the sequential schedule (no nano-batching), on one stream except that
// chunked-prefill attention is forked onto a side stream while decode attention runs.
// The plainest statement of the layer math and the baseline the overlapped schedule must
// agree with.  Operator order follows the reference's
// pipeline/src/pipeline_nonoverlap_local.cu:25-62, wiring :245-304, update :108-126,327-385.
#include "pipeline.h"

NonOverlapLocalPipeline::NonOverlapLocalPipeline(vortexInitData* input_data, int nrank, int nranks,
                                                 int vnranks, bool kqv_bias_)
    : PipelineBase(input_data, nrank, nranks, vnranks) {
  kqv_bias = kqv_bias_;
  stream_all = createPipelineStream(0, 0);
  stream_prefill = createPipelineStream(0, 0);
  HIP_CHECK(hipEventCreateWithFlags(&prefill_fork, hipEventDisableTiming));
  HIP_CHECK(hipEventCreateWithFlags(&prefill_join, hipEventDisableTiming));
  NF_LOG_INFO("Init pipeline (non-overlap local)");
}

NonOverlapLocalPipeline::~NonOverlapLocalPipeline() {
  clearGraphs();
  for (auto g : gemms) delete g;
  delete[] output_data.sampled_token_array;
  if (prefill_fork) (void)hipEventDestroy(prefill_fork);
  if (prefill_join) (void)hipEventDestroy(prefill_join);
  if (stream_prefill) (void)hipStreamDestroy(stream_prefill);
  if (stream_all) (void)hipStreamDestroy(stream_all);
}

void NonOverlapLocalPipeline::setProfiling(int level) {
  profiling = level > 0;
  profile_gemms = level > 1;
  const unsigned stride = profileStride();
  timings.layer_stride = (int)stride;
  const size_t n = profiling ? (size_t)ModelConfig.run_layer : 0;
  GEMV.enableProfiling(n, stride);
  prefill.enableProfiling(n, stride);
  const size_t ng = profile_gemms ? (size_t)ModelConfig.run_layer : 0;
  for (auto g : gemms)
    if (g) g->enableProfiling(ng, stride);
  dual.enableProfiling(ng, stride);
}

vortexOutputData NonOverlapLocalPipeline::run() {
  setWeight(0);
  HIP_CHECK(hipEventRecord(events[EventManager::GEMM_TIMING_START], stream_all));
  runIteration(stream_all, baseSignature(), [this] {
    genEmbedding.run().log();
    for (int iter = 0; iter < ModelConfig.run_layer; ++iter) {
      setWeight(iter % ModelConfig.model_layer);
      layerNormAttention.run().log();
      KQV->run().log();
      roPEAppend.run().log();
      // fork: prefill attention beside decode attention; join before the O projection
      const bool side = update_data.prefillNum > 0 && GEMV.batch_size > 0;
      if (side) {
        HIP_CHECK(hipEventRecord(prefill_fork, stream_all));
        HIP_CHECK(hipStreamWaitEvent(stream_prefill, prefill_fork, 0));
        prefill.setStream(stream_prefill);
        prefill.run().log();
        HIP_CHECK(hipEventRecord(prefill_join, stream_prefill));
      }
      if (GEMV.batch_size > 0) GEMV.run().log();
      if (side) {
        HIP_CHECK(hipStreamWaitEvent(stream_all, prefill_join, 0));
      } else if (update_data.prefillNum > 0) {
        prefill.setStream(stream_all);
        prefill.run().log();
      }
      O->run().log();
      layerNormFFN.run().log();
      dual.run().log();
      D->run().log();
    }
    keepToken.run().log();
    layerNormModel.run().log();
    LOGITS->run().log();
    maxSampler.run().log();
  });
  HIP_CHECK(hipEventRecord(events[EventManager::GEMM_TIMING_END], stream_all));
  HIP_CHECK(hipMemcpyAsync(output_data.sampled_token_array, maxSampler.d_argMax.ptr,
                           output_data.sampled_tokens * sizeof(int), hipMemcpyDeviceToHost,
                           stream_all));
  HIP_CHECK(hipStreamSynchronize(stream_all));
  float runtime_ms = 0;
  HIP_CHECK(hipEventElapsedTime(&runtime_ms, events[EventManager::GEMM_TIMING_START],
                                events[EventManager::GEMM_TIMING_END]));
  timings.iter_ms = runtime_ms;
  if (profiling) {
    GEMV.collectProfile(timings.decode_attn_ms, timings.decode_attn_launches);
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
    add(dual, dual.totalCompute());
  }
  NF_LOG_INFO("Total running cost (ms) of one microbatch is %f", runtime_ms);
  return output_data;
}

void NonOverlapLocalPipeline::update(vortexUpdateData* update_data_) {
  this->update_data = *update_data_;
  const int T = config_data.global_batch_size;
  genEmbedding.setInput(pllmTensor<int>(update_data.input_tokens, T, 1, PllmLayout::ROW_MAJOR));
  const int req_num = update_data.decodePrefillBorder + update_data.prefillNum;
  update_token_num = update_data.decodePrefillBorder + update_data.prefillTokensNum;
  for (BaseGEMMWrapper* g : {O, D, KQV}) g->set_live_rows((size_t)update_token_num);
  dual.set_live_rows(update_token_num);
  genEmbedding.set_live_rows(update_token_num);
  layerNormAttention.set_live_rows(update_token_num);
  layerNormFFN.set_live_rows(update_token_num);
  maxSampler.set_batch_size(req_num / nranks);
  keepToken.update(req_num, update_data.input_indptr);
  LOGITS->set_shape(std::min((req_num / nranks + 127) / 128 * 128, T), (int)ModelConfig.vocab_size,
                    ModelConfig.model_hidden_dim);
  LOGITS->init();
  layerNormModel.set_live_rows((int)LOGITS->M);  // the rows the LM head reads (sampled rows padded to 128)
  output_data.sampled_tokens = req_num;
  GEMVOpUpdate();
}

void NonOverlapLocalPipeline::config(vortexConfigData* config_data_) {
  NF_LOG_INFO("Config non-overlap local pipeline");
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
      configFail("NonOverlapLocalPipeline::config: cannot build GEMM %d from tag \"%s\"", i,
                   tag.c_str());
      return;
    }
  }
  const int globalbatch = config_data.global_batch_size;
  if (globalbatch <= 0 || globalbatch > ModelConfig.max_batch_size) {
    configFail("NonOverlapLocalPipeline::config: global batch %d exceeds max batch %d",
                 globalbatch, ModelConfig.max_batch_size);
      return;
  }
  O->set_shape(globalbatch, ModelConfig.model_hidden_dim_pergpu, ModelConfig.model_hidden_dim);
  D->set_shape(globalbatch, ModelConfig.model_hidden_dim, ModelConfig.model_ff_dim_gpu);
  KQV->set_shape(globalbatch,
                 (2 * ModelConfig.model_kv_heads_gpu + ModelConfig.model_qo_heads_gpu) *
                     ModelConfig.model_head_dim,
                 ModelConfig.model_hidden_dim);
  LOGITS->set_shape(globalbatch, (int)ModelConfig.vocab_size, ModelConfig.model_hidden_dim);
  dual.set_shape(globalbatch, ModelConfig.model_ff_dim_gpu, ModelConfig.model_hidden_dim);
  dual.setWeightFormat(weight_format);
  dual.setWeightLayout(pairWeightLayout(gemms, static_cast<int>(GEMM_NAME::LOGITS)));
  ScheduleInit();
  GEMMOpInit();
  GEMVOpInit();
  OtherOpInit();
  setName();
  output_data = vortexOutputData();
  output_data.sampled_token_array = new int[globalbatch];
  output_data.global_batch_size = globalbatch;
  if (profiling) setProfiling(profilingLevel());
}

void NonOverlapLocalPipeline::setName() {
  SET_NAME_PTR(KQV);
  SET_NAME_PTR(LOGITS);
  SET_NAME_PTR(O);
  SET_NAME_REF(dual);
  SET_NAME_PTR(D);
  SET_NAME_REF(genEmbedding);
  SET_NAME_REF(layerNormAttention);
  SET_NAME_REF(layerNormFFN);
  SET_NAME_REF(layerNormModel);
  SET_NAME_REF(GEMV);
  SET_NAME_REF(prefill);
  SET_NAME_REF(roPEAppend);
  SET_NAME_REF(maxSampler);
  SET_NAME_REF(keepToken);
}

void NonOverlapLocalPipeline::setWeight(int layer) {
  auto& lw = input_data->weight.layer_weight[layer];
  bool success = true;
  success &= O->set_weight(lw.W_O1);
  success &= D->set_weight(lw.W_D);
  success &= KQV->set_weight(lw.W_KQV);
  success &= bindKQVBias(KQV, lw.B_KQV);
  success &= layerNormAttention.setWeight(lw.W_LN_Attention);
  success &= layerNormFFN.setWeight(lw.W_LN_FFN);
  success &= dual.set_weight(lw.W_G, lw.W_U);
  if (!success) NF_LOG_ERROR("Failed to set weight for layer %d", layer);
  GEMV.setKVData(input_data->kv_data[layer]);
  prefill.setKVData(input_data->kv_data[layer]);
  roPEAppend.setKVData(input_data->kv_data[layer]);
}

void NonOverlapLocalPipeline::ScheduleInit() {
  const auto ROW = PllmLayout::ROW_MAJOR;
  const int T = config_data.global_batch_size;
  const int qdim = ModelConfig.model_head_dim * ModelConfig.model_qo_heads_gpu;
  gemvOutput = tmpBufferM.allocTensor(T, qdim, ROW);
  const auto O_output = tmpBufferM.allocTensor((int)O->M, (int)O->N, ROW);
  O->setA(gemvOutput);
  O->setD(O_output);
  const auto LayerNormFFN_output = tmpBufferM.allocTensor(dual.M, dual.K, ROW);
  layerNormFFN.setInput(O_output).setOutput(LayerNormFFN_output);
  const auto activation_output = tmpBufferM.allocTensor((int)D->M, (int)D->K, ROW);
  dual.setA(LayerNormFFN_output);
  dual.setD(pllmTensor<half>(), pllmTensor<half>(), activation_output);
  const auto D_output = tmpBufferM.allocTensor((int)D->M, (int)D->N, ROW);
  D->setA(activation_output);
  D->setC(O_output);   // residual: output of the attention block
  D->setOutput(D_output);
  const auto layerNormAttention_output = tmpBufferM.allocTensor((int)D->M, (int)D->N, ROW);
  layerNormAttention.setInput(D_output).setOutput(layerNormAttention_output);
  O->setC(D_output);   // residual stream lives in the D output
  KQV->setA(layerNormAttention_output).setOutput(tmpBufferM.allocTensor((int)KQV->M, (int)KQV->N, ROW));
  gemvInput = tmpBufferM.allocTensor(T, qdim, ROW);
  const auto keepTokenOutput = tmpBufferM.allocTensor(T, (int)D->N, ROW);
  keepToken.setInput(D_output).setOutput(keepTokenOutput);
  const auto layerNormModel_output = tmpBufferM.allocTensor(T, (int)D->N, ROW);
  layerNormModel.setInput(keepTokenOutput).setOutput(layerNormModel_output);
  const auto LOGITS_output = tmpBufferM.allocTensor(T, (int)LOGITS->N, ROW);
  LOGITS->setA(layerNormModel_output);
  LOGITS->setOutput(LOGITS_output);
  int* sample_output_alloc = (int*)tmpBufferM.alloc((size_t)T * sizeof(int) / sizeof(half));
  pllmTensor<int> sample_output = {sample_output_alloc, T, 1, ROW};
  const auto maxSampler_maxVals = tmpBufferM.allocTensor(T, 1, ROW);
  maxSampler.init(LOGITS_output, maxSampler_maxVals, sample_output);
  genEmbedding.setOutput(D->getD());
  // scratch of the fp8-weight wrappers (none for fp16 weights)
  for (int i = 0; i < gemmNum; ++i)
    gemms[i]->setWorkspace(tmpBufferM.allocBytes(gemms[i]->workspaceBytes()), gemms[i]->workspaceBytes());
  dual.setWorkspace(tmpBufferM.allocBytes(dual.workspaceBytes()), dual.workspaceBytes());
  // e4m3 weights: the two RMSNorms hand their consumers quantised rows
  if (const QuantRows qa = allocQuantRows(KQV->M); qa && KQV->setQuantizedA(qa.q, qa.scale))
    layerNormAttention.setQuantOutput(qa.q, qa.scale);
  if (const QuantRows qf = allocQuantRows(dual.M); qf && dual.setQuantizedA(qf.q, qf.scale))
    layerNormFFN.setQuantOutput(qf.q, qf.scale);
  NF_LOG_INFO("allocated %zu halfs", tmpBufferM.getAllocation());
}

void NonOverlapLocalPipeline::GEMMOpInit() {
  setWeight(0);
  O->init(1.f);
  dual.init();
  D->init(1.f);
  KQV->init(kqv_bias ? 1.f : 0.f);
  // one stream, nobody waits on an operator: no start / end events (each record is a packet
  // between two kernels)
  for (int i = 0; i < gemmNum; ++i) {
    gemms[i]->setStream(stream_all);
    gemms[i]->updateEventExistance(false, false);
  }
  LOGITS->set_weight(input_data->weight.lm_head);
  LOGITS->init();
  dual.setStream(stream_all).updateEventExistance(false, false);
}

void NonOverlapLocalPipeline::GEMVOpUpdate() {
  const uint32_t dpb = update_data.decodePrefillBorder;
  uint32_t arr[] = {dpb, uint32_t(update_data.prefillNum)};
  std::span<uint32_t, 2> batch_sizes(arr, 2);
  const size_t total_batch_size = arr[0] + arr[1];
  const uint32_t T = config_data.global_batch_size;
  const auto kv_indptr_split = pllmTensor<int32_t>{update_data.kv_indptr, total_batch_size + 1}
                                   .splitTensor(PllmDimension::ROW, batch_sizes, 1U);
  const auto kv_last_page_len_split = pllmTensor<int32_t>{update_data.kv_last_page_len, total_batch_size}
                                          .splitTensor(PllmDimension::ROW, batch_sizes);
  const auto input_ptr_split = pllmTensor<int32_t>{update_data.input_indptr, total_batch_size + 1}
                                   .splitTensor(PllmDimension::ROW, batch_sizes, 1U);
  GEMV.init(dpb, update_data.gemv_num_blocks[0], input_ptr_split[0], kv_indptr_split[0],
            update_data.kv_indices, kv_last_page_len_split[0], gemvInput, gemvOutput);
  prefill.init(update_data.prefillNum, 0, input_ptr_split[1], kv_indptr_split[1],
               update_data.kv_indices, kv_last_page_len_split[1], gemvInput, gemvOutput);
  roPEAppend.update(update_token_num, KQV->getD(), gemvInput,
                    pllmTensor<int32_t>(update_data.rev_input_indptr, (size_t)T),
                    pllmTensor<int32_t>(update_data.per_token_offset, (size_t)T),
                    pllmTensor<int32_t>(update_data.kv_indices, ModelConfig.max_page_num),
                    pllmTensor<int32_t>(update_data.kv_indptr, (size_t)T + 1),
                    pllmTensor<int32_t>(update_data.kv_last_page_len, (size_t)T));
}

void NonOverlapLocalPipeline::OtherOpInit() {
  layerNormAttention.setStream(stream_all).updateEventExistance(false, false);
  layerNormFFN.setStream(stream_all).updateEventExistance(false, false);
  genEmbedding.setStream(stream_all).updateEventExistance(false, false);
  layerNormModel.setStream(stream_all).updateEventExistance(false, false);
  roPEAppend.setStream(stream_all).updateEventExistance(false, false);
  maxSampler.setStream(stream_all).updateEventExistance(false, false);
  keepToken.setStream(stream_all).updateEventExistance(false, false);
  genEmbedding.setWeight(input_data->weight.embedding);
  layerNormModel.setWeight(input_data->weight.model_layernorm);
}

void NonOverlapLocalPipeline::GEMVOpInit() {
  GEMV.setStream(stream_all).updateEventExistance(false, false);
  prefill.setStream(stream_all).updateEventExistance(false, false);
}

double NonOverlapLocalPipeline::totalCompute() {
  double total = 0;
  for (auto gemm : gemms) total += gemm->totalCompute();
  return total;
}
