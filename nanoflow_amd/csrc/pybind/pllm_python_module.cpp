// The Python extension module `pllm_python`: the names, arguments and behaviour of the reference's
// pybind11 module (pipeline/src/pybind.cu:189-284), so that Python written against the reference
// (pipeline/utils/{serve_8B,pybindUtil,weightLoader,kv_cache}.py) imports and drives this build
// unchanged.  Everything below goes through the control plane's C ABI (include/nanoflow_pllm.h);
// the module adds no logic of its own beyond converting between Python objects and the flat structs.
//
//   * weights handed to init() are HOST pointers (torch CPU tensors' data_ptr(), or what
//     createModelWeight allocated); init uploads them (pybind.cu:73-98) and then starts the pipeline;
//   * createModelWeight allocates HOST memory (the reference binds createModelWeightCPU, pybind.cu:281);
//   * update-data setters take raw addresses as integers (pybind.cu:31-63);
//   * getPipelineOutput is constructed exactly as the reference constructs it (pybind.cu:178-184).
#include <pybind11/numpy.h>
#include <pybind11/pybind11.h>
#include <pybind11/stl.h>

#include <stdexcept>
#include <string>
#include <vector>

#include "nanoflow_pllm.h"

namespace py = pybind11;

namespace {

struct VortexWeight {
  size_t ptr = 0;
  int N = 0, K = 0;
  nf_vortex_weight c() const { return nf_vortex_weight{reinterpret_cast<uint16_t*>(ptr), N, K}; }
  static VortexWeight from(const nf_vortex_weight& w) {
    VortexWeight v;
    v.ptr = reinterpret_cast<size_t>(w.ptr);
    v.N = w.N;
    v.K = w.K;
    return v;
  }
};

struct VortexLayerWeight {
  VortexWeight W_O1, W_O2, W_U, W_G, W_D, W_KQV, B_KQV, W_LN_Attention, W_LN_FFN, W_ROT;
  nf_vortex_layer_weight c() const {
    return nf_vortex_layer_weight{W_O1.c(), W_O2.c(), W_U.c(), W_G.c(), W_D.c(), W_KQV.c(), B_KQV.c(),
                                  W_LN_Attention.c(), W_LN_FFN.c(), W_ROT.c()};
  }
  static VortexLayerWeight from(const nf_vortex_layer_weight& l) {
    VortexLayerWeight v;
    v.W_O1 = VortexWeight::from(l.W_O1);
    v.W_O2 = VortexWeight::from(l.W_O2);
    v.W_U = VortexWeight::from(l.W_U);
    v.W_G = VortexWeight::from(l.W_G);
    v.W_D = VortexWeight::from(l.W_D);
    v.W_KQV = VortexWeight::from(l.W_KQV);
    v.B_KQV = VortexWeight::from(l.B_KQV);
    v.W_LN_Attention = VortexWeight::from(l.W_LN_Attention);
    v.W_LN_FFN = VortexWeight::from(l.W_LN_FFN);
    v.W_ROT = VortexWeight::from(l.W_ROT);
    return v;
  }
};

struct VortexModelWeight {
  VortexWeight lm_head, embedding, model_layernorm;
  std::vector<VortexLayerWeight> layer_weight;
};

struct VortexInitData {
  std::vector<size_t> kv_data;  // device address of each layer's pool
  VortexModelWeight weight;
  size_t weight_size = 0;
  size_t tmp_buffer = 0;
  size_t tmp_buffer_size = 0;
};

struct VortexOutputData {};

struct VortexUpdateData {
  nf_vortex_update_data c{};
  std::vector<int32_t> gemv_batch_size, gemv_num_blocks;  // owned copies, as the reference makes
};

struct VortexConfigData {
  std::vector<std::string> gemm_op_tag;
  int global_batch_size = 0, nanobatch_1_size = 0, kqv1_size = 0, kqv3_size = 0;
};

[[noreturn]] void fail(const char* what) {
  throw std::runtime_error(std::string(what) + ": " + pllm_last_error());
}
void check(int rc, const char* what) {
  if (rc != 0) fail(what);
}

int g_nranks = 1;
// what the pipeline keeps pointers into for the life of the process (as the reference leaks its
// `new half*[]` in setKVdata)
std::vector<std::vector<uint16_t*>> g_kv_arrays;

// flat copy of a weight set; `layers` is the storage the returned struct points into
nf_vortex_model_weight flatten(const VortexModelWeight& w, std::vector<nf_vortex_layer_weight>& layers) {
  layers.clear();
  for (const auto& l : w.layer_weight) layers.push_back(l.c());
  return nf_vortex_model_weight{w.lm_head.c(), w.embedding.c(), w.model_layernorm.c(), layers.data(),
                                (int)layers.size()};
}
VortexModelWeight unflatten(const nf_vortex_model_weight& c) {
  VortexModelWeight w;
  w.lm_head = VortexWeight::from(c.lm_head);
  w.embedding = VortexWeight::from(c.embedding);
  w.model_layernorm = VortexWeight::from(c.model_layernorm);
  for (int i = 0; i < c.num_layers; ++i) w.layer_weight.push_back(VortexLayerWeight::from(c.layer_weight[i]));
  return w;
}

void setRank(int nranks, int vnranks) {
  check(pllm_set_rank(nranks, vnranks), "setRank");
  g_nranks = nranks;
}

void setModelConfig(const std::string& filename) { check(pllm_set_model_config(filename.c_str()), "setModelConfig"); }

void createModelWeight(VortexModelWeight& weight, int rank) {
  if (rank != 0) throw std::runtime_error("createModelWeight: this build runs one rank");
  const int n = pllm_num_layers();
  std::vector<nf_vortex_layer_weight> layers((size_t)std::max(n, 1));
  nf_vortex_model_weight c{};
  check(pllm_create_model_weight_host(&c, layers.data(), (int)layers.size()), "createModelWeight");
  weight = unflatten(c);
}

void createInitData(VortexInitData& data, VortexModelWeight& weight, int rank) {
  if (rank != 0) throw std::runtime_error("createInitData: this build runs one rank");
  std::vector<nf_vortex_layer_weight> layers;
  const nf_vortex_model_weight cw = flatten(weight, layers);
  std::vector<uint16_t*> kv((size_t)std::max(pllm_num_layers(), 1));
  nf_vortex_init_data c{};
  check(pllm_create_init_data(&c, kv.data(), (int)kv.size(), &cw), "createInitData");
  data.kv_data.clear();
  for (int i = 0; i < pllm_num_layers(); ++i) data.kv_data.push_back(reinterpret_cast<size_t>(kv[i]));
  data.weight = weight;
  data.weight_size = c.weight_size;
  data.tmp_buffer = reinterpret_cast<size_t>(c.tmp_buffer);
  data.tmp_buffer_size = c.tmp_buffer_size;
}

// init: upload the host-resident weights of every rank, then start the pipeline (pybind.cu:73-98).
// As in the reference, input[i].weight is replaced by the device copy.
void init(std::vector<VortexInitData*> input, int pipeline_type) {
  if ((int)input.size() != g_nranks || g_nranks != 1)
    throw std::runtime_error("init: this build runs exactly one rank (setRank(1, ...), one VortexInitData)");
  VortexInitData& d = *input[0];
  std::vector<nf_vortex_layer_weight> host_layers;
  const nf_vortex_model_weight hw = flatten(d.weight, host_layers);
  std::vector<nf_vortex_layer_weight> dev_layers(std::max<size_t>(host_layers.size(), 1));
  nf_vortex_model_weight dw{};
  {
    py::gil_scoped_release nogil;  // gigabytes of copies
    check(pllm_model_weight_to_gpu(&hw, &dw, dev_layers.data()), "init (weight upload)");
  }
  d.weight = unflatten(dw);
  g_kv_arrays.emplace_back();
  for (size_t a : d.kv_data) g_kv_arrays.back().push_back(reinterpret_cast<uint16_t*>(a));
  nf_vortex_init_data ci{};
  ci.kv_data = g_kv_arrays.back().data();
  ci.weight = dw;
  ci.weight_size = d.weight_size;
  ci.tmp_buffer = reinterpret_cast<uint16_t*>(d.tmp_buffer);
  ci.tmp_buffer_size = d.tmp_buffer_size;
  check(pllm_init(&ci, pipeline_type), "init");
}

void config(std::vector<VortexConfigData*> configs) {
  if (configs.size() != 1) throw std::runtime_error("config: this build runs exactly one rank");
  const VortexConfigData& c = *configs[0];
  std::vector<const char*> tags;
  for (const auto& t : c.gemm_op_tag) tags.push_back(t.c_str());
  nf_vortex_config_data cc{tags.data(), (int)tags.size(), c.global_batch_size, c.nanobatch_1_size, c.kqv1_size,
                           c.kqv3_size};
  check(pllm_config(&cc), "config");
}

void update(std::vector<VortexUpdateData*> updates) {
  if (updates.size() != 1) throw std::runtime_error("update: this build runs exactly one rank");
  VortexUpdateData& u = *updates[0];
  u.c.gemv_batch_size = u.gemv_batch_size.data();
  u.c.gemv_num_blocks = u.gemv_num_blocks.data();
  if (u.gemv_batch_size.size() < 4 || u.gemv_num_blocks.size() < 4)
    throw std::runtime_error("update: setGemvBatchSize / setGemvNumBlocks need 4 entries each");
  py::gil_scoped_release nogil;
  check(pllm_update(&u.c), "update");
}

void run() {
  py::gil_scoped_release nogil;
  check(pllm_run(), "run");
}
void run_async() { check(pllm_run_async(), "run_async"); }
void run_async_wait() {
  py::gil_scoped_release nogil;
  check(pllm_run_async_wait(), "run_async_wait");
}
void finalize() { check(pllm_finalize(), "finalize"); }

py::array getPipelineOutput() {
  const int32_t* tokens = nullptr;
  int count = 0;
  check(pllm_get_pipeline_output(&tokens, &count), "getPipelineOutput");
  // dtype, shape, strides, data and no base object: the reference's own constructor call
  return py::array(py::dtype("int32"), {(size_t)count}, {sizeof(int32_t)}, tokens);
}

std::vector<int32_t> copy_int_array(const py::array_t<int>& a) {
  const py::buffer_info info = a.request();
  const int* p = static_cast<const int*>(info.ptr);
  return std::vector<int32_t>(p, p + (info.ndim ? info.shape[0] : 0));
}

}  // namespace

PYBIND11_MODULE(pllm_python, m) {
  m.doc() = "MI355X-native NanoFlow pipeline behind the reference's pllm_python interface";

  py::class_<VortexInitData>(m, "VortexInitData")
      .def(py::init<>())
      .def("setKVdata",
           [](VortexInitData& d, py::array_t<size_t> kv) {
             const py::buffer_info info = kv.request();
             const size_t* p = static_cast<const size_t*>(info.ptr);
             d.kv_data.assign(p, p + (info.ndim ? info.shape[0] : 0));
           })
      .def("setWeight",
           [](VortexInitData& d, const VortexModelWeight& w, size_t weight_size) {
             d.weight = w;
             d.weight_size = weight_size;
           })
      .def("setTmpBuffer",
           [](VortexInitData& d, size_t tmp_buffer, size_t tmp_buffer_size) {
             d.tmp_buffer = tmp_buffer;
             d.tmp_buffer_size = tmp_buffer_size;
           })
      .def_readwrite("weight_size", &VortexInitData::weight_size)
      .def_readwrite("tmp_buffer_size", &VortexInitData::tmp_buffer_size);

  py::class_<VortexOutputData>(m, "VortexOutputData").def(py::init<>());

#define NF_UPD_FIELD(name) \
  def_property(#name, [](const VortexUpdateData& u) { return u.c.name; }, [](VortexUpdateData& u, int v) { u.c.name = v; })
#define NF_UPD_PTR(pyname, field) \
  def(pyname, [](VortexUpdateData& u, size_t addr) { u.c.field = reinterpret_cast<int32_t*>(addr); })
  py::class_<VortexUpdateData>(m, "VortexUpdateData")
      .def(py::init<>())
      .NF_UPD_FIELD(decodePrefillBorder)
      .NF_UPD_FIELD(prefillNum)
      .NF_UPD_FIELD(prefillTokensNum)
      .NF_UPD_FIELD(keepTokenListLength)
      .NF_UPD_PTR("setKVIndices", kv_indices)
      .NF_UPD_PTR("setKVIndptr", kv_indptr)
      .NF_UPD_PTR("setKVLastPageLen", kv_last_page_len)
      .NF_UPD_PTR("setInputIndptr", input_indptr)
      .NF_UPD_PTR("setRevInputIndptr", rev_input_indptr)
      .NF_UPD_PTR("setInputEmbedding", input_tokens)
      .NF_UPD_PTR("setPerTokenOffset", per_token_offset)
      .NF_UPD_PTR("setKeepTokenList", keep_token_list)
      .def("setGemvBatchSize", [](VortexUpdateData& u, py::array_t<int> a) { u.gemv_batch_size = copy_int_array(a); })
      .def("setGemvNumBlocks", [](VortexUpdateData& u, py::array_t<int> a) { u.gemv_num_blocks = copy_int_array(a); });
#undef NF_UPD_FIELD
#undef NF_UPD_PTR

  py::class_<VortexConfigData>(m, "VortexConfigData")
      .def(py::init<>())
      .def_readwrite("gemmOpTag", &VortexConfigData::gemm_op_tag)
      .def_readwrite("globalBatchSize", &VortexConfigData::global_batch_size)
      .def_readwrite("nanobatch1Size", &VortexConfigData::nanobatch_1_size)
      .def_readwrite("kqv1Size", &VortexConfigData::kqv1_size)
      .def_readwrite("kqv3Size", &VortexConfigData::kqv3_size)
      .def("setGemmOpTag", [](VortexConfigData& c, py::list tags) {
        c.gemm_op_tag.clear();
        for (auto t : tags) c.gemm_op_tag.push_back(t.cast<std::string>());
      });

  py::enum_<nf_pipeline_type>(m, "PipelineType")
      .value("PLLM", NF_PIPE_PLLM)
      .value("NONOVERLAP", NF_PIPE_NONOVERLAP)
      .value("NANOBATCH", NF_PIPE_NANOBATCH)
      .value("PLLMOFFLOAD", NF_PIPE_PLLMOFFLOAD)
      .value("LOCAL", NF_PIPE_LOCAL)
      .value("NON_OVERLAP_LOCAL", NF_PIPE_NON_OVERLAP_LOCAL)
      .value("NANOBATCH_LOCAL", NF_PIPE_NANOBATCH_LOCAL)
      .value("NONOVERLAP_KQVBIAS", NF_PIPE_NONOVERLAP_KQVBIAS)
      .value("NANOBATCH_KQVBIAS", NF_PIPE_NANOBATCH_KQVBIAS)
      .value("KQVBIAS", NF_PIPE_KQVBIAS);

  py::class_<VortexWeight>(m, "VortexWeight")
      .def(py::init<>())
      .def("setPtr", [](VortexWeight& w, size_t ptr) { w.ptr = ptr; })
      .def_readwrite("N", &VortexWeight::N)
      .def_readwrite("K", &VortexWeight::K);

  py::class_<VortexLayerWeight>(m, "VortexLayerWeight")
      .def(py::init<>())
      .def_readwrite("W_O1", &VortexLayerWeight::W_O1)
      .def_readwrite("W_O2", &VortexLayerWeight::W_O2)
      .def_readwrite("W_U", &VortexLayerWeight::W_U)
      .def_readwrite("W_G", &VortexLayerWeight::W_G)
      .def_readwrite("W_D", &VortexLayerWeight::W_D)
      .def_readwrite("W_KQV", &VortexLayerWeight::W_KQV)
      .def_readwrite("B_KQV", &VortexLayerWeight::B_KQV)
      .def_readwrite("W_LN_Attention", &VortexLayerWeight::W_LN_Attention)
      .def_readwrite("W_LN_FFN", &VortexLayerWeight::W_LN_FFN)
      .def_readwrite("W_ROT", &VortexLayerWeight::W_ROT);

  py::class_<VortexModelWeight>(m, "VortexModelWeight")
      .def(py::init<>())
      .def_readwrite("lm_head", &VortexModelWeight::lm_head)
      .def_readwrite("embedding", &VortexModelWeight::embedding)
      .def_readwrite("model_layernorm", &VortexModelWeight::model_layernorm)
      .def_readwrite("layer_weight", &VortexModelWeight::layer_weight);

  m.def("init", [](std::vector<VortexInitData*> input, nf_pipeline_type t) { init(std::move(input), (int)t); },
        "Initializes the Pipeline.");
  m.def("update", &update, "Updates the Pipeline.");
  m.def("config", &config, "Configures the Pipeline.");
  m.def("run", &run, "Runs the Pipeline.");
  m.def("finalize", &finalize, "Finalizes the Pipeline.");
  m.def("run_async", &run_async, "Runs the Pipeline asynchronously.");
  m.def("run_async_wait", &run_async_wait, "Waits for the Pipeline to finish.");
  m.def("getPipelineOutput", &getPipelineOutput, "Returns the output of the Pipeline.");
  m.def("setRank", &setRank, "Sets the rank of the Pipeline.");
  m.def("createModelWeight", &createModelWeight, "Creates a weight.");
  m.def("setModelConfig", &setModelConfig, "Sets the model configuration.");
  m.def("createInitData", &createInitData, "Creates an initialization data.");
  // a pipeline left open must not keep the interpreter from exiting (its worker thread waits
  // on a barrier); finalize is a no-op when nothing is initialised
  py::module_::import("atexit").attr("register")(py::cpp_function([] { (void)pllm_finalize(); }));
}
