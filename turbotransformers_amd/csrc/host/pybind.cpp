// Python boundary: module `turbo_transformers_cxx` with the reference's Python-visible
// surface (turbo_transformers/python/pybind.cpp:141-371): Tensor (DLPack in/out), the layer
// classes whose constructors move their weight tensors in, numpy converters, and the
// allocator / profiler / thread knobs.  Additions for this build are grouped at the end
// (stream hand-over, allocator statistics).
#include <pybind11/numpy.h>
#include <pybind11/pybind11.h>
#include <pybind11/stl.h>

#include <cstring>
#include <memory>

#include "bert_model.h"
#include "core/allocator.h"
#include "core/device_context.h"
#include "core/tensor.h"
#include "layers/bert_layers.h"
#include "layers/multi_headed_attention.h"
#include "layers/quantized_layers.h"
#include "loaders/npz_load.h"
#include "ttmi.h"

namespace py = pybind11;
using namespace turbo_transformers;
using core::Tensor;

static void DLPackCapsuleDestructor(PyObject* data) {
  auto* t = static_cast<DLManagedTensor*>(PyCapsule_GetPointer(data, "dltensor"));
  if (t) {
    if (t->deleter) t->deleter(t);  // never consumed: release it ourselves
  } else {
    PyErr_Clear();  // consumed and renamed by the importer
  }
}

template <typename T>
static Tensor NpArray2Tensor(py::array_t<T, py::array::c_style | py::array::forcecast> array, const std::string& dev_name) {
  if (array.ndim() == 0) throw std::runtime_error("nparray2tensor: numpy array shall not be empty!");
  std::vector<int64_t> shape(array.ndim());
  for (py::ssize_t i = 0; i < array.ndim(); ++i) shape[i] = array.shape(i);
  DLDeviceType dev;
  if (dev_name == "CPU") dev = kDLCPU;
  else if (dev_name == "GPU") dev = kDLROCM;
  else TT_THROW("nparray2tensor dev_name should be CPU or GPU!");
  Tensor tensor(core::NewDLPackTensorT<T>(shape, dev));
  core::CopyBytes(tensor.mutable_raw(), dev, array.data(), kDLCPU, (size_t)tensor.numel() * sizeof(T));
  return tensor;
}

template <typename T>
static py::array_t<T> Tensor2NpArray(const Tensor& tensor) {
  std::vector<py::ssize_t> shape(tensor.n_dim());
  for (size_t i = 0; i < tensor.n_dim(); ++i) shape[i] = tensor.shape((int)i);
  py::array_t<T> out(shape);
  core::CopyBytes(out.mutable_data(), kDLCPU, tensor.data<T>(), tensor.device_type(), (size_t)tensor.numel() * sizeof(T));
  return out;
}

enum class BlasProvider { MKL, OpenBlas };

PYBIND11_MODULE(turbo_transformers_cxx, m) {
  py::register_exception<core::EnforceNotMet>(m, "EnforceNotMet", PyExc_RuntimeError);

  auto config = m.def_submodule("config", "compile configuration of turbo_transformers");
  py::enum_<BlasProvider>(config, "BlasProvider").value("MKL", BlasProvider::MKL).value("OpenBlas", BlasProvider::OpenBlas);
  // "compiled with cuda" is what the Python callers test before taking the GPU path
  // (python/tests/*_test.py): the device build answers True.
  config.def("is_compiled_with_cuda", [] { return true; });
  config.def("get_blas_provider", [] { return BlasProvider::OpenBlas; });

  m.def("nparray2tensor", &NpArray2Tensor<float>, "Convert Numpy to Tensor.");
  m.def("nparray2tensor", &NpArray2Tensor<int64_t>, "Convert Numpy to Tensor.");
  m.def("tensor2nparrayf", &Tensor2NpArray<float>, "Convert Tensor to Numpy, float data only.");
  m.def("tensor2nparrayl", &Tensor2NpArray<int64_t>, "Convert Tensor to Numpy, int64 data only.");

  m.def("set_stderr_verbose_level", [](int) {});
  m.def("enable_perf", [](const std::string&) {});  // profiling is rocprofv3's job
  m.def("disable_perf", [] {});
  m.def("set_num_threads", [](int) {});             // no host-side compute threads
  m.def("bert_opt_mem_allocate_api", &core::allocator::bert_opt_mem_allocate_api);
  m.def("reset_allocator_schema", &core::allocator::reset_allocator_schema);

  py::class_<Tensor>(m, "Tensor")
      .def_static("from_dlpack",
                  [](py::capsule capsule) -> std::unique_ptr<Tensor> {
                    auto* tensor = static_cast<DLManagedTensor*>(PyCapsule_GetPointer(capsule.ptr(), "dltensor"));
                    if (tensor == nullptr) throw py::error_already_set();
                    TT_ENFORCE(tensor->dl_tensor.strides == nullptr || tensor->dl_tensor.ndim == 0 ||
                                   [&] {
                                     int64_t expect = 1;
                                     for (int i = tensor->dl_tensor.ndim - 1; i >= 0; --i) {
                                       if (tensor->dl_tensor.shape[i] != 1 && tensor->dl_tensor.strides[i] != expect) return false;
                                       expect *= tensor->dl_tensor.shape[i];
                                     }
                                     return true;
                                   }(),
                               "from_dlpack: tensor must be contiguous");
                    PyCapsule_SetName(capsule.ptr(), "used_tensor");
                    return std::make_unique<Tensor>(tensor);
                  })
      .def("to_dlpack",
           [](Tensor& tensor) -> py::capsule {
             auto* dlpack = tensor.ToDLPack();
             return py::capsule(dlpack, "dltensor", DLPackCapsuleDestructor);
           })
      // The unrounded fp32 values a bfloat16 LayerNorm output travels with (None when there are none): the final
      // hidden state of a bfloat16 model before its rounding to 8 mantissa bits.  No counterpart in the reference.
      .def("take_fp32_shadow", [](Tensor& tensor) -> std::unique_ptr<Tensor> { return tensor.TakeShadow(); })
      .def("n_dim", &Tensor::n_dim)
      .def("shape", [](const Tensor& t, int pos) { return t.shape(pos); })
      .def("float_data", [](const Tensor& t) { return reinterpret_cast<uintptr_t>(t.data<float>()); })
      .def("is_null", &Tensor::is_null)
      .def("data_ptr", [](const Tensor& t) { return reinterpret_cast<uintptr_t>(t.raw()); })
      .def_static("create_empty", [] { return Tensor(nullptr); });

  py::class_<layers::BERTEmbedding>(m, "BERTEmbedding")
      .def(py::init([](Tensor& word, Tensor& position, Tensor& token_type, Tensor& ln_w, Tensor& ln_b) {
        return new layers::BERTEmbedding(std::move(word), std::move(position), std::move(token_type), std::move(ln_w),
                                         std::move(ln_b));
      }))
      .def("__call__", &layers::BERTEmbedding::operator());

  py::class_<layers::BertAttention>(m, "BertAttention")
      .def(py::init([](Tensor& qkv_w, Tensor& qkv_b, Tensor& dense_w, Tensor& dense_b, Tensor& ln_w, Tensor& ln_b, int heads) {
        return new layers::BertAttention(std::move(qkv_w), std::move(qkv_b), std::move(dense_w), std::move(dense_b),
                                         std::move(ln_w), std::move(ln_b), heads);
      }))
      .def("__call__", &layers::BertAttention::operator(), py::arg("input_tensor"), py::arg("attention_mask"),
           py::arg("output"), py::arg("attn") = nullptr, py::arg("is_trans_weight") = false);

  py::class_<layers::MultiHeadedAttention>(m, "MultiHeadedAttention")
      .def(py::init([](Tensor& kw, Tensor& kb, Tensor& vw, Tensor& vb, Tensor& qw, Tensor& qb, Tensor& dw, Tensor& db,
                       Tensor& qkvw, Tensor& qkvb, int heads) {
        return new layers::MultiHeadedAttention(std::move(kw), std::move(kb), std::move(vw), std::move(vb), std::move(qw),
                                                std::move(qb), std::move(dw), std::move(db), std::move(qkvw), std::move(qkvb),
                                                heads);
      }))
      .def(py::init([](Tensor& kw, Tensor& kb, Tensor& vw, Tensor& vb, Tensor& qw, Tensor& qb, Tensor& dw, Tensor& db,
                       Tensor& qkvw, Tensor& qkvb, Tensor& gamma, Tensor& beta, int heads) {
        return new layers::MultiHeadedAttention(std::move(kw), std::move(kb), std::move(vw), std::move(vb), std::move(qw),
                                                std::move(qb), std::move(dw), std::move(db), std::move(qkvw), std::move(qkvb),
                                                std::move(gamma), std::move(beta), heads);
      }))
      .def("__call__", &layers::MultiHeadedAttention::operator());

  py::class_<layers::MultiHeadedAttentionSmartBatch>(m, "MultiHeadedAttentionSmartBatch")
      .def(py::init([](Tensor& kw, Tensor& kb, Tensor& vw, Tensor& vb, Tensor& qw, Tensor& qb, Tensor& dw, Tensor& db,
                       Tensor& qkvw, Tensor& qkvb, int heads) {
        return new layers::MultiHeadedAttentionSmartBatch(std::move(kw), std::move(kb), std::move(vw), std::move(vb),
                                                          std::move(qw), std::move(qb), std::move(dw), std::move(db),
                                                          std::move(qkvw), std::move(qkvb), heads);
      }))
      .def(py::init([](Tensor& kw, Tensor& kb, Tensor& vw, Tensor& vb, Tensor& qw, Tensor& qb, Tensor& dw, Tensor& db,
                       Tensor& qkvw, Tensor& qkvb, Tensor& gamma, Tensor& beta, int heads) {
        return new layers::MultiHeadedAttentionSmartBatch(std::move(kw), std::move(kb), std::move(vw), std::move(vb),
                                                          std::move(qw), std::move(qb), std::move(dw), std::move(db),
                                                          std::move(qkvw), std::move(qkvb), std::move(gamma), std::move(beta),
                                                          heads);
      }))
      .def("__call__", &layers::MultiHeadedAttentionSmartBatch::operator());

  py::class_<layers::BertIntermediate>(m, "BertIntermediate")
      .def(py::init([](Tensor& w, Tensor& b) { return new layers::BertIntermediate(std::move(w), std::move(b)); }))
      .def("__call__", &layers::BertIntermediate::operator());

  py::class_<layers::BertOutput>(m, "BertOutput")
      .def(py::init([](Tensor& w, Tensor& b, Tensor& ln_w, Tensor& ln_b) {
        return new layers::BertOutput(std::move(w), std::move(b), std::move(ln_w), std::move(ln_b));
      }))
      .def("__call__", &layers::BertOutput::operator());

  py::class_<layers::SequencePool>(m, "SequencePool")
      .def(py::init([](const std::string& pool_type) { return new layers::SequencePool(pool_type); }))
      .def("__call__", &layers::SequencePool::operator());

  py::class_<layers::BertPooler>(m, "BertPooler")
      .def(py::init([](Tensor& w, Tensor& b) { return new layers::BertPooler(std::move(w), std::move(b)); }))
      .def("__call__", &layers::BertPooler::operator());

  py::class_<layers::PrepareBertMasks>(m, "PrepareBertMasks").def(py::init()).def("__call__", &layers::PrepareBertMasks::operator());

  py::class_<layers::AlbertLayer>(m, "AlbertLayer")
      .def(py::init([](Tensor& w1, Tensor& b1, Tensor& w2, Tensor& b2, Tensor& ln_w, Tensor& ln_b) {
        return new layers::AlbertLayer(std::move(w1), std::move(b1), std::move(w2), std::move(b2), std::move(ln_w),
                                       std::move(ln_b));
      }))
      .def("__call__", &layers::AlbertLayer::operator());

  py::class_<layers::PositionwiseFeedForward>(m, "PositionwiseFeedForward")
      .def(py::init([](Tensor& w1, Tensor& b1, Tensor& w2, Tensor& b2, Tensor& ln_w, Tensor& ln_b) {
        return new layers::PositionwiseFeedForward(std::move(w1), std::move(b1), std::move(w2), std::move(b2), std::move(ln_w),
                                                   std::move(ln_b));
      }))
      .def("__call__", &layers::PositionwiseFeedForward::operator());

  py::class_<layers::DistrillFFN>(m, "DistrillFFN")
      .def(py::init([](Tensor& w1, Tensor& b1, Tensor& w2, Tensor& b2, Tensor& ln_w, Tensor& ln_b) {
        return new layers::DistrillFFN(std::move(w1), std::move(b1), std::move(w2), std::move(b2), std::move(ln_w),
                                       std::move(ln_b));
      }))
      .def("__call__", &layers::DistrillFFN::operator());

  py::class_<layers::FusedAddBiasGELU>(m, "FusedAddBiasGELU")
      .def(py::init([](Tensor& bias) { return new layers::FusedAddBiasGELU(std::move(bias)); }))
      .def("__call__", &layers::FusedAddBiasGELU::operator());

  py::class_<layers::FusedAddBiasLayerNorm>(m, "FusedAddBiasLayerNorm")
      .def(py::init([](Tensor& bias, Tensor& ln_w, Tensor& ln_b) {
        return new layers::FusedAddBiasLayerNorm(std::move(bias), std::move(ln_w), std::move(ln_b));
      }))
      .def("__call__", &layers::FusedAddBiasLayerNorm::operator());

  py::class_<layers::LinearBias>(m, "LinearBias")
      .def(py::init([](Tensor& w, Tensor& b) { return new layers::LinearBias(std::move(w), std::move(b)); }))
      .def("__call__", &layers::LinearBias::operator());

  py::class_<layers::QuantizedLinear>(m, "QuantizedLinear")
      .def(py::init([](Tensor& w) { return new layers::QuantizedLinear(std::move(w)); }))
      .def(py::init([](Tensor& w, Tensor& bias, const std::string& activation) {
        return new layers::QuantizedLinear(std::move(w), std::move(bias), activation);
      }))
      .def("__call__", &layers::QuantizedLinear::operator());

  py::class_<layers::QuantizedBertAttention>(m, "QuantizedBertAttention")
      .def(py::init([](Tensor& qkv_w, Tensor& qkv_b, Tensor& dense_w, Tensor& dense_b, Tensor& ln_w, Tensor& ln_b, int heads) {
        return new layers::QuantizedBertAttention(std::move(qkv_w), std::move(qkv_b), std::move(dense_w), std::move(dense_b),
                                                  std::move(ln_w), std::move(ln_b), heads);
      }))
      .def("__call__", &layers::QuantizedBertAttention::operator(), py::arg("input_tensor"), py::arg("attention_mask"),
           py::arg("output"), py::arg("attn") = nullptr);

  m.def("build_smart_pad_mask",
        [](const std::vector<int64_t>& lens, Tensor* out) {
          auto plan = core::DeviceContext::GetInstance().GetSeqPlan(lens);
          float* mask = out->Reshape<float>({plan.batch, 1, plan.max_seq}, kDLROCM, 0, "SmartBatch/mask");
          TT_DEVICE_CALL(ttmi_smart_pad_mask(mask, plan.cu_seqlens, plan.batch, plan.max_seq,
                                             core::DeviceContext::GetInstance().stream()));
        },
        "Key-padding mask of a packed batch: fp32 [B,1,max_len], 0 on valid columns and -1e9 on columns >= len[b].");

  // ---- the C++ BertModel of example/cpp/bert_model.h, usable from Python as well ----------
  py::class_<BertModel>(m, "CxxBertModel")
      .def(py::init([](std::map<std::string, Tensor*> weights, size_t n_layers, int64_t n_heads) {
             BertModel::WeightMap owned;
             for (auto& kv : weights) owned.emplace(kv.first, std::move(*kv.second));
             return new BertModel(std::move(owned), kDLROCM, n_layers, n_heads);
           }),
           py::arg("weights"), py::arg("n_layers"), py::arg("n_heads"))
      .def(py::init([](const std::string& npz, size_t n_layers, int64_t n_heads) {
             return new BertModel(npz, kDLROCM, n_layers, n_heads);
           }),
           py::arg("npz_file"), py::arg("n_layers"), py::arg("n_heads"))
      .def("__call__",
           [](const BertModel& model, const std::vector<std::vector<int64_t>>& ids,
              const std::vector<std::vector<int64_t>>& pos, const std::vector<std::vector<int64_t>>& seg,
              const std::string& pooling, bool use_pooler) {
             layers::kernels::PoolType pt = layers::kernels::PoolType::kFirst;
             if (pooling == "Last") pt = layers::kernels::PoolType::kLast;
             else if (pooling == "Mean") pt = layers::kernels::PoolType::kMean;
             else if (pooling == "Max") pt = layers::kernels::PoolType::kMax;
             return model(ids, pos, seg, pt, use_pooler);
           },
           py::arg("inputs"), py::arg("position_ids"), py::arg("segment_ids"), py::arg("pooling") = "First",
           py::arg("use_pooler") = false)
      .def("encode",
           [](const BertModel& model, const Tensor& ids, Tensor* out) { model.Encode(ids, out); },
           "input_ids int64 [B,S] on the GPU -> last hidden state [B,S,H]; the whole forward in C++");

  // ---- additions of this build --------------------------------------------------------------
  // The layer loop of an encoder in one call: hidden -> [attention -> intermediate -> output] x layers -> out.  What the
  // Python BertEncoder does layer by layer, without a round trip through the interpreter per sub-layer (three calls,
  // three temporaries and a stream query each: at batch 1 x seq 128 the interpreter, not the GPU, set the pace).
  // `layer_list` is a sequence of (BertAttention, BertIntermediate, BertOutput).  No counterpart in the reference.
  m.def("run_bert_layers", [](const py::sequence& layer_list, const Tensor& hidden, const Tensor& mask, Tensor* out) {
    struct Sub {
      const layers::BertAttention* attention;
      const layers::BertIntermediate* intermediate;
      const layers::BertOutput* output;
    };
    std::vector<Sub> subs;
    subs.reserve(py::len(layer_list));
    for (const py::handle& item : layer_list) {
      const py::tuple t = py::cast<py::tuple>(item);
      TT_ENFORCE_EQ(py::len(t), (size_t)3, "each layer is (attention, intermediate, output)");
      subs.push_back(Sub{&py::cast<const layers::BertAttention&>(t[0]), &py::cast<const layers::BertIntermediate&>(t[1]),
                         &py::cast<const layers::BertOutput&>(t[2])});
    }
    TT_ENFORCE(!subs.empty() && out != nullptr, "run_bert_layers needs layers and an output tensor");
    Tensor attention_out(nullptr), intermediate_out(nullptr), even(nullptr), odd(nullptr);
    const Tensor* current = &hidden;
    for (size_t i = 0; i < subs.size(); ++i) {
      // the last layer writes the caller's tensor; before it two buffers alternate (a layer never writes what it reads)
      Tensor* target = (i + 1 == subs.size()) ? out : (i % 2 == 0 ? &even : &odd);
      (*subs[i].attention)(*current, mask, &attention_out, nullptr, false);
      (*subs[i].intermediate)(attention_out, &intermediate_out);
      (*subs[i].output)(intermediate_out, attention_out, target);
      current = target;
    }
  });

  m.def("set_stream", [](uintptr_t s) { core::DeviceContext::GetInstance().set_stream(reinterpret_cast<void*>(s)); },
        "Enqueue all following kernels on this hipStream_t (pass torch.cuda.current_stream().cuda_stream).");
  m.def("synchronize", [] { core::DeviceContext::GetInstance().Wait(); },
        "Wait for the work stream and raise if a kernel reported an error (e.g. embedding id out of range).");
  m.def("free_all_cached", [] { core::allocator::Allocator::GetInstance().FreeAllCached(); });
  m.def("allocator_stats", [] {
    auto s = core::allocator::Allocator::GetInstance().stats();
    py::dict d;
    d["device_mallocs"] = s.device_mallocs;
    d["cache_hits"] = s.cache_hits;
    d["bytes_live"] = s.bytes_live;
    d["bytes_cached"] = s.bytes_cached;
    d["oom_retries"] = s.oom_retries;
    return d;
  });
  m.def("allocator_schema", [] { return core::allocator::Allocator::GetInstance().schema(); });
  m.def("model_aware_chunks", [] { return core::allocator::Allocator::GetInstance().model_aware_chunks(); },
        "(number of chunks, total bytes) held by the model-aware plan");
  // The planner as plain functions, for tests: records are (name, start_op, end_op, size).
  using Rec = std::tuple<std::string, int64_t, int64_t, int64_t>;
  auto to_records = [](const std::vector<Rec>& in) {
    std::vector<core::allocator::TensorRecord> out;
    for (const auto& r : in) out.push_back({std::get<0>(r), std::get<1>(r), std::get<2>(r), std::get<3>(r)});
    return out;
  };
  m.def("bert_tensor_usage_records", [](int64_t b, int64_t s, int64_t h, int64_t hidden, int64_t layers) {
    std::vector<Rec> out;
    for (const auto& r : core::allocator::BertTensorUsageRecords(b, s, h, hidden, layers))
      out.emplace_back(r.name, r.start_op, r.end_op, r.size);
    return out;
  });
  m.def("plan_memory", [to_records](const std::vector<Rec>& records, std::vector<int64_t> chunk_sizes) {
    std::vector<core::allocator::Placement> placements;
    std::vector<bool> used;
    core::allocator::ChunkedGreedyBySizeOffsetCalculation(to_records(records), &chunk_sizes, &placements, &used);
    std::vector<std::pair<int, int64_t>> pl;
    for (const auto& p : placements) pl.emplace_back(p.chunk, p.offset);
    return py::make_tuple(pl, chunk_sizes, used);
  }, "-> (placements [(chunk, offset)], chunk sizes, chunk used flags)");
  m.def("placement_is_valid", [to_records](const std::vector<Rec>& records, const std::vector<int64_t>& chunk_sizes,
                                           const std::vector<std::pair<int, int64_t>>& placements) {
    std::vector<core::allocator::Placement> pl;
    for (const auto& p : placements) pl.push_back({p.first, p.second});
    return core::allocator::PlacementIsValid(to_records(records), chunk_sizes, pl);
  });
  m.def("set_allocator_device_limit_for_test",
        [](size_t bytes) { core::allocator::Allocator::GetInstance().set_device_limit_for_test(bytes); });
  m.def("load_npz",
        [](const std::string& path) {
          py::dict out;
          for (auto& kv : loaders::LoadNpz(path)) {
            const loaders::NpyArray& a = kv.second;
            py::dtype dt = a.kind == 'i' ? py::dtype::of<int64_t>() : (a.word_size == 4 ? py::dtype::of<float>() : py::dtype("float16"));
            py::array arr(dt, std::vector<py::ssize_t>(a.shape.begin(), a.shape.end()));
            std::memcpy(arr.mutable_data(), a.bytes.data(), a.bytes.size());
            out[py::str(kv.first)] = arr;
          }
          return out;
        },
        "Read an uncompressed .npz with the in-tree reader the C++ BertModel uses.");
  m.def("device_info", [] {
    char name[128];
    int cu = 0, clock = 0, lds = 0;
    int64_t hbm = 0;
    TT_DEVICE_CALL(ttmi_device_info(name, sizeof(name), &cu, &clock, &hbm, &lds));
    py::dict d;
    d["name"] = std::string(name);
    d["compute_units"] = cu;
    d["clock_khz"] = clock;
    d["hbm_bytes"] = hbm;
    d["lds_bytes_per_cu"] = lds;
    return d;
  });
}
