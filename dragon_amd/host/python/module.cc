// pybind11 module of the host layer: what the reference's compiled module
// (dragon/modules/python/module.cc:26-173) exposes of Workspace and Tensor for
// this path, the HIP counterpart of its device sub-module
// (dragon/modules/python/cuda.h:24-176: device queries, current device, seed,
// stream synchronisation, the stream class), and the numpy <-> tensor
// conversions with a HIP branch (dragon/modules/python/numpy.h:31-150).
// Everything binds the C++ classes of this directory directly.
//
// 16-bit types: float16 maps to numpy float16. numpy has no bfloat16 (the
// reference falls back to a run-time registered type, numpy.h:40-45,93-99);
// here a bfloat16 tensor goes to numpy as its uint16 bit patterns, and
// FromNumpy takes the type name beside a uint16 array.
#include <pybind11/numpy.h>
#include <pybind11/pybind11.h>
#include <pybind11/stl.h>

#include "core/context.h"
#include "core/gradient.h"
#include "core/operator.h"
#include "core/workspace.h"
#include "dragon_hip.h"

namespace py = pybind11;

namespace dragon {
namespace python {
namespace {

py::dtype NumpyTypeOf(DType meta) {
  switch (meta) {
    case DType::kFloat16: return py::dtype("float16");
    case DType::kBFloat16: return py::dtype("uint16");
    case DType::kFloat32: return py::dtype("float32");
    case DType::kFloat64: return py::dtype("float64");
    case DType::kInt64: return py::dtype("int64");
    case DType::kInt32: return py::dtype("int32");
    case DType::kUInt8: return py::dtype("uint8");
    default: break;
  }
  LOG(FATAL) << "Unsupported " << NameOf(meta) << " tensor to numpy.";
  return py::dtype("uint8");
}

DType TypeOfNumpy(const py::array& array, const string& dtype) {
  if (!dtype.empty()) {
    const DType meta = DTypeFromName(dtype);
    CHECK(meta != DType::kUndefined) << "\nUnsupported dtype: " << dtype;
    CHECK_EQ(static_cast<size_t>(array.itemsize()), SizeOf(meta))
        << "\nArray items of " << array.itemsize() << " bytes cannot hold " << dtype << ".";
    return meta;
  }
  const char kind = array.dtype().kind();
  const auto size = array.itemsize();
  if (kind == 'f' && size == 2) return DType::kFloat16;
  if (kind == 'f' && size == 4) return DType::kFloat32;
  if (kind == 'f' && size == 8) return DType::kFloat64;
  if (kind == 'i' && size == 8) return DType::kInt64;
  if (kind == 'i' && size == 4) return DType::kInt32;
  if (kind == 'u' && size == 1) return DType::kUInt8;
  LOG(FATAL) << "Unsupported numpy type to tensor.";
  return DType::kUndefined;
}

void* MutableData(Tensor* t, DType meta, bool on_device) {
#define DRAGON_CASE(T)                                                  \
  return on_device ? static_cast<void*>(t->mutable_data<T, HIPContext>()) \
                   : static_cast<void*>(t->mutable_data<T, CPUContext>())
  switch (meta) {
    case DType::kFloat16: DRAGON_CASE(float16);
    case DType::kBFloat16: DRAGON_CASE(bfloat16);
    case DType::kFloat32: DRAGON_CASE(float);
    case DType::kFloat64: DRAGON_CASE(double);
    case DType::kInt64: DRAGON_CASE(int64_t);
    case DType::kInt32: DRAGON_CASE(int);
    case DType::kUInt8: DRAGON_CASE(uint8_t);
    default: break;
  }
#undef DRAGON_CASE
  LOG(FATAL) << "Unsupported dtype: " << NameOf(meta);
  return nullptr;
}

// NumpyWrapper::To with copy: a new array filled from wherever the tensor's
// up-to-date copy lives, straight from device memory when that is the device.
py::array TensorToNumpy(Tensor* self) {
  CHECK(self->meta() != DType::kUndefined) << "\nAn empty tensor to numpy.";
  CHECK(self->has_memory()) << "\nAn empty tensor to numpy.";
  std::vector<py::ssize_t> dims(self->dims().begin(), self->dims().end());
  py::array array(NumpyTypeOf(self->meta()), dims);
  if (self->nbytes() == 0) return array;
  UnifiedMemory* memory = self->memory();
  if (memory->device_type() == "hip") {
    HIPDeviceGuard guard(memory->device());
    HIPContext::Memcpy<CPUContext, HIPContext>(self->nbytes(), array.mutable_data(),
                                               self->raw_data<HIPContext>());
  } else {
    std::memcpy(array.mutable_data(), self->raw_data<CPUContext>(), self->nbytes());
  }
  return array;
}

// NumpyWrapper::From with copy. `device_type` "hip" writes the array straight
// into device memory of `device_id` (the branch numpy.h:104-113 takes for a
// tensor that lives on the device); "cpu" leaves the move to the first
// operator that reads the tensor there.
void TensorFromNumpy(Tensor* self, const py::array& obj, const string& dtype,
                     const string& device_type, int device_id) {
  const py::array array = py::array::ensure(obj, py::array::c_style);
  CHECK(array) << "\nExpected a numpy array.";
  const DType meta = TypeOfNumpy(array, dtype);
  vec64_t dims(array.shape(), array.shape() + array.ndim());
  self->Reshape(dims);
  if (device_type == "hip") {
    HIPDeviceGuard guard(device_id);
    void* dst = MutableData(self, meta, true);
    if (self->nbytes() > 0) {
      HIPContext::Memcpy<HIPContext, CPUContext>(self->nbytes(), dst, array.data());
    }
  } else {
    CHECK(device_type == "cpu") << "\nUnsupported device type: " << device_type;
    void* dst = MutableData(self, meta, false);
    if (self->nbytes() > 0) std::memcpy(dst, array.data(), self->nbytes());
  }
}

int ResolveDevice(int device_id) { return device_id < 0 ? HIPContext::current_device() : device_id; }

}  // namespace

void RegisterModule_hip(py::module& m) {
  m.def("hipIsDriverSufficient", []() {
    int count = 0;
    return dragon_hip_device_count(&count) == 0;
  });
  m.def("hipGetDevice", []() { return HIPContext::current_device(); });
  m.def("hipGetDeviceCount", []() { return HIPContext::device_count(); });
  m.def("hipGetDeviceName", [](int device_id) {
    char name[256] = {0};
    HIP_CHECK(dragon_hip_device_name(ResolveDevice(device_id), name, sizeof(name)));
    return string(name);
  });
  m.def("hipGetDeviceCapability", [](int device_id) {
    int major = 0, minor = 0;
    HIP_CHECK(dragon_hip_device_capability(ResolveDevice(device_id), &major, &minor));
    return std::tuple<int, int>(major, minor);
  });
  m.def("hipSetDevice", [](int device_id) { HIPContext::objects().SetDevice(device_id); });
  m.def("hipSetRandomSeed", [](int device_id, int seed) {
    HIPContext::objects().SetRandomSeed(ResolveDevice(device_id), seed);
  });
  m.def("hipGetRandomSeed",
        [](int device_id) { return HIPContext::objects().GetRandomSeed(ResolveDevice(device_id)); });
  m.def("hipStreamSynchronize", [](int device_id, int stream_id) {
    const int device = ResolveDevice(device_id);
    HIPDeviceGuard guard(device);
    py::gil_scoped_release g;
    HIPContext::SynchronizeStream(HIPContext::objects().stream(device, stream_id));
  });
  m.def("hipDeviceSynchronize", [](int device_id) {
    HIPDeviceGuard guard(ResolveDevice(device_id));
    py::gil_scoped_release g;
    HIP_CHECK(dragon_hip_device_sync());
  });

  py::class_<HIPStream>(m, "HIPStream")
      .def(py::init<int>())
      .def_property_readonly("index", &HIPStream::stream_id)
      .def_property_readonly("device_index", &HIPStream::device_id)
      .def_property_readonly("ptr", [](HIPStream* self) { return (intptr_t)self->impl(); })
      .def("Query", &HIPStream::Query)
      .def("Synchronize", [](HIPStream* self) {
        py::gil_scoped_release g;
        self->Synchronize();
      });
}

void RegisterModule_tensor(py::module& m) {
  py::class_<Tensor>(m, "Tensor")
      .def_property_readonly("name", &Tensor::name)
      .def_property_readonly("ndim", &Tensor::ndim)
      .def_property_readonly("dims", &Tensor::dims)
      .def_property_readonly("size", &Tensor::size)
      .def_property_readonly("itemsize", [](Tensor* self) { return SizeOf(self->meta()); })
      .def_property_readonly("nbytes", &Tensor::nbytes)
      .def_property_readonly("capacity", &Tensor::capacity)
      .def_property_readonly("dtype", [](Tensor* self) { return string(NameOf(self->meta())); })
      .def_property_readonly("device",
                             [](Tensor* self) {
                               if (!self->has_memory()) return std::tuple<string, int>("unknown", 0);
                               UnifiedMemory* memory = self->memory();
                               const string type = memory->device_type();
                               return std::tuple<string, int>(type, type == "hip" ? memory->device() : 0);
                             })
      .def("data",
           [](Tensor* self, const string& device_type) {
             if (device_type == "cpu") return (intptr_t)self->raw_data<CPUContext>();
             CHECK(device_type == "hip") << "\nUnsupported device type: " << device_type;
             return (intptr_t)self->raw_data<HIPContext>();
           })
      .def("mutable_data",
           [](Tensor* self, const string& device_type) {
             if (device_type == "cpu") return (intptr_t)self->raw_mutable_data<CPUContext>();
             CHECK(device_type == "hip") << "\nUnsupported device type: " << device_type;
             return (intptr_t)self->raw_mutable_data<HIPContext>();
           })
      .def("Reshape", [](Tensor* self, const vec64_t& dims) { self->Reshape(dims); })
      .def("ToNumpy", [](Tensor* self) { return TensorToNumpy(self); })
      .def("FromNumpy", &TensorFromNumpy, py::arg("array"), py::arg("dtype") = "",
           py::arg("device_type") = "cpu", py::arg("device_id") = 0);
}

void RegisterModule_workspace(py::module& m) {
  py::class_<Workspace>(m, "Workspace")
      .def(py::init<const string&>())
      .def_property_readonly("name", &Workspace::name)
      .def_property_readonly("tensors", &Workspace::tensors)
      .def_property_readonly("num_cached_operators", &Workspace::num_cached_operators)
      .def("HasTensor",
           [](Workspace* self, const string& name) {
             Tensor* t = self->TryGetTensor(name);
             return t != nullptr && t->has_memory();
           })
      .def("CreateTensor", &Workspace::CreateTensor, py::return_value_policy::reference)
      .def("GetTensor", [](Workspace* self, const string& name) { return self->TryGetTensor(name); },
           py::return_value_policy::reference)
      .def("ResetTensor", &Workspace::ResetTensor)
      .def("MemoryAllocated",
           [](Workspace* self, const string& device_type, int device_id) {
             size_t size = 0;
             for (const auto& name : self->tensors()) {
               Tensor* t = self->TryGetTensor(name);
               if (t == nullptr || !t->has_memory()) continue;
               size += t->memory()->size(device_type, device_id);
             }
             return size;
           })
      // An OperatorDef travels as protobuf text (this build has no protobuf
      // runtime to parse the serialized form the reference passes).
      .def("RunOperator",
           [](Workspace* self, const string& def_text, int stream, bool sync) {
             const OperatorDef def = ParseOperatorDef(def_text);
             py::gil_scoped_release g;
             self->RunOperator(def, stream, sync);
           },
           py::arg("def_text"), py::arg("stream") = 0, py::arg("sync") = true)
      .def("RunOperator",
           [](Workspace* self, const vector<string>& def_texts, int stream, bool sync) {
             vector<OperatorDef> defs;
             for (const auto& text : def_texts) defs.push_back(ParseOperatorDef(text));
             py::gil_scoped_release g;
             for (const auto& def : defs) self->RunOperator(def, stream, sync);
           },
           py::arg("def_texts"), py::arg("stream") = 0, py::arg("sync") = true);
}

}  // namespace python
}  // namespace dragon

PYBIND11_MODULE(libdragon_hip_python, m) {
  using namespace dragon;
  m.doc() = "Workspace, Tensor, operator execution and HIP device utilities of the host layer";
  // A fatal condition (the reference's LOG(FATAL)) surfaces as a Python exception.
  SetFatalHandler(ThrowingFatalHandler);
  python::RegisterModule_hip(m);
  python::RegisterModule_tensor(m);
  python::RegisterModule_workspace(m);
  m.def("RegisteredOperators", []() { return HIPOperatorRegistry()->keys(); });
  m.def("MakeGradientDefs", [](const string& def_text, const vector<string>& grad_outputs) {
    vector<string> grad_inputs, defs;
    for (const auto& g : MakeGradientDefs(ParseOperatorDef(def_text), grad_outputs, &grad_inputs)) {
      defs.push_back(PrintOperatorDef(g));
    }
    return std::make_tuple(defs, grad_inputs);
  });
}
