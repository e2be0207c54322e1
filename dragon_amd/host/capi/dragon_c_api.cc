#include "capi/dragon_c_api.h"

#include <cstdio>

#include "core/gradient.h"
#include "core/operator.h"
#include "core/workspace.h"

namespace {

thread_local std::string g_last_error;

// Inside this library a fatal condition unwinds to the API boundary instead of
// aborting the embedding process.
struct InstallHandler {
  InstallHandler() { dragon::SetFatalHandler(dragon::ThrowingFatalHandler); }
} g_install_handler;

template <typename F>
int Guarded(F f) {
  try {
    f();
    return 0;
  } catch (const std::exception& e) {
    g_last_error = e.what();
  } catch (...) {
    g_last_error = "unknown error";
  }
  return -1;
}

void CopyOut(const std::string& s, char* out, size_t bytes) {
  CHECK(out != nullptr && bytes > s.size()) << "\nOutput buffer too small: need " << s.size() + 1 << " bytes.";
  std::memcpy(out, s.c_str(), s.size() + 1);
}

dragon::Workspace* WS(void* ws) {
  CHECK(ws != nullptr) << "\nNull workspace.";
  return static_cast<dragon::Workspace*>(ws);
}

} // namespace

extern "C" {

const char* dragon_c_last_error(void) { return g_last_error.c_str(); }

int dragon_c_device_count(int* count) {
  return Guarded([&] { *count = dragon::HIPContext::device_count(); });
}

int dragon_c_registered_operators(char* out, size_t out_bytes) {
  return Guarded([&] {
    std::string s;
    for (const auto& k : dragon::HIPOperatorRegistry()->keys()) s += k + "\n";
    CopyOut(s, out, out_bytes);
  });
}

int dragon_c_workspace_create(const char* name, void** ws) {
  return Guarded([&] { *ws = new dragon::Workspace(name ? name : "default"); });
}

int dragon_c_workspace_destroy(void* ws) {
  return Guarded([&] { delete static_cast<dragon::Workspace*>(ws); });
}

int dragon_c_has_tensor(void* ws, const char* name, int* has) {
  return Guarded([&] {
    dragon::Tensor* t = WS(ws)->TryGetTensor(name);
    *has = (t != nullptr && t->has_memory()) ? 1 : 0;
  });
}

int dragon_c_reset_tensor(void* ws, const char* name) {
  return Guarded([&] { WS(ws)->ResetTensor(name); });
}

int dragon_c_feed_tensor(void* ws, const char* name, const char* dtype, int ndim,
                         const int64_t* dims, const void* host_data) {
  return Guarded([&] {
    const dragon::DType meta = dragon::DTypeFromName(dtype);
    CHECK(meta != dragon::DType::kUndefined) << "\nUnsupported dtype: " << dtype;
    dragon::Tensor* t = WS(ws)->CreateTensor(name);
    t->Reshape(dragon::vec64_t(dims, dims + ndim));
    void* dst = nullptr;
    switch (meta) {
      case dragon::DType::kFloat16: dst = t->mutable_data<dragon::float16, dragon::CPUContext>(); break;
      case dragon::DType::kBFloat16: dst = t->mutable_data<dragon::bfloat16, dragon::CPUContext>(); break;
      case dragon::DType::kFloat32: dst = t->mutable_data<float, dragon::CPUContext>(); break;
      case dragon::DType::kFloat64: dst = t->mutable_data<double, dragon::CPUContext>(); break;
      case dragon::DType::kInt64: dst = t->mutable_data<int64_t, dragon::CPUContext>(); break;
      case dragon::DType::kInt32: dst = t->mutable_data<int, dragon::CPUContext>(); break;
      default: LOG(FATAL) << "Unsupported dtype: " << dtype;
    }
    if (t->nbytes() > 0) std::memcpy(dst, host_data, t->nbytes());
  });
}

int dragon_c_tensor_info(void* ws, const char* name, char* dtype_buf, size_t dtype_bytes,
                         int* ndim, int64_t* dims) {
  return Guarded([&] {
    dragon::Tensor* t = WS(ws)->GetTensor(name);
    CopyOut(dragon::NameOf(t->meta()), dtype_buf, dtype_bytes);
    CHECK_LE(t->ndim(), 8) << "\nTensor has more than 8 dimensions.";
    *ndim = t->ndim();
    for (int i = 0; i < t->ndim(); ++i) dims[i] = t->dim(i);
  });
}

int dragon_c_fetch_tensor(void* ws, const char* name, void* host_out, size_t out_bytes) {
  return Guarded([&] {
    dragon::Tensor* t = WS(ws)->GetTensor(name);
    CHECK(t->has_memory()) << "\nTensor(" << name << ") was never written.";
    CHECK_GE(out_bytes, t->nbytes()) << "\nOutput buffer too small for Tensor(" << name << ").";
    const void* src = t->raw_data<dragon::CPUContext>();
    if (t->nbytes() > 0) std::memcpy(host_out, src, t->nbytes());
  });
}

int dragon_c_run_operator(void* ws, const char* def_text, int stream, int sync) {
  return Guarded([&] {
    const dragon::OperatorDef def = dragon::ParseOperatorDef(def_text);
    WS(ws)->RunOperator(def, stream, sync != 0);
  });
}

int dragon_c_make_gradient_defs(const char* def_text, const char* const* g_outputs,
                                int num_g_outputs, char* defs_out, size_t defs_bytes,
                                char* grad_inputs_out, size_t grad_inputs_bytes) {
  return Guarded([&] {
    const dragon::OperatorDef def = dragon::ParseOperatorDef(def_text);
    std::vector<std::string> gos(g_outputs, g_outputs + num_g_outputs), gis;
    std::string defs, inputs;
    for (const auto& g : dragon::MakeGradientDefs(def, gos, &gis)) defs += dragon::PrintOperatorDef(g) + "\n";
    for (const auto& g : gis) inputs += g + "\n";
    CopyOut(defs, defs_out, defs_bytes);
    CopyOut(inputs, grad_inputs_out, grad_inputs_bytes);
  });
}

} // extern "C"
