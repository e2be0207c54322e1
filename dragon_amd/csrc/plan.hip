// Plan query: which kernels an entry point would launch for a shape, found by
// running the entry point itself in plan-only mode (no launch, no device) with
// made-up 16-byte-aligned addresses. It has no counterpart in the reference; it
// exists so that a test without a GPU can pin the routing of the shapes that
// matter: a changed predicate that sends a shape to a slower fallback then fails
// a test and not only a benchmark.
#include <string.h>

#include "common.h"

namespace dragon_hip {
namespace {

// Distinct, aligned, never dereferenced.
inline void* fake(int k) { return reinterpret_cast<void*>(static_cast<uintptr_t>(0x100000000ull) * (k + 1)); }

struct PlanScope {
  PlanScope() {
    LaunchTrace& t = launch_trace();
    t.recording = true;
    t.plan_only = true;
    t.used = 0;
    t.text[0] = 0;
  }
  ~PlanScope() {
    LaunchTrace& t = launch_trace();
    t.recording = false;
    t.plan_only = false;
  }
};

}  // namespace
}  // namespace dragon_hip

extern "C" int dragon_hip_plan_name(const char* op, int dtype, int layout, const int64_t* dims,
                                    int num_dims, char* buf, size_t buf_bytes) {
  using dragon_hip::fake;
  if (!op || !dims || !buf || buf_bytes == 0) return DRAGON_HIP_EINVAL;
  auto dim = [&](int i) { return i < num_dims ? dims[i] : 1; };
  const size_t big = static_cast<size_t>(1) << 40;  // scratch is assumed large enough
  int rc = DRAGON_HIP_OK;
  bool known = true;
  {
    dragon_hip::PlanScope scope;
    void* s = nullptr;  // the default stream
    if (!strcmp(op, "layer_norm")) {
      rc = dragon_hip_layer_norm(dtype, dim(0), dim(1), 1e-5f, fake(0), fake(1), fake(2), fake(3),
                                 fake(4), fake(5), s);
    } else if (!strcmp(op, "layer_norm_grad")) {
      rc = dragon_hip_group_norm_grad(dtype, dim(0), 1, dim(1), 1, DRAGON_HIP_NHWC, fake(0), fake(1),
                                      fake(2), fake(3), fake(4), fake(5), fake(5), fake(6), fake(7),
                                      fake(8), fake(9), big, s);
    } else if (!strcmp(op, "group_norm_forward")) {
      rc = dragon_hip_group_norm_forward(dtype, dim(0), dim(1), dim(2), dim(3), layout, 1e-5f, fake(0),
                                         fake(1), fake(2), fake(3), fake(4), fake(5), fake(6), big, s);
    } else if (!strcmp(op, "group_norm_grad")) {
      rc = dragon_hip_group_norm_grad(dtype, dim(0), dim(1), dim(2), dim(3), layout, fake(0), fake(1),
                                      fake(2), fake(3), fake(4), fake(5), fake(5), fake(6), fake(7),
                                      fake(8), fake(9), big, s);
    } else if (!strcmp(op, "batch_norm_training_forward")) {
      rc = dragon_hip_batch_norm_training_forward(dtype, dim(0), dim(1), dim(2), layout, 0.9f, 1e-5f,
                                                  fake(0), fake(1), fake(2), fake(3), fake(4), fake(5),
                                                  fake(6), fake(7), fake(8), fake(9), big, s);
    } else if (!strcmp(op, "batch_norm_training_backward")) {
      rc = dragon_hip_batch_norm_training_backward(
          dtype, dim(0), dim(1), dim(2), static_cast<float>(dim(0) * dim(2)), layout, fake(0), fake(1),
          fake(2), fake(3), fake(4), fake(5), fake(5), fake(6), fake(7), big, s);
    } else if (!strcmp(op, "softmax")) {
      rc = dragon_hip_softmax(dtype, dim(0), dim(1), dim(2), fake(0), fake(1), fake(2), big, s);
    } else if (!strcmp(op, "log_softmax")) {
      rc = dragon_hip_log_softmax(dtype, dim(0), dim(1), dim(2), fake(0), fake(1), fake(2), big, s);
    } else if (!strcmp(op, "softmax_grad")) {
      rc = dragon_hip_softmax_grad(dtype, dim(0), dim(1), dim(2), fake(0), fake(1), fake(2), fake(3),
                                   big, s);
    } else if (!strcmp(op, "log_softmax_grad")) {
      rc = dragon_hip_log_softmax_grad(dtype, dim(0), dim(1), dim(2), fake(0), fake(1), fake(2),
                                       fake(3), big, s);
    } else if (!strcmp(op, "l2_norm")) {
      rc = dragon_hip_l2_norm(dtype, dim(0), dim(1), dim(2), 1.0f, 1e-12f, fake(0), fake(1), s);
    } else if (!strcmp(op, "l2_norm_grad")) {
      rc = dragon_hip_l2_norm_grad(dtype, dim(0), dim(1), dim(2), 1.0f, 1e-12f, fake(0), fake(1),
                                   fake(2), s);
    } else if (!strcmp(op, "l1_norm")) {
      rc = dragon_hip_l1_norm(dtype, dim(0), dim(1), dim(2), 1.0f, 1e-12f, fake(0), fake(1), s);
    } else if (!strcmp(op, "l1_norm_grad")) {
      rc = dragon_hip_l1_norm_grad(dtype, dim(0), dim(1), dim(2), 1.0f, 1e-12f, fake(0), fake(1),
                                   fake(2), s);
    } else if (!strcmp(op, "softmax_cross_entropy_loss_forward")) {
      rc = dragon_hip_softmax_cross_entropy_loss_forward(dtype, DRAGON_HIP_I64, dim(0), dim(1), dim(2),
                                                         255, 4 /* VALID */, fake(0), fake(1),
                                                         fake(2), fake(3), fake(4), big, s);
    } else if (!strcmp(op, "softmax_cross_entropy_loss_backward")) {
      rc = dragon_hip_softmax_cross_entropy_loss_backward(dtype, DRAGON_HIP_I64, dim(0), dim(1),
                                                          dim(2), 255, 4 /* VALID */, fake(0),
                                                          fake(1), fake(2), fake(3), fake(4), big, s);
    } else {
      known = false;
    }
    (void)hipGetLastError();  // without a device the launch paths' queries fail: not an error here
    if (known) {
      const dragon_hip::LaunchTrace& t = dragon_hip::launch_trace();
      const size_t n = t.used < buf_bytes - 1 ? t.used : buf_bytes - 1;
      memcpy(buf, t.text, n);
      buf[n] = 0;
    }
  }
  if (!known) return DRAGON_HIP_EINVAL;
  // An argument error of the entry point itself (a shape it rejects) is the caller's to see.
  if (rc == DRAGON_HIP_EINVAL || rc == DRAGON_HIP_EDTYPE) return rc;
  return static_cast<int>(strlen(buf));
}
