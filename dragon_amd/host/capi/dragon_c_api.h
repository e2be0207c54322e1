/*
 * C API of the host layer: create a workspace, feed and fetch tensors, run
 * operator definitions given in protobuf text format, and derive gradient
 * definitions. It plays the role the pybind11 module and the C++ runtime API
 * play in the reference (dragon/modules/python/module.cc:84-173,
 * dragon/modules/runtime/dragon_runtime.h:30-128) for the operators of this
 * path, so that tests can drive the C++ operators from Python through ctypes.
 *
 * Every function returns 0 on success and -1 on failure; the message of the
 * failure (what the reference would print before aborting) is available from
 * dragon_c_last_error() on the calling thread.
 */
#ifndef DRAGON_C_API_H_
#define DRAGON_C_API_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

const char* dragon_c_last_error(void);

int dragon_c_device_count(int* count);
/* Newline-separated names of the operator types registered for the HIP device. */
int dragon_c_registered_operators(char* out, size_t out_bytes);

int dragon_c_workspace_create(const char* name, void** ws);
int dragon_c_workspace_destroy(void* ws);
int dragon_c_has_tensor(void* ws, const char* name, int* has);
int dragon_c_reset_tensor(void* ws, const char* name);

/* Copies `host_data` (dtype: float16|bfloat16|float32|float64|int64) into the
 * tensor; it moves to the device when an operator first reads it there. */
int dragon_c_feed_tensor(void* ws, const char* name, const char* dtype, int ndim,
                         const int64_t* dims, const void* host_data);
/* dims must hold 8 entries; dtype_buf receives the type name. */
int dragon_c_tensor_info(void* ws, const char* name, char* dtype_buf, size_t dtype_bytes,
                         int* ndim, int64_t* dims);
/* Copies the tensor to `host_out` (synchronising device -> host if needed). */
int dragon_c_fetch_tensor(void* ws, const char* name, void* host_out, size_t out_bytes);

/* Runs one OperatorDef (protobuf text format) on stream `stream`; `sync` != 0
 * waits for the stream before returning. */
int dragon_c_run_operator(void* ws, const char* def_text, int stream, int sync);

/* Gradient definitions of `def_text` given the names of the output gradients.
 * `defs_out` receives the definitions, one per line; `grad_inputs_out` the
 * newline-separated names of the input gradients ("" for inputs without one). */
int dragon_c_make_gradient_defs(const char* def_text, const char* const* g_outputs,
                                int num_g_outputs, char* defs_out, size_t defs_bytes,
                                char* grad_inputs_out, size_t grad_inputs_bytes);

#ifdef __cplusplus
}
#endif

#endif /* DRAGON_C_API_H_ */
