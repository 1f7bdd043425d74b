// TVM-FFI plugin entry points: decode the TVMFFIAny argument array the reference's executor passes to
// `executor.call_plugin` (mlir-tensorrt/executor/lib/Runtime/FFI/FFI.cpp:56-104) and forward to the cluster
// layer.  The argument layout is the one of mlir-tensorrt/executor/lib/Passes/TVMFFIUtils.cpp:304-423.
#include <cstdarg>
#include <cstdio>
#include <cstring>

#include "mtrt_hip_tvm_ffi.h"
#include "runtime_internal.hpp"

extern "C" {
// libtvm_ffi's own entry points (apache-tvm-ffi 0.1.3, c_api.h / extra/c_env_api.h); absent unless the host
// process has loaded that library
void *TVMFFIEnvGetStream(int32_t device_type, int32_t device_id) __attribute__((weak));
void TVMFFIErrorSetRaisedFromCStr(const char *kind, const char *message) __attribute__((weak));
}

namespace {

struct Failure {
  char text[512];
};

int fail(const char *kind, const char *fmt, ...) {
  Failure f;
  va_list ap;
  va_start(ap, fmt);
  std::vsnprintf(f.text, sizeof(f.text), fmt, ap);
  va_end(ap);
  mtrt_rt::set_error(MTRT_INVALID_ARGUMENT, "%s: %s", kind, f.text);   // also readable through mtrt_hip_last_error()
  if (TVMFFIErrorSetRaisedFromCStr)
    TVMFFIErrorSetRaisedFromCStr(kind, f.text);
  return -1;
}

// the message of a failed cluster call travels on as the plugin's error
int forward(int32_t status) {
  if (status == MTRT_OK)
    return 0;
  const std::string message = mtrt_hip_last_error();    // fail() rewrites the buffer it points into
  return fail(status == MTRT_INVALID_ARGUMENT ? "ValueError" : "RuntimeError", "%s", message.c_str());
}

bool is_gpu(const mtrt_dl_tensor *t) { return t->device_type == 2 || t->device_type == 10; }

int64_t numel(const mtrt_dl_tensor *t) {
  int64_t n = 1;
  for (int32_t i = 0; i < t->ndim; ++i)
    n *= t->shape[i];
  return n;
}

bool contiguous(const mtrt_dl_tensor *t) {
  if (!t->strides)
    return true;
  int64_t expect = 1;
  for (int32_t i = t->ndim - 1; i >= 0; --i) {
    if (t->shape[i] != 1 && t->strides[i] != expect)
      return false;
    expect *= t->shape[i];
  }
  return true;
}

void *data_of(const mtrt_dl_tensor *t) { return static_cast<char *>(t->data) + t->byte_offset; }

// DLPack dtype -> mtrt_hip_dtype, or -1
int32_t dtype_of(const mtrt_dl_tensor *t) {
  if (t->dtype_lanes != 1)
    return -1;
  if (t->dtype_code == 2 && t->dtype_bits == 32)
    return MTRT_F32;
  if (t->dtype_code == 2 && t->dtype_bits == 16)
    return MTRT_F16;
  if (t->dtype_code == 4 && t->dtype_bits == 16)
    return MTRT_BF16;
  if (t->dtype_code == 0 && t->dtype_bits == 8)
    return MTRT_I8;
  if (t->dtype_code == 10 && t->dtype_bits == 8)
    return MTRT_F8E4M3FN;
  return -1;
}

struct Args {
  const char *func;
  const mtrt_tvm_ffi_any *args;
  int32_t n;
  // argument i as a contiguous GPU tensor; null (and the error raised) otherwise
  const mtrt_dl_tensor *tensor(int32_t i, const char *name) const {
    if (i >= n || args[i].type_index != MTRT_TVM_FFI_DLTENSOR_PTR || !args[i].value.v_ptr) {
      fail("TypeError", "%s: argument %d (%s) must be a tensor", func, i, name);
      return nullptr;
    }
    const auto *t = static_cast<const mtrt_dl_tensor *>(args[i].value.v_ptr);
    if (!is_gpu(t)) {
      fail("ValueError", "%s: %s must live in GPU memory (device type %d)", func, name, t->device_type);
      return nullptr;
    }
    if (t->ndim < 0 || (t->ndim > 0 && !t->shape) || !contiguous(t)) {
      fail("ValueError", "%s: %s must be a contiguous tensor", func, name);
      return nullptr;
    }
    return t;
  }
  // optional integer argument i: false when absent or None
  bool integer(int32_t i, int64_t *out) const {
    if (i >= n || args[i].type_index == MTRT_TVM_FFI_NONE)
      return false;
    *out = args[i].value.v_int64;
    return args[i].type_index == MTRT_TVM_FFI_INT || args[i].type_index == MTRT_TVM_FFI_BOOL;
  }
  bool real(int32_t i, double *out) const {
    if (i >= n)
      return false;
    if (args[i].type_index == MTRT_TVM_FFI_FLOAT) {
      *out = args[i].value.v_float64;
      return true;
    }
    if (args[i].type_index == MTRT_TVM_FFI_INT) {
      *out = double(args[i].value.v_int64);
      return true;
    }
    return false;
  }
};

mtrt_stream_t stream_for(const mtrt_dl_tensor *t) {
  if (!TVMFFIEnvGetStream)
    return nullptr;
  return static_cast<mtrt_stream_t>(TVMFFIEnvGetStream(t->device_type, t->device_id));
}

void set_none(mtrt_tvm_ffi_any *result) {
  if (result) {
    result->type_index = MTRT_TVM_FFI_NONE;
    result->zero_padding = 0;
    result->value.v_int64 = 0;
  }
}

// (scale kind, d0, d1, nb) of the cluster layer from the shapes, by the op's own rules
// (mlir-tensorrt/tensorrt/lib/TensorRT/IR/Verification.cpp:1182-1265): one scale element = per-tensor; a 1-D
// scale with an axis = per-channel; a scale of the data's rank that differs in the last or second-to-last
// extent = block.
int addressing(const char *func, const mtrt_dl_tensor *data, const mtrt_dl_tensor *scale, bool has_axis, int64_t axis,
               int32_t *kind, int64_t *d0, int64_t *d1, int64_t *nb) {
  const int32_t rank = data->ndim;
  const int64_t n = numel(data);
  if (!has_axis && numel(scale) == 1 && scale->ndim <= 1) {
    *kind = MTRT_SCALE_UNIFORM;
    *d1 = rank ? data->shape[rank - 1] : 1;
    *d0 = *d1 ? n / *d1 : 0;
    *nb = 1;
    return 0;
  }
  if (has_axis) {
    if (axis < 0 || axis >= rank)
      return fail("ValueError", "%s: axis %lld is outside [0, %d)", func, (long long)axis, rank);
    if (scale->ndim != 1 || scale->shape[0] != data->shape[axis])
      return fail("ValueError", "%s: per-channel scale must be 1-D with %lld elements", func, (long long)data->shape[axis]);
    const int64_t c = data->shape[axis];
    int64_t inner = 1;
    for (int32_t i = int32_t(axis) + 1; i < rank; ++i)
      inner *= data->shape[i];
    if (inner == 1) {
      *kind = MTRT_SCALE_COL;
      *d0 = c ? n / c : 0;
      *d1 = c;
      *nb = *d0 > 0 ? *d0 : 1;
    } else {
      *kind = MTRT_SCALE_ROW;
      *d0 = n / inner;
      *d1 = inner;
      *nb = c;
    }
    return 0;
  }
  if (scale->ndim != rank || rank < 1)
    return fail("ValueError", "%s: scale must have one element, or be 1-D with an axis, or have the data's rank", func);
  int32_t blocked = -1;
  for (int32_t i = 0; i < rank; ++i)
    if (scale->shape[i] != data->shape[i]) {
      if (blocked >= 0)
        return fail("ValueError", "%s: block scale may differ from the data in one dimension only", func);
      blocked = i;
    }
  if (blocked < 0 || (blocked != rank - 1 && blocked != rank - 2))
    return fail("ValueError", "%s: the blocked dimension must be the last or the second-to-last", func);
  if (scale->shape[blocked] <= 0 || data->shape[blocked] % scale->shape[blocked] != 0)
    return fail("ValueError", "%s: the scale extent must divide the blocked extent", func);
  const int64_t block = data->shape[blocked] / scale->shape[blocked];
  if (blocked == rank - 1) {
    *kind = MTRT_SCALE_ROW;
    *d0 = n / block;
    *d1 = block;
    *nb = *d0 > 0 ? *d0 : 1;
  } else {
    *kind = MTRT_SCALE_COL;
    *d1 = data->shape[rank - 1];
    *d0 = *d1 ? n / *d1 : 0;
    *nb = block;
  }
  return 0;
}

int qdq(const char *func, bool quantize, const mtrt_tvm_ffi_any *args, int32_t num_args, mtrt_tvm_ffi_any *result) {
  const Args a{func, args, num_args};
  if (num_args < 3 || num_args > 4)
    return fail("TypeError", "%s expects (input, scale, output [, axis]), got %d arguments", func, num_args);
  const mtrt_dl_tensor *in = a.tensor(0, "input"), *scale = in ? a.tensor(1, "scale") : nullptr,
                       *out = scale ? a.tensor(2, "output") : nullptr;
  if (!out)
    return -1;
  int64_t axis = 0;
  const bool has_axis = a.integer(3, &axis);
  if (dtype_of(scale) != MTRT_F32)
    return fail("TypeError", "%s: scale must be float32", func);
  if (numel(in) != numel(out) || in->ndim != out->ndim)
    return fail("ValueError", "%s: input and output must have the same shape", func);
  const mtrt_dl_tensor *data = quantize ? in : out;    // the float side carries the shape rules
  int32_t kind = MTRT_SCALE_UNIFORM;
  int64_t d0 = 0, d1 = 0, nb = 1;
  if (addressing(func, data, scale, has_axis, axis, &kind, &d0, &d1, &nb) != 0)
    return -1;
  const int32_t in_dt = dtype_of(in), out_dt = dtype_of(out);
  if (in_dt < 0 || out_dt < 0)
    return fail("TypeError", "%s: unsupported element type", func);
  const mtrt_stream_t stream = stream_for(in);
  const int32_t st = quantize ? mtrt_hip_quantize(stream, data_of(in), in_dt, data_of(out), out_dt,
                                                  static_cast<const float *>(data_of(scale)), kind, d0, d1, nb, 0)
                              : mtrt_hip_dequantize(stream, data_of(in), in_dt, data_of(out), out_dt,
                                                    static_cast<const float *>(data_of(scale)), kind, d0, d1, nb);
  set_none(result);
  return forward(st);
}

} // namespace

extern "C" {

int __tvm_ffi_mtrt_quantize(void *, const mtrt_tvm_ffi_any *args, int32_t num_args, mtrt_tvm_ffi_any *result) {
  return qdq("mtrt_quantize", true, args, num_args, result);
}

int __tvm_ffi_mtrt_dequantize(void *, const mtrt_tvm_ffi_any *args, int32_t num_args, mtrt_tvm_ffi_any *result) {
  return qdq("mtrt_dequantize", false, args, num_args, result);
}

int __tvm_ffi_mtrt_amax(void *, const mtrt_tvm_ffi_any *args, int32_t num_args, mtrt_tvm_ffi_any *result) {
  const Args a{"mtrt_amax", args, num_args};
  if (num_args != 3)
    return fail("TypeError", "mtrt_amax expects (x, amax_and_scale, qmax), got %d arguments", num_args);
  const mtrt_dl_tensor *x = a.tensor(0, "x"), *out = x ? a.tensor(1, "amax_and_scale") : nullptr;
  if (!out)
    return -1;
  double qmax = 0.0;
  if (!a.real(2, &qmax))
    return fail("TypeError", "mtrt_amax: qmax must be a number");
  if (dtype_of(out) != MTRT_F32 || numel(out) != 2)
    return fail("ValueError", "mtrt_amax: amax_and_scale must be float32[2]");
  float *o = static_cast<float *>(data_of(out));
  set_none(result);
  return forward(mtrt_hip_amax(stream_for(x), data_of(x), dtype_of(x), numel(x), float(qmax), o, o + 1));
}

int __tvm_ffi_mtrt_layernorm(void *, const mtrt_tvm_ffi_any *args, int32_t num_args, mtrt_tvm_ffi_any *result) {
  const Args a{"mtrt_layernorm", args, num_args};
  if (num_args != 5)
    return fail("TypeError", "mtrt_layernorm expects (x, gamma, beta, y, eps), got %d arguments", num_args);
  const mtrt_dl_tensor *x = a.tensor(0, "x"), *g = x ? a.tensor(1, "gamma") : nullptr, *b = g ? a.tensor(2, "beta") : nullptr,
                       *y = b ? a.tensor(3, "y") : nullptr;
  if (!y)
    return -1;
  double eps = 0.0;
  if (!a.real(4, &eps))
    return fail("TypeError", "mtrt_layernorm: eps must be a number");
  if (x->ndim < 1)
    return fail("ValueError", "mtrt_layernorm: x must have at least one dimension");
  const int64_t d = x->shape[x->ndim - 1];
  const int32_t dt = dtype_of(x);
  if (dtype_of(g) != dt || dtype_of(b) != dt || dtype_of(y) != dt)
    return fail("TypeError", "mtrt_layernorm: x, gamma, beta and y must share one element type");
  if (numel(g) != d || numel(b) != d || numel(y) != numel(x))
    return fail("ValueError", "mtrt_layernorm: gamma and beta must have the last extent of x, y the shape of x");
  set_none(result);
  return forward(mtrt_hip_layernorm(stream_for(x), data_of(x), data_of(g), data_of(b), data_of(y), dt, d ? numel(x) / d : 0, d,
                                    float(eps)));
}

int __tvm_ffi_mtrt_softmax(void *, const mtrt_tvm_ffi_any *args, int32_t num_args, mtrt_tvm_ffi_any *result) {
  const Args a{"mtrt_softmax", args, num_args};
  if (num_args != 2)
    return fail("TypeError", "mtrt_softmax expects (x, y), got %d arguments", num_args);
  const mtrt_dl_tensor *x = a.tensor(0, "x"), *y = x ? a.tensor(1, "y") : nullptr;
  if (!y)
    return -1;
  if (x->ndim < 1 || dtype_of(x) != dtype_of(y) || numel(x) != numel(y))
    return fail("ValueError", "mtrt_softmax: y must have the shape and element type of x (at least one dimension)");
  const int64_t d = x->shape[x->ndim - 1];
  set_none(result);
  return forward(mtrt_hip_softmax(stream_for(x), data_of(x), data_of(y), dtype_of(x), d ? numel(x) / d : 0, d));
}

int __tvm_ffi_mtrt_gemm_w8a8(void *, const mtrt_tvm_ffi_any *args, int32_t num_args, mtrt_tvm_ffi_any *result) {
  const Args a{"mtrt_gemm_w8a8", args, num_args};
  if (num_args != 5)
    return fail("TypeError", "mtrt_gemm_w8a8 expects (a, w_nk, a_scale, w_scale, y), got %d arguments", num_args);
  const mtrt_dl_tensor *x = a.tensor(0, "a"), *w = x ? a.tensor(1, "w_nk") : nullptr, *xs = w ? a.tensor(2, "a_scale") : nullptr,
                       *ws = xs ? a.tensor(3, "w_scale") : nullptr, *y = ws ? a.tensor(4, "y") : nullptr;
  if (!y)
    return -1;
  if (x->ndim != 2 || w->ndim != 2 || y->ndim != 2 || dtype_of(x) != MTRT_I8 || dtype_of(w) != MTRT_I8 ||
      dtype_of(xs) != MTRT_F32 || dtype_of(ws) != MTRT_F32 || dtype_of(y) != MTRT_F16)
    return fail("TypeError", "mtrt_gemm_w8a8: a [M,K] int8, w_nk [N,K] int8, scales float32, y [M,N] float16");
  const int64_t M = x->shape[0], K = x->shape[1], N = w->shape[0];
  if (w->shape[1] != K || y->shape[0] != M || y->shape[1] != N || numel(xs) != M || numel(ws) != N)
    return fail("ValueError", "mtrt_gemm_w8a8: shapes do not agree (M=%lld K=%lld N=%lld)", (long long)M, (long long)K, (long long)N);
  set_none(result);
  return forward(mtrt_hip_gemm_w8a8(stream_for(x), data_of(x), data_of(w), static_cast<const float *>(data_of(xs)),
                                    static_cast<const float *>(data_of(ws)), data_of(y), M, K, N));
}

} // extern "C"
