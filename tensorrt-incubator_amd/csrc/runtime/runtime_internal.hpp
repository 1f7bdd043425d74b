// Internal helpers shared by the launch-ABI layer and the cluster layer.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <string>
#include <vector>

#include "mtrt_hip.h"

namespace mtrt_rt {

inline hipStream_t as_hip(mtrt_stream_t s) { return reinterpret_cast<hipStream_t>(s); }

[[noreturn]] void fatal(const char *file, int line, const char *msg);
bool read_file(const std::string &path, std::vector<char> &out);
// Reads a program artifact by name: absolute names as they are, relative ones under $MTRT_ARTIFACTS_DIR first and
// then under the working directory.  MTRT_NOT_FOUND (message lists what was tried) / MTRT_IO_ERROR via set_error.
int32_t read_artifact(const char *filename, std::vector<char> &out);

// Thread-local error text for the status-returning entry points.
int32_t set_error(int32_t code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
void clear_error();
const char *last_error();
const char *last_kernel_name();

// Validates that `data` looks like an AMDGPU code object (ELF or clang offload
// bundle) and loads it on the current device.
int32_t load_code_object(const char *data, size_t len, hipModule_t *out, std::string *err);

// Per-device state of the cluster layer: the built-in module, a function cache and
// the pool of zeroed reduction blocks handed out per stream.
struct DeviceState;
DeviceState *device_state();                 // nullptr + set_error on failure
hipModule_t builtin_module(DeviceState *);
int num_compute_units(DeviceState *);
hipFunction_t find_kernel(DeviceState *, const std::string &name);   // nullptr + set_error
uint32_t *reduction_slot(DeviceState *, hipStream_t stream);         // nullptr + set_error
int32_t reset_reduction_slot(DeviceState *, hipStream_t stream);     // stream-ordered clear of the stream's block
void forget_stream(hipStream_t stream);                              // before a stream is destroyed

// Set-up half of the allocation-free entry point (no_alloc.hip): looks up, with `device` current, the
// device address of that file's scratch array and the kernel handles it launches.
int32_t no_alloc_setup(DeviceState *, int device);

// A kernel name put together on the stack (no heap, no locale): KernelName("mtrt_q_") + kind + "_" + x.
struct KernelName {
  char text[72];
  uint32_t len = 0;
  KernelName(const char *s) { text[0] = '\0'; *this + s; }
  KernelName &operator+(const char *s) {
    while (*s && len + 1 < sizeof(text))
      text[len++] = *s++;
    text[len] = '\0';
    return *this;
  }
  KernelName &operator+(int v) {                       // small non-negative numbers (vector counts)
    char digits[12];
    int n = 0;
    do {
      digits[n++] = char('0' + v % 10);
      v /= 10;
    } while (v > 0 && n < 11);
    while (n > 0 && len + 1 < sizeof(text))
      text[len++] = digits[--n];
    text[len] = '\0';
    return *this;
  }
};

// Launch through the same driver call as mtrt_cuda_launch_kernel, returning a status.  The name is resolved
// through a per-thread table first (no lock, no allocation); only the first use of a kernel on a thread goes to
// the device state's table under its mutex.
int32_t launch(DeviceState *, const KernelName &kernel, uint32_t grid, uint32_t block,
               hipStream_t stream, void **args);

} // namespace mtrt_rt
