// The one entry point of the cluster layer that allocates nothing: mtrt_hip_amax_no_alloc.
//
// It is mtrt_hip_amax with the cross-workgroup reduction block (arrival tickets and running
// maxima, see kernels/amax.hip) taken from an array that lives in this library's own device
// image instead of from the pool that mtrt_hip_init allocates with hipMalloc.  Callers that
// must not allocate (code under stream capture, tight serving loops, harnesses that forbid
// hipMalloc) use it; the reference has no counterpart.
//
// Rules kept here:
//  * `scratch` below is a device array.  In host code its NAME is only a stand-in: the device
//    address is asked for once per device with hipGetSymbolAddress while that device is current
//    (no_alloc_setup, called from the per-device set-up that mtrt_hip_init runs) and only that
//    pointer is handed to kernels.  Every GPU has its own copy of the array at its own address.
//  * The entry point itself calls no hipMalloc / hipFree and builds no heap objects: the kernel
//    handles were resolved at set-up.
//  * All calls on one GPU share that GPU's array.  Each call first clears the block with the
//    built-in module's fill kernel on the caller's stream (a kernel, not a memset node, so the
//    pair can be captured into a graph; launched through the driver call, whose own return value
//    says whether THIS launch was accepted), then runs the reduction.  Two calls that overlap in time on one GPU (different
//    streams) race on the block; callers serialise them.
#include <hip/hip_runtime.h>

#include <atomic>

#include "runtime_internal.hpp"

// (1 + 32) lines of 128 bytes are used by the reduction tree; rounded up to 40 lines = 5 KiB per GPU.
// Plain file-scope `static __device__`: the compiler gives such an array a global device symbol because host
// code below names it; marked `used` or put into an unnamed namespace it would stay a local symbol of the
// device image, and the address look-up could not find it.
constexpr int kScratchWords = 40 * 32;
static __device__ __align__(256) uint32_t scratch[kScratchWords];

namespace {

constexpr int kMaxDevices = 64;
struct PerDevice {
  // device address of `scratch` on this device; written last by the set-up (release) and read first by the entry
  // point (acquire), so a thread that sees it also sees the handles below
  std::atomic<uint32_t *> ptr{nullptr};
  hipFunction_t amax[3] = {nullptr, nullptr, nullptr};   // indexed by MTRT_F32 / MTRT_F16 / MTRT_BF16
  hipFunction_t fill = nullptr;          // mtrt_fill of the built-in module
  int num_cus = 0;
};
PerDevice g_dev[kMaxDevices];

} // namespace

namespace mtrt_rt {

int32_t no_alloc_setup(DeviceState *st, int device) {
  if (device < 0 || device >= kMaxDevices)
    return MTRT_OK;   // the allocation-free entry point reports such a device itself
  void *p = nullptr;
  const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
  if (e != hipSuccess || !p)
    return set_error(MTRT_RUNTIME_ERROR, "hipGetSymbolAddress(scratch) on device %d: %s", device,
                     hipGetErrorString(e));
  PerDevice &d = g_dev[device];
  static const char *kNames[3] = {"mtrt_amax_f32", "mtrt_amax_f16", "mtrt_amax_bf16"};
  for (int i = 0; i < 3; ++i) {
    d.amax[i] = find_kernel(st, kNames[i]);
    if (!d.amax[i])
      return MTRT_NOT_FOUND;
  }
  d.fill = find_kernel(st, "mtrt_fill");
  if (!d.fill)
    return MTRT_NOT_FOUND;
  d.num_cus = num_compute_units(st);
  d.ptr.store(static_cast<uint32_t *>(p), std::memory_order_release);
  return MTRT_OK;
}

} // namespace mtrt_rt

extern "C" int32_t mtrt_hip_amax_no_alloc(mtrt_stream_t stream, const void *x, int32_t dtype, int64_t n, float qmax,
                                          float *amax_out, float *scale_out) {
  using namespace mtrt_rt;
  clear_error();
  if (dtype != MTRT_F32 && dtype != MTRT_F16 && dtype != MTRT_BF16)
    return set_error(MTRT_INVALID_ARGUMENT, "amax input dtype %d is not one of f32/f16/bf16", dtype);
  if (n < 0)
    return set_error(MTRT_INVALID_ARGUMENT, "negative element count %lld", (long long)n);
  if (n > MTRT_HIP_AMAX_NO_ALLOC_MAX_ELEMENTS)
    return set_error(MTRT_INVALID_ARGUMENT,
                     "%lld elements exceed the %lld that the allocation-free amax accepts; use mtrt_hip_amax",
                     (long long)n, (long long)MTRT_HIP_AMAX_NO_ALLOC_MAX_ELEMENTS);
  if (n > 0 && !x)
    return set_error(MTRT_INVALID_ARGUMENT, "null input");
  const uintptr_t elem = dtype == MTRT_F32 ? 4 : 2;
  if (reinterpret_cast<uintptr_t>(x) & (elem - 1))
    return set_error(MTRT_INVALID_ARGUMENT, "input is not aligned to its element size");
  int device = -1;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess)
    return set_error(MTRT_RUNTIME_ERROR, "no usable HIP device: %s", hipGetErrorString(e));
  uint32_t *block = device >= 0 && device < kMaxDevices ? g_dev[device].ptr.load(std::memory_order_acquire) : nullptr;
  if (!block)
    return set_error(MTRT_RUNTIME_ERROR,
                     "device %d is not set up: call mtrt_hip_init() on it first (set-up loads code and "
                     "allocates, this entry point does neither)", device);
  const PerDevice &d = g_dev[device];
  hipStream_t s = as_hip(stream);

  {
    uint8_t *p = reinterpret_cast<uint8_t *>(block);
    int64_t count = kScratchWords;
    uint32_t fill = 0;
    int32_t width = 4;
    void *fargs[] = {&p, &count, &fill, &width};
    e = hipModuleLaunchKernel(d.fill, 1, 1, 1, 256, 1, 1, 0, s, fargs, nullptr);
    if (e != hipSuccess)
      return set_error(MTRT_DRIVER_ERROR, "launching the clear kernel: %s", hipGetErrorString(e));
  }

  // launch shape of mtrt_hip_amax: at most two workgroups per compute unit, 4 x 128-bit loads per lane and trip
  const int per_vec = dtype == MTRT_F32 ? 4 : 8;
  const int64_t nvec = n / per_vec;
  int64_t grid = (nvec + 256 * 4 - 1) / (256 * 4);
  if (grid > int64_t(d.num_cus) * 2) grid = int64_t(d.num_cus) * 2;
  if (grid < 1) grid = 1;
  const void *x_arg = x;
  int64_t n_arg = n;
  float qmax_arg = qmax;
  void *args[] = {&x_arg, &n_arg, &qmax_arg, &amax_out, &scale_out, &block};
  e = hipModuleLaunchKernel(d.amax[dtype], uint32_t(grid), 1, 1, 256, 1, 1, 0, s, args, nullptr);
  if (e != hipSuccess) {
    return set_error(MTRT_DRIVER_ERROR, "launching the amax kernel grid %lld: %s", (long long)grid, hipGetErrorString(e));
  }
  return MTRT_OK;
}
