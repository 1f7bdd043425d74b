// Per-device state of the cluster layer and the embedded kernel module.
//
// The gfx950 code object built from csrc/kernels/*.hip is linked into this
// library as read-only data (the role PTX text plays inside a reference
// executable's data segment,
// mlir-tensorrt/compiler/lib/Passes/2_Host/HostToExecutor/CUDAToExecutor/CUDAToExecutor.cpp:858-905)
// and loaded once per device, lazily, the way the reference initialises its module
// and function globals on first use (CUDAToExecutor.cpp:797-905).
#include "runtime_internal.hpp"

#include <cstdio>
#include <cstring>
#include <map>
#include <mutex>
#include <unordered_map>
#include <vector>

#ifndef MTRT_HSACO_PATH
#error "MTRT_HSACO_PATH must name the code object to embed"
#endif

__asm__(".section .rodata\n"
        ".balign 4096\n"
        ".global mtrt_hip_hsaco_begin\n"
        "mtrt_hip_hsaco_begin:\n"
        ".incbin \"" MTRT_HSACO_PATH "\"\n"
        ".global mtrt_hip_hsaco_end\n"
        "mtrt_hip_hsaco_end:\n"
        ".byte 0\n"
        ".previous\n");
extern "C" const char mtrt_hip_hsaco_begin[];
extern "C" const char mtrt_hip_hsaco_end[];

namespace mtrt_rt {

namespace {
thread_local char tl_error[1024] = {0};
thread_local char tl_kernel[128] = {0};
} // namespace

int32_t set_error(int32_t code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  std::vsnprintf(tl_error, sizeof(tl_error), fmt, ap);
  va_end(ap);
  return code;
}
void clear_error() { tl_error[0] = '\0'; }
const char *last_error() { return tl_error; }

int32_t load_code_object(const char *data, size_t len, hipModule_t *out, std::string *err) {
  static const char kBundle[] = "__CLANG_OFFLOAD_BUNDLE__";
  const bool elf = len >= 4 && std::memcmp(data, "\x7f" "ELF", 4) == 0;
  const bool bundle = len >= sizeof(kBundle) - 1 && std::memcmp(data, kBundle, sizeof(kBundle) - 1) == 0;
  if (!data || (!elf && !bundle)) {
    *err = "module data is not an AMDGPU code object (expected ELF or a clang offload bundle; "
           "PTX is not accepted)";
    return MTRT_INVALID_ARGUMENT;
  }
  // The loader reads sizes from the image's own headers; hand it a private copy so
  // a caller's buffer that is not NUL-padded or is freed early cannot matter.
  std::vector<char> copy(data, data + len);
  copy.push_back('\0');
  hipModule_t module = nullptr;
  const hipError_t e = hipModuleLoadData(&module, copy.data());
  if (e != hipSuccess) {
    *err = std::string("hipModuleLoadData: ") + hipGetErrorString(e);
    return MTRT_DRIVER_ERROR;
  }
  *out = module;
  return MTRT_OK;
}

struct DeviceState {
  int device = -1;
  int num_cus = 0;
  hipModule_t module = nullptr;
  std::mutex mu;
  std::unordered_map<std::string, hipFunction_t> funcs;
  // One block per stream for single-launch grid reductions, zero when a stream first uses it: 33 lines of
  // 128 bytes for the arrival tree (root + 32 first-level groups, see amax.hip), which the kernels return to
  // zero, and 18 for the tagged slots and counters of dynq.hip, which never need clearing; rounded up to 64.
  static constexpr int kSlots = 256;
  static constexpr int kSlotWords = 64 * 32;
  uint32_t *slots = nullptr;
  // The stream -> block mapping has a mutex of its own (slot_mu), which reduction_slot holds across the launch of
  // a fresh block's clear; that launch may take `mu` to resolve the fill kernel.  Order: slot_mu, then mu.
  std::mutex slot_mu;
  std::map<hipStream_t, int> slot_of;
  std::vector<int> free_slots;   // slots of destroyed streams, handed out again before new ones
  std::vector<bool> pinned = std::vector<bool>(kSlots, false);   // handed out under stream capture: never recycled
  int next_slot = 0;
};

namespace {
std::mutex g_mu;
std::map<int, DeviceState *> g_states;
} // namespace

DeviceState *device_state() {
  int device = -1;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) {
    set_error(MTRT_RUNTIME_ERROR, "no usable HIP device: %s", hipGetErrorString(e));
    return nullptr;
  }
  std::lock_guard<std::mutex> lock(g_mu);
  auto it = g_states.find(device);
  if (it != g_states.end())
    return it->second;

  hipDeviceProp_t prop;
  e = hipGetDeviceProperties(&prop, device);
  if (e != hipSuccess) {
    set_error(MTRT_RUNTIME_ERROR, "hipGetDeviceProperties: %s", hipGetErrorString(e));
    return nullptr;
  }
  if (std::strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
    set_error(MTRT_RUNTIME_ERROR, "device %d is %s; this library carries gfx950 code only", device,
              prop.gcnArchName);
    return nullptr;
  }
  auto *st = new DeviceState();
  st->device = device;
  st->num_cus = prop.multiProcessorCount;
  std::string err;
  const size_t len = size_t(mtrt_hip_hsaco_end - mtrt_hip_hsaco_begin);
  if (load_code_object(mtrt_hip_hsaco_begin, len, &st->module, &err) != MTRT_OK) {
    set_error(MTRT_DRIVER_ERROR, "loading the built-in kernel module failed: %s", err.c_str());
    delete st;
    return nullptr;
  }
  const size_t bytes = size_t(DeviceState::kSlots) * DeviceState::kSlotWords * sizeof(uint32_t);
  e = hipMalloc(reinterpret_cast<void **>(&st->slots), bytes);
  if (e == hipSuccess)
    e = hipMemset(st->slots, 0, bytes);
  if (e != hipSuccess) {
    set_error(MTRT_RUNTIME_ERROR, "allocating reduction slots: %s", hipGetErrorString(e));
    (void)hipModuleUnload(st->module);
    delete st;
    return nullptr;
  }
  if (no_alloc_setup(st, device) != MTRT_OK) {
    (void)hipFree(st->slots);
    (void)hipModuleUnload(st->module);
    delete st;
    return nullptr;
  }
  g_states[device] = st;
  return st;
}

hipModule_t builtin_module(DeviceState *st) { return st->module; }
int num_compute_units(DeviceState *st) { return st->num_cus; }

hipFunction_t find_kernel(DeviceState *st, const std::string &name) {
  std::lock_guard<std::mutex> lock(st->mu);
  auto it = st->funcs.find(name);
  if (it != st->funcs.end())
    return it->second;
  hipFunction_t f = nullptr;
  const hipError_t e = hipModuleGetFunction(&f, st->module, name.c_str());
  if (e != hipSuccess) {
    set_error(MTRT_NOT_FOUND, "kernel '%s' is not in the built-in module: %s", name.c_str(),
              hipGetErrorString(e));
    return nullptr;
  }
  st->funcs.emplace(name, f);
  return f;
}

namespace {
// Stream-ordered clear of one reduction block (a fill kernel, so that it may sit inside a captured graph).
int32_t clear_slot(DeviceState *st, uint32_t *block, hipStream_t stream) {
  uint8_t *p = reinterpret_cast<uint8_t *>(block);
  int64_t count = DeviceState::kSlotWords;
  uint32_t fill = 0;
  int32_t width = 4;
  void *args[] = {&p, &count, &fill, &width};
  return launch(st, KernelName("mtrt_fill"), 1, 256, stream, args);
}
} // namespace

uint32_t *reduction_slot(DeviceState *st, hipStream_t stream) {
  // A kernel recorded into a graph keeps the block's address in its arguments for as long as the graph is replayed,
  // which can be long after the capture stream is gone: a block handed out while its stream is capturing stays out
  // of the free list for good (256 blocks per device; a capture stream is normally bound once).
  hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
  const bool capturing = hipStreamIsCapturing(stream, &capture) == hipSuccess && capture != hipStreamCaptureStatusNone;
  std::lock_guard<std::mutex> lock(st->slot_mu);
  auto it = st->slot_of.find(stream);
  if (it != st->slot_of.end()) {
    if (capturing)
      st->pinned[size_t(it->second)] = true;
    return st->slots + size_t(it->second) * DeviceState::kSlotWords;
  }
  int slot;
  if (!st->free_slots.empty()) {
    slot = st->free_slots.back();
    st->free_slots.pop_back();
  } else if (st->next_slot < DeviceState::kSlots) {
    slot = st->next_slot++;
  } else {
    set_error(MTRT_RUNTIME_ERROR, "more than %d live streams use grid reductions", DeviceState::kSlots);
    return nullptr;
  }
  uint32_t *block = st->slots + size_t(slot) * DeviceState::kSlotWords;
  // A block newly bound to a stream is cleared in stream order before its first use: whatever an earlier
  // owner (a destroyed stream, or a launch that never finished) left in it cannot reach this stream's results.
  // The clear is queued before the mapping becomes visible (the lock is held), so no other thread's reduction on
  // this stream can be queued in front of it.
  if (clear_slot(st, block, stream) != MTRT_OK) {
    st->free_slots.push_back(slot);
    return nullptr;
  }
  st->slot_of.emplace(stream, slot);
  if (capturing)
    st->pinned[size_t(slot)] = true;
  return block;
}

int32_t reset_reduction_slot(DeviceState *st, hipStream_t stream) {
  int slot = -1;
  {
    std::lock_guard<std::mutex> lock(st->slot_mu);
    auto it = st->slot_of.find(stream);
    if (it != st->slot_of.end())
      slot = it->second;
  }
  if (slot < 0)
    return MTRT_OK;   // nothing bound: the next reduction on this stream clears its block itself
  return clear_slot(st, st->slots + size_t(slot) * DeviceState::kSlotWords, stream);
}

void forget_stream(hipStream_t stream) {
  // Called by every stream-destroy entry point before the stream goes away.  The stream's block returns
  // to the free list only after the stream has drained, so a kernel still running on the old stream can
  // never share the block with its next owner; HIP reusing the handle value for a new stream is harmless
  // for the same reason (the mapping is gone by then).
  std::vector<DeviceState *> states;
  {
    std::lock_guard<std::mutex> lock(g_mu);
    for (auto &kv : g_states)
      states.push_back(kv.second);
  }
  for (DeviceState *st : states) {
    bool bound;
    {
      std::lock_guard<std::mutex> lock(st->slot_mu);
      bound = st->slot_of.count(stream) != 0;
    }
    if (!bound)
      continue;
    (void)hipStreamSynchronize(stream);
    std::lock_guard<std::mutex> lock(st->slot_mu);
    auto it = st->slot_of.find(stream);
    if (it != st->slot_of.end()) {
      if (!st->pinned[size_t(it->second)])             // a captured graph may still name a pinned block
        st->free_slots.push_back(it->second);
      st->slot_of.erase(it);
    }
  }
}

namespace {
// Per-thread cache of resolved kernels: open addressing on the name's hash, entries never removed (the set of
// kernel names is fixed).  A hit costs one hash of a short string and one compare.
struct CachedKernel {
  DeviceState *st = nullptr;
  hipFunction_t fn = nullptr;
  uint64_t hash = 0;
  char name[72] = {0};
};
constexpr uint32_t kCacheSlots = 512;                // a thread uses a few dozen kernels; a full table falls back to the locked look-up
thread_local CachedKernel tl_cache[kCacheSlots];
thread_local const char *tl_kernel_ptr = "";

uint64_t name_hash(const KernelName &k, DeviceState *st) {
  uint64_t h = 1469598103934665603ull ^ reinterpret_cast<uintptr_t>(st);
  for (uint32_t i = 0; i < k.len; ++i)
    h = (h ^ uint8_t(k.text[i])) * 1099511628211ull;
  return h | 1;                                      // 0 marks an empty slot
}
} // namespace

int32_t launch(DeviceState *st, const KernelName &kernel, uint32_t grid, uint32_t block, hipStream_t stream, void **args) {
  const uint64_t h = name_hash(kernel, st);
  CachedKernel *hit = nullptr;
  for (uint32_t probe = 0; probe < kCacheSlots; ++probe) {
    CachedKernel &c = tl_cache[(h + probe) & (kCacheSlots - 1)];
    if (c.hash == h && c.st == st && std::strcmp(c.name, kernel.text) == 0) {
      hit = &c;
      break;
    }
    if (c.hash == 0) {
      hipFunction_t f = find_kernel(st, kernel.text);
      if (!f)
        return MTRT_NOT_FOUND;
      c.st = st;
      c.fn = f;
      std::memcpy(c.name, kernel.text, kernel.len + 1);
      c.hash = h;
      hit = &c;
      break;
    }
  }
  hipFunction_t f = hit ? hit->fn : find_kernel(st, kernel.text);   // table full: the locked look-up
  if (!f)
    return MTRT_NOT_FOUND;
  const hipError_t e =
      hipModuleLaunchKernel(f, grid, 1, 1, block, 1, 1, /*sharedMemBytes=*/0, stream, args, nullptr);
  if (e != hipSuccess) {
    (void)hipGetLastError(); // reported through the status; do not leave it for the caller's next HIP call
    return set_error(MTRT_DRIVER_ERROR, "launching '%s' grid %u block %u: %s", kernel.text, grid, block,
                     hipGetErrorString(e));
  }
  if (hit) {
    tl_kernel_ptr = hit->name;
  } else {
    std::snprintf(tl_kernel, sizeof(tl_kernel), "%s", kernel.text);
    tl_kernel_ptr = tl_kernel;
  }
  return MTRT_OK;
}

const char *last_kernel_name() { return tl_kernel_ptr; }

} // namespace mtrt_rt

extern "C" {

const char *mtrt_hip_last_error(void) { return mtrt_rt::last_error(); }
const char *mtrt_hip_last_kernel(void) { return mtrt_rt::last_kernel_name(); }

int32_t mtrt_hip_init(void) {
  mtrt_rt::clear_error();
  return mtrt_rt::device_state() ? MTRT_OK : MTRT_RUNTIME_ERROR;
}

int32_t mtrt_hip_reset_reductions(mtrt_stream_t stream) {
  mtrt_rt::clear_error();
  mtrt_rt::DeviceState *st = mtrt_rt::device_state();
  if (!st)
    return MTRT_RUNTIME_ERROR;
  return mtrt_rt::reset_reduction_slot(st, mtrt_rt::as_hip(stream));
}

mtrt_module_t mtrt_hip_builtin_module(void) {
  mtrt_rt::DeviceState *st = mtrt_rt::device_state();
  return st ? reinterpret_cast<mtrt_module_t>(mtrt_rt::builtin_module(st)) : nullptr;
}

const char *mtrt_hip_builtin_code_object(size_t *size) {
  if (size)
    *size = size_t(mtrt_hip_hsaco_end - mtrt_hip_hsaco_begin);
  return mtrt_hip_hsaco_begin;
}

} // extern "C"
