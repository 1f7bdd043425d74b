// Device-independent half of the `namespace mtrt` flavour: the thread-local message setter, aligned host
// memory and the loading of constant blobs (a compiled program's weights) from the artifacts directory into a
// named memory space.  Behaviour follows the reference's StandaloneCPP core
// (mlir-tensorrt/executor/lib/Runtime/StandaloneCPP/MTRTRuntimeCore.cpp:76-93, 168-189, 246-358 and the two
// constant hooks of MTRTRuntimeCuda.cpp:319-372) with HIP allocations where that one uses CUDA's.
#include "mtrt_hip_standalone.h"
#include "runtime_internal.hpp"

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

using namespace mtrt_rt;

namespace {

// memory spaces as the compiler numbers them (plan dialect), MTRTRuntimeCore.cpp:59-63
constexpr int32_t kSpaceUnknown = 0, kSpaceHost = 1, kSpaceHostPinned = 2, kSpaceDevice = 3, kSpaceUnified = 4;

std::vector<std::string> candidates_for(const std::string &name) {
  std::vector<std::string> out;
  if (name.empty())
    return out;
  if (name[0] == '/') {
    out.push_back(name);
    return out;
  }
  if (const char *dir = std::getenv("MTRT_ARTIFACTS_DIR")) {
    std::string base(dir);
    if (!base.empty())
      out.push_back(base.back() == '/' ? base + name : base + "/" + name);
  }
  out.push_back(name);   // relative to the working directory
  return out;
}

} // namespace

namespace mtrt_rt {

int32_t read_artifact(const char *filename, std::vector<char> &bytes) {
  const std::vector<std::string> tried = candidates_for(filename);
  for (const std::string &path : tried) {
    std::FILE *f = std::fopen(path.c_str(), "rb");
    if (!f)
      continue;
    bool ok = std::fseek(f, 0, SEEK_END) == 0;
    const long size = ok ? std::ftell(f) : -1;
    ok = ok && size >= 0 && std::fseek(f, 0, SEEK_SET) == 0;
    if (ok) {
      bytes.resize(size_t(size));
      ok = size == 0 || std::fread(bytes.data(), 1, size_t(size), f) == size_t(size);
    }
    std::fclose(f);
    if (!ok)
      return set_error(MTRT_IO_ERROR, "Error reading file '%s'", path.c_str());
    return MTRT_OK;
  }
  std::string msg = std::string("Error opening file '") + filename + "'.\nTried:\n";
  for (const std::string &path : tried)
    msg += "  - " + path + "\n";
  msg += "Hint: set MTRT_ARTIFACTS_DIR to the directory containing manifest.json\n";
  return set_error(MTRT_NOT_FOUND, "%s", msg.c_str());
}

} // namespace mtrt_rt

namespace mtrt {

namespace detail {
void set_last_error_message_v(const char *fmt, va_list ap) {
  char buf[1024];
  std::vsnprintf(buf, sizeof(buf), fmt, ap);
  set_error(MTRT_INTERNAL_ERROR, "%s", buf);
}
} // namespace detail

Status host_aligned_alloc(int64_t sizeBytes, int32_t alignment, void **outPtr) {
  if (!outPtr)
    return set_error(MTRT_INVALID_ARGUMENT, "outPtr must not be null");
  *outPtr = nullptr;
  if (sizeBytes < 0)
    return set_error(MTRT_INVALID_ARGUMENT, "sizeBytes must be >= 0");
  if (alignment <= 0 || (uint32_t(alignment) & (uint32_t(alignment) - 1)) != 0)
    return set_error(MTRT_INVALID_ARGUMENT, "alignment must be a power-of-two > 0 (got %d)", alignment);
  if (sizeBytes == 0)
    return ok();
  const size_t a = size_t(alignment);
  const size_t rounded = (size_t(sizeBytes) + a - 1) / a * a;
  void *p = std::aligned_alloc(a, rounded);
  if (!p)
    return set_error(MTRT_INTERNAL_ERROR, "aligned_alloc failed (size=%zu align=%d)", rounded, alignment);
  *outPtr = p;
  return ok();
}

void host_free(void *ptr) { std::free(ptr); }

Status constant_load_from_file(const char *filename, int32_t align, int32_t space, void **outPtr) {
  if (!outPtr)
    return set_error(MTRT_INVALID_ARGUMENT, "outPtr must not be null");
  *outPtr = nullptr;
  if (!filename || filename[0] == '\0')
    return set_error(MTRT_INVALID_ARGUMENT, "filename must not be empty");
  std::vector<char> bytes;
  const int32_t st = read_artifact(filename, bytes);
  if (st != MTRT_OK)
    return st;
  if (space == kSpaceUnknown || space == kSpaceHost) {
    void *buf = nullptr;
    const Status a = host_aligned_alloc(int64_t(bytes.size()), align > 1 ? align : 1, &buf);
    if (a != ok())
      return a;
    if (!bytes.empty())
      std::memcpy(buf, bytes.data(), bytes.size());
    *outPtr = buf;
    return ok();
  }
  if (bytes.empty())
    return ok();
  void *dst = nullptr;
  hipError_t e = hipSuccess;
  switch (space) {
  case kSpaceHostPinned:
    e = hipHostMalloc(&dst, bytes.size(), hipHostMallocDefault);
    if (e == hipSuccess)
      std::memcpy(dst, bytes.data(), bytes.size());
    break;
  case kSpaceUnified:
    e = hipMallocManaged(&dst, bytes.size(), hipMemAttachGlobal);
    if (e == hipSuccess)
      std::memcpy(dst, bytes.data(), bytes.size());
    break;
  case kSpaceDevice:
    e = hipMalloc(&dst, bytes.size());
    if (e == hipSuccess) {
      e = hipMemcpy(dst, bytes.data(), bytes.size(), hipMemcpyHostToDevice);
      if (e != hipSuccess)
        (void)hipFree(dst);
    }
    break;
  default:
    return set_error(MTRT_INVALID_ARGUMENT, "unsupported memory space for constant load: %d", space);
  }
  if (e != hipSuccess) {
    (void)hipGetLastError();
    return set_error(MTRT_RUNTIME_ERROR, "HIP runtime error: %s (loading constant '%s' into space %d)",
                     hipGetErrorString(e), filename, space);
  }
  *outPtr = dst;
  return ok();
}

void constant_destroy(void *data, int32_t space) {
  if (!data)
    return;
  hipError_t e = hipSuccess;
  switch (space) {
  case kSpaceUnknown:
  case kSpaceHost:
    host_free(data);
    return;
  case kSpaceHostPinned:
    e = hipHostFree(data);
    break;
  case kSpaceUnified:
  case kSpaceDevice:
    e = hipFree(data);
    break;
  default:
    set_error(MTRT_INVALID_ARGUMENT, "unsupported memory space for constant free: %d", space);
    return;
  }
  if (e != hipSuccess) {
    (void)hipGetLastError();
    set_error(MTRT_RUNTIME_ERROR, "HIP runtime error: %s (freeing a constant of space %d)", hipGetErrorString(e), space);
  }
}

} // namespace mtrt
