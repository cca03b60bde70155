// extern "C" boundary of libspnc_hip: translates exceptions of the C++ layer into return codes
// plus a thread-local message, the way the reference's pybind11 module turns its C++ exceptions
// into Python RuntimeErrors (python-interface/src/python-interface.cpp:19-64).
#include <hip/hip_runtime.h>

#include <cstring>
#include <map>
#include <string>

#include "../../include/spnc_hip.h"
#include "kernel.h"

#include "interp_kernel.h"
static_assert(SPNC_HIP_STATIC_SCRATCH_BYTES == spnc_hip::INTERP_SCRATCH_BYTES, "the header states the size of the scratch array");

struct spnc_hip_kernel {
  std::unique_ptr<spnc_hip::Kernel> impl;
};

namespace {
thread_local std::string g_lastError;

template <typename Fn>
int guarded(Fn&& fn) {
  try {
    g_lastError.clear();
    fn();
    return 0;
  } catch (const std::exception& e) {
    g_lastError = e.what();
    return 1;
  } catch (...) {
    g_lastError = "unknown error";
    return 1;
  }
}
}  // namespace

extern "C" {

int spnc_hip_available(void) {
  int count = 0;
  if (hipGetDeviceCount(&count) != hipSuccess || count <= 0) {
    (void)hipGetLastError();
    return 0;
  }
  for (int d = 0; d < count; ++d) {
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, d) == hipSuccess && std::strncmp(prop.gcnArchName, "gfx950", 6) == 0) return 1;
  }
  return 0;
}

int spnc_hip_compile(const char* query_path, const char* const* keys, const char* const* vals, size_t n_opts, spnc_hip_kernel** out) {
  return guarded([&] {
    if (!query_path || !out) throw std::runtime_error("null argument");
    std::map<std::string, std::string> opts;
    for (size_t i = 0; i < n_opts; ++i) {
      if (!keys || !vals || !keys[i] || !vals[i]) throw std::runtime_error("null option string");
      opts[keys[i]] = vals[i];
    }
    auto k = spnc_hip::Kernel::compile(query_path, opts);
    *out = new spnc_hip_kernel{std::move(k)};
  });
}

int spnc_hip_load(const char* kernel_file, spnc_hip_kernel** out) {
  return guarded([&] {
    if (!kernel_file || !out) throw std::runtime_error("null argument");
    auto k = spnc_hip::Kernel::load(kernel_file);
    *out = new spnc_hip_kernel{std::move(k)};
  });
}

int spnc_hip_kernel_info(const spnc_hip_kernel* k, spnc_hip_info* info) {
  return guarded([&] {
    if (!k || !info) throw std::runtime_error("null argument");
    k->impl->fillInfo(info);
  });
}

int spnc_hip_execute(spnc_hip_kernel* k, size_t n, const void* in, void* out) {
  return guarded([&] {
    if (!k) throw std::runtime_error("null kernel");
    k->impl->execute(n, in, out);
  });
}

int spnc_hip_execute_device(spnc_hip_kernel* k, size_t n, const void* d_in, void* d_out, void* stream) {
  return guarded([&] {
    if (!k) throw std::runtime_error("null kernel");
    k->impl->executeDevice(n, d_in, d_out, static_cast<hipStream_t>(stream));
  });
}

int spnc_hip_execute_device_static(spnc_hip_kernel* k, size_t n, const void* d_in, void* d_out, void* stream) {
  return guarded([&] {
    if (!k) throw std::runtime_error("null kernel");
    k->impl->executeDeviceStatic(n, d_in, d_out, static_cast<hipStream_t>(stream));
  });
}

int spnc_hip_kernel_source(const spnc_hip_kernel* k, const char** text, size_t* len) {
  return guarded([&] {
    if (!k || !text || !len) throw std::runtime_error("null argument");
    *text = k->impl->text().c_str();
    *len = k->impl->text().size();
  });
}

void spnc_hip_destroy(spnc_hip_kernel* k) { delete k; }

const char* spnc_hip_last_error(void) { return g_lastError.c_str(); }

}  // extern "C"
