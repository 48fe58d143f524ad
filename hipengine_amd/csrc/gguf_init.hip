// Library set-up: hipengine_gfx950_init() does, once per device, everything a launch would otherwise
// have to do on first use through a call that is not a stream operation - raising dynamic-LDS limits,
// looking up the address of library-held scratch - so that every entry point can be captured into a HIP
// graph from its very first call.  Launch paths call ensure_init() and so stay correct without it.

#include <hip/hip_runtime.h>

#include <atomic>
#include <mutex>

#include "gguf_init.hpp"

#include "../../include/hipengine_gfx950.h"

namespace {

constexpr int kMaxDevices = 64;
std::atomic<bool> device_ready[kMaxDevices];
std::mutex init_mutex;

}  // namespace

extern "C" int hipengine_gfx950_abi_version(void) { return 2; }

extern "C" int hipengine_gfx950_init(void) {
  int device = -1;
  const hipError_t err = hipGetDevice(&device);
  if (err != hipSuccess) return static_cast<int>(err);
  if (device < 0 || device >= kMaxDevices) return static_cast<int>(hipErrorInvalidDevice);
  if (device_ready[device].load(std::memory_order_acquire)) return static_cast<int>(hipSuccess);
  std::lock_guard<std::mutex> lock(init_mutex);
  if (device_ready[device].load(std::memory_order_relaxed)) return static_cast<int>(hipSuccess);
  int rc = hipengine_gfx950::gemv_raise_lds_limits();
  if (rc != static_cast<int>(hipSuccess)) return rc;
  rc = hipengine_gfx950::argmax_noalloc_setup(device);
  if (rc != static_cast<int>(hipSuccess)) return rc;
  rc = hipengine_gfx950::prefill_pack_setup(device);
  if (rc != static_cast<int>(hipSuccess)) return rc;
  int (*const loads[])() = {hipengine_gfx950::quantize_load, hipengine_gfx950::mmq_load, hipengine_gfx950::moe_load,
                            hipengine_gfx950::embedding_load};
  for (auto load : loads) {
    rc = load();
    if (rc != static_cast<int>(hipSuccess)) return rc;
  }
  device_ready[device].store(true, std::memory_order_release);
  return static_cast<int>(hipSuccess);
}

namespace hipengine_gfx950 {

int ensure_init() {
  int device = -1;
  const hipError_t err = hipGetDevice(&device);
  if (err != hipSuccess) return static_cast<int>(err);
  if (device >= 0 && device < kMaxDevices && device_ready[device].load(std::memory_order_acquire)) {
    return static_cast<int>(hipSuccess);
  }
  return hipengine_gfx950_init();
}

}  // namespace hipengine_gfx950
