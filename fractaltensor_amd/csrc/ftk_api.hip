// Library-wide entry points of include/ftk.h: version, error text, device info.
#include <string.h>

#include <mutex>

#include "ftk_common.h"

namespace ftk {

char* last_error_buffer() {
  static thread_local char buf[kErrLen] = {0};
  return buf;
}

int device_props(const DeviceProps** out) {
  constexpr int kMaxDev = 16;
  static DeviceProps cache[kMaxDev];
  static bool ready[kMaxDev] = {false};
  static std::mutex mu;
  int dev = 0;
  FTK_HIP(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDev) return fail(FTK_ERR_DEVICE, "device id %d out of range", dev);
  std::lock_guard<std::mutex> lock(mu);
  if (!ready[dev]) {
    hipDeviceProp_t p;
    FTK_HIP(hipGetDeviceProperties(&p, dev));
    DeviceProps d;
    d.cus = p.multiProcessorCount;
    d.lds_optin = (int)p.sharedMemPerBlockOptin;
    if (d.lds_optin <= 0) d.lds_optin = (int)p.sharedMemPerBlock;
    d.clock_khz = p.clockRate;
    d.wave = p.warpSize;
    strncpy(d.arch, p.gcnArchName, sizeof(d.arch) - 1);
    // gfx950 has 160 KB of LDS per compute unit, all of it addressable by one workgroup
    if (strncmp(d.arch, "gfx950", 6) == 0 && d.lds_optin < 163840) d.lds_optin = 163840;
    cache[dev] = d;
    ready[dev] = true;
  }
  *out = &cache[dev];
  return FTK_OK;
}

}  // namespace ftk

extern "C" {

int ftk_version(void) { return 100; }

const char* ftk_last_error(void) { return ftk::last_error_buffer(); }

int ftk_device_info_query(ftk_device_info* out) {
  if (!out) return ftk::fail(FTK_ERR_INVALID_ARGUMENT, "ftk_device_info_query: out is NULL");
  const ftk::DeviceProps* d = nullptr;
  int rc = ftk::device_props(&d);
  if (rc) return rc;
  out->compute_units = d->cus;
  out->lds_bytes_per_block = d->lds_optin;
  out->clock_khz = d->clock_khz;
  out->wavefront_size = d->wave;
  out->persistent_slots = d->cus;  // one 256-thread workgroup with all 512 registers per lane fills a CU
  memset(out->arch, 0, sizeof(out->arch));
  strncpy(out->arch, d->arch, sizeof(out->arch) - 1);
  return FTK_OK;
}

}  // extern "C"
