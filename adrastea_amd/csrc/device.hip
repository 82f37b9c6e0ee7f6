// Properties of the current device, queried once per device and never changed afterwards
// (the only state the library keeps): architecture check, compute-unit and die counts that the
// launchers size their grids and tile walks by.
#include <atomic>
#include <string.h>

#include "adr_common.hpp"

namespace adr {

namespace {

constexpr int MAX_DEVICES = 64;
constexpr DeviceInfo GFX950_DEFAULT = {ADR_OK, 256, 8};

struct Slot {
  std::atomic<int> ready{0};
  DeviceInfo info;
};
Slot slots[MAX_DEVICES];

DeviceInfo query(int dev) {
  DeviceInfo d = GFX950_DEFAULT;
  hipDeviceProp_t prop;
  const hipError_t e = hipGetDeviceProperties(&prop, dev);
  if (e != hipSuccess) {
    d.status = (int)e;
    return d;
  }
  // "gfx950:sramecc+:xnack-": the target name up to the first colon decides
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0 ||
      (prop.gcnArchName[6] != 0 && prop.gcnArchName[6] != ':')) {
    d.status = ADR_EUNSUPPORTED_DEVICE;
    return d;
  }
  if (prop.multiProcessorCount > 0) d.cus = prop.multiProcessorCount;
  int xcc = 0;
  if (hipDeviceGetAttribute(&xcc, hipDeviceAttributeNumberOfXccs, dev) == hipSuccess && xcc > 0)
    d.xcds = xcc;
  return d;
}

}  // namespace

DeviceInfo device_info() {
  int dev = -1;
  const hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0) {
    (void)hipGetLastError();  // the failed query must not surface in a later launch check
    DeviceInfo d = GFX950_DEFAULT;
    d.status = e != hipSuccess ? (int)e : (int)hipErrorNoDevice;
    return d;
  }
  if (dev >= MAX_DEVICES) return query(dev);
  Slot& s = slots[dev];
  if (s.ready.load(std::memory_order_acquire) == 2) return s.info;
  const DeviceInfo d = query(dev);
  // a failed query (a positive hipError_t) may be transient: reported, not remembered
  if (d.status > 0) {
    (void)hipGetLastError();
    return d;
  }
  int expect = 0;
  if (s.ready.compare_exchange_strong(expect, 1, std::memory_order_acq_rel)) {
    s.info = d;
    s.ready.store(2, std::memory_order_release);
  }
  return d;  // (a thread that lost the race returns its own, identical, copy)
}

namespace {
std::atomic<int> knobs[KNOB_COUNT];
}
int knob(int id) { return id >= 0 && id < KNOB_COUNT ? knobs[id].load(std::memory_order_relaxed) : 0; }
int set_knob(int id, int value) {
  if (id < 0 || id >= KNOB_COUNT) return ADR_EINVAL_ENUM;
  knobs[id].store(value, std::memory_order_relaxed);
  return ADR_OK;
}

DeviceInfo device_info_for_plan() {
  // the plan queries answer without a device too (a build machine): then for an MI355X
  DeviceInfo d = device_info();
  if (d.status != ADR_OK) d = GFX950_DEFAULT;
  return d;
}

}  // namespace adr
