// Scan scratch that lives in a static device array instead of an allocation, for the one
// entry point that must not allocate (acchip_execute_into).  Implemented in scratch.hip,
// the only file of the library compiled by hipcc: it holds the array and resolves its
// per-device address.
#pragma once
#include <hip/hip_runtime.h>

#include <cstddef>

namespace acchip {

// device scratch of the single-pass scans: tile descriptors, ticket counter, and the host's
// view of both (value the counter will have when the next launch starts, tag of the last launch)
struct ScanState {
  void* desc = nullptr;
  size_t descBytes = 0;
  unsigned long long* ticket = nullptr;
  unsigned long long ticketBase = 0;
  unsigned epoch = 0;
};

// bytes of descriptors the static array holds per device
size_t staticScratchDescBytes();

// Resolve the static array's address on `device` (made current by the call); once per
// device, at context creation.  Throws Error when HIP refuses.
void staticScratchSetup(int device);

// The device's static scan state, advanced to a fresh epoch for one launch on `stream`.
// Throws Error when descBytes exceeds staticScratchDescBytes() or the device was never set
// up.  Allocates nothing.  All contexts of a device share the array: launches that use it
// must not overlap.
ScanState& staticScanState(int device, hipStream_t stream, size_t descBytes);

}  // namespace acchip
