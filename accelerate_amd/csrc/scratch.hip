// The static device scratch behind acchip_execute_into (see scratch.hpp).
//
// `scratch` is a file-scope device array: every GPU the library runs on holds its own copy,
// at its own address, until the process ends.  In host code the array's name is only a
// stand-in for the symbol; the address a kernel can use comes from hipGetSymbolAddress,
// once per device, and host code uses nothing but that pointer afterwards.
#include "scratch.hpp"

#include <mutex>
#include <string>

#include "sx.hpp"

namespace acchip {

namespace {

constexpr size_t kTicketBytes = 256;          // the ticket counter has the first 256 bytes to itself
constexpr size_t kDescBytes = (size_t)1 << 20;  // 131072 descriptor words: e.g. 65536 tiles of Int64
constexpr int kMaxDevices = 64;

static __device__ __align__(256) unsigned char scratch[kTicketBytes + kDescBytes];

// clears descriptor words when the epoch tag wraps (a fill kernel, not a memset node: callers may
// be capturing the stream)
__global__ void acchip_scratch_clear(unsigned long long* p, size_t words) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < words; i += (size_t)gridDim.x * blockDim.x)
    p[i] = 0;
}

struct PerDevice {
  bool ready = false;
  unsigned char* ptr = nullptr;  // device address of `scratch` on this device
  ScanState scan;
};
std::mutex g_mu;
PerDevice g_dev[kMaxDevices];

}  // namespace

size_t staticScratchDescBytes() { return kDescBytes; }

void staticScratchSetup(int device) {
  if (device < 0 || device >= kMaxDevices) throw Error("static scratch: device number out of range");
  std::lock_guard<std::mutex> g(g_mu);
  PerDevice& d = g_dev[device];
  if (d.ready) return;
  hipError_t e = hipSetDevice(device);
  if (e != hipSuccess) throw Error(std::string("static scratch: hipSetDevice: ") + hipGetErrorString(e));
  void* p = nullptr;
  e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
  if (e != hipSuccess || !p) {
    (void)hipGetLastError();
    throw Error(std::string("static scratch: hipGetSymbolAddress: ") + hipGetErrorString(e));
  }
  d.ptr = static_cast<unsigned char*>(p);
  // The array starts as zeros (static storage): a zero word carries no launch's tag, and the
  // ticket counter starts at 0, which is what ticketBase says.
  d.scan.ticket = reinterpret_cast<unsigned long long*>(d.ptr);
  d.scan.desc = d.ptr + kTicketBytes;
  d.scan.descBytes = kDescBytes;
  d.scan.ticketBase = 0;
  d.scan.epoch = 0;
  d.ready = true;
}

ScanState& staticScanState(int device, hipStream_t stream, size_t descBytes) {
  if (device < 0 || device >= kMaxDevices) throw Error("static scratch: device number out of range");
  std::lock_guard<std::mutex> g(g_mu);
  PerDevice& d = g_dev[device];
  if (!d.ready) throw Error("static scratch: this device was never set up");
  if (descBytes > kDescBytes)
    throw Error("this scan needs " + std::to_string(descBytes) + " bytes of tile descriptors; the static scratch of " +
                "acchip_execute_into holds " + std::to_string(kDescBytes) + " (use acchip_execute)");
  if (++d.scan.epoch >= (1u << 30)) {
    // tags would repeat: wipe the descriptors left by earlier launches and start over
    (void)hipSetDevice(device);
    hipLaunchKernelGGL(acchip_scratch_clear, dim3(256), dim3(256), 0, stream,
                       reinterpret_cast<unsigned long long*>(d.scan.desc), kDescBytes / 8);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) throw Error(std::string("static scratch: clear kernel: ") + hipGetErrorString(e));
    d.scan.epoch = 1;
  }
  return d.scan;
}

}  // namespace acchip
