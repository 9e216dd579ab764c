// Scratch memory that exists without any allocation call: one file-scope
// device array per GPU, for the entry point that serves callers who cannot
// allocate device memory (code under graph capture, serving loops, harnesses
// that forbid it). Each GPU the library runs on holds its own copy of the
// array, at its own address, until the process ends.
//
// The array's name is only a host-side handle: host code must never pass it to
// a kernel or a memory routine. Its device address is looked up once per
// device with hipGetSymbolAddress, with that device current, and only that
// address is used from then on.
#include <hip/hip_runtime.h>

#include <mutex>

#include "static_scratch.h"

namespace ruyamd {
namespace {

static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
std::mutex g_mutex;
void* g_address[kMaxDevices] = {};

__global__ void FillZeroKernel(uint32_t* p, uint32_t words) {
  for (uint32_t i = blockIdx.x * blockDim.x + threadIdx.x; i < words; i += gridDim.x * blockDim.x) p[i] = 0;
}

}  // namespace

hipError_t StaticScratchOfCurrentDevice(void** address) {
  *address = nullptr;
  int device = -1;
  hipError_t status = hipGetDevice(&device);
  if (status != hipSuccess) return status;
  if (device < 0 || device >= kMaxDevices) return hipErrorInvalidDevice;
  std::lock_guard<std::mutex> lock(g_mutex);
  if (!g_address[device]) {
    void* ptr = nullptr;
    status = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (status != hipSuccess) return status;
    if (!ptr) return hipErrorInvalidSymbol;
    g_address[device] = ptr;
  }
  *address = g_address[device];
  return hipSuccess;
}

hipError_t LaunchFillZero(hipStream_t stream, uint32_t* p, uint32_t words) {
  if (words == 0) return hipSuccess;
  const unsigned blocks = (words + 255) / 256 < 64 ? (words + 255) / 256 : 64;
  hipLaunchKernelGGL(FillZeroKernel, dim3(blocks), dim3(256), 0, stream, p, words);
  return hipGetLastError();
}

}  // namespace ruyamd
