// fbfft_conv_fprop_static: the forward convolution layer for callers that cannot
// allocate device memory (code under HIP graph capture, tight serving loops,
// harnesses that forbid hipMalloc).  It runs the kernels of fbfft_conv_fprop; the
// workspace those kernels hand their spectra through is a fixed array in this
// library's device image instead of a buffer the caller brings.
//
// Every GPU holds its own copy of the array at its own address for as long as the
// process lives.  The array's name is only a host-side handle: the address the
// kernels receive is looked up once per device with hipGetSymbolAddress and kept.
// All calls on one GPU share that GPU's array, so calls that overlap in time on
// one GPU (different streams, or host threads on different streams) race; calls
// on one stream are ordered.  Nothing in the array has to survive between calls
// and nothing has to start at zero: the forward-transform kernels write every
// element the contraction reads, padding rows included.
//
// The look-up happens in the first call on a device, whatever its operands - a call
// with an empty batch does it and launches nothing - and may make the runtime load
// this library's device image.  Callers that capture into a graph or must not
// touch the allocator in their loop make that first call beforehand, outside
// capture; later calls only enqueue kernels.
#include "common.h"

#include <atomic>
#include <mutex>

namespace fbfft_amd {
namespace {

static __device__ __align__(256) unsigned char scratch[FBFFT_STATIC_SCRATCH_BYTES];

constexpr int kMaxDevices = 64;
std::atomic<void*> scratchOnDevice[kMaxDevices];
std::mutex setupLock;

// device address of `scratch` on the current device; nullptr on failure
void* scratchAddress() {
  int device = -1;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= kMaxDevices) return nullptr;
  void* p = scratchOnDevice[device].load(std::memory_order_acquire);
  if (p) return p;
  std::lock_guard<std::mutex> hold(setupLock);
  p = scratchOnDevice[device].load(std::memory_order_relaxed);
  if (p) return p;
  void* found = nullptr;
  if (hipGetSymbolAddress(&found, HIP_SYMBOL(scratch)) != hipSuccess || !found) {
    (void)hipGetLastError();
    return nullptr;
  }
  scratchOnDevice[device].store(found, std::memory_order_release);
  return found;
}

}  // namespace
}  // namespace fbfft_amd

using namespace fbfft_amd;

extern "C" int fbfft_conv_fprop_static(const fbfft_tensor* input, const fbfft_tensor* weight,
                                       const fbfft_tensor* output, int fftSize,
                                       fbfft_stream_t stream) {
  if (!input || !weight || !output || input->dim != 4 || weight->dim != 4 || output->dim != 4)
    return FBFFT_UNSUPPORTED_DIMENSION;
  const size_t need = fbfft_conv_workspace_image(0, input->size[0], input->size[1], weight->size[0],
                                                 input->size[2], input->size[3], weight->size[2],
                                                 weight->size[3], fftSize);
  // need == 0: empty or unsupported shapes; fbfft_conv_fprop sorts those out and
  // never touches the workspace
  void* ws = scratchAddress();  // before any other outcome: the first call is the set-up call
  if (!ws) return FBFFT_HIP_ERROR;
  if (need > (size_t)FBFFT_STATIC_SCRATCH_BYTES) return FBFFT_UNSUPPORTED_SIZE;
  return fbfft_conv_fprop(input, weight, output, fftSize, ws, FBFFT_STATIC_SCRATCH_BYTES, stream);
}
