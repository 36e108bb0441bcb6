// frnn_launch_static: the launch entry point that allocates nothing (see include/frnn_rt.h).
//
// The hidden buffers of a launch (state checkpoints, saved row sums, any zero-filled accumulator) are
// placed in one file-scope device array instead of memory the caller allocated (which buffers is the caller's
// choice: the Python host puts state / d-state checkpoints and the saved sums there).  Every GPU has its own
// copy of the array at its own address; that address is asked for once per device and is what kernels,
// fills and copies are given.  The array's name itself is only meaningful to hipGetSymbolAddress.
#include <hip/hip_runtime.h>

#include <dlfcn.h>
#include <stdint.h>
#include <string.h>

#include <mutex>

#include "frnn_rt.h"
#include "frnn_internal.h"

namespace {

static __device__ __align__(256) unsigned char scratch[FRNN_STATIC_SCRATCH_BYTES];

constexpr int kMaxDevices = 64;
constexpr size_t kMaxArgBytes = 4096;     // (the hardware's limit for an argument segment)
constexpr size_t kMaxSlots = 64;

std::mutex g_mu;
unsigned char* g_base[kMaxDevices];       // per device: where that GPU's copy of `scratch` lives
bool g_checked = false;                   // the one-runtime check below has passed

// 16 bytes per thread and trip; the grid is sized by the host and every thread leaves after its share
__global__ void __launch_bounds__(256) frnn_fill_zero(uint4* p, size_t n16) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += stride) p[i] = make_uint4(0u, 0u, 0u, 0u);
}

int scratch_of_current_device(unsigned char** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return frnn_detail_fail(FRNN_ERR_HIP, "hipGetDevice failed: %s (%d)", hipGetErrorString(e), (int)e);
  if (dev < 0 || dev >= kMaxDevices) return frnn_detail_fail(FRNN_ERR_ARG, "frnn_launch_static: device %d is beyond the %d supported", dev, kMaxDevices);
  std::lock_guard<std::mutex> lock(g_mu);
  if (!g_checked) {
    // This file is linked against the HIP runtime; the rest of the library resolves it at run time from what the
    // process already holds.  A kernel handle made by one copy of the runtime must not be launched through another:
    // refuse when the two bindings live in different shared objects.
    void* theirs = frnn_detail_runtime_launch_symbol();
    void* mine = (void*)&hipModuleLaunchKernel;
    Dl_info a, b;
    if (theirs && theirs != mine && dladdr(theirs, &a) && dladdr(mine, &b) && a.dli_fname && b.dli_fname && strcmp(a.dli_fname, b.dli_fname) != 0)
      return frnn_detail_fail(FRNN_ERR_NO_HIP, "frnn_launch_static: two HIP runtimes in one process (%s and %s); load the one the "
                              "application uses before this library", a.dli_fname, b.dli_fname);
    g_checked = true;
  }
  if (!g_base[dev]) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p)
      return frnn_detail_fail(FRNN_ERR_HIP, "hipGetSymbolAddress(scratch) failed on device %d: %s (%d)", dev, hipGetErrorString(e), (int)e);
    g_base[dev] = (unsigned char*)p;
  }
  *out = g_base[dev];
  return FRNN_OK;
}

}  // namespace

extern "C" int frnn_launch_static(frnn_kernel_t k, const uint32_t grid[3], const uint32_t block[3], uint32_t lds_bytes,
                                  void* stream, const void* args, size_t arg_bytes, const frnn_scratch_slot* slots,
                                  size_t nslots) {
  if (!k || !grid || !block || !args || (!slots && nslots)) return frnn_detail_fail(FRNN_ERR_ARG, "frnn_launch_static: null argument");
  for (int i = 0; i < 3; i++)
    if (grid[i] == 0 || block[i] == 0) return frnn_detail_fail(FRNN_ERR_ARG, "frnn_launch_static: empty grid or block");
  if ((uint64_t)block[0] * block[1] * block[2] > 1024) return frnn_detail_fail(FRNN_ERR_ARG, "frnn_launch_static: block larger than 1024 threads");
  if (grid[1] > 65535 || grid[2] > 65535) return frnn_detail_fail(FRNN_ERR_ARG, "frnn_launch_static: grid y/z larger than 65535");
  if (arg_bytes == 0 || arg_bytes % 8 != 0 || arg_bytes > kMaxArgBytes)
    return frnn_detail_fail(FRNN_ERR_ARG, "frnn_launch_static: argument block of %zu bytes (must be a multiple of 8, at most %zu)", arg_bytes, kMaxArgBytes);
  if (k->kernarg && arg_bytes != k->kernarg)
    return frnn_detail_fail(FRNN_ERR_ARG, "frnn_launch_static: argument block of %zu bytes, the kernel's code object declares %zu", arg_bytes, k->kernarg);
  if (nslots > kMaxSlots) return frnn_detail_fail(FRNN_ERR_ARG, "frnn_launch_static: %zu scratch regions, at most %zu", nslots, kMaxSlots);
  for (size_t i = 0; i < nslots; i++) {
    const frnn_scratch_slot& s = slots[i];
    if (s.arg_offset % 8 != 0 || s.arg_offset > arg_bytes - 8)
      return frnn_detail_fail(FRNN_ERR_ARG, "frnn_launch_static: region %zu: pointer field at byte %llu is outside the %zu-byte argument block or misaligned",
                              i, (unsigned long long)s.arg_offset, arg_bytes);
    if (s.scratch_offset % 256 != 0)
      return frnn_detail_fail(FRNN_ERR_ARG, "frnn_launch_static: region %zu: offset %llu is not a multiple of 256", i, (unsigned long long)s.scratch_offset);
    if (s.bytes == 0 || s.bytes > FRNN_STATIC_SCRATCH_BYTES || s.scratch_offset > FRNN_STATIC_SCRATCH_BYTES - s.bytes)
      return frnn_detail_fail(FRNN_ERR_ARG, "frnn_launch_static: region %zu: bytes %llu..%llu do not fit the static scratch buffer of %llu bytes; use frnn_launch with caller-allocated buffers for this size",
                              i, (unsigned long long)s.scratch_offset, (unsigned long long)(s.scratch_offset + s.bytes),
                              (unsigned long long)FRNN_STATIC_SCRATCH_BYTES);
    for (size_t j = 0; j < i; j++) {
      const frnn_scratch_slot& o = slots[j];
      if (s.arg_offset == o.arg_offset)
        return frnn_detail_fail(FRNN_ERR_ARG, "frnn_launch_static: regions %zu and %zu fill the same pointer field", j, i);
      if (s.scratch_offset < o.scratch_offset + o.bytes && o.scratch_offset < s.scratch_offset + s.bytes)
        return frnn_detail_fail(FRNN_ERR_ARG, "frnn_launch_static: regions %zu and %zu overlap", j, i);
    }
  }
  unsigned char* base = nullptr;
  int rc = scratch_of_current_device(&base);
  if (rc != FRNN_OK) return rc;

  alignas(8) unsigned char buf[kMaxArgBytes];
  memcpy(buf, args, arg_bytes);
  hipStream_t st = (hipStream_t)stream;
  for (size_t i = 0; i < nslots; i++) {
    const frnn_scratch_slot& s = slots[i];
    unsigned char* p = base + s.scratch_offset;
    memcpy(buf + s.arg_offset, &p, sizeof p);
    if (s.clear) {
      // whole 16-byte words: the region starts 256-aligned, and rounding its end up stays inside the array
      const size_t n16 = (size_t)((s.bytes + 15) / 16);
      const unsigned blocks = (unsigned)(n16 / 256 + 1 < 2048 ? n16 / 256 + 1 : 2048);
      (void)hipGetLastError();         // (an error an earlier, unrelated call left behind is not this launch's)
      hipLaunchKernelGGL(frnn_fill_zero, dim3(blocks), dim3(256), 0, st, (uint4*)p, n16);
      hipError_t e = hipGetLastError();
      if (e != hipSuccess) return frnn_detail_fail(FRNN_ERR_HIP, "frnn_launch_static: clearing region %zu failed: %s (%d)", i, hipGetErrorString(e), (int)e);
    }
  }
  size_t sz = arg_bytes;
  void* extra[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, buf, HIP_LAUNCH_PARAM_BUFFER_SIZE, &sz, HIP_LAUNCH_PARAM_END};
  hipError_t e = hipModuleLaunchKernel((hipFunction_t)k->fn, grid[0], grid[1], grid[2], block[0], block[1], block[2], lds_bytes, st,
                                       nullptr, extra);
  if (e != hipSuccess) return frnn_detail_fail(FRNN_ERR_HIP, "hipModuleLaunchKernel failed: %s (%d)", hipGetErrorString(e), (int)e);
  return FRNN_OK;
}
