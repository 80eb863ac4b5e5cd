// aitamd_gemm_rcr_noalloc: aitamd_gemm_rcr_ws with its scratch memory taken from an array in the library's device
// image, for callers that cannot allocate.  A translation unit of its own: a model library links the static archive
// and pulls only the objects it refers to, and compiled models pass their own workspace, so they must not carry a
// copy of the array (16 MiB of device memory per loaded library and GPU).
#include <mutex>

#include "../../include/aitemplate_amd_kernels.h"
#include "errors.hpp"

#include <hip/hip_runtime.h>

using aitamd::fail;

namespace {

// Scratch memory of aitamd_gemm_rcr_noalloc: 16 MiB per GPU, part of the library's device image (zero when the
// image is loaded; every launch leaves the counters at its start zero again).  In host code `scratch` is only a
// handle for hipGetSymbolAddress: the device address is looked up once per device and used from then on.
constexpr int64_t kScratchBytes = 16ll << 20;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

constexpr int kMaxScratchDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxScratchDevices];

// Device address of `scratch` on the current device (null with a message on failure).
void* scratch_of_current_device() {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= kMaxScratchDevices) {
    fail("aitamd_gemm_rcr_noalloc: cannot identify the current device: %s", hipGetErrorString(e));
    return nullptr;
  }
  std::lock_guard<std::mutex> lk(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || ptr == nullptr) {
      fail("aitamd_gemm_rcr_noalloc: hipGetSymbolAddress failed on device %d: %s", dev, hipGetErrorString(e));
      return nullptr;
    }
    g_scratch_ptr[dev] = ptr;
  }
  return g_scratch_ptr[dev];
}

}  // namespace

extern "C" {

int aitamd_gemm_rcr_noalloc(int epilogue, int dtype, int algo, const void* a, const void* b, const void* bias,
                            const void* d0, const void* d1, void* c, int64_t M, int64_t N, int64_t K, int64_t lda,
                            int64_t ldb, int64_t ldc, int64_t ldd, void* stream) {
  if (algo >= 0) {
    const int64_t need = aitamd_gemm_workspace_bytes(epilogue, dtype, algo, 1, M, N, K);
    if (need > kScratchBytes)
      return fail("aitamd_gemm_rcr_noalloc: this instance needs %lld bytes of scratch memory for M=%lld N=%lld K=%lld; "
                  "the built-in buffer holds %lld (use aitamd_gemm_rcr_ws with a buffer of the caller's)",
                  (long long)need, (long long)M, (long long)N, (long long)K, (long long)kScratchBytes);
  }
  void* ws = scratch_of_current_device();
  if (ws == nullptr) return 1;
  return aitamd_gemm_rcr_ws(epilogue, dtype, algo, a, b, bias, d0, d1, c, M, N, K, lda, ldb, ldc, ldd, ws, kScratchBytes,
                            stream);
}

// Also resolves the array's address on the current device when there is one, so that a caller who asks for the
// capacity at set-up has the look-up (and its lock) behind it before the first launch: a first launch made under
// stream capture then does nothing but launch.  Without a device the capacity is still answered.
int64_t aitamd_gemm_noalloc_scratch_bytes(void) {
  int dev = 0;
  if (hipGetDevice(&dev) == hipSuccess)
    (void)scratch_of_current_device();
  else
    (void)hipGetLastError();
  return kScratchBytes;
}

}  // extern "C"
