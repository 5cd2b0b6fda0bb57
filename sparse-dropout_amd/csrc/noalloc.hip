// sd_gemm_dsd_noalloc: the mask form of the DSD product for callers that can neither allocate device memory
// nor hand over a workspace (code under graph capture, serving loops, harnesses that forbid hipMalloc).  The
// kept-block list that sd_gemm_dsd builds into the caller's workspace is built into a fixed array in device
// memory instead; each GPU the library runs on holds its own copy of that array until the process ends.
#include <mutex>

#include "common.h"

namespace {

// room for the CSR list of a 64-granular block grid: row_ptr (padded to 16 bytes) + one int32 per block
constexpr int64_t kScratchBytes = SD_NOALLOC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

constexpr int kMaxDevices = 64;
std::mutex scratch_mutex;
void* scratch_ptr[kMaxDevices] = {};  // device address of `scratch` on each device, looked up at first use

// The array's name is only a host-side handle; the address kernels can use comes from the runtime, once per
// device with that device current.
int scratch_address(void** out) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return sd::fail(SD_ERR_RUNTIME, "hipGetDevice: %s", hipGetErrorString(e));
  if (dev < 0 || dev >= kMaxDevices) return sd::fail(SD_ERR_RUNTIME, "device index %d out of range", dev);
  std::lock_guard<std::mutex> lock(scratch_mutex);
  if (scratch_ptr[dev] == nullptr) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || p == nullptr)
      return sd::fail(SD_ERR_RUNTIME, "hipGetSymbolAddress(scratch): %s", hipGetErrorString(e));
    scratch_ptr[dev] = p;
  }
  *out = scratch_ptr[dev];
  return SD_OK;
}

}  // namespace

extern "C" {

int64_t sd_noalloc_scratch_bytes(void) { return kScratchBytes; }

int sd_gemm_dsd_noalloc(const void* A, int64_t asr, int64_t asc, const void* B, int64_t bsr, int64_t bsc, void* C,
                        int64_t csr, int64_t csc, const uint8_t* mask, int64_t msr, int64_t msc, int64_t M,
                        int64_t N, int64_t K, int64_t bs, float scale, int dtype, void* stream) {
  SD_REQUIRE(M >= 0 && N >= 0 && K >= 0 && bs > 0, "gemm_dsd_noalloc: negative dimension or block size");
  // the list the mask form would build: at 64 granularity when the block size is a larger multiple of 64, or 32
  const int64_t g = bs % 32 == 0 ? 64 : bs;
  const int64_t mb = sd::ceil_div(M, g), kb = sd::ceil_div(K, g);
  SD_REQUIRE(mb < (1 << 24) && kb < (1 << 24), "gemm_dsd_noalloc: block grid %lld x %lld too large", (long long)mb,
             (long long)kb);
  const int64_t need = sd_workspace_bytes(mb, kb);
  const int64_t need16 = (need + 15) / 16 * 16;
  SD_REQUIRE(need16 <= kScratchBytes,
             "gemm_dsd_noalloc: the kept-block list of a %lld x %lld operand in blocks of %lld needs %lld bytes, "
             "the built-in scratch holds %lld; use sd_gemm_dsd with a workspace",
             (long long)M, (long long)K, (long long)bs, (long long)need16, (long long)kScratchBytes);
  void* ws = nullptr;
  if (int rc = scratch_address(&ws)) return rc;
  // exactly the list's bytes: nothing is left over for split-reduction partials, so none are made
  return sd_gemm_dsd(A, asr, asc, B, bsr, bsc, C, csr, csc, mask, msr, msc, M, N, K, bs, scale, dtype, ws,
                     need16, stream);
}

}  // extern "C"
