// The library's static scratch: device memory no call has to allocate.
//
// ogm_matmul_dev_static (ogm_api.cpp) serves callers that cannot call hipMalloc -- code under HIP
// graph capture, tight serving loops, harnesses that forbid allocation.  Its kernels take their
// scratch buffer (the int8 activations, their scales and side sums) as pointer arguments like every
// other launch; the memory behind those pointers is this file-scope array instead of a buffer the
// context grew on demand.  Every GPU the library runs on holds its own copy of the array, at its own
// address, until the process ends.  In host code the array's name is only a handle for
// hipGetSymbolAddress: the address that kernels, copies and memsets may use is the one that call
// returns for the device that is current, resolved once per device in ogm_init.
#include <hip/hip_runtime.h>

#include "ogm_kernels.h"

namespace {

// q: 1 byte per element; d: one f32 per 32; sums: one i32 per 16; bsum: one i16 per 32; bs16: one
// u16 per 16.  Every piece is a multiple of 256 bytes, so each starts 256-byte aligned.
constexpr size_t kQ = OGM_STATIC_MAX_ELEMS;
constexpr size_t kD = OGM_STATIC_MAX_ELEMS / 32 * 4;
constexpr size_t kSums = OGM_STATIC_MAX_ELEMS / 16 * 4;
constexpr size_t kBsum = OGM_STATIC_MAX_ELEMS / 32 * 2;
constexpr size_t kBs16 = OGM_STATIC_MAX_ELEMS / 16 * 2;
constexpr size_t kTotal = kQ + kD + kSums + kBsum + kBs16;
static_assert(kQ % 256 == 0 && kD % 256 == 0 && kSums % 256 == 0 && kBsum % 256 == 0, "pieces stay aligned");

static __device__ __align__(256) uint8_t scratch[kTotal];

}  // namespace

hipError_t ogm_static_scratch_address(uint8_t **ptr) {
  void *p = nullptr;
  const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
  if (e != hipSuccess) return e;
  *ptr = (uint8_t *)p;
  return hipSuccess;
}

OgmActDev ogm_static_act_view(uint8_t *base) {
  OgmActDev a;
  a.q = (int8_t *)base;
  a.d = (float *)(base + kQ);
  a.sums = (int32_t *)(base + kQ + kD);
  a.bsum = (int16_t *)(base + kQ + kD + kSums);
  a.bs16 = (uint16_t *)(base + kQ + kD + kSums + kBsum);
  return a;
}
