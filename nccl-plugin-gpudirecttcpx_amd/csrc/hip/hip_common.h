// Shared by the translation units of the HIP layer: error plumbing and per-device helpers.
#ifndef TCPXU_HIP_COMMON_H_
#define TCPXU_HIP_COMMON_H_

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "tcpx_unpack_hip.h"

namespace tcpxu {

constexpr int kMaxDevices = 64;

void set_error(const char* fmt, ...) __attribute__((format(printf, 1, 2)));
int use_device(int device);            // hipSetDevice + cache properties
int device_compute_units(int device);  // valid after use_device
void batch_geometry(int device, uint64_t n_descs, uint32_t* descs_per_wg, uint64_t* n_batches, uint32_t* grid);

}  // namespace tcpxu

// A failing HIP call returns the "unhandled device error" code, as CUCHECK does in the reference
// (src/misc/cuda_checks.h:38-49); nothing in this layer calls exit().
#define TCPXU_HIP(call)                                                                              \
  do {                                                                                               \
    hipError_t e_ = (call);                                                                          \
    if (e_ != hipSuccess) {                                                                          \
      ::tcpxu::set_error("%s:%d %s -> %s", __FILE__, __LINE__, #call, hipGetErrorString(e_));        \
      return TCPXU_DEVICE_ERROR;                                                                     \
    }                                                                                                \
  } while (0)

#define TCPXU_TRY(call)                   \
  do {                                    \
    int rc_ = (call);                     \
    if (rc_ != TCPXU_SUCCESS) return rc_; \
  } while (0)

#endif  // TCPXU_HIP_COMMON_H_
