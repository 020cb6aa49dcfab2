// dsx_q8_0_kernels.hpp -- Q8_0 expert products (int8 MFMA).  Filled in below.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/dsx_moe.h"

namespace dsx {

int q8_0_unsupported(const char *what);

inline void q8_0_raise_lds_limits() {}

inline int q8_0_gate_up_decode(hipStream_t, float *, const uint8_t *, const uint8_t *,
                               const uint8_t *, const float *, const int32_t *, const uint8_t *,
                               const uint8_t *, float, uint64_t, uint64_t, uint32_t, float,
                               uint32_t, uint32_t) {
    return q8_0_unsupported("moe_gate_up_batch");
}
inline int q8_0_down_decode(hipStream_t, float *, const uint8_t *, const uint8_t *, const int32_t *,
                            const uint8_t *, uint64_t, uint32_t, uint32_t, uint32_t, uint32_t) {
    return q8_0_unsupported("moe_down_batched");
}
inline int q8_0_gate_up_by_expert(hipStream_t, float *, const uint8_t *, const uint8_t *,
                                  const uint8_t *, const float *, const int32_t *, const int32_t *,
                                  const int32_t *, const int32_t *, const int32_t *, uint32_t,
                                  uint64_t, uint64_t, uint32_t, uint32_t, float, uint32_t,
                                  uint32_t) {
    return q8_0_unsupported("moe_gate_up_chunked_rows");
}
inline int q8_0_down_by_expert(hipStream_t, float *, const uint8_t *, const uint8_t *,
                               const int32_t *, const int32_t *, const int32_t *, const int32_t *,
                               const int32_t *, uint32_t, uint64_t, uint32_t, uint32_t, uint32_t,
                               uint32_t, uint32_t) {
    return q8_0_unsupported("moe_down_by_expert");
}

}  // namespace dsx
