// int4 decode attention kernels (placeholder launcher until the kernel lands).
#include "kvx_device.h"

int kvx_decode_int4_launch(const kvx_storage *, kvx_kv_layer, uint32_t, const void *, void *,
                           const uint64_t *const *, const kvx_verify_params *, uint32_t, uint32_t,
                           void *, uint64_t, hipStream_t) {
  return 1;  // declined: the caller runs the generic tile
}
