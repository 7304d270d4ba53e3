// Paged decode attention, MLA latent-KV variant, for gfx950 (placeholder translation unit).
#include "common.cuh"
#include "launch.h"

namespace xllm_mi355 {

int paged_decode_mla(const void*, const void*, const void*, void*, float*, const PageAddressing&,
                     int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, float, void*,
                     size_t, int, hipStream_t) {
  return XLLM_MI355_ESHAPE;
}

}  // namespace xllm_mi355
