// Placeholder entry points; replaced by the real kernels.
#include "common.h"
using namespace mi355;
extern "C" size_t mi355_fp8_blockwise_mm_workspace_bytes(int64_t, int64_t, int64_t) { return 0; }
extern "C" int mi355_fp8_blockwise_mm(const void*, const void*, const float*, const float*, void*, int, int64_t, int64_t,
                                      int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, void*,
                                      size_t, void*) {
  set_error("mi355_fp8_blockwise_mm: not built yet");
  return MI355_ERR_UNSUPPORTED;
}
extern "C" size_t mi355_int8_scaled_mm_workspace_bytes(int64_t, int64_t, int64_t) { return 0; }
extern "C" int mi355_int8_scaled_mm(const void*, const void*, const float*, const float*, const void*, void*, int,
                                    int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, void*, size_t, void*) {
  set_error("mi355_int8_scaled_mm: not built yet");
  return MI355_ERR_UNSUPPORTED;
}
extern "C" int mi355_per_token_quant_int8(const void*, int, void*, float*, int64_t, int64_t, void*) {
  set_error("mi355_per_token_quant_int8: not built yet");
  return MI355_ERR_UNSUPPORTED;
}
