// MFMA form of attn_mixq_prefill for bf16 models (see mix_attn.hip for the math).
#include "mix_common.h"

namespace rfqmix {

bool launch_attn_mixq_prefill_mfma(const float*, const void*, const void*, const int32_t*, int,
                                   const int32_t*, const int32_t*, const int32_t*, const int32_t*,
                                   const int32_t*, int, void*, int64_t, const float*, const float*,
                                   int, int, int, int, int, int, hipStream_t) {
  return false;
}

}  // namespace rfqmix
