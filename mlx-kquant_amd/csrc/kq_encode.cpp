// Host-side wire encoders (kq_quantize).  Placeholder until the first encoder lands.
#include "kq_common.h"

extern "C" int kq_quantize(const float*, const float*, uint8_t*, int64_t, int64_t, int codec) {
  return kq_set_error(KQ_ERR_UNSUPPORTED, "quantize: no encoder for codec id %d in this build", codec);
}
