// Tuned MFMA kernels (placeholder until the first tuned kernel lands).
#include "kq_common.h"

int kq_launch_qmm_tuned(const void*, const uint8_t*, void*, int, int, int, int, int, hipStream_t) {
  return KQ_ERR_UNSUPPORTED;
}
