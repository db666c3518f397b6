#include "moa_common.h"
using namespace moa;
extern "C" int moa_prefill_fwd(const void* q, const void* k, const void* v, void* o,
                               const int64_t* q_strides, const int64_t* k_strides,
                               const int64_t* v_strides, const int64_t* o_strides, int B, int Hq,
                               int Hkv, int N, int D, const int64_t* sink_blocks,
                               const int64_t* local_blocks, float sm_scale, int dtype, void* stream) {
  return fail(MOA_ERR_UNSUPPORTED, "moa_prefill_fwd: not built yet");
}
