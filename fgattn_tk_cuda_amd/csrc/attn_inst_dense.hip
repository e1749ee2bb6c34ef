// Dense attention / row-statistics instantiations (q-block 128).
#include "attn_fwd.h"
#include "dispatch.h"

namespace spattn {

hipError_t run_attn_dense(const AttnParams& p, int D, bool has_v, bool stats, hipStream_t stream) {
  if (D == 128) {
    if (has_v && !stats) return launch_attn_fwd<128, 128, KV_DENSE, true, false>(p, stream);
    if (has_v && stats) return launch_attn_fwd<128, 128, KV_DENSE, true, true>(p, stream);
    if (!has_v && stats) return launch_attn_fwd<128, 128, KV_DENSE, false, true>(p, stream);
  } else if (D == 64) {
    if (has_v && !stats) return launch_attn_fwd<64, 128, KV_DENSE, true, false>(p, stream);
    if (has_v && stats) return launch_attn_fwd<64, 128, KV_DENSE, true, true>(p, stream);
    if (!has_v && stats) return launch_attn_fwd<64, 128, KV_DENSE, false, true>(p, stream);
  }
  return hipErrorInvalidValue;
}

hipError_t prepare_attn_dense() {
  hipError_t e = prepare_attn_fwd<128, 128, KV_DENSE, true, false>();
  if (e == hipSuccess) e = prepare_attn_fwd<128, 128, KV_DENSE, true, true>();
  if (e == hipSuccess) e = prepare_attn_fwd<128, 128, KV_DENSE, false, true>();
  if (e == hipSuccess) e = prepare_attn_fwd<64, 128, KV_DENSE, true, false>();
  if (e == hipSuccess) e = prepare_attn_fwd<64, 128, KV_DENSE, true, true>();
  if (e == hipSuccess) e = prepare_attn_fwd<64, 128, KV_DENSE, false, true>();
  return e;
}

}  // namespace spattn
