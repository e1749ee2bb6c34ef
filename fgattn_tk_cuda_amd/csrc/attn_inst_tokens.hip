// Token-list (gathered) sparse attention instantiations.
#include "attn_fwd.h"
#include "dispatch.h"

namespace spattn {

hipError_t run_attn_tokens(const AttnParams& p, int D, int qblk, hipStream_t stream) {
  if (D == 128 && qblk == 128) return launch_attn_fwd<128, 128, KV_TOKENS, true, false>(p, stream);
  if (D == 128 && qblk == 64) return launch_attn_fwd<128, 64, KV_TOKENS, true, false>(p, stream);
  if (D == 64 && qblk == 128) return launch_attn_fwd<64, 128, KV_TOKENS, true, false>(p, stream);
  if (D == 64 && qblk == 64) return launch_attn_fwd<64, 64, KV_TOKENS, true, false>(p, stream);
  return hipErrorInvalidValue;
}

hipError_t prepare_attn_tokens() {
  hipError_t e = prepare_attn_fwd<128, 128, KV_TOKENS, true, false>();
  if (e == hipSuccess) e = prepare_attn_fwd<128, 64, KV_TOKENS, true, false>();
  if (e == hipSuccess) e = prepare_attn_fwd<64, 128, KV_TOKENS, true, false>();
  if (e == hipSuccess) e = prepare_attn_fwd<64, 64, KV_TOKENS, true, false>();
  return e;
}

}  // namespace spattn
