#include "attn_common.h"
extern "C" int rswa_attn_bwd(const rswa_attn_params* p, void* stream) {
  return rswa::fail(RSWA_ERR_UNSUPPORTED, "attn_bwd: not built yet");
}
