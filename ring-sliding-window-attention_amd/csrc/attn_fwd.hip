#include "rswa_common.h"
extern "C" int rswa_attn_fwd(const rswa_attn_params* p, void* stream) {
  return rswa::fail(RSWA_ERR_UNSUPPORTED, "attn_fwd: not built yet");
}
