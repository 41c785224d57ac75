#include "fg_common.h"
extern "C" int fg_flash_attn_varlen_fwd(const FgFlashParams* p, void* stream) {
  fg_set_error("flash_attn_varlen_fwd: not built yet");
  return FG_ERR_UNSUPPORTED;
}
