#include "gemm_tile.h"
namespace fgk {
int skinny_supported(const GemmArgs&, int, bool, bool) { return 0; }
size_t skinny_workspace_bytes(int64_t, int64_t, int64_t, int) { return 0; }
int skinny_launch(const GemmArgs&, int, void*, size_t, int, hipStream_t) { return FG_ERR_UNSUPPORTED; }
size_t streamk_workspace_bytes(int64_t, int64_t, int64_t, int, int) { return 0; }
int streamk_launch(GemmArgs, int, int, int, void*, size_t, int, hipStream_t) { return FG_ERR_UNSUPPORTED; }
}
