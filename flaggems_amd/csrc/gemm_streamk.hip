// Host side of the general-shape stream-K schedule over the 128x128 MFMA tile (16-bit inputs).
//
// Tiles are split as in the partition rule exported by fg_streamk_partition: the ragged last wave
// of tiles (plus, when it is small, one full wave) is shared K-step by K-step between one
// persistent workgroup per CU; the remaining full waves run data-parallel.  Two launches on the
// same stream: the data-parallel tiles [sk_tiles, tiles) first, then the stream-K workgroups.
#include <mutex>
#include "gemm_tile.h"

namespace fgk {

namespace {
constexpr int kBM = 128, kBN = 128, kBK = 64;

template <typename T, int AMODE, int BMODE>
int launch(const GemmArgs& g, int dp_tiles, hipStream_t st) {
  typedef TileCompute<T, kBM, kBN, AMODE, BMODE> TC;
  static std::once_flag once;
  static hipError_t attr_err = hipSuccess;
  auto dp = gemm_dp_kernel<T, kBM, kBN, AMODE, BMODE>;
  auto sk = gemm_streamk_kernel<T, kBM, kBN, AMODE, BMODE>;
  std::call_once(once, [&] {
    attr_err = hipFuncSetAttribute(reinterpret_cast<const void*>(dp), hipFuncAttributeMaxDynamicSharedMemorySize, TC::LDS_BYTES);
    if (attr_err == hipSuccess)
      attr_err = hipFuncSetAttribute(reinterpret_cast<const void*>(sk), hipFuncAttributeMaxDynamicSharedMemorySize, TC::LDS_BYTES);
  });
  if (attr_err != hipSuccess) {
    fg_set_error("gemm(stream-K): cannot reserve LDS: %s", hipGetErrorString(attr_err));
    return FG_ERR_LAUNCH;
  }
  if (dp_tiles > 0) hipLaunchKernelGGL(dp, dim3((unsigned)dp_tiles), dim3(kThreads), TC::LDS_BYTES, st, g);
  if (g.sk_tiles > 0) hipLaunchKernelGGL(sk, dim3((unsigned)g.sk_workers), dim3(kThreads), TC::LDS_BYTES, st, g);
  return fg_check_launch("gemm(stream-K)");
}

template <typename T>
int launch_modes(const GemmArgs& g, int amode, int bmode, int dp_tiles, hipStream_t st) {
  if (amode == LOAD_K && bmode == LOAD_K) return launch<T, LOAD_K, LOAD_K>(g, dp_tiles, st);
  if (amode == LOAD_K && bmode == LOAD_MN) return launch<T, LOAD_K, LOAD_MN>(g, dp_tiles, st);
  if (amode == LOAD_MN && bmode == LOAD_K) return launch<T, LOAD_MN, LOAD_K>(g, dp_tiles, st);
  if (amode == LOAD_MN && bmode == LOAD_MN) return launch<T, LOAD_MN, LOAD_MN>(g, dp_tiles, st);
  return launch<T, LOAD_GEN, LOAD_GEN>(g, dp_tiles, st);
}
}  // namespace

size_t streamk_workspace_bytes(int64_t M, int64_t N, int64_t K, int dtype, int num_cu) {
  if (dtype != FG_F16 && dtype != FG_BF16) return 0;
  if (M <= 0 || N <= 0 || K <= 0) return 0;
  return kPartialOffset + (size_t)num_cu * 2 * kBM * kBN * sizeof(float);
}

int streamk_launch(GemmArgs g, int dtype, int amode, int bmode, void* workspace, size_t workspace_bytes, int num_cu,
                   hipStream_t st) {
  FG_REQUIRE(workspace != nullptr && workspace_bytes >= streamk_workspace_bytes(g.M, g.N, g.K, dtype, num_cu),
             FG_ERR_WORKSPACE, "gemm(stream-K): workspace too small");
  FG_REQUIRE(fg_aligned(workspace, 256), FG_ERR_WORKSPACE, "gemm(stream-K): workspace must be 256-byte aligned");
  g.tiles_m = (int)fg_cdiv(g.M, kBM);
  g.tiles_n = (int)fg_cdiv(g.N, kBN);
  g.iters_per_tile = (int)fg_cdiv(g.K, kBK);
  const int64_t tiles = (int64_t)g.tiles_m * g.tiles_n;
  FG_REQUIRE(tiles < ((int64_t)1 << 30), FG_ERR_UNSUPPORTED, "gemm(stream-K): too many tiles");
  int64_t sk_tiles = 0;
  fg_streamk_partition(tiles, g.iters_per_tile, num_cu, &sk_tiles, nullptr, nullptr);
  FG_REQUIRE(num_cu <= kMaxWorkers, FG_ERR_UNSUPPORTED, "gemm(stream-K): more CUs than ticket counters");
  const int64_t total_iters = sk_tiles * g.iters_per_tile;
  int workers = num_cu;
  if (total_iters < workers) workers = (int)total_iters;
  g.sk_tiles = (int)sk_tiles;
  g.sk_workers = workers;
  g.sk_per = workers > 0 ? total_iters / workers : 0;
  g.sk_rem = workers > 0 ? total_iters % workers : 0;
  g.tile_base = (int)sk_tiles;
  char* ws = (char*)workspace;
  g.tickets = (unsigned*)(ws + kTicketOffset);
  g.partials = (float*)(ws + kPartialOffset);
  const int dp_tiles = (int)(tiles - sk_tiles);
  if (dtype == FG_BF16) return launch_modes<bf16_t>(g, amode, bmode, dp_tiles, st);
  return launch_modes<f16_t>(g, amode, bmode, dp_tiles, st);
}

}  // namespace fgk
