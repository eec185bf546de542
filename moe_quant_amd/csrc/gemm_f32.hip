// fp32 MFMA GEMM for gfx950: 128x128 workgroup tile, four wave64 each owning 64x64
// (2x2 blocks of v_mfma_f32_32x32x2_f32), operands staged through LDS as [k][m] / [k][n]
// so every fragment read is a conflict-free ds_read_b32 whatever the global layout was.
// Used by the factorisation (trailing update, panel solve, triangular inverse) and by the
// GPTQ lazy-batch trailing update.
#include <mutex>

#include "gemm_f32_tile.hpp"

namespace {

using namespace gemmf32;

// pair_rows > 0 (triangular-K problems): the workgroup computes row tile tm and then its mirror
// pair_rows-1-tm, so every workgroup sees the same total K and the triangle no longer unbalances the grid.
template <bool A_KC, bool B_KC>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2))) void gemm_f32_kernel(GemmF32 g, int tiles_n, int total, int vecA, int vecB,
                                                      int pair_rows) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  int tm, tn;
  decode_tile(g, xcd_remap(blockIdx.x, total), tiles_n, tm, tn);
  tile_body<A_KC, B_KC>(g, tm, tn, blockIdx.z, reinterpret_cast<float*>(smem_raw), vecA, vecB);
  if (pair_rows > 0) {
    const int tm2 = pair_rows - 1 - tm;
    if (tm2 != tm) tile_body<A_KC, B_KC>(g, tm2, tn, blockIdx.z, reinterpret_cast<float*>(smem_raw), vecA, vecB);
  }
}

template <bool A_KC, bool B_KC>
int launch(const GemmF32& g, int tiles_n, int total, int vecA, int vecB, int pair_rows, hipStream_t stream) {
  static std::once_flag once;
  std::call_once(once, [] {
    (void)hipFuncSetAttribute((const void*)gemm_f32_kernel<A_KC, B_KC>, hipFuncAttributeMaxDynamicSharedMemorySize,
                              (int)SMEM_BYTES);
  });
  hipLaunchKernelGGL((gemm_f32_kernel<A_KC, B_KC>), dim3(total, 1, g.batch), dim3(256), SMEM_BYTES, stream, g, tiles_n,
                     total, vecA, vecB, pair_rows);
  return mq_check_launch();
}

}  // namespace

bool mq_gemm_operand_aligned(const float* p, long ld, long batch) {
  return ((uintptr_t)p % 16 == 0) && (ld % 4 == 0) && (batch % 4 == 0);
}

int mq_launch_gemm_f32(const GemmF32& g, hipStream_t stream) {
  if (g.M <= 0 || g.N <= 0 || g.batch <= 0) return MQ_OK;
  if (!g.A || !g.B || !g.C) return MQ_ERR_ARG;
  const bool a_kc = (g.sak == 1), b_kc = (g.sbk == 1);
  if (!a_kc && g.sam != 1) return MQ_ERR_ARG;
  if (!b_kc && g.sbn != 1) return MQ_ERR_ARG;
  if (g.tri && g.M != g.N) return MQ_ERR_ARG;
  const int tiles_m = (g.M + BM - 1) / BM, tiles_n = (g.N + BN - 1) / BN;
  int total = g.tri ? tiles_m * (tiles_m + 1) / 2 : tiles_m * tiles_n;
  int pair_rows = 0;
  if (!g.tri && g.ktrim != 0 && tiles_m >= 2) {
    pair_rows = tiles_m;
    total = ((tiles_m + 1) / 2) * tiles_n;
  }
  const int vecA = mq_gemm_operand_aligned(g.A, a_kc ? g.sam : g.sak, g.batchA);
  const int vecB = mq_gemm_operand_aligned(g.B, b_kc ? g.sbn : g.sbk, g.batchB);
  if (a_kc && b_kc) return launch<true, true>(g, tiles_n, total, vecA, vecB, pair_rows, stream);
  if (a_kc && !b_kc) return launch<true, false>(g, tiles_n, total, vecA, vecB, pair_rows, stream);
  if (!a_kc && b_kc) return launch<false, true>(g, tiles_n, total, vecA, vecB, pair_rows, stream);
  return launch<false, false>(g, tiles_n, total, vecA, vecB, pair_rows, stream);
}

// Test hook: plain GEMM through the C ABI so the MFMA core can be checked on its own.
extern "C" int mq_gemm_f32(const float* A, long sam, long sak, const float* B, long sbk, long sbn, float* C, long ldc,
                           int M, int N, int K, float alpha, float beta, int tri, int ktrim, void* stream) {
  GemmF32 g{A, B, C, sam, sak, sbk, sbn, ldc, M, N, K, alpha, beta, tri, ktrim, 1, 0, 0, 0};
  return mq_launch_gemm_f32(g, (hipStream_t)stream);
}
