// GPTQ column loop for gfx950.
//
// Layout follows the loop's natural access: Wt is the transposed weight (C x R, one weight column per
// memory row), so a wavefront that gives one lane to each output row reads and writes fully coalesced.
// Rows of W never interact, so there is no grid-wide synchronisation anywhere.
//
//   per block of <=128 columns [i1, i2):
//     gptq_block_kernel : each lane keeps its row's 128 block weights in registers, walks the columns
//                         in order (quantize -> dequantize -> error -> fused-multiply-add of the error
//                         into the remaining block columns, multiplier U[j,k] wave-uniform via scalar
//                         loads), and leaves codes, dequantized weights and the error block in memory.
//     trailing update   : Wt[i2:, :] += U[i1:i2, i2:]^T * E   as an fp32 MFMA GEMM (gemm_f32.hip).
//
// Arithmetic per column is the reference's: q = clamp(floor(x/s + z + 0.5), 0, maxq) with IEEE division,
// y = round_to(dtype)((q - z) * s), e = y - x, w_k = fma(U[j,k], e, w_k).
#include <hip/hip_fp16.h>

#include "common.hpp"

namespace {

constexpr int B = 128;

template <int RD>
__device__ __forceinline__ float round_dtype(float x) {
  if (RD == 1) return round_to_bf16(x);
  if (RD == 2) return __half2float(__float2half_rn(x));
  return x;
}

struct LoopArgs {
  float* Wt;
  long ldw;
  int C, R;
  const float* U;
  long ldu;
  const float* scale;
  long lds;
  const int* scale_row;  // nullable: scale row of column j is scale_row[j], else j
  const float* qzero;    // nullable: same indexing as scale, else qzero_const
  float qzero_const, maxq;
  uint8_t* Qt;
  float* E;
};

constexpr int MB = 16;      // micro-block: columns walked with weights in registers
constexpr int WSTRIDE = 64; // LDS tile is [column][lane]

typedef const float __attribute__((address_space(4))) * cfloat_p;  // constant address space -> scalar loads

// One wavefront owns 64 rows.  The 128-column block of those rows sits in LDS ([column][lane], so
// every access is conflict-free); 16 columns at a time move to registers for the strictly sequential
// part, and their 16 errors are then folded into the rest of the block, 16 columns per pass, with the
// multipliers U[j,k] arriving as scalar operands.  For every weight the updates are applied in
// ascending j with one fma each, exactly the order of the sequential reference.
template <bool FULL, int RD>
__global__ __launch_bounds__(64) void gptq_block_kernel(LoopArgs a, int i1, int nb) {
  __shared__ float tile[B * WSTRIDE];
  const int lane = threadIdx.x;
  const int r0 = blockIdx.x * 64;
  // Lanes past the last row shadow row R-1: they compute and store exactly what that row's own lane
  // does, which keeps every branch wave-uniform (a divergent branch would turn the scalar loads of U
  // into per-lane vector loads).
  const int r = min(r0 + lane, a.R - 1);
  float* __restrict__ wp = a.Wt + (long)i1 * a.ldw + r;
  for (int k = 0; k < B; ++k) tile[k * WSTRIDE + lane] = (FULL || k < nb) ? wp[(long)k * a.ldw] : 0.f;
  cfloat_p U = (cfloat_p)(a.U);
  const float maxq = a.maxq;
#pragma unroll 1
  for (int c0 = 0; c0 < (FULL ? B : nb); c0 += MB) {
    float w[MB], e[MB];
#pragma unroll
    for (int t = 0; t < MB; ++t) w[t] = tile[(c0 + t) * WSTRIDE + lane];
#pragma unroll
    for (int J = 0; J < MB; ++J) {
      e[J] = 0.f;
      if (FULL || c0 + J < nb) {
        const int col = i1 + c0 + J;
        const int srow = a.scale_row ? a.scale_row[col] : col;
        const float s = a.scale[(long)srow * a.lds + r];
        const float z = a.qzero ? a.qzero[(long)srow * a.lds + r] : a.qzero_const;
        const float x = w[J];
        const float v = x / s + z;
        float q = floorf(v + 0.5f);
        q = fminf(fmaxf(q, 0.f), maxq);
        const float y = round_dtype<RD>((q - z) * s);
        e[J] = y - x;
        wp[(long)(c0 + J) * a.ldw] = y;
        a.Qt[(long)col * a.R + r] = (uint8_t)q;
        a.E[(long)(c0 + J) * a.R + r] = e[J];
        cfloat_p urow = U + (long)col * a.ldu + i1 + c0;
#pragma unroll
        for (int t = J + 1; t < MB; ++t) {
          const int tc = FULL ? t : min(t, nb - 1 - c0);  // keep the scalar load inside the matrix
          w[t] = fmaf(urow[tc], e[J], w[t]);
        }
      }
    }
    const int cend = FULL ? B : nb;
#pragma unroll 1
    for (int k0 = c0 + MB; k0 < cend; k0 += MB) {
      float x[MB];
#pragma unroll
      for (int t = 0; t < MB; ++t) x[t] = tile[(k0 + t) * WSTRIDE + lane];
#pragma unroll
      for (int J = 0; J < MB; ++J) {
        const int jr = FULL ? J : min(J, nb - 1 - c0);  // rows past the block carry e = 0; stay inside U
        cfloat_p urow = U + (long)(i1 + c0 + jr) * a.ldu + i1 + k0;
#pragma unroll
        for (int t = 0; t < MB; ++t) {
          const int tc = FULL ? t : min(t, nb - 1 - k0);
          x[t] = fmaf(urow[tc], e[J], x[t]);
        }
      }
#pragma unroll
      for (int t = 0; t < MB; ++t) tile[(k0 + t) * WSTRIDE + lane] = x[t];
    }
  }
}

template <int RD>
int run_loop(const LoopArgs& a, int block, hipStream_t st) {
  const int grid = (a.R + 63) / 64;
  for (int i1 = 0; i1 < a.C; i1 += block) {
    const int i2 = (i1 + block < a.C) ? i1 + block : a.C;
    const int nb = i2 - i1;
    if (nb == B)
      hipLaunchKernelGGL((gptq_block_kernel<true, RD>), dim3(grid), dim3(64), 0, st, a, i1, nb);
    else
      hipLaunchKernelGGL((gptq_block_kernel<false, RD>), dim3(grid), dim3(64), 0, st, a, i1, nb);
    int rc = mq_check_launch();
    if (rc != MQ_OK) return rc;
    if (i2 < a.C) {
      // Wt[i2+m, r] += sum_j U[i1+j, i2+m] * E[j, r]
      GemmF32 g{a.U + (long)i1 * a.ldu + i2, a.E, a.Wt + (long)i2 * a.ldw, 1, a.ldu, a.R, 1, a.ldw,
                a.C - i2, a.R, nb, 1.f, 1.f, 0, 0, 1, 0, 0, 0};
      if ((rc = mq_launch_gemm_f32(g, st)) != MQ_OK) return rc;
    }
  }
  return MQ_OK;
}

}  // namespace

extern "C" int mq_gptq_loop(float* Wt, long ldw, int C, int R, const float* U, long ldu, const float* scale,
                            long ld_scale, const int* scale_row, const float* qzero, float qzero_const, float maxq,
                            int round_dtype, int block, uint8_t* Qt, float* E, void* stream) {
  if (!Wt || !U || !scale || !Qt || !E || C <= 0 || R <= 0) return MQ_ERR_ARG;
  if (ldw < R || ldu < C || ld_scale < R) return MQ_ERR_ARG;
  if (round_dtype < 0 || round_dtype > 2) return MQ_ERR_ARG;
  if (block <= 0 || block > B) block = B;  // wider blocks only reassociate the trailing sums
  LoopArgs a{Wt, ldw, C, R, U, ldu, scale, ld_scale, scale_row, qzero, qzero_const, maxq, Qt, E};
  hipStream_t st = (hipStream_t)stream;
  switch (round_dtype) {
    case 0: return run_loop<0>(a, block, st);
    case 1: return run_loop<1>(a, block, st);
    default: return run_loop<2>(a, block, st);
  }
}
