// Shared declarations for the moequant HIP library (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define MQ_OK 0
#define MQ_ERR_ARG (-1)       // bad pointer / size / alignment
#define MQ_ERR_LAUNCH (-2)    // hipGetLastError() after a launch was not hipSuccess
#define MQ_ERR_WORKSPACE (-3) // workspace too small
#define MQ_ERR_TOO_LARGE (-4) // problem beyond the fixed capacity of an entry point that brings its own scratch memory
// element types of weights, activations and rounding targets
#define MQ_DT_F32 0
#define MQ_DT_BF16 1
#define MQ_DT_F16 2

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef short bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8n __attribute__((ext_vector_type(8)));

static inline int mq_check_launch() { return hipGetLastError() == hipSuccess ? MQ_OK : MQ_ERR_LAUNCH; }

__device__ __forceinline__ float bf16_bits_to_f32(uint16_t b) { return __uint_as_float(((uint32_t)b) << 16); }

// round-to-nearest-even fp32 -> bf16 -> fp32 (finite inputs; NaN stays NaN)
__device__ __forceinline__ float round_to_bf16(float x) {
  uint32_t u = __float_as_uint(x);
  if ((u & 0x7fffffffu) > 0x7f800000u) return x;
  u += 0x7fffu + ((u >> 16) & 1u);
  return __uint_as_float(u & 0xffff0000u);
}
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float x) {
  uint32_t u = __float_as_uint(x);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

// ---------------------------------------------------------------------------------------------
// fp32 MFMA GEMM (gemm_f32.hip):  C[m,n] = beta*C[m,n] + alpha * sum_k A(m,k) * B(k,n)
// A(m,k) lives at A[m*sam + k*sak]; exactly one of sam/sak must be 1 (same for B with sbk/sbn).
// C is row-major with leading dimension ldc.  tri: 0 = all tiles, 1 = only tiles with tile_m <= tile_n
// (upper block triangle, requires M == N).  ktrim: 0 = full K; 1 = K range [0, tile_m_end) (A is the
// transpose of an upper-triangular matrix); 2 = K range [tile_m_begin, K) (A upper triangular).
// batch: blockIdx.z offsets A,B,C by z*batch{A,B,C} elements.
// ---------------------------------------------------------------------------------------------
struct GemmF32 {
  const float* A;
  const float* B;
  float* C;
  long sam, sak, sbk, sbn, ldc;
  int M, N, K;
  float alpha, beta;
  int tri, ktrim;
  int batch;
  long batchA, batchB, batchC;
  // optional: the B operand is the sum of several arrays of the same layout, bsum_stride elements apart;
  // column tile tn adds the first min(bsum, tn / bsum_c + 1) of them (0 = plain B).  Interior tiles only.
  int bsum, bsum_c;
  long bsum_stride;
  // optional: the old C (the beta term) is read from another array of row pitch ldcs (nullptr = from C)
  const float* Csrc;
  long ldcs;
  // 1: interior tiles too run on the fp32 matrix cores (default: operands split into bf16 pieces, bf16 cores)
  int fp32_mfma;
};
int mq_launch_gemm_f32(const GemmF32& g, hipStream_t stream);
bool mq_gemm_operand_aligned(const float* p, long ld, long batch);
