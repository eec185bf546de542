// Damped-Hessian factorisation for GPTQ:  given SPD H (upper triangle read), produce in place the
// unit-diagonal upper-triangular  U = chol(H^-1, upper) / diag  that the column loop consumes.
//
// Instead of the three library calls of the torch path (cholesky, cholesky_inverse, cholesky) this
// uses the identity  H = R R^T (R upper, "reverse" Cholesky)  =>  H^-1 = R^-T R^-1  =>  the unique
// upper Cholesky factor of H^-1 is R^-1.  So: one blocked reverse Cholesky (right-looking, bottom-right
// to top-left), one blocked triangular inverse (recursive doubling, batched), one row scaling.
// (2/3) C^3 flop instead of (4/3) C^3, all in the caller's C x C buffer.
//
//   per 128-block b (last to first):
//     diag kernel  : R_bb = revchol(H_bb), then R_bb^-1 written in place (one workgroup, LDS resident)
//     panel GEMM   : R_ab = H_ab * (R_bb^-1)^T            for a < b   (fp32 MFMA)
//     trailing GEMM: H_aa' -= R_ab R_a'b^T                for a <= a' < b  (fp32 MFMA, upper tiles only)
//   triangular inverse, block size s = 128, 256, ...: for each aligned pair (left, right)
//     T^T = U22^T R12^T  (written to the unused mirror position below the diagonal)
//     U12 = -U11 T
//   finalize: U[j, k] /= U[j, j], strictly lower part zeroed.
#include "common.hpp"

namespace {

constexpr int NB = 128;
constexpr int LDD = 129;

// One workgroup, 256 threads.  Block is staged in LDS; on exit the global block holds R_bb^-1
// (upper, zeros below the diagonal).  A non-positive or NaN pivot records its 1-based global index
// in *info (first one wins) and is replaced by 1 so that every wave still finishes normally.
__global__ __launch_bounds__(256) void revchol_diag_kernel(float* A, long ld, int i1, int* info) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  float* S = reinterpret_cast<float*>(smem);  // [NB][LDD]
  float* colj = S + NB * LDD;                 // [NB]
  float* part = colj + NB;                    // [256]
  const int tid = threadIdx.x;
  float* blk = A + (long)i1 * ld + i1;
  for (int idx = tid; idx < NB * NB; idx += 256) {
    const int r = idx >> 7, c = idx & 127;
    S[r * LDD + c] = (c >= r) ? blk[(long)r * ld + c] : 0.f;
  }
  __syncthreads();

  const int k = tid & 127, h = tid >> 7;
  // ---- reverse Cholesky: S = R R^T, R upper, columns from last to first
  for (int j = NB - 1; j >= 0; --j) {
    float d = S[j * LDD + j];
    if (!(d > 0.f)) {
      if (tid == 0) atomicCAS(info, 0, i1 + j + 1);
      d = 1.f;
    }
    const float r = sqrtf(d);
    float ck = 0.f;
    if (h == 0) {
      if (k < j) ck = S[k * LDD + j] / r;
      else if (k == j) ck = r;
      colj[k] = ck;
    }
    __syncthreads();
    if (h == 0 && k <= j) S[k * LDD + j] = ck;
    ck = colj[k];
    if (k < j) {
      for (int i = h; i <= k; i += 2) S[i * LDD + k] = fmaf(-colj[i], ck, S[i * LDD + k]);
    }
    __syncthreads();
  }
  // ---- in-place inverse of the upper-triangular R, column by column:
  //      X[i,j] = -(sum_{k=i}^{j-1} X[i,k] R[k,j]) / R[j,j],  X[j,j] = 1/R[j,j]
  for (int j = 0; j < NB; ++j) {
    const int i = k;
    float s = 0.f;
    if (i < j) {
      for (int kk = i + h; kk < j; kk += 2) s = fmaf(S[i * LDD + kk], S[kk * LDD + j], s);
    }
    part[tid] = s;
    const float rjj = S[j * LDD + j];
    __syncthreads();
    if (h == 0) {
      if (i < j) S[i * LDD + j] = -(part[i] + part[i + 128]) / rjj;
      else if (i == j) S[j * LDD + j] = 1.f / rjj;
    }
    __syncthreads();
  }
  for (int idx = tid; idx < NB * NB; idx += 256) {
    const int r = idx >> 7, c = idx & 127;
    blk[(long)r * ld + c] = S[r * LDD + c];
  }
}

// U[j,k] <- U[j,k] / U[j,j] for k > j, 1 on the diagonal, 0 for k < j (normalize == 0: only the zeroing).
// One workgroup per row.  The diagonal travels through LDS: the one thread that loads it publishes the
// value before the barrier (a data dependence the compiler cannot reorder), so the thread that later
// overwrites the diagonal cannot be observed by anyone.
__global__ __launch_bounds__(256) void unit_diag_kernel(float* A, long ld, int C, int normalize) {
  __shared__ float dsh;
  const int j = blockIdx.x;
  float* row = A + (long)j * ld;
  if (threadIdx.x == 0) dsh = row[j];
  __syncthreads();
  const float d = dsh;
  if (normalize) {
    for (int k = threadIdx.x; k < C; k += 256) row[k] = (k > j) ? (row[k] / d) : (k == j ? 1.f : 0.f);
  } else {
    for (int k = threadIdx.x; k < j; k += 256) row[k] = 0.f;
  }
}

constexpr size_t DIAG_SMEM = (size_t)(NB * LDD + NB + 256) * sizeof(float);

}  // namespace

extern "C" int mq_factor_upper_inverse(float* A, long ld, int C, int normalize, int* info, void* stream) {
  if (!A || !info || C <= 0 || ld < C) return MQ_ERR_ARG;
  if (C % NB != 0) return MQ_ERR_ARG;  // the host pads with an identity block
  hipStream_t st = (hipStream_t)stream;
  static bool attr_done = false;
  if (!attr_done) {
    (void)hipFuncSetAttribute((const void*)revchol_diag_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                              (int)DIAG_SMEM);
    attr_done = true;
  }
  int rc;
  for (int i1 = C - NB; i1 >= 0; i1 -= NB) {
    hipLaunchKernelGGL(revchol_diag_kernel, dim3(1), dim3(256), DIAG_SMEM, st, A, ld, i1, info);
    if ((rc = mq_check_launch()) != MQ_OK) return rc;
    if (i1 == 0) break;
    float* P = A + i1;                       // panel: rows [0,i1), cols [i1, i1+NB)
    const float* Dinv = A + (long)i1 * ld + i1;
    GemmF32 panel{P, Dinv, P, ld, 1, 1, ld, ld, i1, NB, NB, 1.f, 0.f, 0, 0, 1, 0, 0, 0};
    if ((rc = mq_launch_gemm_f32(panel, st)) != MQ_OK) return rc;
    GemmF32 trail{P, P, A, ld, 1, 1, ld, ld, i1, i1, NB, -1.f, 1.f, 1, 0, 1, 0, 0, 0};
    if ((rc = mq_launch_gemm_f32(trail, st)) != MQ_OK) return rc;
  }
  for (long s = NB; s < C; s *= 2) {
    const int nfull = (int)(C / (2 * s));
    auto level = [&](long p, int w, int batch) -> int {
      float* U11 = A + p * ld + p;
      float* U22 = A + (p + s) * ld + (p + s);
      float* R12 = A + p * ld + (p + s);
      float* Tt = A + (p + s) * ld + p;
      const long bs = 2 * s * (ld + 1);
      // T^T (w x s) = U22^T (w x w) * R12^T (w x s)
      GemmF32 g1{U22, R12, Tt, 1, ld, 1, ld, ld, w, (int)s, w, 1.f, 0.f, 0, 1, batch, bs, bs, bs};
      int r = mq_launch_gemm_f32(g1, st);
      if (r != MQ_OK) return r;
      // U12 (s x w) = -U11 (s x s) * T (s x w),  T(k,n) = Tt[n][k]
      GemmF32 g2{U11, Tt, R12, ld, 1, 1, ld, ld, (int)s, w, (int)s, -1.f, 0.f, 0, 2, batch, bs, bs, bs};
      return mq_launch_gemm_f32(g2, st);
    };
    if (nfull > 0 && (rc = level(0, (int)s, nfull)) != MQ_OK) return rc;
    const long p = (long)nfull * 2 * s;
    if (p + s < C && (rc = level(p, (int)(C - p - s), 1)) != MQ_OK) return rc;
  }
  hipLaunchKernelGGL(unit_diag_kernel, dim3(C), dim3(256), 0, st, A, ld, C, normalize);
  return mq_check_launch();
}
