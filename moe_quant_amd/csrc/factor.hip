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
#include "gemm_f32_tile.hpp"

namespace {

constexpr int NB = 128;
constexpr int SB = 32;     // sub-block edge inside the diagonal-block kernel
constexpr int LDM = 131;   // LDS row pitch (odd: lane-per-row accesses hit 32 distinct banks)

// ---------------------------------------------------------------------------------------------
// Diagonal block: S (128x128, upper valid) -> R^-1 where S = R R^T, R upper.
//
// One LDS array holds two triangular matrices side by side: the upper triangle S(i,k), k >= i, at
// column k+1, and below it Xt(c,k) = X[k][c], k <= c, at column k, where X accumulates R^-1.
// Stacking M = [S; Xt] makes the inverse fall out of the factorisation: every elimination step that
// scales column j of S by 1/R_jj and subtracts its outer product from the columns to its left does,
// applied unchanged to the rows of Xt (initialised to the identity), exactly the right-looking update
// of the triangular inverse.  Nothing extra is computed for the inverse except more rows.
//
// Sub-blocks of 32: the 32x32 diagonal sub-block is eliminated by one wavefront with a row per lane in
// registers -- lanes 0-31 carry S rows, lanes 32-63 the matching Xt rows, same instructions -- and the
// off-diagonal work (column scaling by the sub-block inverse, outer-product updates) runs as 32x32x32
// products on the fp32 matrix cores, one product per wavefront at a time.
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ float& Sv(float* buf, int i, int k) { return buf[i * LDM + k + 1]; }
__device__ __forceinline__ float& Xv(float* buf, int c, int k) { return buf[c * LDM + k]; }

__device__ __forceinline__ float bcast_lane(float v, int lane) {
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), lane));
}

template <int J>
struct ElimStep {
  // one elimination step on column J of the 32x32 sub-block held one row per lane in reg[]
  static __device__ __forceinline__ void run(float (&reg)[SB], int gidx, int& bad) {
    float d = bcast_lane(reg[J], J);
    const bool neg = !(d > 0.f);  // also catches NaN; selects, not branches: one basic block per sub-block
    bad = (neg && bad == 0) ? (gidx + J + 1) : bad;
    d = neg ? 1.f : d;
    float y = __frsqrt_rn(d);
    y = y * (1.5f - 0.5f * d * y * y);  // one Newton step: 1/sqrt(d) to fp32 accuracy
    const float v = reg[J] * y;
    reg[J] = v;
    // nearest column first: the next step's pivot lives in reg[J-1], so its chain can start while the
    // remaining updates of this step are still issuing
#pragma unroll
    for (int k = J - 1; k >= 0; --k) reg[k] = fmaf(-bcast_lane(v, k), v, reg[k]);
    ElimStep<J - 1>::run(reg, gidx, bad);
  }
};
template <>
struct ElimStep<-1> {
  static __device__ __forceinline__ void run(float (&)[SB], int, int&) {}
};

// acc (32x32, MFMA layout) (+)= sum_k a(m,k) * b(k,n); a/b fetch one element for this lane
template <typename FA, typename FB>
__device__ __forceinline__ void mm32(floatx16& acc, FA a, FB b, int lane) {
  const int x = lane & 31, kk = lane >> 5;
  float av[16], bv[16];
#pragma unroll
  for (int t = 0; t < 16; ++t) {
    av[t] = a(x, 2 * t + kk);
    bv[t] = b(2 * t + kk, x);
  }
#pragma unroll
  for (int t = 0; t < 16; ++t) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av[t], bv[t], acc, 0, 0, 0);
}

// buf: LDS, NB*LDM floats.  blk: global 128x128 block (row pitch ld).  gidx0: global index of its first row.
// preloaded: the caller already filled Sv (upper) and zeroed Xv (strictly lower) and synchronised.
// blk rows must be 16-byte aligned (ld % 4 == 0).
__device__ __forceinline__ void diag_block_invert(float* buf, float* blk, long ld, int gidx0, int* info,
                                                  bool preloaded) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  if (!preloaded) {
    float4 v[16];
#pragma unroll
    for (int it = 0; it < 16; ++it) {
      const int idx = tid + it * 256, r = idx >> 5, c = (idx & 31) << 2;
      v[it] = *reinterpret_cast<const float4*>(blk + (long)r * ld + c);
    }
#pragma unroll
    for (int it = 0; it < 16; ++it) {
      const int idx = tid + it * 256, r = idx >> 5, c = (idx & 31) << 2;
      const float e[4] = {v[it].x, v[it].y, v[it].z, v[it].w};
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        if (c + q >= r) Sv(buf, r, c + q) = e[q];
        else Xv(buf, r, c + q) = 0.f;  // strictly lower part of Xt starts at zero (unit diagonal implicit)
      }
    }
    __syncthreads();
  }

  for (int J = NB / SB - 1; J >= 0; --J) {
    const int o = J * SB;
    if (wave == 0) {
      float reg[SB];
      const int li = lane & 31;
      const bool up = lane >= 32;
#pragma unroll
      for (int k = 0; k < SB; ++k) reg[k] = up ? (k == li ? 1.f : 0.f) : (k >= li ? Sv(buf, o + li, o + k) : 0.f);
      int bad = 0;
      ElimStep<SB - 1>::run(reg, gidx0 + o, bad);
      if (bad != 0 && lane == 0) atomicCAS(info, 0, bad);
#pragma unroll
      for (int k = 0; k < SB; ++k) {
        if (!up && k >= li) Sv(buf, o + li, o + k) = reg[k];
        if (up && k <= li) Xv(buf, o + li, o + k) = reg[k];
      }
    }
    __syncthreads();
    // ---- column block J of M times the sub-block inverse: V = M(:,J) * Xinv^T, Xinv[n][k] = Xt(o+k... ) masked
    {
      const int ntask = 3;  // J row blocks of S above the diagonal + (3-J) row blocks of Xt below it
      for (int t = wave; t < ntask; t += 4) {
        const bool is_s = t < J;
        const int rb = is_s ? t : (t + 1);  // S row block I=t, or Xt row block Cb=t+1 (> J)
        const int ro = rb * SB;
        floatx16 acc;
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[v] = 0.f;
        auto bfn = [&](int k, int n) { return (k >= n) ? Xv(buf, o + k, o + n) : 0.f; };  // Xinv[n][k]
        if (is_s) mm32(acc, [&](int m, int k) { return Sv(buf, ro + m, o + k); }, bfn, lane);
        else mm32(acc, [&](int m, int k) { return Xv(buf, ro + m, o + k); }, bfn, lane);
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int m = 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3), n = lane & 31;
          if (is_s) Sv(buf, ro + m, o + n) = acc[v];
          else Xv(buf, ro + m, o + n) = acc[v];
        }
      }
    }
    __syncthreads();
    // ---- outer-product updates of the column blocks K < J:  M(rb,K) -= V(rb) * R(K,J)^T
    {
      // tasks enumerated as (K, rb): for each K < J the S row blocks I <= K, then the Xt row blocks Cb >= J
      const int per_k_x = NB / SB - J;
      int t = 0;
      for (int K = 0; K < J; ++K) {
        const int cnt = (K + 1) + per_k_x;
        for (int q = 0; q < cnt; ++q, ++t) {
          if ((t & 3) != wave) continue;
          const bool is_s = q <= K;
          const int rb = is_s ? q : (J + (q - K - 1));
          const int ro = rb * SB, ko = K * SB;
          floatx16 acc;
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            const int m = 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3), n = lane & 31;
            acc[v] = is_s ? Sv(buf, ro + m, ko + n) : Xv(buf, ro + m, ko + n);
          }
          auto bfn = [&](int k, int n) { return Sv(buf, ko + n, o + k); };  // R(K,J)[n][k]
          if (is_s) {
            mm32(acc, [&](int m, int k) { return -Sv(buf, ro + m, o + k); }, bfn, lane);
          } else if (rb == J) {  // V is the sub-block inverse itself; only its lower triangle is Xt data
            mm32(acc, [&](int m, int k) { return (k <= m) ? -Xv(buf, ro + m, o + k) : 0.f; }, bfn, lane);
          } else {
            mm32(acc, [&](int m, int k) { return -Xv(buf, ro + m, o + k); }, bfn, lane);
          }
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            const int m = 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3), n = lane & 31;
            if (is_s) Sv(buf, ro + m, ko + n) = acc[v];
            else Xv(buf, ro + m, ko + n) = acc[v];
          }
        }
      }
    }
    __syncthreads();
  }
  // R^-1[r][c] = Xt(c, r) for r <= c, zero below the diagonal
#pragma unroll 4
  for (int it = 0; it < 16; ++it) {
    const int idx = tid + it * 256, r = idx >> 5, c = (idx & 31) << 2;
    float4 o4;
    o4.x = (r <= c + 0) ? Xv(buf, c + 0, r) : 0.f;
    o4.y = (r <= c + 1) ? Xv(buf, c + 1, r) : 0.f;
    o4.z = (r <= c + 2) ? Xv(buf, c + 2, r) : 0.f;
    o4.w = (r <= c + 3) ? Xv(buf, c + 3, r) : 0.f;
    *reinterpret_cast<float4*>(blk + (long)r * ld + c) = o4;
  }
}

__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2))) void revchol_diag_kernel(float* A, long ld, int i1, int* info) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  diag_block_invert(reinterpret_cast<float*>(smem), A + (long)i1 * ld + i1, ld, i1, info, false);
}

// One launch per elimination step b (block at offset i1, panel P = A[0:i1, i1:i1+128] already solved):
//   workgroup 0        : updates the next diagonal tile (rows/cols [i1-128, i1)) with the panel, keeps the
//                        result in LDS and inverts it right away (the next step's critical path);
//   workgroups 1..T-1  : the other T-1 upper tiles of the trailing update  A[0:i1,0:i1] -= P P^T.
// The diagonal-block work is thereby hidden behind the bulk of the trailing update.
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2))) void trail_diag_kernel(GemmF32 g, int total, float* A,
                                                                                                  long ld, int i1, int* info) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  float* buf = reinterpret_cast<float*>(smem);
  using namespace gemmf32;
  if (blockIdx.x == 0) {
    const int t = i1 / NB - 1;  // last tile of the column-major upper-triangle order
    tile_body<true, true, true>(g, t, t, 0, buf, 1, 1, [&](int r, int c, float v) {
      if (c >= r) Sv(buf, r, c) = v;
    });
    for (int idx = threadIdx.x; idx < NB * NB; idx += 256) {
      const int r = idx >> 7, c = idx & 127;
      if (c < r) Xv(buf, r, c) = 0.f;
    }
    __syncthreads();
    diag_block_invert(buf, A + (long)(i1 - NB) * ld + (i1 - NB), ld, i1 - NB, info, true);
  } else {
    int tm, tn;
    tri_decode(xcd_remap(blockIdx.x - 1, total - 1), tm, tn);
    tile_body<true, true>(g, tm, tn, 0, buf, 1, 1);
  }
}


// U[j,k] <- U[j,k] / U[j,j] for k > j, 1 on the diagonal, 0 for k < j (normalize == 0: only the zeroing).
// One workgroup per row.  The diagonal travels through LDS: the one thread that loads it publishes the
// value before the barrier (a data dependence the compiler cannot reorder), so the thread that later
// overwrites the diagonal cannot be observed by anyone.
// A failed factorisation (*info != 0) leaves the identity, the fallback GPTQ takes when Cholesky raises.
__global__ __launch_bounds__(256) void unit_diag_kernel(float* A, long ld, int C, int normalize, const int* info) {
  __shared__ float dsh;
  const int j = blockIdx.x;
  float* row = A + (long)j * ld;
  if (*info != 0) {
    for (int k = threadIdx.x; k < C; k += 256) row[k] = (k == j) ? 1.f : 0.f;
    return;
  }
  if (threadIdx.x == 0) dsh = row[j];
  __syncthreads();
  const float d = dsh;
  if (normalize) {
    for (int k = threadIdx.x; k < C; k += 256) row[k] = (k > j) ? (row[k] / d) : (k == j ? 1.f : 0.f);
  } else {
    for (int k = threadIdx.x; k < j; k += 256) row[k] = 0.f;
  }
}

constexpr size_t DIAG_SMEM = (size_t)(NB * LDM) * sizeof(float);
constexpr size_t FUSED_SMEM = DIAG_SMEM > gemmf32::SMEM_BYTES ? DIAG_SMEM : gemmf32::SMEM_BYTES;

}  // namespace

extern "C" int mq_factor_upper_inverse(float* A, long ld, int C, int normalize, int* info, void* stream) {
  if (!A || !info || C <= 0 || ld < C) return MQ_ERR_ARG;
  if (C % NB != 0) return MQ_ERR_ARG;  // the host pads with an identity block
  hipStream_t st = (hipStream_t)stream;
  static bool attr_done = false;
  if (!attr_done) {
    (void)hipFuncSetAttribute((const void*)revchol_diag_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                              (int)DIAG_SMEM);
    (void)hipFuncSetAttribute((const void*)trail_diag_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                              (int)FUSED_SMEM);
    attr_done = true;
  }
  if ((ld & 3) || ((uintptr_t)A & 15)) return MQ_ERR_ARG;  // float4 access to rows of A
  int rc;
  hipLaunchKernelGGL(revchol_diag_kernel, dim3(1), dim3(256), DIAG_SMEM, st, A, ld, C - NB, info);
  if ((rc = mq_check_launch()) != MQ_OK) return rc;
  for (int i1 = C - NB; i1 > 0; i1 -= NB) {
    float* P = A + i1;  // panel: rows [0,i1), cols [i1, i1+NB)
    const float* Dinv = A + (long)i1 * ld + i1;
    GemmF32 panel{P, Dinv, P, ld, 1, 1, ld, ld, i1, NB, NB, 1.f, 0.f, 0, 0, 1, 0, 0, 0};
    if ((rc = mq_launch_gemm_f32(panel, st)) != MQ_OK) return rc;
    GemmF32 trail{P, P, A, ld, 1, 1, ld, ld, i1, i1, NB, -1.f, 1.f, 1, 0, 1, 0, 0, 0};
    const int tiles = i1 / NB, total = tiles * (tiles + 1) / 2;
    hipLaunchKernelGGL(trail_diag_kernel, dim3(total), dim3(256), FUSED_SMEM, st, trail, total, A, ld, i1, info);
    if ((rc = mq_check_launch()) != MQ_OK) return rc;
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
  hipLaunchKernelGGL(unit_diag_kernel, dim3(C), dim3(256), 0, st, A, ld, C, normalize, info);
  return mq_check_launch();
}
