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
//   triangular inverse, one block row at a time, bottom to top, riding along in the same launches:
//     row b:  T^T = U22^T R12^T   (U22 = finished inverse of everything below/right of b, R12 = R[b, b+1:];
//                                  written to the unused mirror position below the diagonal)
//             U[b, b+1:] = -U_bb T
//     Both products only touch rows >= b, the elimination at step b only rows < b, so the first runs as extra
//     workgroups of step b's trailing-update launch and the second as extra workgroups of step b-1's panel
//     launch: the (1/3)C^3 flop of the inverse fill the CUs the late elimination steps leave idle.
//   finalize: U[j, k] /= U[j, j], strictly lower part zeroed.
#include <cstdlib>

#include "gemm_f32_tile.hpp"

namespace {

constexpr int NB = 128;
constexpr int SB = 32;     // sub-block edge inside the diagonal-block kernel
constexpr int LDM = 131;   // LDS row pitch (odd: lane-per-row accesses hit 32 distinct banks)
static int INV_KC = 4;  // the first inverse product is cut into K chunks of 4 blocks (512), one workgroup each

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

// Work item idx of the first inverse product: (row tile tm, K chunk s), enumerated from the bottom row tile up.
// Chunk s of row tile tm is written 128*s columns to the right of chunk 0; the second product adds the chunks
// while it loads its B operand (a fixed order, and no fence or atomic between workgroups: a device-scope fence
// here writes back the L2 of the XCD, dirty with the trailing update, and cost more than it saved).
__device__ __forceinline__ void inv_first_tile(const GemmF32& ginv, int kc, int idx, float* buf) {
  using namespace gemmf32;
  const int T = ginv.M / NB, smax = (T + kc - 1) / kc;
  const int tm = T - 1 - idx / smax, s = idx % smax;
  if (s > tm / kc) return;  // U22 is triangular: row tile tm stops at k = (tm+1)*128
  const int k0 = s * kc * NB, k1 = min((s + 1) * kc * NB, (tm + 1) * NB);
  GemmF32 gl = ginv;
  gl.A += (long)k0 * gl.sak;
  gl.B += (long)k0 * gl.sbk;
  gl.C += s * NB;
  gl.K = k1 - k0;
  gl.ktrim = 0;
  tile_body<false, true>(gl, tm, 0, 0, buf, 1, 1);
}

__global__ __launch_bounds__(256) void inv_first_kernel(GemmF32 ginv, int kc) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  inv_first_tile(ginv, kc, blockIdx.x, reinterpret_cast<float*>(smem));
}

// One launch per elimination step b (block at offset i1, panel P = A[0:i1, i1:i1+128] already solved):
//   workgroup 0          : updates the next diagonal tile (rows/cols [i1-128, i1)) with the panel, keeps the
//                          result in LDS and inverts it right away (the next step's critical path);
//   next inv_tiles ones  : T^T = U22^T R12^T for block row b of the inverse: row tile tm (k <= its last row, U22 is
//                          triangular) times K chunk s of 512; chunk s lands 128*s columns to the right of chunk
//                          0, in the mirror area of block column b+s, free since that row's inverse is complete;
//                          the second product sums the chunks while loading them;
//   the rest             : the other T-1 upper tiles of the trailing update  A[0:i1,0:i1] -= P P^T.
// The diagonal-block work is thereby hidden behind the bulk of the trailing update, and the inverse behind both.
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2))) void trail_diag_kernel(GemmF32 g, int total, GemmF32 ginv,
                                                                                                  int inv_tiles, int kc, float* A,
                                                                                                  long ld, int i1, int* info) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  float* buf = reinterpret_cast<float*>(smem);
  using namespace gemmf32;
  const int bid = blockIdx.x;
  if (bid == 0) {
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
  } else if (bid <= inv_tiles) {
    inv_first_tile(ginv, kc, bid - 1, buf);
  } else {
    int tm, tn;
    tri_decode(xcd_remap(bid - 1 - inv_tiles, total - 1), tm, tn);
    tile_body<true, true>(g, tm, tn, 0, buf, 1, 1);
  }
}

// Panel product of step b (P = H_ab Dinv^T, one tile per row block) together with the second product of the
// inverse's block row b+1 (U12 = -U11 T, one tile per column block): two independent GEMMs in one launch.
__global__ __launch_bounds__(256) void panel_inv_kernel(GemmF32 gp, int panel_tiles, GemmF32 g2, int inv_tiles) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  float* buf = reinterpret_cast<float*>(smem);
  using namespace gemmf32;
  const int bid = blockIdx.x;
  if (bid < panel_tiles) tile_body<true, true>(gp, bid, 0, 0, buf, 1, 1);
  else tile_body<true, true>(g2, 0, bid - panel_tiles, 0, buf, 1, 1);
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
    if (const char* e = getenv("MQ_INV_KC")) INV_KC = atoi(e) > 0 ? atoi(e) : INV_KC;
    (void)hipFuncSetAttribute((const void*)revchol_diag_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                              (int)DIAG_SMEM);
    (void)hipFuncSetAttribute((const void*)trail_diag_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                              (int)FUSED_SMEM);
    (void)hipFuncSetAttribute((const void*)panel_inv_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                              (int)gemmf32::SMEM_BYTES);
    (void)hipFuncSetAttribute((const void*)inv_first_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                              (int)gemmf32::SMEM_BYTES);
    attr_done = true;
  }
  if ((ld & 3) || ((uintptr_t)A & 15)) return MQ_ERR_ARG;  // float4 access to rows of A
  int rc;
  // the two products of block row b of the inverse (w = columns to the right of b)
  auto inv_first = [&](int b, int& tiles) {  // T^T (w x 128) = U22^T (w x w) * R12^T (w x 128), in K chunks
    const long p = (long)b * NB;
    const int w = C - (int)p - NB;
    tiles = (w / NB) * ((w / NB + INV_KC - 1) / INV_KC);
    return GemmF32{A + (p + NB) * ld + (p + NB), A + p * ld + (p + NB), A + (p + NB) * ld + p, 1, ld, 1, ld, ld,
                   w, NB, w, 1.f, 0.f, 0, 1, 1, 0, 0, 0};
  };
  auto inv_second = [&](int b, int& tiles) {  // U12 (128 x w) = -U11 (128 x 128) * T,  T(k,n) = Tt[n][k]
    const long p = (long)b * NB;
    const int w = C - (int)p - NB;
    tiles = w / NB;
    return GemmF32{A + p * ld + p, A + (p + NB) * ld + p, A + p * ld + (p + NB), ld, 1, 1, ld, ld,
                   NB, w, NB, -1.f, 0.f, 0, 0, 1, 0, 0, 0, (w / NB + INV_KC - 1) / INV_KC, INV_KC, NB};
  };
  const int B = C / NB;
  hipLaunchKernelGGL(revchol_diag_kernel, dim3(1), dim3(256), DIAG_SMEM, st, A, ld, C - NB, info);
  if ((rc = mq_check_launch()) != MQ_OK) return rc;
  for (int b = B - 1; b >= 1; --b) {
    const int i1 = b * NB;
    float* P = A + i1;  // panel: rows [0,i1), cols [i1, i1+NB)
    const float* Dinv = A + (long)i1 * ld + i1;
    GemmF32 panel{P, Dinv, P, ld, 1, 1, ld, ld, i1, NB, NB, 1.f, 0.f, 0, 0, 1, 0, 0, 0};
    int t2 = 0;
    GemmF32 g2 = panel;
    if (b + 1 <= B - 2) g2 = inv_second(b + 1, t2);  // row b+1: its T was produced in the previous launch
    hipLaunchKernelGGL(panel_inv_kernel, dim3(b + t2), dim3(256), gemmf32::SMEM_BYTES, st, panel, b, g2, t2);
    if ((rc = mq_check_launch()) != MQ_OK) return rc;
    GemmF32 trail{P, P, A, ld, 1, 1, ld, ld, i1, i1, NB, -1.f, 1.f, 1, 0, 1, 0, 0, 0};
    const int tiles = i1 / NB, total = tiles * (tiles + 1) / 2;
    int t1 = 0;
    GemmF32 g1 = trail;
    if (b <= B - 2) g1 = inv_first(b, t1);  // rows > b of the inverse are complete
    hipLaunchKernelGGL(trail_diag_kernel, dim3(total + t1), dim3(256), FUSED_SMEM, st, trail, total, g1, t1, INV_KC, A, ld,
                       i1, info);
    if ((rc = mq_check_launch()) != MQ_OK) return rc;
  }
  // what is left of the inverse once the elimination has reached the top: second product of row 1, both of row 0
  if (B >= 3) {
    int t2;
    GemmF32 g2 = inv_second(1, t2);
    if ((rc = mq_launch_gemm_f32(g2, st)) != MQ_OK) return rc;
  }
  if (B >= 2) {
    int t;
    GemmF32 g1 = inv_first(0, t);
    hipLaunchKernelGGL(inv_first_kernel, dim3(t), dim3(256), gemmf32::SMEM_BYTES, st, g1, INV_KC);
    if ((rc = mq_check_launch()) != MQ_OK) return rc;
    GemmF32 g2 = inv_second(0, t);
    if ((rc = mq_launch_gemm_f32(g2, st)) != MQ_OK) return rc;
  }
  hipLaunchKernelGGL(unit_diag_kernel, dim3(C), dim3(256), 0, st, A, ld, C, normalize, info);
  return mq_check_launch();
}
