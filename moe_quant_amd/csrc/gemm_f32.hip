// fp32 MFMA GEMM for gfx950: 128x128 workgroup tile, four wave64 each owning 64x64
// (2x2 blocks of v_mfma_f32_32x32x2_f32), operands staged through LDS as [k][m] / [k][n]
// so every fragment read is a conflict-free ds_read_b32 whatever the global layout was.
// Used by the factorisation (trailing update, panel solve, triangular inverse) and by the
// GPTQ lazy-batch trailing update.
#include "common.hpp"

namespace {

constexpr int BM = 128, BN = 128, BK = 16, LDT = 132;  // LDT: padded LDS row length (floats)

// Workgroups are handed to the 8 XCDs round-robin by linear id; give every XCD one contiguous
// run of tiles so that tiles sharing operand panels meet in the same L2.
__device__ __forceinline__ int xcd_remap(int bid, int total) {
  const int q = total >> 3, rem = total & 7;
  const int xcd = bid & 7, idx = bid >> 3;
  return xcd * q + (xcd < rem ? xcd : rem) + idx;
}

// linear index over the upper block triangle, column by column: L = tn(tn+1)/2 + tm, tm <= tn
__device__ __forceinline__ void tri_decode(int L, int& tm, int& tn) {
  int c = (int)((__fsqrt_rn(8.0f * (float)L + 1.0f) - 1.0f) * 0.5f);
  while (c * (c + 1) / 2 > L) --c;
  while ((c + 1) * (c + 2) / 2 <= L) ++c;
  tn = c;
  tm = L - c * (c + 1) / 2;
}

template <bool KCONTIG>
struct TileLoader {
  // Loads a (128 x BK) operand tile: element (x, k) at p[x*sx + k*sk], x in [x0, x0+128), k in [k0, k0+BK).
  float4 r[2];
  __device__ __forceinline__ void load(const float* __restrict__ p, long sx, long sk, int x0, int X, int k0, int Kend,
                                       bool vec_ok, int tid) {
#pragma unroll
    for (int it = 0; it < 2; ++it) {
      const int idx = tid + it * 256;
      int x, k;
      if (KCONTIG) {
        x = idx >> 2;
        k = (idx & 3) << 2;
      } else {
        k = idx >> 5;
        x = (idx & 31) << 2;
      }
      const int gx = x0 + x, gk = k0 + k;
      float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
      if (KCONTIG) {
        if (gx < X) {
          const float* q = p + (long)gx * sx + gk;
          if (vec_ok && gk + 3 < Kend) {
            v = *reinterpret_cast<const float4*>(q);
          } else {
            if (gk + 0 < Kend) v.x = q[0];
            if (gk + 1 < Kend) v.y = q[1];
            if (gk + 2 < Kend) v.z = q[2];
            if (gk + 3 < Kend) v.w = q[3];
          }
        }
      } else {
        if (gk < Kend) {
          const float* q = p + (long)gk * sk + gx;
          if (vec_ok && gx + 3 < X) {
            v = *reinterpret_cast<const float4*>(q);
          } else {
            if (gx + 0 < X) v.x = q[0];
            if (gx + 1 < X) v.y = q[1];
            if (gx + 2 < X) v.z = q[2];
            if (gx + 3 < X) v.w = q[3];
          }
        }
      }
      r[it] = v;
    }
  }
  __device__ __forceinline__ void store(float* __restrict__ s, int tid) const {
#pragma unroll
    for (int it = 0; it < 2; ++it) {
      const int idx = tid + it * 256;
      if (KCONTIG) {
        const int x = idx >> 2, k = (idx & 3) << 2;
        s[(k + 0) * LDT + x] = r[it].x;
        s[(k + 1) * LDT + x] = r[it].y;
        s[(k + 2) * LDT + x] = r[it].z;
        s[(k + 3) * LDT + x] = r[it].w;
      } else {
        const int k = idx >> 5, x = (idx & 31) << 2;
        *reinterpret_cast<float4*>(&s[k * LDT + x]) = r[it];
      }
    }
  }
};

template <bool A_KC, bool B_KC>
__global__ __launch_bounds__(256) void gemm_f32_kernel(GemmF32 g, int tiles_m, int tiles_n, int total, int vecA,
                                                      int vecB) {
  __shared__ __attribute__((aligned(16))) float As[2][BK * LDT];
  __shared__ __attribute__((aligned(16))) float Bs[2][BK * LDT];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  int tm, tn;
  {
    const int L = xcd_remap(blockIdx.x, total);
    if (g.tri) {
      tri_decode(L, tm, tn);
    } else {
      tm = L / tiles_n;
      tn = L - tm * tiles_n;
    }
  }
  const float* __restrict__ A = g.A + (long)blockIdx.z * g.batchA;
  const float* __restrict__ B = g.B + (long)blockIdx.z * g.batchB;
  float* C = g.C + (long)blockIdx.z * g.batchC;
  const int m0 = tm * BM, n0 = tn * BN;
  int kb = 0, ke = g.K;
  if (g.ktrim == 1) ke = min(g.K, m0 + BM);
  if (g.ktrim == 2) kb = m0;

  floatx16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  TileLoader<A_KC> la;
  TileLoader<B_KC> lb;
  const int nk = (ke - kb + BK - 1) / BK;
  if (nk > 0) {
    la.load(A, g.sam, g.sak, m0, g.M, kb, ke, vecA, tid);
    lb.load(B, g.sbn, g.sbk, n0, g.N, kb, ke, vecB, tid);
    la.store(As[0], tid);
    lb.store(Bs[0], tid);
  }
  __syncthreads();
  const int lr = lane & 31, lk = lane >> 5;
  for (int kt = 0; kt < nk; ++kt) {
    const int cur = kt & 1;
    if (kt + 1 < nk) {
      la.load(A, g.sam, g.sak, m0, g.M, kb + (kt + 1) * BK, ke, vecA, tid);
      lb.load(B, g.sbn, g.sbk, n0, g.N, kb + (kt + 1) * BK, ke, vecB, tid);
    }
    const float* as = As[cur] + wm * 64 + lr;
    const float* bs = Bs[cur] + wn * 64 + lr;
#pragma unroll
    for (int kp = 0; kp < BK / 2; ++kp) {
      const int k = 2 * kp + lk;
      const float a0 = as[k * LDT], a1 = as[k * LDT + 32];
      const float b0 = bs[k * LDT], b1 = bs[k * LDT + 32];
      acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b0, acc[0][0], 0, 0, 0);
      acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b1, acc[0][1], 0, 0, 0);
      acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b0, acc[1][0], 0, 0, 0);
      acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b1, acc[1][1], 0, 0, 0);
    }
    if (kt + 1 < nk) {
      la.store(As[cur ^ 1], tid);
      lb.store(Bs[cur ^ 1], tid);
    }
    __syncthreads();
  }

  const float alpha = g.alpha, beta = g.beta;
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int col = n0 + wn * 64 + j * 32 + lr;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int row = m0 + wm * 64 + i * 32 + 8 * (v >> 2) + 4 * lk + (v & 3);
        if (row < g.M && col < g.N) {
          float* c = C + (long)row * g.ldc + col;
          float r = alpha * acc[i][j][v];
          if (beta != 0.f) r = fmaf(beta, *c, r);
          *c = r;
        }
      }
    }
}

}  // namespace

int mq_launch_gemm_f32(const GemmF32& g, hipStream_t stream) {
  if (g.M <= 0 || g.N <= 0 || g.batch <= 0) return MQ_OK;
  if (!g.A || !g.B || !g.C) return MQ_ERR_ARG;
  const bool a_kc = (g.sak == 1), b_kc = (g.sbk == 1);
  if (!a_kc && g.sam != 1) return MQ_ERR_ARG;
  if (!b_kc && g.sbn != 1) return MQ_ERR_ARG;
  if (g.tri && g.M != g.N) return MQ_ERR_ARG;
  const int tiles_m = (g.M + BM - 1) / BM, tiles_n = (g.N + BN - 1) / BN;
  const int total = g.tri ? tiles_m * (tiles_m + 1) / 2 : tiles_m * tiles_n;
  auto aligned = [](const float* p, long ld, long batch) {
    return ((uintptr_t)p % 16 == 0) && (ld % 4 == 0) && (batch % 4 == 0);
  };
  const int vecA = aligned(g.A, a_kc ? g.sam : g.sak, g.batchA);
  const int vecB = aligned(g.B, b_kc ? g.sbn : g.sbk, g.batchB);
  dim3 grid(total, 1, g.batch), block(256);
  if (a_kc && b_kc)
    hipLaunchKernelGGL((gemm_f32_kernel<true, true>), grid, block, 0, stream, g, tiles_m, tiles_n, total, vecA, vecB);
  else if (a_kc && !b_kc)
    hipLaunchKernelGGL((gemm_f32_kernel<true, false>), grid, block, 0, stream, g, tiles_m, tiles_n, total, vecA, vecB);
  else if (!a_kc && b_kc)
    hipLaunchKernelGGL((gemm_f32_kernel<false, true>), grid, block, 0, stream, g, tiles_m, tiles_n, total, vecA, vecB);
  else
    hipLaunchKernelGGL((gemm_f32_kernel<false, false>), grid, block, 0, stream, g, tiles_m, tiles_n, total, vecA, vecB);
  return mq_check_launch();
}

// Test hook: plain GEMM through the C ABI so the MFMA core can be checked on its own.
extern "C" int mq_gemm_f32(const float* A, long sam, long sak, const float* B, long sbk, long sbn, float* C, long ldc,
                           int M, int N, int K, float alpha, float beta, int tri, int ktrim, void* stream) {
  GemmF32 g{A, B, C, sam, sak, sbk, sbn, ldc, M, N, K, alpha, beta, tri, ktrim, 1, 0, 0, 0};
  return mq_launch_gemm_f32(g, (hipStream_t)stream);
}
