// Device-side body of the fp32 MFMA GEMM tile (128x128 per workgroup of 256 threads), shared by the
// plain GEMM kernel and by kernels that mix GEMM tiles with other work in one launch.
#pragma once
#include "common.hpp"

namespace gemmf32 {

constexpr int BM = 128, BN = 128, BK = 32, LDT = 132;  // LDT: padded LDS row length (floats)
constexpr int STAGE = BK * LDT;                        // floats per operand per stage
constexpr size_t SMEM_BYTES = (size_t)4 * STAGE * sizeof(float);  // 2 stages x {A, B}

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
  static constexpr int NV = BM * BK / 4 / 256;  // float4 per thread
  float4 r[NV];
  __device__ __forceinline__ void load(const float* __restrict__ p, long sx, long sk, int x0, int X, int k0, int Kend,
                                       bool vec_ok, int tid) {
#pragma unroll
    for (int it = 0; it < NV; ++it) {
      const int idx = tid + it * 256;
      int x, k;
      if (KCONTIG) {
        x = idx / (BK / 4);
        k = (idx % (BK / 4)) << 2;
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
    for (int it = 0; it < NV; ++it) {
      const int idx = tid + it * 256;
      if (KCONTIG) {
        const int x = idx / (BK / 4), k = (idx % (BK / 4)) << 2;
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

// One 128x128 output tile (tm, tn) of problem g (batch index z).  smem: SMEM_BYTES of LDS.
// The old C tile is fetched before the K loop (when beta != 0) so its latency hides behind the products;
// it is added after the accumulation, never fed through the accumulator.
// With LDS_OUT the result tile is not written to memory: it is handed to `sink(r, c, value)` (tile-local
// coordinates) after the last LDS operand read, so the sink may overwrite the staging buffers.
struct NoSink {
  __device__ __forceinline__ void operator()(int, int, float) const {}
};
template <bool A_KC, bool B_KC, bool LDS_OUT = false, typename Sink = NoSink>
__device__ __forceinline__ void tile_body(const GemmF32& g, int tm, int tn, int z, float* smem, int vecA, int vecB,
                                          Sink sink = Sink()) {
  float* As = smem;
  float* Bs = smem + 2 * STAGE;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const float* __restrict__ A = g.A + (long)z * g.batchA;
  const float* __restrict__ B = g.B + (long)z * g.batchB;
  float* C = g.C + (long)z * g.batchC;
  const int m0 = tm * BM, n0 = tn * BN;
  int kb = 0, ke = g.K;
  if (g.ktrim == 1) ke = min(g.K, m0 + BM);
  if (g.ktrim == 2) kb = m0;
  const int lr = lane & 31, lk = lane >> 5;
  const float alpha = g.alpha, beta = g.beta;

  floatx16 acc[2][2], cold[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        acc[i][j][v] = 0.f;
        cold[i][j][v] = 0.f;
      }

  TileLoader<A_KC> la;
  TileLoader<B_KC> lb;
  const int nk = (ke - kb + BK - 1) / BK;
  if (nk > 0) {
    la.load(A, g.sam, g.sak, m0, g.M, kb, ke, vecA, tid);
    lb.load(B, g.sbn, g.sbk, n0, g.N, kb, ke, vecB, tid);
  }
  if (beta != 0.f) {
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int col = n0 + wn * 64 + j * 32 + lr;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int row = m0 + wm * 64 + i * 32 + 8 * (v >> 2) + 4 * lk + (v & 3);
          if (row < g.M && col < g.N) cold[i][j][v] = C[(long)row * g.ldc + col];
        }
      }
  }
  if (nk > 0) {
    la.store(As, tid);
    lb.store(Bs, tid);
  }
  __syncthreads();
  for (int kt = 0; kt < nk; ++kt) {
    const int cur = kt & 1;
    if (kt + 1 < nk) {
      la.load(A, g.sam, g.sak, m0, g.M, kb + (kt + 1) * BK, ke, vecA, tid);
      lb.load(B, g.sbn, g.sbk, n0, g.N, kb + (kt + 1) * BK, ke, vecB, tid);
    }
    const float* as = As + cur * STAGE + wm * 64 + lr;
    const float* bs = Bs + cur * STAGE + wn * 64 + lr;
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
      la.store(As + (cur ^ 1) * STAGE, tid);
      lb.store(Bs + (cur ^ 1) * STAGE, tid);
    }
    __syncthreads();
  }

#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int col = n0 + wn * 64 + j * 32 + lr;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int row = m0 + wm * 64 + i * 32 + 8 * (v >> 2) + 4 * lk + (v & 3);
        if (row < g.M && col < g.N) {
          float r = alpha * acc[i][j][v];
          if (beta != 0.f) r = fmaf(beta, cold[i][j][v], r);
          if (LDS_OUT) sink(row - m0, col - n0, r);
          else C[(long)row * g.ldc + col] = r;
        }
      }
    }
}

__device__ __forceinline__ void decode_tile(const GemmF32& g, int L, int tiles_n, int& tm, int& tn) {
  if (g.tri) {
    tri_decode(L, tm, tn);
  } else {
    tm = L / tiles_n;
    tn = L - tm * tiles_n;
  }
}

}  // namespace gemmf32
