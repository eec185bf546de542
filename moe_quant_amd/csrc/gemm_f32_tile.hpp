// Device-side body of the fp32 MFMA GEMM tile (128x128 per workgroup of 256 threads), shared by the
// plain GEMM kernel and by kernels that mix GEMM tiles with other work in one launch.
#pragma once
#include "common.hpp"

namespace gemmf32 {

constexpr int BM = 128, BN = 128, BK = 32;
// LDS staging layouts, chosen by how the operand lies in memory so that global float4 loads go to LDS as
// float4 stores, untransposed:
//   k-contiguous operand : [x][LDK]  (x = m or n), LDK = BK + 4; a lane fetches its 4 k-values with one b128 read
//   x-contiguous operand : [k][LDT],  LDT = 128 + 4;              a lane fetches them with four b32 reads
// A 32x32x2 MFMA sums two k-slots (lanes 0-31 and 32-63).  Which two k meet in one instruction is free as
// long as A and B agree: per group of 8 k, lane half h owns k = 4h..4h+3 and instruction t pairs (t, 4+t).
constexpr int LDK = BK + 4, LDT = BM + 4;
constexpr int STAGE = (BM * LDK > BK * LDT) ? BM * LDK : BK * LDT;  // floats per operand per stage
constexpr size_t SMEM_BYTES = (size_t)4 * STAGE * sizeof(float);    // 2 stages x {A, B}

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
  // interior tile: every element exists and every row is 16-byte aligned -> straight-line float4 loads
  __device__ __forceinline__ void load_fast(const float* __restrict__ p, long sx, long sk, int x0, int k0, int tid) {
#pragma unroll
    for (int it = 0; it < NV; ++it) {
      const int idx = tid + it * 256;
      const float* q;
      if (KCONTIG) q = p + (long)(x0 + idx / (BK / 4)) * sx + k0 + ((idx % (BK / 4)) << 2);
      else q = p + (long)(k0 + (idx >> 5)) * sk + x0 + ((idx & 31) << 2);
      // through the native vector type: a struct copy straight from memory left the loader in scratch
      const floatx4 v = *reinterpret_cast<const floatx4*>(q);
      r[it] = make_float4(v[0], v[1], v[2], v[3]);
    }
  }
  // r += the same tile of another array
  __device__ __forceinline__ void add_fast(const float* __restrict__ p, long sx, long sk, int x0, int k0, int tid) {
#pragma unroll
    for (int it = 0; it < NV; ++it) {
      const int idx = tid + it * 256;
      const float* q;
      if (KCONTIG) q = p + (long)(x0 + idx / (BK / 4)) * sx + k0 + ((idx % (BK / 4)) << 2);
      else q = p + (long)(k0 + (idx >> 5)) * sk + x0 + ((idx & 31) << 2);
      const floatx4 v = *reinterpret_cast<const floatx4*>(q);
      r[it].x += v[0];
      r[it].y += v[1];
      r[it].z += v[2];
      r[it].w += v[3];
    }
  }
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
        *reinterpret_cast<float4*>(&s[x * LDK + k]) = r[it];
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

// the four k-values (k = 8j + 4h + t, t = 0..3) of operand row x for this lane
template <bool KC>
__device__ __forceinline__ float4 frag4(const float* __restrict__ s, int x, int j, int h) {
  if (KC) return *reinterpret_cast<const float4*>(&s[x * LDK + 8 * j + 4 * h]);
  const float* q = s + (8 * j + 4 * h) * LDT + x;
  return make_float4(q[0], q[LDT], q[2 * LDT], q[3 * LDT]);
}

template <bool A_KC, bool B_KC, bool FAST, bool LDS_OUT, typename Sink>
__device__ __forceinline__ void tile_core(const GemmF32& g, int m0, int n0, int kb, int ke, const float* __restrict__ A,
                                          const float* __restrict__ B, float* C, float* smem, int vecA, int vecB,
                                          Sink& sink) {
  float* As = smem;
  float* Bs = smem + 2 * STAGE;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
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
  const int nsum = g.bsum ? min(g.bsum, (n0 / BN) / g.bsum_c + 1) : 1;  // arrays summed into the B operand
// (a macro, not a lambda: loaders captured by reference end up in scratch memory)
#define MQ_GEMM_FETCH(k0)                                       \
  do {                                                          \
    if (FAST) {                                                 \
      la.load_fast(A, g.sam, g.sak, m0, (k0), tid);             \
      lb.load_fast(B, g.sbn, g.sbk, n0, (k0), tid);             \
      for (int s_ = 1; s_ < nsum; ++s_) lb.add_fast(B + s_ * g.bsum_stride, g.sbn, g.sbk, n0, (k0), tid); \
    } else {                                                    \
      la.load(A, g.sam, g.sak, m0, g.M, (k0), ke, vecA, tid);   \
      lb.load(B, g.sbn, g.sbk, n0, g.N, (k0), ke, vecB, tid);   \
    }                                                           \
  } while (0)
  const float* Cold = g.Csrc ? g.Csrc + (C - g.C) : C;  // where the beta term is read from
  const long ldcold = g.Csrc ? g.ldcs : g.ldc;
  const int nk = (ke - kb + BK - 1) / BK;
  if (nk > 0) MQ_GEMM_FETCH(kb);
  // Interior tiles that go to memory move C sixteen bytes at a time, row-wise (a wavefront covers two rows of 512
  // bytes per instruction): the old tile is fetched that way here, and the result is turned from the MFMA layout
  // into that layout through LDS once the operand stages are no longer needed.
  constexpr bool ROWWISE_C = FAST && !LDS_OUT;
  constexpr int LDC_S = BN + 4;  // LDS row pitch of the result tile
  static_assert(BM * LDC_S <= 4 * STAGE, "result tile must fit in the operand stages");
  floatx4 cold4[ROWWISE_C ? 16 : 1];
  if (ROWWISE_C) {
    if (beta != 0.f) {
#pragma unroll
      for (int it = 0; it < 16; ++it) {
        const int idx = tid + it * 256;
        cold4[it] = *reinterpret_cast<const floatx4*>(Cold + (long)(m0 + (idx >> 5)) * ldcold + n0 + ((idx & 31) << 2));
      }
    }
  } else if (beta != 0.f) {
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int col = n0 + wn * 64 + j * 32 + lr;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int row = m0 + wm * 64 + i * 32 + 8 * (v >> 2) + 4 * lk + (v & 3);
          if (FAST || (row < g.M && col < g.N)) cold[i][j][v] = Cold[(long)row * ldcold + col];
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
    if (kt + 1 < nk) MQ_GEMM_FETCH(kb + (kt + 1) * BK);
    const float* as = As + cur * STAGE;
    const float* bs = Bs + cur * STAGE;
#pragma unroll
    for (int j = 0; j < BK / 8; ++j) {
      const float4 a0 = frag4<A_KC>(as, wm * 64 + lr, j, lk), a1 = frag4<A_KC>(as, wm * 64 + 32 + lr, j, lk);
      const float4 b0 = frag4<B_KC>(bs, wn * 64 + lr, j, lk), b1 = frag4<B_KC>(bs, wn * 64 + 32 + lr, j, lk);
      const float av0[4] = {a0.x, a0.y, a0.z, a0.w}, av1[4] = {a1.x, a1.y, a1.z, a1.w};
      const float bv0[4] = {b0.x, b0.y, b0.z, b0.w}, bv1[4] = {b1.x, b1.y, b1.z, b1.w};
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(av0[t], bv0[t], acc[0][0], 0, 0, 0);
        acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(av0[t], bv1[t], acc[0][1], 0, 0, 0);
        acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(av1[t], bv0[t], acc[1][0], 0, 0, 0);
        acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(av1[t], bv1[t], acc[1][1], 0, 0, 0);
      }
    }
    if (kt + 1 < nk) {
      la.store(As + (cur ^ 1) * STAGE, tid);
      lb.store(Bs + (cur ^ 1) * STAGE, tid);
    }
    __syncthreads();
  }

  if (ROWWISE_C) {
    float* cs = smem;  // the loop's last barrier has passed: no wavefront reads operands any more
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v)
          cs[(wm * 64 + i * 32 + 8 * (v >> 2) + 4 * lk + (v & 3)) * LDC_S + wn * 64 + j * 32 + lr] = acc[i][j][v];
    __syncthreads();
#pragma unroll
    for (int it = 0; it < 16; ++it) {
      const int idx = tid + it * 256, r = idx >> 5, c = (idx & 31) << 2;
      const floatx4 a4 = *reinterpret_cast<const floatx4*>(cs + r * LDC_S + c);
      floatx4 o;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float x = alpha * a4[e];
        if (beta != 0.f) x = fmaf(beta, cold4[it][e], x);
        o[e] = x;
      }
      *reinterpret_cast<floatx4*>(C + (long)(m0 + r) * g.ldc + n0 + c) = o;
    }
    return;
  }
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int col = n0 + wn * 64 + j * 32 + lr;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int row = m0 + wm * 64 + i * 32 + 8 * (v >> 2) + 4 * lk + (v & 3);
        if (FAST || (row < g.M && col < g.N)) {
          float r = alpha * acc[i][j][v];
          if (beta != 0.f) r = fmaf(beta, cold[i][j][v], r);
          if (LDS_OUT) sink(row - m0, col - n0, r);
          else C[(long)row * g.ldc + col] = r;
        }
      }
    }
#undef MQ_GEMM_FETCH
}

// =============================================================================================
// Interior tiles on the bf16 matrix cores.  Every fp32 operand element is split into three bf16 pieces,
// x = hi + mid + lo (hi = RN(x), mid = RN(x - hi), lo = RN(x - hi - mid); 24 significand bits in all), and the
// product is formed from the six piece products that matter, hi*hi + hi*mid + mid*hi + hi*lo + lo*hi + mid*mid,
// each exact in the fp32 accumulator of v_mfma_f32_32x32x16_bf16 (what is dropped is below 2^-23 of |a||b|).
// The bf16 pipe runs 16 times the fp32 one, so six products cost 0.4 of the fp32 MFMA time; against an fp64
// product the result is as close as the fp32 MFMA path's (1.6e-7 vs 2.0e-7 relative on random 512x512x128).
// BK = 16 per stage.  LDS per operand and stage, three planes:
//   k-contiguous operand : [k/8][x][8]   bf16, 4 KB a plane: a lane's MFMA fragment (8 k of one row) is one b128 read,
//                          lanes 0..31 read 512 contiguous bytes;
//   x-contiguous operand : [k][x] bf16 with 288-byte rows, 4.5 KB a plane: fragments come out of the transposing
//                          read ds_read_b64_tr_b16 (16 lanes fetch a 4 k x 16 x patch, each ends up with 4 k of its x).
// =============================================================================================
namespace split {
constexpr int SBK = 16;
constexpr int KPLANE = 4096, XROW = 288, XPLANE = SBK * XROW;
constexpr int OPB_MAX = 3 * XPLANE;
constexpr int STAGEB = 2 * OPB_MAX;
static_assert(2 * STAGEB <= (int)SMEM_BYTES, "two stages must fit in the fp32 core's LDS");
typedef __bf16 bf16x4v __attribute__((ext_vector_type(4)));
typedef short short4v __attribute__((ext_vector_type(4)));

typedef __bf16 bf16x2v __attribute__((ext_vector_type(2)));
typedef float float2v __attribute__((ext_vector_type(2)));
typedef unsigned uint2v __attribute__((ext_vector_type(2)));
// two floats -> two bf16 (round to nearest even) in one word: one v_cvt_pk_bf16_f32
__device__ __forceinline__ unsigned pk_bf16(float a, float b) {
  return __builtin_bit_cast(unsigned, __builtin_convertvector(float2v{a, b}, bf16x2v));
}
// v = hi + mid + lo, each a bf16 (four elements: two words per piece).  The rounded pieces are turned back
// into floats by a shift or a mask of the packed word: 11 instructions per pair of elements.
__device__ __forceinline__ void split3(const floatx4 v, uint2v& hi, uint2v& mid, uint2v& lo) {
#pragma unroll
  for (int p = 0; p < 2; ++p) {
    const unsigned h = pk_bf16(v[2 * p], v[2 * p + 1]);
    const float r0 = v[2 * p] - __uint_as_float(h << 16), r1 = v[2 * p + 1] - __uint_as_float(h & 0xffff0000u);
    const unsigned m = pk_bf16(r0, r1);
    const float s0 = r0 - __uint_as_float(m << 16), s1 = r1 - __uint_as_float(m & 0xffff0000u);
    hi[p] = h;
    mid[p] = m;
    lo[p] = pk_bf16(s0, s1);
  }
}

template <bool KC>
struct Loader {
  floatx4 r[2];
  // element (x, k) at p[x*sx + k*sk]; KC: sk == 1, else sx == 1.  X: the operand's extent along x; a tile that
  // sticks out past it fetches the last valid row (or quad of rows) again in place of what does not exist --
  // an address clamp, no branch -- and the caller never stores the results computed from those.
  __device__ __forceinline__ const float* addr(const float* p, long sx, long sk, int x0, int X, int k0, int it, int tid) const {
    const int idx = tid + it * 256;
    if (KC) return p + (long)min(x0 + (idx >> 2), X - 1) * sx + k0 + ((idx & 3) << 2);
    return p + (long)(k0 + (idx >> 5)) * sk + min(x0 + ((idx & 31) << 2), X - 4);
  }
  __device__ __forceinline__ void store(unsigned char* op, int tid) const {
#pragma unroll
    for (int it = 0; it < 2; ++it) {
      const int idx = tid + it * 256;
      uint2v hi, mid, lo;
      split3(r[it], hi, mid, lo);
      unsigned char* q;
      int plane;
      if (KC) {
        const int x = idx >> 2, k4 = (idx & 3) << 2;
        q = op + (k4 >> 3) * 2048 + x * 16 + (k4 & 7) * 2;
        plane = KPLANE;
      } else {
        const int k = idx >> 5, x4 = (idx & 31) << 2;
        q = op + k * XROW + x4 * 2;
        plane = XPLANE;
      }
      *reinterpret_cast<uint2v*>(q) = hi;
      *reinterpret_cast<uint2v*>(q + plane) = mid;
      *reinterpret_cast<uint2v*>(q + 2 * plane) = lo;
    }
  }
};

// the three planes of the fragment of rows xt..xt+31 for this lane (row xt + lane%32, k = 8*(lane/32)..+7)
template <bool KC>
__device__ __forceinline__ void frag(const unsigned char* op, int xt, int lane, bf16x8n (&f)[3]) {
  if (KC) {
    const unsigned char* q = op + (lane >> 5) * 2048 + (xt + (lane & 31)) * 16;
#pragma unroll
    for (int p = 0; p < 3; ++p) f[p] = *reinterpret_cast<const bf16x8n*>(q + p * KPLANE);
  } else {
    const int L = lane & 15;
    const unsigned char* q = op + (8 * (lane >> 5) + (L >> 2)) * XROW + (xt + 16 * ((lane >> 4) & 1) + 4 * (L & 3)) * 2;
#pragma unroll
    for (int p = 0; p < 3; ++p) {
      const short4v a = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
          (short4v __attribute__((address_space(3)))*)(q + p * XPLANE));
      const short4v b = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
          (short4v __attribute__((address_space(3)))*)(q + p * XPLANE + 4 * XROW));
      f[p] = __builtin_bit_cast(bf16x8n, __builtin_shufflevector(a, b, 0, 1, 2, 3, 4, 5, 6, 7));
    }
  }
}
}  // namespace split

template <bool A_KC, bool B_KC>
__device__ __forceinline__ void tile_core_split(const GemmF32& g, int m0, int n0, int kb, int ke, const float* __restrict__ A,
                                                const float* __restrict__ B, float* C, float* smem_f) {
  using namespace split;
  unsigned char* smem = reinterpret_cast<unsigned char*>(smem_f);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1, lr = lane & 31, lk = lane >> 5;
  const float alpha = g.alpha, beta = g.beta;
  floatx16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
  // Operand tiles travel memory -> registers -> LDS.  A 16-k step is 768 MFMA cycles per wavefront, a memory
  // round trip under load several times that: the registers hold the next two steps, so a step's loads have
  // two steps of products to arrive in.
  Loader<A_KC> la[2];
  Loader<B_KC> lb[2];
  const float* Cold = g.Csrc ? g.Csrc + (C - g.C) : C;
  const long ldcold = g.Csrc ? g.ldcs : g.ldc;
  const int nk = (ke - kb) / SBK;
  // Where the next step to fetch lies, kept in registers of their own and moved on by a wave-uniform stride:
  // address arithmetic in temporaries tempts the register allocator to compute it in the registers a load
  // still in flight will write, and the hazard costs a wait for every load.  Past the last step the pointers
  // stay (the last step is fetched again and never used): no branch around a load, at whose join the
  // compiler would wait for all of them as well.
  const float* qa[2];
  const float* qb[2];
#pragma unroll
  for (int it = 0; it < 2; ++it) {
    qa[it] = la[0].addr(A, g.sam, g.sak, m0, g.M, kb, it, tid);
    qb[it] = lb[0].addr(B, g.sbn, g.sbk, n0, g.N, kb, it, tid);
  }
  const long inca = (long)SBK * g.sak, incb = (long)SBK * g.sbk;
  int fetched = 0;  // steps fetched so far
  auto fetch = [&](Loader<A_KC>& xa, Loader<B_KC>& xb) {
#pragma unroll
    for (int it = 0; it < 2; ++it) {
      xa.r[it] = *reinterpret_cast<const floatx4*>(qa[it]);
      xb.r[it] = *reinterpret_cast<const floatx4*>(qb[it]);
    }
    ++fetched;
    const long ia = fetched < nk ? inca : 0, ib = fetched < nk ? incb : 0;
#pragma unroll
    for (int it = 0; it < 2; ++it) {
      qa[it] += ia;
      qb[it] += ib;
    }
  };
  if (nk > 0) {
    fetch(la[0], lb[0]);
    fetch(la[1], lb[1]);
  }
  constexpr int LDC_S = BN + 4;
  floatx4 cold4[16];
  if (beta != 0.f) {
#pragma unroll
    for (int it = 0; it < 16; ++it) {
      const int idx = tid + it * 256;
      cold4[it] = *reinterpret_cast<const floatx4*>(Cold + (long)min(m0 + (idx >> 5), g.M - 1) * ldcold +
                                                    min(n0 + ((idx & 31) << 2), g.N - 4));
    }
  }
  if (nk > 0) {
    la[0].store(smem, tid);
    lb[0].store(smem + OPB_MAX, tid);
  }
  __syncthreads();
  // step kt: LDS stage kt%2 holds its operands, `nxt` those of step kt+1 (in flight), `fre` is free
  auto step = [&](int kt, Loader<A_KC>& fa_free, Loader<B_KC>& fb_free, Loader<A_KC>& fa_next, Loader<B_KC>& fb_next) {
    const int cur = kt & 1;
    fetch(fa_free, fb_free);  // step kt + 2
    const unsigned char* as = smem + cur * STAGEB;
    const unsigned char* bs = as + OPB_MAX;
    bf16x8n fa[2][3], fb[2][3];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      frag<A_KC>(as, wm * 64 + i * 32, lane, fa[i]);
      frag<B_KC>(bs, wn * 64 + i * 32, lane, fb[i]);
    }
    // small terms first; the four accumulators take turns, so consecutive instructions never depend on each other
    constexpr int PA[6] = {1, 0, 2, 0, 1, 0}, PB[6] = {1, 2, 0, 1, 0, 0};
#pragma unroll
    for (int t = 0; t < 6; ++t)
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i][PA[t]], fb[j][PB[t]], acc[i][j], 0, 0, 0);
    // (no branch here either: after the last step this writes a stage nobody reads, and the whole step stays
    // one block of code in which the conversions can be scheduled between the matrix instructions)
    fa_next.store(smem + (cur ^ 1) * STAGEB, tid);
    fb_next.store(smem + (cur ^ 1) * STAGEB + OPB_MAX, tid);
    __syncthreads();
  };
  for (int kt = 0; kt < nk; kt += 2) {
    step(kt, la[0], lb[0], la[1], lb[1]);
    if (kt + 1 < nk) step(kt + 1, la[1], lb[1], la[0], lb[0]);
  }
  float* cs = smem_f;  // the loop's last barrier has passed: no wavefront reads operands any more
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v)
        cs[(wm * 64 + i * 32 + 8 * (v >> 2) + 4 * lk + (v & 3)) * LDC_S + wn * 64 + j * 32 + lr] = acc[i][j][v];
  __syncthreads();
#pragma unroll
  for (int it = 0; it < 16; ++it) {
    const int idx = tid + it * 256, r = idx >> 5, c = (idx & 31) << 2;
    const floatx4 a4 = *reinterpret_cast<const floatx4*>(cs + r * LDC_S + c);
    floatx4 o;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      float x = alpha * a4[e];
      if (beta != 0.f) x = fmaf(beta, cold4[it][e], x);
      o[e] = x;
    }
    if (m0 + r < g.M && n0 + c < g.N) *reinterpret_cast<floatx4*>(C + (long)(m0 + r) * g.ldc + n0 + c) = o;
  }
}

// A 64 x (64 NH) output tile with K = 128, both operands K-contiguous, beta == 0: for launches of a few
// short products, which are nothing but latency (the core above waits one memory round trip per 16 k, and
// a 128x128 tile keeps one CU busy where several could share the work).  All of K is requested at once;
// the arrays of a summed B operand are fetched eight at a time.  Operands pass through LDS in two halves of
// 64 k (short_smem_bytes(NH)).  Same piece products, same k order and same order of additions as the core
// above: the results are the same bits.
// The tile reads all of its A rows before it writes any of C: with NH = 2 and N == 128 a product may
// overwrite its own A operand (C == A), since no other tile touches those rows.
constexpr int SHORT_K = 128;
constexpr size_t short_smem_bytes(int nh) { return (size_t)4 * 3 * 2048 * (1 + nh); }
template <int NH>
__device__ __forceinline__ void tile_short(const GemmF32& g, int m0, int n0, float* smem_f) {
  using namespace split;
  constexpr int PLA = 2048, PLB = 2048 * NH;  // plane: 64 (A) or 64 NH (B) rows x 16 k of bf16
  constexpr int OPA = 3 * PLA, STG = OPA + 3 * PLB;
  unsigned char* smem = reinterpret_cast<unsigned char*>(smem_f);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1, lr = lane & 31, lk = lane >> 5;
  const float* __restrict__ A = g.A;
  const float* __restrict__ B = g.B;
  const int nsum = g.bsum ? min(g.bsum, (n0 / BN) / g.bsum_c + 1) : 1;
  // thread -> (row x, four k) of a 64-k half: idx = tid + 256 it, x = idx / 16, k = 4 (idx % 16)
  floatx4 ra[2][4], rb[2][4 * NH];
#pragma unroll
  for (int h = 0; h < 2; ++h) {
#pragma unroll
    for (int it = 0; it < 4; ++it) {
      const int idx = tid + it * 256, x = idx >> 4, k = 64 * h + ((idx & 15) << 2);
      ra[h][it] = *reinterpret_cast<const floatx4*>(A + (long)(m0 + x) * g.sam + k);
    }
#pragma unroll
    for (int it = 0; it < 4 * NH; ++it) {
      const int idx = tid + it * 256, x = idx >> 4, k = 64 * h + ((idx & 15) << 2);
      rb[h][it] = *reinterpret_cast<const floatx4*>(B + (long)(n0 + x) * g.sbn + k);
    }
  }
  constexpr int R = 8 / NH;
  for (int s0 = 1; s0 < nsum; s0 += R) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      floatx4 t[R][4 * NH];
#pragma unroll
      for (int u = 0; u < R; ++u) {
        const float* Bu = B + (long)min(s0 + u, nsum - 1) * g.bsum_stride;  // past the last: re-read, dropped below
#pragma unroll
        for (int it = 0; it < 4 * NH; ++it) {
          const int idx = tid + it * 256, x = idx >> 4, k = 64 * h + ((idx & 15) << 2);
          t[u][it] = *reinterpret_cast<const floatx4*>(Bu + (long)(n0 + x) * g.sbn + k);
        }
      }
#pragma unroll
      for (int u = 0; u < R; ++u)
#pragma unroll
        for (int it = 0; it < 4 * NH; ++it)
          if (s0 + u < nsum) rb[h][it] += t[u][it];
    }
  }
  floatx16 acc[NH];
#pragma unroll
  for (int j = 0; j < NH; ++j)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[j][v] = 0.f;
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    if (h) __syncthreads();  // every wavefront has read the first half
#pragma unroll
    for (int it = 0; it < 4 * (1 + NH); ++it) {
      const bool isb = it >= 4;
      const int idx = tid + (isb ? it - 4 : it) * 256, x = idx >> 4, k4 = (idx & 15) << 2;
      unsigned char* q = smem + (k4 >> 4) * STG + (isb ? OPA : 0) + ((k4 & 15) >> 3) * (isb ? 1024 * NH : 1024) + x * 16 +
                         (k4 & 7) * 2;
      const int plane = isb ? PLB : PLA;
      uint2v hi, mid, lo;
      split3(isb ? rb[h][it - 4] : ra[h][it], hi, mid, lo);
      *reinterpret_cast<uint2v*>(q) = hi;
      *reinterpret_cast<uint2v*>(q + plane) = mid;
      *reinterpret_cast<uint2v*>(q + 2 * plane) = lo;
    }
    __syncthreads();
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const unsigned char* as = smem + s * STG + lk * 1024 + (wm * 32 + lr) * 16;
      const unsigned char* bs = smem + s * STG + OPA + lk * (1024 * NH) + (wn * 32 * NH + lr) * 16;
      bf16x8n fa[3], fb[NH][3];
#pragma unroll
      for (int p = 0; p < 3; ++p) {
        fa[p] = *reinterpret_cast<const bf16x8n*>(as + p * PLA);
#pragma unroll
        for (int j = 0; j < NH; ++j) fb[j][p] = *reinterpret_cast<const bf16x8n*>(bs + p * PLB + j * 32 * 16);
      }
      constexpr int PA[6] = {1, 0, 2, 0, 1, 0}, PB[6] = {1, 2, 0, 1, 0, 0};
#pragma unroll
      for (int t = 0; t < 6; ++t)
#pragma unroll
        for (int j = 0; j < NH; ++j)
          acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[PA[t]], fb[j][PB[t]], acc[j], 0, 0, 0);
    }
  }
  __syncthreads();
  constexpr int LDC_S = 64 * NH + 4;
  float* cs = smem_f;
#pragma unroll
  for (int j = 0; j < NH; ++j)
#pragma unroll
    for (int v = 0; v < 16; ++v)
      cs[(wm * 32 + 8 * (v >> 2) + 4 * lk + (v & 3)) * LDC_S + wn * 32 * NH + j * 32 + lr] = acc[j][v];
  __syncthreads();
  const float alpha = g.alpha;
#pragma unroll
  for (int it = 0; it < 4 * NH; ++it) {
    const int idx = tid + it * 256, r = idx / (16 * NH), c = (idx % (16 * NH)) << 2;
    floatx4 o = *reinterpret_cast<const floatx4*>(cs + r * LDC_S + c);
#pragma unroll
    for (int e = 0; e < 4; ++e) o[e] = alpha * o[e];
    *reinterpret_cast<floatx4*>(g.C + (long)(m0 + r) * g.ldc + n0 + c) = o;
  }
}

// One 128x128 output tile (tm, tn) of problem g (batch index z).  smem: SMEM_BYTES of LDS.
// The old C tile is fetched before the K loop (when beta != 0) so its latency hides behind the products;
// it is added after the accumulation, never fed through the accumulator.
// Interior tiles (whole tile inside the matrix, aligned rows, K range a multiple of BK) run a copy of the
// body without any bounds test: guarded loads sit in branches, and a branch makes the wavefront wait for
// every load in flight.
// With LDS_OUT the result tile is not written to memory: it is handed to `sink(r, c, value)` (tile-local
// coordinates) after the last LDS operand read, so the sink may overwrite the staging buffers.
template <bool A_KC, bool B_KC, bool LDS_OUT = false, typename Sink = NoSink>
__device__ __forceinline__ void tile_body(const GemmF32& g, int tm, int tn, int z, float* smem, int vecA, int vecB,
                                          Sink sink = Sink()) {
  const float* __restrict__ A = g.A + (long)z * g.batchA;
  const float* __restrict__ B = g.B + (long)z * g.batchB;
  float* C = g.C + (long)z * g.batchC;
  const int m0 = tm * BM, n0 = tn * BN;
  int kb = 0, ke = g.K;
  if (g.ktrim == 1) ke = min(g.K, m0 + BM);
  if (g.ktrim == 2) kb = m0;
  const bool c_vec = LDS_OUT || ((((uintptr_t)C) & 15) == 0 && (g.ldc & 3) == 0 &&  // C moves 16 bytes at a time
                                 (!g.Csrc || ((((uintptr_t)g.Csrc) & 15) == 0 && (g.ldcs & 3) == 0)));
  const bool inside = vecA && vecB && c_vec && m0 + BM <= g.M && n0 + BN <= g.N;
  // a tile that sticks out of the matrix still takes the fast path when whole quads of rows and columns exist (its
  // loads clamp their addresses, its stores are masked): K-contiguous operands need nothing, the others and C move
  // four elements of M or N at a time
  const bool quads = vecA && vecB && c_vec && g.M >= 4 && g.N >= 4 && (g.N & 3) == 0 && (A_KC || (g.M & 3) == 0);
  if (!LDS_OUT && !g.fp32_mfma && !g.bsum && (inside || quads) && ((ke - kb) % split::SBK == 0)) {
    tile_core_split<A_KC, B_KC>(g, m0, n0, kb, ke, A, B, C, smem);
    return;
  }
  const bool interior = inside && ((ke - kb) % BK == 0);
  if (interior) tile_core<A_KC, B_KC, true, LDS_OUT, Sink>(g, m0, n0, kb, ke, A, B, C, smem, vecA, vecB, sink);
  else tile_core<A_KC, B_KC, false, LDS_OUT, Sink>(g, m0, n0, kb, ke, A, B, C, smem, vecA, vecB, sink);
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
