// HBM-bound helpers around the column loop: group scales, transposed fp32 weights, code
// transposition and int4 -> int32 packing.  All streaming kernels; lanes always run along the
// contiguous dimension of whatever they read or write, transposes go through LDS.
#include <hip/hip_fp16.h>

#include "common.hpp"

namespace {

enum { DT_F32 = 0, DT_BF16 = 1, DT_F16 = 2 };

__device__ __forceinline__ float load_as_f32(const void* p, long idx, int dt) {
  if (dt == DT_BF16) return bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(p)[idx]);
  if (dt == DT_F16) return __half2float(reinterpret_cast<const __half*>(p)[idx]);
  return reinterpret_cast<const float*>(p)[idx];
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
  return v;
}

// ---------------------------------------------------------------------------------------------
// Symmetric group scales: one wavefront per (row, group).
//   scale = round_to(dtype)( (2/maxq as fp32) * max|w| + 1e-12 )
// written compact (R,G) and, optionally, transposed (G,R) for the column loop.
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void grid_sym_kernel(const void* __restrict__ W, int wdt, long ldw, int R, int C, int g,
                                                       int G, const uint8_t* __restrict__ dead, float two_over_maxq,
                                                       int round_dt, float* __restrict__ scale_rg,
                                                       float* __restrict__ scale_gr) {
  const int lane = threadIdx.x & 63;
  const long item = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (item >= (long)R * G) return;
  const int row = (int)(item / G), grp = (int)(item - (long)row * G);
  const int c0 = grp * g, c1 = min(C, c0 + g);
  float m = 0.f;
  for (int c = c0 + lane; c < c1; c += 64) {
    float v = load_as_f32(W, (long)row * ldw + c, wdt);
    if (dead && dead[c]) v = 0.f;
    m = fmaxf(m, fabsf(v));
  }
  m = wave_max(m);
  if (lane == 0) {
    float s = two_over_maxq * m;
    s = s + 1e-12f;
    if (round_dt == DT_BF16) s = round_to_bf16(s);
    if (round_dt == DT_F16) s = __half2float(__float2half_rn(s));
    scale_rg[(long)row * G + grp] = s;
    if (scale_gr) scale_gr[(long)grp * R + row] = s;
  }
}

// The same for bf16 weights in 16-byte-aligned rows and power-of-two groups of 32..512: a lane takes 8 consecutive
// weights per 16-byte load, a group is g/8 neighbouring lanes, and a wavefront issues four such loads (2048 columns
// of one row) before it reduces anything: 14x fewer wavefronts, four loads in flight in each.
__global__ __launch_bounds__(256) void grid_sym_vec_kernel(const uint16_t* __restrict__ W, long ldw, int R, int C, int g,
                                                           int G, const uint8_t* __restrict__ dead, float two_over_maxq,
                                                           int round_dt, float* __restrict__ scale_rg,
                                                           float* __restrict__ scale_gr, int spans) {
  const int lane = threadIdx.x & 63;
  const long item = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (item >= (long)R * spans) return;
  const int row = (int)(item / spans), sp = (int)(item - (long)row * spans);
  uint4 v[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int col = sp * 2048 + i * 512 + lane * 8;
    v[i] = col < C ? *reinterpret_cast<const uint4*>(W + (long)row * ldw + col) : make_uint4(0, 0, 0, 0);
  }
  const int L = g >> 3;  // lanes per group
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int col = sp * 2048 + i * 512 + lane * 8;
    const unsigned wds[4] = {v[i].x, v[i].y, v[i].z, v[i].w};
    float m = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const unsigned bits = (e & 1) ? (wds[e >> 1] & 0xffff0000u) : (wds[e >> 1] << 16);
      float a = fabsf(__uint_as_float(bits));
      if (dead && col < C && dead[col + e]) a = 0.f;
      m = fmaxf(m, a);
    }
    for (int off = L >> 1; off > 0; off >>= 1) m = fmaxf(m, __shfl_xor(m, off, 64));
    if ((lane & (L - 1)) == 0 && col < C) {
      const int grp = col / g;
      float s = two_over_maxq * m;
      s = s + 1e-12f;
      if (round_dt == DT_BF16) s = round_to_bf16(s);
      if (round_dt == DT_F16) s = __half2float(__float2half_rn(s));
      scale_rg[(long)row * G + grp] = s;
      if (scale_gr) scale_gr[(long)grp * R + row] = s;
    }
  }
}

// ---------------------------------------------------------------------------------------------
// Scale search: for every (row, group) try the shrunken scales round(s0 * p_i) and keep the one whose
// quantize-dequantize error sum |dq - x|^norm is smallest, the last one among equals.
// One wavefront per group, one LANE PER CANDIDATE (up to 4 per lane): the group's weights are handed round as
// wave-uniform values (v_readlane), every lane runs the quantizer of the column loop on them for its own
// candidate scales and keeps its own running sums, so no reduction is needed until the final arg-min.
// |d|^norm = exp2(norm * log2|d|), which is 0 for d = 0 like the reference's exp(log|d| * norm).
// ---------------------------------------------------------------------------------------------
constexpr int MSE_NC = 4;  // candidates per lane: P <= 256

__device__ __forceinline__ float round_sel(float x, int rd) {
  const float b = round_to_bf16(x);
  const float h = __half2float(__float2half_rn(x));
  return rd == DT_BF16 ? b : (rd == DT_F16 ? h : x);
}

// rounding to the scale/weight dtype known at compile time (RD: 0 fp32, 1 bf16, 2 fp16); the hardware bf16
// conversion rounds to nearest even like round_to_bf16
template <int RD>
__device__ __forceinline__ float round_rd(float x) {
  if (RD == DT_BF16) return (float)(__bf16)x;
  if (RD == DT_F16) return __half2float(__float2half_rn(x));
  return x;
}

template <int RD>
__global__ __launch_bounds__(256) void mse_scale_kernel(const void* __restrict__ W, int wdt, long ldw, int R, int C, int g,
                                                        int G, const uint8_t* __restrict__ dead, const float* __restrict__ p,
                                                        int P, float qzero, float maxq, float norm, int rd,
                                                        float* __restrict__ scale_rg, float* __restrict__ scale_gr) {
  const int lane = threadIdx.x & 63;
  const long item = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (item >= (long)R * G) return;
  const int row = (int)(item / G), grp = (int)(item - (long)row * G);
  const float s0 = scale_rg[(long)row * G + grp];
  // x / s with IEEE rounding from a reciprocal computed once per candidate: q0 = RN(x*rcp), q1 = RN(q0 +
  // (x - q0*s)*rcp) is the correctly rounded quotient when rcp = RN(1/s) (Markstein); infinities and NaNs keep q0,
  // which is what the division gives there
  float sp[MSE_NC], rcp[MSE_NC], loss[MSE_NC];
#pragma unroll
  for (int c = 0; c < MSE_NC; ++c) {
    const int idx = lane + 64 * c;
    sp[c] = round_sel(s0 * p[min(idx, P - 1)], rd);
    rcp[c] = 1.0f / sp[c];
    loss[c] = 0.f;
  }
  const int c0 = grp * g;
  for (int e0 = 0; e0 < g; e0 += 64) {
    const int col = c0 + e0 + lane;
    float xv = 0.f;
    if (e0 + lane < g) {
      xv = load_as_f32(W, (long)row * ldw + col, wdt);
      if (dead && dead[col]) xv = 0.f;
    }
    const int cnt = min(64, g - e0);
#pragma unroll 4
    for (int j = 0; j < cnt; ++j) {
      const float x = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(xv), j));
#pragma unroll
      for (int c = 0; c < MSE_NC; ++c) {
        if (64 * c < P) {  // wave-uniform
          const float q0 = x * rcp[c];
          const float q1 = fmaf(fmaf(-q0, sp[c], x), rcp[c], q0);
          float q = floorf((fabsf(q0) < 3.0e38f ? q1 : q0) + qzero + 0.5f);
          q = fminf(fmaxf(q, 0.f), maxq);
          const float d = fabsf(round_rd<RD>((q - qzero) * sp[c]) - x);
          loss[c] += __builtin_amdgcn_exp2f(norm * __builtin_amdgcn_logf(d));
        }
      }
    }
  }
  // arg-min with the larger index winning ties: inside the lane, then across the wavefront
  float bl = __builtin_inff();
  int bi = -1;
#pragma unroll
  for (int c = 0; c < MSE_NC; ++c) {
    const int idx = lane + 64 * c;
    if (idx < P && (loss[c] < bl || (loss[c] == bl && idx > bi))) {
      bl = loss[c];
      bi = idx;
    }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const float ol = __shfl_xor(bl, off, 64);
    const int oi = __shfl_xor(bi, off, 64);
    if (oi >= 0 && (bi < 0 || ol < bl || (ol == bl && oi > bi))) {
      bl = ol;
      bi = oi;
    }
  }
  if (lane == 0) {
    const float s = round_sel(s0 * p[max(bi, 0)], rd);
    scale_rg[(long)row * G + grp] = s;
    if (scale_gr) scale_gr[(long)grp * R + row] = s;
  }
}

// ---------------------------------------------------------------------------------------------
// Wt[j, r] = W[r, perm[j]] as fp32 (0 for dead columns).  64x64 tiles through LDS.
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void prepare_wt_kernel(const void* __restrict__ W, int wdt, long ldw, int R, int C,
                                                         const int* __restrict__ perm, const uint8_t* __restrict__ dead,
                                                         float* __restrict__ Wt, float* __restrict__ Wt2, long ldwt) {
  __shared__ float t[64][65];
  const int j0 = blockIdx.x * 64, r0 = blockIdx.y * 64;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  const int j = j0 + tx;
  int src = -1;
  if (j < C) {
    src = perm ? perm[j] : j;
    if (dead && dead[src]) src = -1;
  }
  for (int rr = ty; rr < 64; rr += 4) {
    const int r = r0 + rr;
    float v = 0.f;
    if (r < R && src >= 0) v = load_as_f32(W, (long)r * ldw + src, wdt);
    t[rr][tx] = v;
  }
  __syncthreads();
  for (int jj = ty; jj < 64; jj += 4) {
    if (j0 + jj < C && r0 + tx < R) {
      Wt[(long)(j0 + jj) * ldwt + r0 + tx] = t[tx][jj];
      if (Wt2) Wt2[(long)(j0 + jj) * ldwt + r0 + tx] = t[tx][jj];  // second copy: the loop keeps one read-only
    }
  }
}

// ---------------------------------------------------------------------------------------------
// codes[r, c] = Qt[perm_inv[c], r]  (u8), 64x64 tiles through LDS.
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void untranspose_codes_kernel(const uint8_t* __restrict__ Qt, int R, int C,
                                                                const int* __restrict__ perm_inv,
                                                                uint8_t* __restrict__ codes, long ldc) {
  __shared__ uint8_t t[64][68];
  const int c0 = blockIdx.x * 64, r0 = blockIdx.y * 64;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  for (int cc = ty; cc < 64; cc += 4) {
    const int c = c0 + cc;
    uint8_t v = 0;
    if (c < C && r0 + tx < R) {
      const int j = perm_inv ? perm_inv[c] : c;
      v = Qt[(long)j * R + r0 + tx];
    }
    t[cc][tx] = v;
  }
  __syncthreads();
  for (int rr = ty; rr < 64; rr += 4) {
    if (r0 + rr < R && c0 + tx < C) codes[(long)(r0 + rr) * ldc + c0 + tx] = t[tx][rr];
  }
}

// ---------------------------------------------------------------------------------------------
// int4 -> int32: word[r, k] = sum_{i<8} ((codes[r, 8k+i] - zero + 8) & 15) << 4i ; columns past C pack as 0.
// One thread reads 16 codes (one 16-byte load) and writes two words (one 8-byte store).
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void pack_int4_kernel(const uint8_t* __restrict__ codes, long ldc, int R, int C,
                                                        const float* __restrict__ zero, int G, int g,
                                                        int32_t* __restrict__ out, long ldo, int words, int vec_ok) {
  const int pairs = (words + 1) / 2;
  const long idx = (long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (long)R * pairs) return;
  const int r = (int)(idx / pairs), p = (int)(idx - (long)r * pairs);
  const int c0 = p * 16;
  const uint8_t* src = codes + (long)r * ldc + c0;
  uint8_t b[16];
  if (vec_ok && c0 + 16 <= C) {
    const uint4 v = *reinterpret_cast<const uint4*>(src);
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 16; ++i) b[i] = (uint8_t)(w[i >> 2] >> (8 * (i & 3)));
  } else {
#pragma unroll
    for (int i = 0; i < 16; ++i) b[i] = (c0 + i < C) ? src[i] : 0;
  }
  uint32_t lo = 0, hi = 0;
  if (zero == nullptr) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      lo |= (uint32_t)(b[i] & 15u) << (4 * i);
      hi |= (uint32_t)(b[8 + i] & 15u) << (4 * i);
    }
  } else {
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      uint32_t u = 0;
      if (c0 + i < C) {
        const int z = (int)zero[(long)r * G + (c0 + i) / g];
        u = (uint32_t)((int)b[i] - z + 8) & 15u;
      }
      if (i < 8) lo |= u << (4 * i);
      else hi |= u << (4 * (i - 8));
    }
  }
  int32_t* dst = out + (long)r * ldo + 2 * p;
  if (vec_ok && 2 * p + 1 < words) {
    *reinterpret_cast<int2*>(dst) = make_int2((int)lo, (int)hi);
  } else {
    dst[0] = (int)lo;
    if (2 * p + 1 < words) dst[1] = (int)hi;
  }
}

// Packed words straight from the loop's transposed codes: word[r, k] from Qt[perm_inv[8k+i], r].
// 64 rows x 64 columns per workgroup; reads are 64-byte runs along r, writes 8 words per row.
__global__ __launch_bounds__(256) void pack_from_qt_kernel(const uint8_t* __restrict__ Qt, int R, int C,
                                                           const int* __restrict__ perm_inv,
                                                           int32_t* __restrict__ out, long ldo, int words) {
  __shared__ uint8_t t[64][68];
  const int c0 = blockIdx.x * 64, r0 = blockIdx.y * 64;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  for (int cc = ty; cc < 64; cc += 4) {
    const int c = c0 + cc;
    uint8_t v = 0;
    if (c < C && r0 + tx < R) {
      const int j = perm_inv ? perm_inv[c] : c;
      v = Qt[(long)j * R + r0 + tx] & 15u;
    }
    t[cc][tx] = v;
  }
  __syncthreads();
  // 64 rows x 8 words = 512 words, two per thread
  for (int it = threadIdx.x; it < 512; it += 256) {
    const int rr = it >> 3, k = it & 7;
    const int wk = (c0 >> 3) + k;
    if (r0 + rr < R && wk < words) {
      uint32_t w = 0;
#pragma unroll
      for (int i = 0; i < 8; ++i) w |= (uint32_t)t[8 * k + i][rr] << (4 * i);
      out[(long)(r0 + rr) * ldo + wk] = (int)w;
    }
  }
}

// ---------------------------------------------------------------------------------------------
// FP8 (e4m3fn) checkpoint weights with one fp32 inverse scale per 128x128 block -> bf16 / fp16:
//   out = round_to(dtype)( fp8_value * round_to(dtype)(scale_inv[block]) ),
// the value of `W.to(dtype) * s.to(dtype)` (fp8 -> 16-bit float is exact).  16 weights per thread:
// one 16-byte load, two 16-byte stores.
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ float e4m3fn_to_f32(uint32_t b) {
  const uint32_t sign = (b & 0x80u) << 24, e = (b >> 3) & 0xFu, m = b & 7u;
  float v;
  if (e == 0) v = (float)m * 0.001953125f;  // subnormal: m * 2^-9
  else if (e == 15 && m == 7) v = __uint_as_float(0x7fc00000u);
  else v = __uint_as_float(((e + 120u) << 23) | (m << 20));
  return __uint_as_float(__float_as_uint(v) | sign);
}

__device__ __forceinline__ uint16_t to_16bit(float x, int dt) {
  return dt == DT_BF16 ? f32_to_bf16_bits(x) : __half_as_ushort(__float2half_rn(x));
}

__global__ __launch_bounds__(256) void dequant_fp8_kernel(const uint8_t* __restrict__ W, long ldw, int R, int C,
                                                          const float* __restrict__ sinv, long lds, int dt,
                                                          uint16_t* __restrict__ out, long ldo, int vec) {
  const int chunks = (C + 15) / 16;
  const long item = (long)blockIdx.x * 256 + threadIdx.x;
  if (item >= (long)R * chunks) return;
  const int r = (int)(item / chunks), c0 = (int)(item - (long)r * chunks) * 16;
  const float s = round_sel(sinv[(long)(r >> 7) * lds + (c0 >> 7)], dt);  // a 16-chunk never straddles a block
  const uint8_t* src = W + (long)r * ldw + c0;
  uint16_t* dst = out + (long)r * ldo + c0;
  if (vec && c0 + 16 <= C) {
    const uint4 v = *reinterpret_cast<const uint4*>(src);
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
    uint32_t o[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const uint32_t lo = (w[k >> 1] >> (16 * (k & 1))) & 0xffu, hi = (w[k >> 1] >> (16 * (k & 1) + 8)) & 0xffu;
      o[k] = (uint32_t)to_16bit(e4m3fn_to_f32(lo) * s, dt) | ((uint32_t)to_16bit(e4m3fn_to_f32(hi) * s, dt) << 16);
    }
    *reinterpret_cast<uint4*>(dst) = make_uint4(o[0], o[1], o[2], o[3]);
    *reinterpret_cast<uint4*>(dst + 8) = make_uint4(o[4], o[5], o[6], o[7]);
  } else {
    for (int k = 0; k < 16 && c0 + k < C; ++k) dst[k] = to_16bit(e4m3fn_to_f32(src[k]) * s, dt);
  }
}

// SwiGLU product of an expert: out[r, j] = round(round(silu(GU[r, j])) * GU[r, I + j]) for 16-bit GU (n x 2I: the gate
// projection's outputs, then the up projection's), both roundings to the tensors' own type as the chained torch ops
// `silu(g) * u` round.  Eight columns per thread, 16-byte accesses.
__device__ __forceinline__ uint4 swiglu8(const uint4 gv, const uint4 uv, int dt) {
  const uint32_t g[4] = {gv.x, gv.y, gv.z, gv.w}, u[4] = {uv.x, uv.y, uv.z, uv.w};
  uint32_t o[4];
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    uint32_t w = 0;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const uint16_t gb = (uint16_t)(g[k] >> (16 * h)), ub = (uint16_t)(u[k] >> (16 * h));
      const float gf = dt == DT_BF16 ? bf16_bits_to_f32(gb) : __half2float(__ushort_as_half(gb));
      const float uf = dt == DT_BF16 ? bf16_bits_to_f32(ub) : __half2float(__ushort_as_half(ub));
      const uint16_t sb = to_16bit(gf / (1.0f + expf(-gf)), dt);
      const float sf = dt == DT_BF16 ? bf16_bits_to_f32(sb) : __half2float(__ushort_as_half(sb));
      w |= (uint32_t)to_16bit(sf * uf, dt) << (16 * h);
    }
    o[k] = w;
  }
  return make_uint4(o[0], o[1], o[2], o[3]);
}

__global__ __launch_bounds__(256) void swiglu_kernel(const uint16_t* __restrict__ GU, long ldg, int n, int I, int dt,
                                                     uint16_t* __restrict__ out, long ldo) {
  const int chunks = I / 8;
  const long item = (long)blockIdx.x * 256 + threadIdx.x;
  if (item >= (long)n * chunks) return;
  const int r = (int)(item / chunks), c0 = (int)(item - (long)r * chunks) * 8;
  const uint4 gv = *reinterpret_cast<const uint4*>(GU + (long)r * ldg + c0);
  const uint4 uv = *reinterpret_cast<const uint4*>(GU + (long)r * ldg + I + c0);
  *reinterpret_cast<uint4*>(out + (long)r * ldo + c0) = swiglu8(gv, uv, dt);
}

// The same product written in the packed-token layout the Hessian kernel reads (out[o][c][j] = value of token 8 o + j,
// channel c; channels padded with zeros to Ip, tokens to a whole octet grid): the product's only reader is the down
// projection's Hessian, so it never exists token-major.  G and U: the gate and the up projection's outputs, n x I each
// (two matrices, or the two halves of one stacked GEMM output).  One thread per (token octet, channel octet).
__global__ __launch_bounds__(256) void swiglu_packed_kernel(const uint16_t* __restrict__ G, long ldg,
                                                            const uint16_t* __restrict__ U, long ldu, int n, int I, int Ip,
                                                            int dt, uint16_t* __restrict__ out) {
  const int o = blockIdx.y;
  const int c8 = (blockIdx.x * 256 + threadIdx.x) * 8;
  if (c8 >= Ip) return;
  uint4 r[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const int t = 8 * o + j;
    r[j] = make_uint4(0, 0, 0, 0);
    if (t < n && c8 < I)
      r[j] = swiglu8(*reinterpret_cast<const uint4*>(G + (long)t * ldg + c8), *reinterpret_cast<const uint4*>(U + (long)t * ldu + c8), dt);
  }
  uint4* dst = reinterpret_cast<uint4*>(out + ((long)o * Ip + c8) * 8);
#pragma unroll
  for (int k = 0; k < 4; ++k) {  // word k of a row holds channels 2k (low half) and 2k+1 (high half)
    uint32_t w[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) w[j] = k == 0 ? r[j].x : (k == 1 ? r[j].y : (k == 2 ? r[j].z : r[j].w));
    dst[2 * k] = make_uint4((w[0] & 0xffffu) | (w[1] << 16), (w[2] & 0xffffu) | (w[3] << 16), (w[4] & 0xffffu) | (w[5] << 16),
                            (w[6] & 0xffffu) | (w[7] << 16));
    dst[2 * k + 1] = make_uint4((w[0] >> 16) | (w[1] & 0xffff0000u), (w[2] >> 16) | (w[3] & 0xffff0000u),
                                (w[4] >> 16) | (w[5] & 0xffff0000u), (w[6] >> 16) | (w[7] & 0xffff0000u));
  }
}

}  // namespace

extern "C" int mq_swiglu(const void* GU, long ldg, int n, int I, int dtype, void* out, long ldo, void* stream) {
  if (n < 0 || I <= 0 || (I & 7) || ldg < 2 * (long)I || ldo < I || (ldg & 7) || (ldo & 7)) return MQ_ERR_ARG;
  if (dtype != DT_BF16 && dtype != DT_F16) return MQ_ERR_ARG;
  if (n == 0) return MQ_OK;
  if (!GU || !out || ((uintptr_t)GU & 15) || ((uintptr_t)out & 15)) return MQ_ERR_ARG;
  const long items = (long)n * (I / 8);
  hipLaunchKernelGGL(swiglu_kernel, dim3((unsigned)((items + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                     (const uint16_t*)GU, ldg, n, I, dtype, (uint16_t*)out, ldo);
  return mq_check_launch();
}

extern "C" int mq_swiglu_packed(const void* G, long ldg, const void* U, long ldu, int n, int I, int dtype, void* out,
                                void* stream) {
  if (n < 0 || I <= 0 || (I & 7) || ldg < I || ldu < I || (ldg & 7) || (ldu & 7)) return MQ_ERR_ARG;
  if (dtype != DT_BF16 && dtype != DT_F16) return MQ_ERR_ARG;
  if (n == 0) return MQ_OK;
  if (!G || !U || !out || ((uintptr_t)G & 15) || ((uintptr_t)U & 15) || ((uintptr_t)out & 15)) return MQ_ERR_ARG;
  const int Ip = (I + 255) / 256 * 256, octets = (n + 127) / 128 * 16;  // the packed layout's padding
  hipLaunchKernelGGL(swiglu_packed_kernel, dim3((Ip / 8 + 255) / 256, octets), dim3(256), 0, (hipStream_t)stream,
                     (const uint16_t*)G, ldg, (const uint16_t*)U, ldu, n, I, Ip, dtype, (uint16_t*)out);
  return mq_check_launch();
}

extern "C" int mq_quant_grid_sym(const void* W, int w_dtype, long ldw, int R, int C, int group_size, int bits,
                                 const uint8_t* dead_cols, int round_dtype, float* scale_rg, float* scale_gr,
                                 void* stream) {
  if (!W || !scale_rg || R <= 0 || C <= 0 || group_size <= 0 || C % group_size != 0) return MQ_ERR_ARG;
  if (w_dtype < 0 || w_dtype > 2 || round_dtype < 0 || round_dtype > 2 || bits < 2 || bits > 8 || ldw < C)
    return MQ_ERR_ARG;
  const int G = C / group_size;
  const float maxq = (float)((1 << bits) - 1);
  const float two_over_maxq = 2.0f / maxq;
  const long items = (long)R * G;
  const bool pow2 = (group_size & (group_size - 1)) == 0;
  if (w_dtype == DT_BF16 && pow2 && group_size >= 32 && group_size <= 512 && (ldw & 7) == 0 && ((uintptr_t)W & 15) == 0) {
    const int spans = (C + 2047) / 2048;
    const long witems = (long)R * spans;
    hipLaunchKernelGGL(grid_sym_vec_kernel, dim3((unsigned)((witems + 3) / 4)), dim3(256), 0, (hipStream_t)stream,
                       (const uint16_t*)W, ldw, R, C, group_size, G, dead_cols, two_over_maxq, round_dtype, scale_rg,
                       scale_gr, spans);
    return mq_check_launch();
  }
  hipLaunchKernelGGL(grid_sym_kernel, dim3((unsigned)((items + 3) / 4)), dim3(256), 0, (hipStream_t)stream, W, w_dtype,
                     ldw, R, C, group_size, G, dead_cols, two_over_maxq, round_dtype, scale_rg, scale_gr);
  return mq_check_launch();
}

extern "C" int mq_mse_scale_sym(const void* W, int w_dtype, long ldw, int R, int C, int group_size,
                                const uint8_t* dead_cols, const float* p, int P, float qzero, float maxq, float norm,
                                int round_dtype, float* scale_rg, float* scale_gr, void* stream) {
  if (!W || !p || !scale_rg || R <= 0 || C <= 0 || group_size <= 0 || C % group_size != 0) return MQ_ERR_ARG;
  if (w_dtype < 0 || w_dtype > 2 || round_dtype < 0 || round_dtype > 2 || ldw < C) return MQ_ERR_ARG;
  if (P <= 0 || P > 64 * MSE_NC) return MQ_ERR_ARG;
  const int G = C / group_size;
  const long items = (long)R * G;
  const dim3 grid((unsigned)((items + 3) / 4));
#define MQ_MSE(RD_)                                                                                                   \
  hipLaunchKernelGGL(mse_scale_kernel<RD_>, grid, dim3(256), 0, (hipStream_t)stream, W, w_dtype, ldw, R, C, group_size, G, \
                     dead_cols, p, P, qzero, maxq, norm, round_dtype, scale_rg, scale_gr)
  if (round_dtype == DT_BF16) MQ_MSE(DT_BF16);
  else if (round_dtype == DT_F16) MQ_MSE(DT_F16);
  else MQ_MSE(0);
#undef MQ_MSE
  return mq_check_launch();
}

extern "C" int mq_prepare_wt_pair(const void* W, int w_dtype, long ldw, int R, int C, const int* perm,
                                  const uint8_t* dead_cols, float* Wt, float* Wt2, long ldwt, void* stream) {
  if (!W || !Wt || Wt == Wt2 || R <= 0 || C <= 0 || ldw < C || ldwt < R || w_dtype < 0 || w_dtype > 2) return MQ_ERR_ARG;
  hipLaunchKernelGGL(prepare_wt_kernel, dim3((C + 63) / 64, (R + 63) / 64), dim3(256), 0, (hipStream_t)stream, W,
                     w_dtype, ldw, R, C, perm, dead_cols, Wt, Wt2, ldwt);
  return mq_check_launch();
}

extern "C" int mq_prepare_wt(const void* W, int w_dtype, long ldw, int R, int C, const int* perm,
                             const uint8_t* dead_cols, float* Wt, long ldwt, void* stream) {
  return mq_prepare_wt_pair(W, w_dtype, ldw, R, C, perm, dead_cols, Wt, nullptr, ldwt, stream);
}

extern "C" int mq_untranspose_codes(const uint8_t* Qt, int R, int C, const int* perm_inv, uint8_t* codes, long ldc,
                                    void* stream) {
  if (!Qt || !codes || R <= 0 || C <= 0 || ldc < C) return MQ_ERR_ARG;
  hipLaunchKernelGGL(untranspose_codes_kernel, dim3((C + 63) / 64, (R + 63) / 64), dim3(256), 0, (hipStream_t)stream,
                     Qt, R, C, perm_inv, codes, ldc);
  return mq_check_launch();
}

extern "C" int mq_pack_int4(const uint8_t* codes, long ldc, int R, int C, const float* zero, int group_size,
                            int32_t* out, long ldo, void* stream) {
  if (!codes || !out || R <= 0 || C <= 0 || ldc < C) return MQ_ERR_ARG;
  const int words = (C + 7) / 8;
  if (ldo < words) return MQ_ERR_ARG;
  int G = 0;
  if (zero) {
    if (group_size <= 0 || C % group_size != 0) return MQ_ERR_ARG;
    G = C / group_size;
  }
  const int vec_ok = ((uintptr_t)codes % 16 == 0) && (ldc % 16 == 0) && ((uintptr_t)out % 8 == 0) && (ldo % 2 == 0);
  const long threads = (long)R * ((words + 1) / 2);
  hipLaunchKernelGGL(pack_int4_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, (hipStream_t)stream, codes,
                     ldc, R, C, zero, G, group_size, out, ldo, words, vec_ok);
  return mq_check_launch();
}

extern "C" int mq_pack_from_qt(const uint8_t* Qt, int R, int C, const int* perm_inv, int32_t* out, long ldo,
                               void* stream) {
  if (!Qt || !out || R <= 0 || C <= 0) return MQ_ERR_ARG;
  const int words = (C + 7) / 8;
  if (ldo < words) return MQ_ERR_ARG;
  hipLaunchKernelGGL(pack_from_qt_kernel, dim3((C + 63) / 64, (R + 63) / 64), dim3(256), 0, (hipStream_t)stream, Qt, R,
                     C, perm_inv, out, ldo, words);
  return mq_check_launch();
}

extern "C" int mq_dequant_fp8_block(const uint8_t* W, long ldw, int R, int C, const float* scale_inv, long ld_scale,
                                    int out_dtype, void* out, long ldo, void* stream) {
  if (!W || !scale_inv || !out || R <= 0 || C <= 0 || ldw < C || ldo < C) return MQ_ERR_ARG;
  if (out_dtype != DT_BF16 && out_dtype != DT_F16) return MQ_ERR_ARG;
  if (ld_scale < (C + 127) / 128) return MQ_ERR_ARG;
  const int vec = ((uintptr_t)W % 16 == 0) && (ldw % 16 == 0) && ((uintptr_t)out % 16 == 0) && (ldo % 8 == 0);
  const long items = (long)R * ((C + 15) / 16);
  hipLaunchKernelGGL(dequant_fp8_kernel, dim3((unsigned)((items + 255) / 256)), dim3(256), 0, (hipStream_t)stream, W, ldw, R,
                     C, scale_inv, ld_scale, out_dtype, (uint16_t*)out, ldo, vec);
  return mq_check_launch();
}
