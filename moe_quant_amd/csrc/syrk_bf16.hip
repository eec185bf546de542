// Hessian accumulation  H <- beta*H + alpha * X^T X  for 16-bit activations X (n x C, row-major; bf16 or
// fp16) and an fp32 Hessian, on the 16-bit matrix cores of gfx950 (v_mfma_f32_32x32x16_bf16 / _f16).
//
// bf16*bf16 and fp16*fp16 products are exact in fp32 (8+8 and 11+11 significand bits), so reading the
// 16-bit tokens directly gives the same terms as up-casting X to fp32 first; only the summation order
// differs.  Data movement is the same for both types: only the matrix instruction changes (template flag F16).
// fp32 activations go through the fp32 GEMM tiles instead (see mq_hessian_syrk).
//
// Only tiles of the upper block triangle are computed.  X is token-major, the matrix cores want the
// reduction index (tokens) contiguous per lane, so every thread loads a 2-channel x 8-token patch with
// eight coalesced 4-byte loads, transposes it in registers and writes two 16-byte rows into an LDS
// tile laid out [channel][token].  With too few tiles to fill 256 CUs the token range is split; the
// partial tiles go to a caller-provided workspace and are reduced in a fixed order (deterministic).
#include <cstdlib>
#include <mutex>
#include <type_traits>

#include "common.hpp"

extern "C" int mq_symmetrize_upper(float* H, long ldh, int C, void* stream);

namespace {

constexpr int T = 128;         // tile edge (channels)
constexpr int KT = 32;         // tokens per LDS stage
constexpr int LDS_ROW = 40;    // bf16 per LDS row: 32 tokens + 8 pad (80 B keeps b128 reads conflict-free)
constexpr int TILE_ELEMS = T * LDS_ROW;
constexpr int EPI_LD = 129;

__device__ __forceinline__ int xcd_remap(int bid, int total) {
  const int q = total >> 3, rem = total & 7;
  const int xcd = bid & 7, idx = bid >> 3;
  return xcd * q + (xcd < rem ? xcd : rem) + idx;
}
__device__ __forceinline__ void tri_decode(int L, int& tm, int& tn) {
  int c = (int)((__fsqrt_rn(8.0f * (float)L + 1.0f) - 1.0f) * 0.5f);
  while (c * (c + 1) / 2 > L) --c;
  while ((c + 1) * (c + 2) / 2 <= L) ++c;
  tn = c;
  tm = L - c * (c + 1) / 2;
}

typedef _Float16 half8n __attribute__((ext_vector_type(8)));
// one 32x32x16 product on 16-bit operands, fp32 accumulation; the operands travel as bf16x8n bit patterns
template <bool F16>
__device__ __forceinline__ floatx16 mfma16(bf16x8n a, bf16x8n b, floatx16 c) {
  if constexpr (F16)
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8n, a), __builtin_bit_cast(half8n, b), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}

struct Patch {
  uint32_t d[8];  // d[i] = {X[t0+i][c], X[t0+i][c+1]}
  __device__ __forceinline__ void load(const uint16_t* __restrict__ X, long ldx, int t0, int tend, int c, int C) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      uint32_t v = 0;
      if (t0 + i < tend && c < C) v = *reinterpret_cast<const uint32_t*>(X + (long)(t0 + i) * ldx + c);
      d[i] = v;
    }
  }
  // rows for channel c (low halves) and c+1 (high halves), 8 tokens each
  __device__ __forceinline__ void store(uint16_t* __restrict__ tile, int ch, int tok) const {
    uint4 lo, hi;
    lo.x = (d[0] & 0xffffu) | (d[1] << 16);
    lo.y = (d[2] & 0xffffu) | (d[3] << 16);
    lo.z = (d[4] & 0xffffu) | (d[5] << 16);
    lo.w = (d[6] & 0xffffu) | (d[7] << 16);
    hi.x = (d[0] >> 16) | (d[1] & 0xffff0000u);
    hi.y = (d[2] >> 16) | (d[3] & 0xffff0000u);
    hi.z = (d[4] >> 16) | (d[5] & 0xffff0000u);
    hi.w = (d[6] >> 16) | (d[7] & 0xffff0000u);
    *reinterpret_cast<uint4*>(tile + ch * LDS_ROW + tok) = lo;
    *reinterpret_cast<uint4*>(tile + (ch + 1) * LDS_ROW + tok) = hi;
  }
};

// The 128x128 tile of raw sums is staged in LDS as epi[r*EPI_LD + c].  Pass 1 folds alpha and the
// beta*H term into LDS (coalesced read of the upper tile); pass 2 writes the upper tile row-wise and,
// for off-diagonal tiles, the mirrored lower tile column-wise out of LDS, both coalesced.
__device__ __forceinline__ void write_tile(float* __restrict__ H, long ldh, int C, int m0, int n0, float* epi,
                                           float alpha, float beta, bool mirror, int tid) {
  for (int idx = tid; idx < T * T; idx += 256) {
    const int r = idx >> 7, c = idx & 127;
    float v = alpha * epi[r * EPI_LD + c];
    if (beta != 0.f && m0 + r < C && n0 + c < C) v = fmaf(beta, H[(long)(m0 + r) * ldh + n0 + c], v);
    epi[r * EPI_LD + c] = v;
  }
  __syncthreads();
  for (int idx = tid; idx < T * T; idx += 256) {
    const int r = idx >> 7, c = idx & 127;
    if (m0 + r < C && n0 + c < C) H[(long)(m0 + r) * ldh + n0 + c] = epi[r * EPI_LD + c];
  }
  if (mirror) {
    for (int idx = tid; idx < T * T; idx += 256) {
      const int c = idx >> 7, r = idx & 127;
      if (m0 + r < C && n0 + c < C) H[(long)(n0 + c) * ldh + m0 + r] = epi[r * EPI_LD + c];
    }
  }
}

template <bool F16>
__global__ __launch_bounds__(256) void syrk_bf16_kernel(float* __restrict__ H, long ldh, const uint16_t* __restrict__ X,
                                                        long ldx, int n, int C, float alpha, float beta, int ntri,
                                                        int splits, int tokens_per_split, float* __restrict__ ws,
                                                        int mirror) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  uint16_t* tiles = reinterpret_cast<uint16_t*>(smem);  // [2 stages][A,B][TILE_ELEMS]
  float* epi = reinterpret_cast<float*>(smem);          // reused after the main loop: [T][EPI_LD]

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int L = xcd_remap(blockIdx.x, ntri * splits);
  const int split = L / ntri;
  int tm, tn;
  tri_decode(L - split * ntri, tm, tn);
  const int m0 = tm * T, n0 = tn * T;
  const int tbeg = split * tokens_per_split;
  const int tend = min(n, tbeg + tokens_per_split);

  floatx16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  const int pair = tid & 63;  // channel pair inside the tile
  const int oct = wave;       // token octet inside the stage
  Patch pa, pb;
  const int nk = (tend - tbeg + KT - 1) / KT;
  if (nk > 0) {
    pa.load(X, ldx, tbeg + oct * 8, tend, m0 + 2 * pair, C);
    pb.load(X, ldx, tbeg + oct * 8, tend, n0 + 2 * pair, C);
    pa.store(tiles, 2 * pair, oct * 8);
    pb.store(tiles + TILE_ELEMS, 2 * pair, oct * 8);
  }
  __syncthreads();
  const int lr = lane & 31, lk = lane >> 5;
  for (int kt = 0; kt < nk; ++kt) {
    const int cur = kt & 1;
    if (kt + 1 < nk) {
      const int t0 = tbeg + (kt + 1) * KT + oct * 8;
      pa.load(X, ldx, t0, tend, m0 + 2 * pair, C);
      pb.load(X, ldx, t0, tend, n0 + 2 * pair, C);
    }
    const uint16_t* as = tiles + cur * 2 * TILE_ELEMS + (wm * 64 + lr) * LDS_ROW + lk * 8;
    const uint16_t* bs = tiles + cur * 2 * TILE_ELEMS + TILE_ELEMS + (wn * 64 + lr) * LDS_ROW + lk * 8;
#pragma unroll
    for (int kk = 0; kk < KT / 16; ++kk) {
      const bf16x8n a0 = *reinterpret_cast<const bf16x8n*>(as + kk * 16);
      const bf16x8n a1 = *reinterpret_cast<const bf16x8n*>(as + 32 * LDS_ROW + kk * 16);
      const bf16x8n b0 = *reinterpret_cast<const bf16x8n*>(bs + kk * 16);
      const bf16x8n b1 = *reinterpret_cast<const bf16x8n*>(bs + 32 * LDS_ROW + kk * 16);
      acc[0][0] = mfma16<F16>(a0, b0, acc[0][0]);
      acc[0][1] = mfma16<F16>(a0, b1, acc[0][1]);
      acc[1][0] = mfma16<F16>(a1, b0, acc[1][0]);
      acc[1][1] = mfma16<F16>(a1, b1, acc[1][1]);
    }
    if (kt + 1 < nk) {
      uint16_t* nx = tiles + (cur ^ 1) * 2 * TILE_ELEMS;
      pa.store(nx, 2 * pair, oct * 8);
      pb.store(nx + TILE_ELEMS, 2 * pair, oct * 8);
    }
    __syncthreads();
  }

  if (splits > 1) {  // partial tile -> workspace [split][tile][128][128], lanes along columns
    float* out = ws + ((long)split * ntri + (L - split * ntri)) * (T * T);
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int r = wm * 64 + i * 32 + 8 * (v >> 2) + 4 * lk + (v & 3);
          out[r * T + wn * 64 + j * 32 + lr] = acc[i][j][v];
        }
    return;
  }
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int r = wm * 64 + i * 32 + 8 * (v >> 2) + 4 * lk + (v & 3);
        epi[r * EPI_LD + wn * 64 + j * 32 + lr] = acc[i][j][v];
      }
  __syncthreads();
  write_tile(H, ldh, C, m0, n0, epi, alpha, beta, mirror && tm != tn, tid);
}

__global__ __launch_bounds__(256) void syrk_reduce_kernel(float* __restrict__ H, long ldh, int C, float alpha, float beta,
                                                          int ntri, int splits, const float* __restrict__ ws,
                                                          int mirror) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  float* epi = reinterpret_cast<float*>(smem);
  const int tid = threadIdx.x;
  const int L = blockIdx.x;
  int tm, tn;
  tri_decode(L, tm, tn);
  for (int idx = tid; idx < T * T; idx += 256) {
    float s = 0.f;
    for (int k = 0; k < splits; ++k) s += ws[((long)k * ntri + L) * (T * T) + idx];
    epi[(idx >> 7) * EPI_LD + (idx & 127)] = s;
  }
  __syncthreads();
  write_tile(H, ldh, C, tm * T, tn * T, epi, alpha, beta, mirror && tm != tn, tid);
}

// =============================================================================================
// Large tiles: 256x256 channels per workgroup.
// =============================================================================================
constexpr int T2 = 256;
// Tile order for the 256x256 kernel.  Upper-triangle tiles are enumerated super-tile by super-tile
// (4 row tiles x 8 column tiles): the ~32 workgroups an XCD runs at any moment then touch about a dozen
// distinct channel panels instead of ~30, so more of their loads hit that XCD's L2.
__device__ __forceinline__ void blocked_tri_decode(int L, int T, int& tm, int& tn) {
  constexpr int SM = 4, SN = 8;
  int cum = 0;
  for (int a = 0; a * SM < T; ++a) {
    for (int b = (a * SM) / SN; b * SN < T; ++b) {
      int cnt = 0;
      for (int i = 0; i < SM; ++i) {
        const int r = a * SM + i;
        if (r >= T) break;
        const int lo = max(r, b * SN), hi = min(T, b * SN + SN);
        cnt += max(0, hi - lo);
      }
      if (L < cum + cnt) {
        int k = L - cum;
        for (int i = 0; i < SM; ++i) {
          const int r = a * SM + i;
          const int lo = max(r, b * SN), hi = min(T, b * SN + SN);
          const int w = max(0, hi - lo);
          if (k < w) {
            tm = r;
            tn = lo + k;
            return;
          }
          k -= w;
        }
      }
      cum += cnt;
    }
  }
  tm = tn = 0;  // not reached for L < T(T+1)/2
}

// =============================================================================================
// Same 256x256 workgroup tile, staged without touching the vector registers: the token-major rows of X go
// from memory straight into LDS (16 bytes per lane per instruction) and the matrix-core operands, which want
// the tokens of one channel side by side, are read back with the transposing LDS load.
//
// LDS stage = 32 tokens x 512 channels (the 256 of the row tile, then the 256 of the column tile) cut into
// 1 KB chunks [token quad q][channel group G of 128]; a chunk is what one wavefront-wide direct load writes
// (lane i fills bytes 16i..16i+15).  Inside a chunk, eight blocks of 128 bytes hold 4 tokens x 16 channels
// each, token-major: lane i of the load fetches token (i%8)/2, channels 16*(i/8) + 8*(i%2) ... +7.
// A transposing read (ds_read_b64_tr_b16) has the 16 lanes of a group fetch 8 bytes each from one such block
// -- 128 contiguous bytes, no bank conflict -- and hands lane s the 4 tokens of channel s.  Two of them give a
// lane its 8 tokens of a 32x32x16 operand; which tokens share a lane is irrelevant as long as both operands
// use the same rule, and both are read by the same code.
// Four stages are allocated: while stage s feeds the matrix cores, stages s+1..s+3 are in flight, tracked
// with the vector-memory counter (32 loads per stage, shared evenly by the wavefronts), one barrier per stage.
// =============================================================================================
constexpr int KT3 = 32, NST3 = 4, CHUNK3 = 1024;
constexpr int STAGE3 = (KT3 / 4) * 4 * CHUNK3;  // bytes
constexpr size_t DMA_SMEM = (size_t)NST3 * STAGE3;

typedef __attribute__((address_space(3))) void* lds_void_p;
typedef __attribute__((address_space(1))) const void* gbl_void_p;
typedef short short4v __attribute__((ext_vector_type(4)));

// One wavefront-wide direct load: lane i copies 16 bytes from its own global address to LDS byte lds_addr + 16 i.
// Written as inline assembly on purpose: told about an LDS-writing load, the compiler drains all of them
// (vmcnt(0)) before the next LDS read, which would serialise the stages this kernel keeps in flight.  The
// kernel orders loads and reads itself (s_waitcnt vmcnt + barrier below).
// The address is a scalar base plus a 32-bit per-lane byte offset, so a stage costs scalar arithmetic only.
__device__ __forceinline__ void dma16(const void* sbase, unsigned lane_off, unsigned lds_addr) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(lane_off), "s"(sbase), "s"(lds_addr)
               : "memory", "m0");
}

// issues (or, for ragged stages, completes) the LPW chunk loads of this wavefront for the stage starting at token t0.
// wave_u is the wavefront index as a scalar; lane_off = 2*(tau*ldx + 16*b + 8*half), the byte offset of this
// lane's slot inside a chunk's source (4 token rows x 128 channels).
template <bool FAST, int LPW>  // LPW: chunk loads per wavefront per stage (32 chunks / number of wavefronts)
__device__ __forceinline__ void dma_stage(const uint16_t* __restrict__ X, unsigned lane_off, long ldx, int t0, int tend,
                                          int C, int m0, int n0, unsigned char* buf, unsigned lds_base, int wave_u,
                                          int lane) {
  const int b = lane >> 3, tau = (lane & 7) >> 1, half = lane & 1;
#pragma unroll
  for (int i = 0; i < LPW; ++i) {
    const int ch = wave_u * LPW + i, q = ch >> 2, G = ch & 3;
    const int chan0 = ((G & 2) ? n0 : m0) + (G & 1) * 128;  // scalar
    if (FAST) {
      const long off = (long)(t0 + 4 * q) * ldx + chan0;  // scalar
      dma16(X + off, lane_off, lds_base + (unsigned)(ch * CHUNK3));
    } else {
      const int chan = chan0 + 16 * b + 8 * half;
      const int tok = t0 + 4 * q + tau;
      const bool ok = (tok < tend) && (chan + 8 <= C);
      const uint16_t* src = X + (long)(tok < tend ? tok : tend - 1) * ldx + (chan + 8 <= C ? chan : 0);
      uint4 v = *reinterpret_cast<const uint4*>(src);
      if (!ok) v = make_uint4(0, 0, 0, 0);
      *reinterpret_cast<uint4*>(buf + ch * CHUNK3 + lane * 16) = v;
    }
  }
}

// How a call's tiles are dealt to workgroups.  The first `head` upper-triangle tiles (in blocked order) are computed
// whole, one workgroup each, and written straight to H.  The remaining `ntail` tiles are cut into `splits` token
// ranges of `tps` tokens, one workgroup per piece; the pieces go to the workspace as raw fp32 sums,
// ws[(split * ntail + tail tile) * 256 * 256], and a second kernel adds them up in a fixed order.  Two uses: few
// tiles in all (head = 0: the token ranges supply the parallelism), and the last, partly filled round of a large
// triangle (406 tiles on 256 CUs: the 150 left over would keep the chip 59% busy for a whole round).
struct SyrkPlan {
  int ntri, head, ntail, splits, tps;
};

// one 256x256 tile (or one token range of it); (bid, yrow) = workgroup index in a grid of max(head, ntail) x (1 + splits),
// or of head x 1 when nothing is cut.
// NW = 4: four wavefronts of 128x128 (one per SIMD, all 512 registers).  NW = 8: eight of 128x64, two per SIMD:
// while one waits for the address unit to take its direct loads the other keeps the matrix pipe busy.
template <int NW, bool F16>
__device__ __forceinline__ void syrk_dma_tile(float* __restrict__ H, long ldh, const uint16_t* __restrict__ X, long ldx,
                                              int n, int C, float alpha, float beta, SyrkPlan pl, float* __restrict__ ws,
                                              int bid, int yrow, unsigned char* smem) {
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // a scalar: LDS targets of the direct loads live in M0
  constexpr int NJ = 16 / NW;     // 32-column blocks per wavefront: 4 (128 columns) or 2 (64 columns)
  constexpr int WCOLS = NW / 2;   // wavefronts side by side along the columns
  constexpr int LPW = 32 / NW;    // direct loads per wavefront per stage
  const int wm = wave / WCOLS, wn = wave % WCOLS;
  // grid row 0: the whole tiles; grid row 1 + s: token range s of the tail tiles (pieces of one token range lie
  // side by side: they share the rows of X they read).  Rows are as wide as the longer of the two: the rest leaves.
  const int split = max(yrow - 1, 0);
  const bool partial = yrow > 0;
  if (bid >= (partial ? pl.ntail : pl.head)) return;
  const int L = partial ? pl.head + bid : xcd_remap(bid, pl.head);
  int tm, tn;
  blocked_tri_decode(L, (C + T2 - 1) / T2, tm, tn);
  // uniform values that the division and the square root above left in vector registers: back to scalars,
  // the direct loads take their base address and LDS target from scalar registers
  tm = __builtin_amdgcn_readfirstlane(tm);
  tn = __builtin_amdgcn_readfirstlane(tn);
  const int m0 = tm * T2, n0 = tn * T2;
  const int tbeg = partial ? __builtin_amdgcn_readfirstlane(min(n, split * pl.tps)) : 0;
  const int tend = partial ? min(n, tbeg + pl.tps) : n;
  const int nk = (tend - tbeg + KT3 - 1) / KT3;
  const bool interior = (m0 + T2 <= C) && (n0 + T2 <= C);
  // LDS byte address of the staging area plus this wavefront's share of a stage, as a scalar
  const unsigned smem_lds = __builtin_amdgcn_readfirstlane(
      (unsigned)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)smem);
  const unsigned lane_off = 2u * (unsigned)(((lane & 7) >> 1) * ldx + 16 * (lane >> 3) + 8 * (lane & 1));

  floatx16 acc[4][NJ];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < NJ; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

#define MQ_SYRK_ISSUE(st)                                                                         \
  do {                                                                                            \
    const int t0_ = tbeg + (st)*KT3;                                                              \
    unsigned char* buf_ = smem + ((st) % NST3) * STAGE3;                                          \
    const unsigned lds_ = smem_lds + (unsigned)(((st) % NST3) * STAGE3);                          \
    if (interior && t0_ + KT3 <= tend) dma_stage<true, LPW>(X, lane_off, ldx, t0_, tend, C, m0, n0, buf_, lds_, wave, lane);  \
    else dma_stage<false, LPW>(X, lane_off, ldx, t0_, tend, C, m0, n0, buf_, lds_, wave, lane);        \
  } while (0)

#pragma unroll
  for (int st = 0; st < NST3 - 1; ++st)
    if (st < nk) MQ_SYRK_ISSUE(st);

  // fragment addressing: 16-lane group g16 = lane/16 -> channel block parity g16&1, token half g16>>1
  const int g16 = lane >> 4, s16 = lane & 15;
  const int a_off = wm * CHUNK3 + (g16 & 1) * 128 + s16 * 8;        // + i*256 (block pair i) + quad*4*CHUNK3
  const int co = wn * NJ * 32;  // first column of this wavefront inside the column tile
  const int b_off = (2 + co / 128) * CHUNK3 + ((co % 128) / 16 + (g16 & 1)) * 128 + s16 * 8;  // + j*256
  const int hq = g16 >> 1;

  for (int kt = 0; kt < nk; ++kt) {
    // stage kt must have landed: at most the loads of the stages issued after it may still be in flight
    const int ahead = min(nk, kt + NST3 - 1) - (kt + 1);
    // (lgkmcnt(0) as well: LDS writes of a ragged stage must have landed before the barrier lets others read)
    asm volatile("" ::: "memory");
    // s_waitcnt immediates: vmcnt in bits 3:0 and 15:14, expcnt 6:4 left at its maximum, lgkmcnt(0) in 11:8
    constexpr int W2 = 0x0070 | ((2 * LPW) & 15) | (((2 * LPW) >> 4) << 14), W1 = 0x0070 | LPW;
    if (ahead >= 2) __builtin_amdgcn_s_waitcnt(W2);       // vmcnt(2*LPW) lgkmcnt(0)
    else if (ahead == 1) __builtin_amdgcn_s_waitcnt(W1);  // vmcnt(LPW) lgkmcnt(0)
    else __builtin_amdgcn_s_waitcnt(0x0070);              // vmcnt(0) lgkmcnt(0)
    // a bare barrier: __syncthreads() carries a fence that makes the compiler drain every direct load in flight.
    // The empty asm statements keep the compiler from moving LDS accesses across it.
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    if (kt + NST3 - 1 < nk) MQ_SYRK_ISSUE(kt + NST3 - 1);
    const unsigned char* stg = smem + (kt % NST3) * STAGE3;
#pragma unroll
    for (int kk = 0; kk < KT3 / 16; ++kk) {
      short4v fa[4][2], fb[NJ][2];
#pragma unroll
      for (int r = 0; r < 2; ++r) {
        const int quad = 4 * kk + 2 * r + hq;
#pragma unroll
        for (int i = 0; i < 4; ++i)
          fa[i][r] = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
              (short4v __attribute__((address_space(3)))*)(stg + quad * 4 * CHUNK3 + a_off + i * 256));
#pragma unroll
        for (int j = 0; j < NJ; ++j)
          fb[j][r] = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
              (short4v __attribute__((address_space(3)))*)(stg + quad * 4 * CHUNK3 + b_off + j * 256));
      }
      bf16x8 va[4], vb[NJ];
#pragma unroll
      for (int i = 0; i < 4; ++i) va[i] = __builtin_shufflevector(fa[i][0], fa[i][1], 0, 1, 2, 3, 4, 5, 6, 7);
#pragma unroll
      for (int j = 0; j < NJ; ++j) vb[j] = __builtin_shufflevector(fb[j][0], fb[j][1], 0, 1, 2, 3, 4, 5, 6, 7);
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < NJ; ++j)
          acc[i][j] = mfma16<F16>(__builtin_bit_cast(bf16x8n, vb[j]), __builtin_bit_cast(bf16x8n, va[i]), acc[i][j]);
    }
  }
#undef MQ_SYRK_ISSUE

  // The products were issued with the operands swapped (block rows = channels of the column tile), so of every 32x32
  // block a lane holds four runs of four consecutive COLUMNS of one row of H: 16-byte accesses where H allows them.
  const int lr = lane & 31, lk = lane >> 5;
  float* out = partial ? ws + ((long)split * pl.ntail + (L - pl.head)) * (T2 * T2) : H;
  const bool vec = partial || ((((uintptr_t)H) & 15) == 0 && (ldh & 3) == 0 && (C & 3) == 0);
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = wm * 128 + i * 32 + lr;
#pragma unroll
    for (int j = 0; j < NJ; ++j)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int c = co + j * 32 + 8 * g + 4 * lk;
        const floatx16& a = acc[i][j];
        if (partial) {
          *reinterpret_cast<float4*>(out + r * T2 + c) = float4{a[4 * g], a[4 * g + 1], a[4 * g + 2], a[4 * g + 3]};
        } else if (m0 + r < C && n0 + c < C) {
          float* q = H + (long)(m0 + r) * ldh + n0 + c;
          if (vec) {
            float4 val = {alpha * a[4 * g], alpha * a[4 * g + 1], alpha * a[4 * g + 2], alpha * a[4 * g + 3]};
            if (beta != 0.f) {
              const float4 o = *reinterpret_cast<const float4*>(q);
              val.x = fmaf(beta, o.x, val.x), val.y = fmaf(beta, o.y, val.y), val.z = fmaf(beta, o.z, val.z),
              val.w = fmaf(beta, o.w, val.w);
            }
            *reinterpret_cast<float4*>(q) = val;
          } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
              if (n0 + c + e < C) {
                float val = alpha * a[4 * g + e];
                if (beta != 0.f) val = fmaf(beta, q[e], val);
                q[e] = val;
              }
          }
        }
      }
  }
}

template <bool F16>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2))) void syrk_bf16_dma8_kernel(
    float* __restrict__ H, long ldh, const uint16_t* __restrict__ X, long ldx, int n, int C, float alpha, float beta,
    SyrkPlan pl, float* __restrict__ ws) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
  syrk_dma_tile<8, F16>(H, ldh, X, ldx, n, C, alpha, beta, pl, ws, blockIdx.x, blockIdx.y, smem);
}

// Several independent accumulations (one Hessian each, same C) in one launch: blockIdx.y picks the problem.
// Each workgroup runs the whole token range of its tile, so no partial tiles and no workspace: the groups,
// not token splits, supply the parallelism (C = 2048 has only 36 tiles per problem).
constexpr int SYRK_MAX_GROUP = 16;
struct SyrkGroupTable {
  float* H[SYRK_MAX_GROUP];
  const uint16_t* X[SYRK_MAX_GROUP];
  long ldh[SYRK_MAX_GROUP], ldx[SYRK_MAX_GROUP];
  int n[SYRK_MAX_GROUP];
  float alpha[SYRK_MAX_GROUP], beta[SYRK_MAX_GROUP];
};
template <bool F16>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2))) void syrk_bf16_dma_grouped_kernel(
    SyrkGroupTable t, int C, int ntri) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
  const int z = blockIdx.y;
  syrk_dma_tile<8, F16>(t.H[z], t.ldh[z], t.X[z], t.ldx[z], t.n[z], C, t.alpha[z], t.beta[z], SyrkPlan{ntri, ntri, 0, 1, 0},
                        nullptr, blockIdx.x, 0, smem);
}

// fixed-order sum of the token-range pieces of the tail tiles (see SyrkPlan)
__global__ __launch_bounds__(256) void syrk_big_reduce_kernel(float* __restrict__ H, long ldh, int C, float alpha,
                                                              float beta, SyrkPlan pl, const float* __restrict__ ws) {
  const int lt = blockIdx.y;  // tail tile
  int tm, tn;
  blocked_tri_decode(pl.head + lt, (C + T2 - 1) / T2, tm, tn);
  const int idx = blockIdx.x * 256 + threadIdx.x;  // one float4 of the tile
  const int r = idx >> 6, c = (idx & 63) << 2;
  float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
  for (int k = 0; k < pl.splits; ++k) {
    const float4 v = *reinterpret_cast<const float4*>(ws + ((long)k * pl.ntail + lt) * (T2 * T2) + r * T2 + c);
    s.x += v.x;
    s.y += v.y;
    s.z += v.z;
    s.w += v.w;
  }
  const float e[4] = {s.x, s.y, s.z, s.w};
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const int gr = tm * T2 + r, gc = tn * T2 + c + q;
    if (gr < C && gc < C) {
      float* p = H + (long)gr * ldh + gc;
      float val = alpha * e[q];
      if (beta != 0.f) val = fmaf(beta, *p, val);
      *p = val;
    }
  }
}

// lower triangle <- transpose of the upper triangle, 64x64 tiles through LDS
__global__ __launch_bounds__(256) void symmetrize_kernel(float* __restrict__ H, long ldh, int C) {
  __shared__ float t[64][65];
  int bi, bj;
  tri_decode(blockIdx.x, bi, bj);  // bi <= bj: source tile rows bi, cols bj
  if (bi == bj) {
    for (int idx = threadIdx.x; idx < 64 * 64; idx += 256) {
      const int r = idx >> 6, c = idx & 63;
      if (c > r && bi * 64 + c < C) t[r][c] = H[(long)(bi * 64 + r) * ldh + bi * 64 + c];
    }
    __syncthreads();
    for (int idx = threadIdx.x; idx < 64 * 64; idx += 256) {
      const int r = idx >> 6, c = idx & 63;
      if (c < r && bi * 64 + r < C) H[(long)(bi * 64 + r) * ldh + bi * 64 + c] = t[c][r];
    }
    return;
  }
  for (int idx = threadIdx.x; idx < 64 * 64; idx += 256) {
    const int r = idx >> 6, c = idx & 63;
    if (bi * 64 + r < C && bj * 64 + c < C) t[r][c] = H[(long)(bi * 64 + r) * ldh + bj * 64 + c];
  }
  __syncthreads();
  for (int idx = threadIdx.x; idx < 64 * 64; idx += 256) {
    const int r = idx >> 6, c = idx & 63;  // destination row bj*64+r, col bi*64+c
    if (bj * 64 + r < C && bi * 64 + c < C) H[(long)(bj * 64 + r) * ldh + bi * 64 + c] = t[c][r];
  }
}

// =============================================================================================
// Packed tokens.  The matrix cores want, per lane, eight consecutive tokens of one channel; token-major X has them
// 2*ldx bytes apart, which is what the transposing LDS reads above are for.  Where the tokens are copied anyway (the
// routed tokens of an expert are gathered; the output of the SiLU product is written by this library) the copy can
// be laid out for the matrix cores instead:
//     Xp[o][c][j] = X[8 o + j][c],   o = token octet, c = channel (padded to a multiple of 256), j = 0..7,
// tokens padded with zeros to a multiple of 32.  A lane's operand fragment is then one aligned 16-byte cell, a
// direct load moves 64 cells = 1 KB of contiguous memory to 1 KB of contiguous LDS, and fragments come out of LDS
// with plain 16-byte reads (ds_read_b128, conflict-free: 16 lanes read 256 contiguous bytes).
// Workgroup = eight wavefronts of 128x64 on a 256x256 tile, two per SIMD, as in the kernel above.  Stage = 32 tokens x
// 512 channels = 32 KB ([token octet][channel][8 tokens]); four stages in LDS.  The loop is software-pipelined by hand
// and its instruction order pinned: per 16-token step, eight matrix instructions with the next step's six fragment
// reads and two direct loads of a later stage dealt between them; one barrier per stage, placed between the stage's two
// steps, so that the fragments of the next stage's first step are fetched while the second step's products run.  Step A
// of stage kt issues the second half of stage kt+3 (into the buffer of stage kt-1, free since that stage's barrier),
// step B the first half of stage kt+4 (into the buffer of stage kt itself, which nobody reads after this stage's
// barrier): three and a half stages in flight.  Loads past the last stage are not branched around: they fetch the last
// stage again into a fifth, unread LDS area, which keeps the loop one basic block and the load counter's arithmetic
// uniform.
// Timing experiments on this loop (65536 tokens x 7168 channels; results discarded): no direct loads in the loop 1.34
// PFLOP/s, loads that always hit the same L2-resident cells 1.22, no fragment reads 1.15, nothing but the matrix
// instructions 1.43 -- the rate this chip sustains on dense bf16 products under its power limit with these tile
// counts -- against 1.03-1.10 for the kernel as it is (the token-major kernel above: 0.93-0.98).
// =============================================================================================
constexpr int PK_PLANE = 512 * 16;            // bytes of one token octet of a stage
constexpr int PK_STAGE = 4 * PK_PLANE;        // 32 KB
constexpr int PK_NST = 4;
constexpr size_t PK_SMEM = (size_t)(PK_NST + 1) * PK_STAGE;  // + the dump area: 160 KB, all the LDS of a CU

static inline int pk_pad_tokens(int n) { return (n + 127) / 128 * 128; }
static inline int pk_pad_channels(int C) { return (C + 255) / 256 * 256; }

template <bool F16>
__device__ __forceinline__ void syrk_packed_tile(float* __restrict__ H, long ldh, const uint16_t* __restrict__ Xp, int n_pad,
                                                  int Cp, int C, float alpha, float beta, SyrkPlan pl, float* __restrict__ ws,
                                                  int bid, int yrow, unsigned char* smem) {
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 2, wn = wave & 3;
  const int split = max(yrow - 1, 0);
  const bool partial = yrow > 0;
  if (bid >= (partial ? pl.ntail : pl.head)) return;
  const int L = partial ? pl.head + bid : xcd_remap(bid, pl.head);
  int tm, tn;
  blocked_tri_decode(L, Cp / T2, tm, tn);
  tm = __builtin_amdgcn_readfirstlane(tm);
  tn = __builtin_amdgcn_readfirstlane(tn);
  const int m0 = tm * T2, n0 = tn * T2;
  const int tbeg = partial ? __builtin_amdgcn_readfirstlane(min(n_pad, split * pl.tps)) : 0;
  const int tend = partial ? min(n_pad, tbeg + pl.tps) : n_pad;
  const int nk = (tend - tbeg) / 32;
  const int s0 = tbeg / 32;
  const unsigned smem_lds = __builtin_amdgcn_readfirstlane(
      (unsigned)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)smem);
  const unsigned lane_off = 16u * (unsigned)lane;
  floatx16 acc[4][2];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
  if (nk > 0) {
    // direct load q (0..3) of stage s: token octet wave/2 of the stage; even wavefronts fetch the row tile's four
    // 64-channel groups, odd ones the column tile's
    const int oct = wave >> 1, side = wave & 1;
    auto issue = [&](int s, int q) {
      const int src = min(s, nk - 1);
      const long cell = ((long)(s0 + src) * 4 + oct) * Cp + (side ? n0 : m0) + 64 * q;
      const unsigned dst = smem_lds + (unsigned)((s < nk ? s % PK_NST : PK_NST) * PK_STAGE + oct * PK_PLANE + (4 * side + q) * 1024);
      dma16(Xp + cell * 8, lane_off, dst);
    };
#pragma unroll
    for (int s = 0; s < PK_NST - 1; ++s)
#pragma unroll
      for (int q = 0; q < 4; ++q) issue(s, q);
#pragma unroll
    for (int q = 0; q < 2; ++q) issue(PK_NST - 1, q);
    const int lr = lane & 31, lk = lane >> 5;
    const int a_off = lk * PK_PLANE + (wm * 128 + lr) * 16;
    const int b_off = lk * PK_PLANE + (256 + wn * 64 + lr) * 16;
    bf16x8n fa0[4], fb0[2], fa1[4], fb1[2];
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_waitcnt(0x0070 | 10);  // stage 0 landed: at most the 10 loads of stages 1, 2, 3 in flight
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
#pragma unroll
    for (int i = 0; i < 4; ++i) fa0[i] = *reinterpret_cast<const bf16x8n*>(smem + a_off + i * 512);
#pragma unroll
    for (int j = 0; j < 2; ++j) fb0[j] = *reinterpret_cast<const bf16x8n*>(smem + b_off + j * 512);
#pragma unroll 1
    for (int kt = 0; kt < nk; ++kt) {
      const unsigned char* stg = smem + (kt % PK_NST) * PK_STAGE;
      const unsigned char* nxt = smem + ((kt + 1) % PK_NST) * PK_STAGE;
#pragma unroll
      for (int m = 0; m < 8; ++m) {
        acc[m >> 1][m & 1] = mfma16<F16>(fb0[m & 1], fa0[m >> 1], acc[m >> 1][m & 1]);
        if (m < 4) fa1[m] = *reinterpret_cast<const bf16x8n*>(stg + 2 * PK_PLANE + a_off + m * 512);
        else if (m < 6) fb1[m - 4] = *reinterpret_cast<const bf16x8n*>(stg + 2 * PK_PLANE + b_off + (m - 4) * 512);
        else issue(kt + PK_NST - 1, 2 + (m - 6));
        __builtin_amdgcn_sched_barrier(0);
      }
      asm volatile("" ::: "memory");
      __builtin_amdgcn_s_waitcnt(0x0070 | 8);  // stage kt+1 landed: at most the 8 loads of stages kt+2, kt+3 in flight
      __builtin_amdgcn_s_barrier();
      asm volatile("" ::: "memory");
#pragma unroll
      for (int m = 0; m < 8; ++m) {
        acc[m >> 1][m & 1] = mfma16<F16>(fb1[m & 1], fa1[m >> 1], acc[m >> 1][m & 1]);
        if (m < 4) fa0[m] = *reinterpret_cast<const bf16x8n*>(nxt + a_off + m * 512);
        else if (m < 6) fb0[m - 4] = *reinterpret_cast<const bf16x8n*>(nxt + b_off + (m - 4) * 512);
        else issue(kt + PK_NST, m - 6);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    __builtin_amdgcn_s_waitcnt(0x0070);
  }
  // The products were issued with the operands swapped (block rows = channels of the column tile), so of every 32x32
  // block a lane holds four runs of four consecutive COLUMNS of one row of H: 16-byte accesses where the rows of H allow
  // them (the padded channels beyond C are whole runs: C is a multiple of 8 here).
  const int lr = lane & 31, lk = lane >> 5;
  float* out = partial ? ws + ((long)split * pl.ntail + (L - pl.head)) * (T2 * T2) : H;
  const bool vec = partial || ((((uintptr_t)H) & 15) == 0 && (ldh & 3) == 0 && (C & 3) == 0);
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = wm * 128 + i * 32 + lr;
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int c = wn * 64 + j * 32 + 8 * g + 4 * lk;
        const floatx16& a = acc[i][j];
        if (partial) {
          *reinterpret_cast<float4*>(out + r * T2 + c) = float4{a[4 * g], a[4 * g + 1], a[4 * g + 2], a[4 * g + 3]};
        } else if (m0 + r < C && n0 + c < C) {
          float* q = H + (long)(m0 + r) * ldh + n0 + c;
          if (vec) {
            float4 val = {alpha * a[4 * g], alpha * a[4 * g + 1], alpha * a[4 * g + 2], alpha * a[4 * g + 3]};
            if (beta != 0.f) {
              const float4 o = *reinterpret_cast<const float4*>(q);
              val.x = fmaf(beta, o.x, val.x), val.y = fmaf(beta, o.y, val.y), val.z = fmaf(beta, o.z, val.z),
              val.w = fmaf(beta, o.w, val.w);
            }
            *reinterpret_cast<float4*>(q) = val;
          } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
              if (n0 + c + e < C) {
                float val = alpha * a[4 * g + e];
                if (beta != 0.f) val = fmaf(beta, q[e], val);
                q[e] = val;
              }
          }
        }
      }
  }
}
template <bool F16>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2))) void syrk_packed_kernel(
    float* __restrict__ H, long ldh, const uint16_t* __restrict__ Xp, int n_pad, int Cp, int C, float alpha, float beta,
    SyrkPlan pl, float* __restrict__ ws) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
  syrk_packed_tile<F16>(H, ldh, Xp, n_pad, Cp, C, alpha, beta, pl, ws, blockIdx.x, blockIdx.y, smem);
}

// Several independent accumulations on packed tokens (one Hessian each, same C) in one launch: blockIdx.y picks the
// problem, every workgroup runs the whole token range of its tile (no partial tiles, no workspace).
struct SyrkPackedTable {
  float* H[SYRK_MAX_GROUP];
  const uint16_t* Xp[SYRK_MAX_GROUP];
  long ldh[SYRK_MAX_GROUP];
  int n_pad[SYRK_MAX_GROUP];
  float alpha[SYRK_MAX_GROUP], beta[SYRK_MAX_GROUP];
};
template <bool F16>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2))) void syrk_packed_grouped_kernel(SyrkPackedTable t,
                                                                                                              int Cp, int C,
                                                                                                              int ntri) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
  const int z = blockIdx.y;
  syrk_packed_tile<F16>(t.H[z], t.ldh[z], t.Xp[z], t.n_pad[z], Cp, C, t.alpha[z], t.beta[z], SyrkPlan{ntri, ntri, 0, 1, 0},
                        nullptr, blockIdx.x, 0, smem);
}

// X (n x C, 16-bit, row pitch ldx; rows != nullptr: row t of the input is X[rows[t]]) -> the packed layout above and,
// when Xg != nullptr, the gathered rows once more in token-major order (n x C, row pitch ldg: what a GEMM of the
// model's forward wants).  A wavefront handles one token octet x 64 channels: lane (token j = lane % 8, channel octet
// q = lane / 8) loads 16 bytes (eight rows x 128 bytes per instruction), the 8 x 64 patch is turned in LDS, and lane c
// stores the finished cell of channel c: 1 KB of contiguous memory per store instruction.  Tokens past n and channels
// past C are zeros.
__global__ __launch_bounds__(256) void pack_tokens_kernel(const uint16_t* __restrict__ X, long ldx, const long* __restrict__ rows,
                                                         int n, int C, int Cp, uint16_t* __restrict__ Xp,
                                                         uint16_t* __restrict__ Xg, long ldg) {
  constexpr int PITCH = 64 + 8;  // 16-bit elements per LDS row: 144 bytes, so the eight rows of a column start in eight banks
  __shared__ __attribute__((aligned(16))) uint16_t patch[4][8 * PITCH];
  const int o = blockIdx.y, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int c0 = (blockIdx.x * 4 + wave) * 64;
  const int j = lane & 7, q = lane >> 3;
  const int t = 8 * o + j, c8 = c0 + 8 * q;
  uint4 v = make_uint4(0, 0, 0, 0);
  if (t < n && c8 < C) {
    const long row = rows ? rows[t] : (long)t;
    v = *reinterpret_cast<const uint4*>(X + row * ldx + c8);
    if (Xg) *reinterpret_cast<uint4*>(Xg + (long)t * ldg + c8) = v;
  }
  uint16_t* p = patch[wave];
  *reinterpret_cast<uint4*>(p + j * PITCH + 8 * q) = v;
  __syncthreads();  // (every wavefront of the grid has work: Cp is a multiple of the 256 channels a workgroup covers)
  uint32_t w[4];
#pragma unroll
  for (int k = 0; k < 4; ++k)
    w[k] = (uint32_t)p[(2 * k) * PITCH + lane] | ((uint32_t)p[(2 * k + 1) * PITCH + lane] << 16);
  *reinterpret_cast<uint4*>(Xp + ((long)o * Cp + c0 + lane) * 8) = make_uint4(w[0], w[1], w[2], w[3]);
}

constexpr int NCU = 256;  // workgroups the large-tile kernel keeps resident (one per CU)

SyrkPlan plan_big(int n, int C) {
  const int tiles = (C + T2 - 1) / T2;
  SyrkPlan pl;
  pl.ntri = tiles * (tiles + 1) / 2;
  pl.head = pl.ntri, pl.ntail = 0, pl.splits = 1, pl.tps = 0;
  int splits = 1;
  if (pl.ntri < 224) {  // too few tiles for the chip: every tile is cut, at least 2048 tokens per piece
    splits = (NCU + pl.ntri - 1) / pl.ntri;
    const int max_splits = (n + 2047) / 2048;
    if (splits > max_splits) splits = max_splits;
    if (splits > 64) splits = 64;
    if (splits > 1) pl.head = 0;
  } else {
    // The last round holds rem = ntri % NCU tiles.  Cutting them into S pieces shortens that round from 1 to
    // ceil(rem * S / NCU) / S tile times at the price of 256 KB written and read per piece, which pays when a
    // tile time is long: from 32768 tokens on, at least 4096 tokens per piece.
    static const bool tail_split = !(getenv("MQ_SYRK_TAIL") && atoi(getenv("MQ_SYRK_TAIL")) == 0);
    const int rem = pl.ntri % NCU;
    if (tail_split && rem > 0 && rem < 224 && n >= 32768) {
      double best = 1.0;
      for (int S = 2; S <= 8 && n / S >= 4096; ++S) {
        const double cost = (double)((rem * S + NCU - 1) / NCU) / S;
        if (cost < best - 0.04) best = cost, splits = S;
      }
      if (splits > 1) pl.head = pl.ntri - rem;
    }
  }
  if (splits > 1) {
    int tps = (n + splits - 1) / splits;
    tps = (tps + KT3 - 1) / KT3 * KT3;
    splits = (n + tps - 1) / tps;
    if (splits > 1) {
      pl.ntail = pl.ntri - pl.head, pl.splits = splits, pl.tps = tps;
    } else {
      pl.head = pl.ntri;
    }
  }
  return pl;
}
size_t plan_big_ws_bytes(const SyrkPlan& pl) { return (size_t)pl.ntail * pl.splits * T2 * T2 * sizeof(float); }

bool use_big(const void* X, long ldx, int n, int C) {
  return n >= 256 && C >= 256 && (C % 8 == 0) && (ldx % 8 == 0) && (((uintptr_t)X & 15) == 0);
}

constexpr size_t SMEM_BYTES = (size_t)T * EPI_LD * sizeof(float);  // 66048 >= 4*TILE_ELEMS*2 = 40960

void pick_split(int n, int C, int& ntri, int& splits, int& tps) {
  const int tiles = (C + T - 1) / T;
  ntri = tiles * (tiles + 1) / 2;
  splits = 1;
  if (ntri < 512) splits = (512 + ntri - 1) / ntri;
  const int max_splits = (n + 1023) / 1024;  // at least 1024 tokens per split
  if (splits > max_splits) splits = max_splits;
  if (splits > 64) splits = 64;
  if (splits < 1) splits = 1;
  tps = (n + splits - 1) / splits;
  tps = (tps + KT - 1) / KT * KT;
  splits = (n + tps - 1) / tps;
  if (splits < 1) splits = 1;
}

}  // namespace

extern "C" size_t mq_packed_tokens_bytes(int n, int C);
extern "C" int mq_pack_tokens(const void* X, int x_dtype, long ldx, const long* rows, int n, int C, void* Xp, void* Xg,
                              long ldg, void* stream);
extern "C" size_t mq_hessian_syrk_packed_workspace_bytes(int n, int C);
extern "C" int mq_hessian_syrk_packed(float* H, long ldh, const void* Xp, int x_dtype, int n, int C, float beta, float alpha,
                                      int mirror, void* workspace, size_t workspace_bytes, void* stream);
extern "C" int mq_hessian_syrk_packed_grouped(int groups, float* const* H, const long* ldh, const void* const* Xp, int x_dtype,
                                              const int* n, int C, const float* beta, const float* alpha, int mirror,
                                              void* stream);

// Wide Hessians with many tokens: one pass re-lays the token-major activations out for the matrix cores (6 TB/s, a
// tenth of the product's time) and the product runs on the packed-token kernel: 0.44 against 0.52 ms for 8192 tokens
// x 7168 channels, 0.385 against 0.44 ms per Hessian in calls of eight.  Narrow ones (2048 channels) and short token
// runs gain nothing and stay on the token-major kernel.
static bool route_packed(const void* X, long ldx, int n, int C) {
  return n >= 4096 && C >= 4096 && (C % 8 == 0) && (ldx % 8 == 0) && (((uintptr_t)X & 15) == 0);
}
static size_t packed_route_ws_bytes(int n, int C) {
  return n >= 4096 && C >= 4096 ? mq_packed_tokens_bytes(n, C) + mq_hessian_syrk_packed_workspace_bytes(n, C) : 0;
}

extern "C" size_t mq_hessian_syrk_workspace_bytes(int n, int C) {
  if (n <= 0 || C <= 0) return 0;
  int ntri, splits, tps;
  pick_split(n, C, ntri, splits, tps);
  const size_t small = splits > 1 ? (size_t)splits * ntri * T * T * sizeof(float) : 0;
  const size_t big = plan_big_ws_bytes(plan_big(n, C));
  const size_t packed = packed_route_ws_bytes(n, C);
  const size_t m = small > big ? small : big;  // any of the kernels may be chosen, depending on alignment
  return m > packed ? m : packed;
}

extern "C" int mq_symmetrize_upper(float* H, long ldh, int C, void* stream) {
  if (!H || C <= 0 || ldh < C) return MQ_ERR_ARG;
  const int t = (C + 63) / 64;
  hipLaunchKernelGGL(symmetrize_kernel, dim3(t * (t + 1) / 2), dim3(256), 0, (hipStream_t)stream, H, ldh, C);
  return mq_check_launch();
}

// fp32 activations: the same accumulation as upper 128x128 tiles of the fp32 GEMM core (gemm_f32_tile.hpp), whose
// products are fp32-accurate (what `input.float()` followed by addmm_ computes, up to summation order).
static int syrk_f32(float* H, long ldh, const float* X, long ldx, int n, int C, float beta, float alpha, int mirror,
                    hipStream_t st) {
  const float* Xp = X ? X : H;  // n == 0: never dereferenced, the tiles only scale H by beta
  GemmF32 g{Xp, Xp, H, 1, ldx, ldx, 1, ldh, C, C, n, alpha, beta, 1, 0, 1, 0, 0, 0};
  const int rc = mq_launch_gemm_f32(g, st);
  if (rc != MQ_OK) return rc;
  return mirror ? mq_symmetrize_upper(H, ldh, C, st) : MQ_OK;
}

extern "C" int mq_hessian_syrk(float* H, long ldh, const void* X, int x_dtype, long ldx, int n, int C, float beta,
                               float alpha, int mirror, void* workspace, size_t workspace_bytes, void* stream) {
  if (!H || C <= 0 || n < 0 || ldh < C || (n > 0 && (!X || ldx < C))) return MQ_ERR_ARG;
  if (x_dtype != MQ_DT_F32 && x_dtype != MQ_DT_BF16 && x_dtype != MQ_DT_F16) return MQ_ERR_ARG;
  hipStream_t st = (hipStream_t)stream;
  if (x_dtype == MQ_DT_F32) {
    if ((uintptr_t)X & 3) return MQ_ERR_ARG;
    return syrk_f32(H, ldh, (const float*)X, ldx, n, C, beta, alpha, mirror, st);
  }
  const bool f16 = x_dtype == MQ_DT_F16;
  if ((C & 1) || (ldx & 1) || ((uintptr_t)X & 3)) return MQ_ERR_ARG;  // 4-byte channel-pair loads
  int ntri, splits, tps;
  static std::once_flag once;
  std::call_once(once, [] {
    (void)hipFuncSetAttribute((const void*)syrk_bf16_dma8_kernel<false>, hipFuncAttributeMaxDynamicSharedMemorySize,
                              (int)DMA_SMEM);
    (void)hipFuncSetAttribute((const void*)syrk_bf16_dma8_kernel<true>, hipFuncAttributeMaxDynamicSharedMemorySize,
                              (int)DMA_SMEM);
    (void)hipFuncSetAttribute((const void*)syrk_bf16_kernel<false>, hipFuncAttributeMaxDynamicSharedMemorySize,
                              (int)SMEM_BYTES);
    (void)hipFuncSetAttribute((const void*)syrk_bf16_kernel<true>, hipFuncAttributeMaxDynamicSharedMemorySize,
                              (int)SMEM_BYTES);
    (void)hipFuncSetAttribute((const void*)syrk_reduce_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)SMEM_BYTES);
  });
  if (route_packed(X, ldx, n, C)) {
    const size_t pb = mq_packed_tokens_bytes(n, C), need = pb + mq_hessian_syrk_packed_workspace_bytes(n, C);
    if (!workspace || workspace_bytes < need || ((uintptr_t)workspace & 15)) return MQ_ERR_WORKSPACE;
    const int rc = mq_pack_tokens(X, x_dtype, ldx, nullptr, n, C, workspace, nullptr, 0, stream);
    if (rc != MQ_OK) return rc;
    return mq_hessian_syrk_packed(H, ldh, workspace, x_dtype, n, C, beta, alpha, mirror, (char*)workspace + pb,
                                  workspace_bytes - pb, stream);
  }
  if (n > 0 && use_big(X, ldx, n, C)) {
    const SyrkPlan pl = plan_big(n, C);
    const size_t need = plan_big_ws_bytes(pl);
    if (need && (!workspace || workspace_bytes < need)) return MQ_ERR_WORKSPACE;
    const dim3 grid(pl.head > pl.ntail ? pl.head : pl.ntail, pl.ntail ? 1 + pl.splits : 1);
    if (f16)
      hipLaunchKernelGGL(syrk_bf16_dma8_kernel<true>, grid, dim3(512), DMA_SMEM, st, H, ldh, (const uint16_t*)X, ldx,
                         n, C, alpha, beta, pl, (float*)workspace);
    else
      hipLaunchKernelGGL(syrk_bf16_dma8_kernel<false>, grid, dim3(512), DMA_SMEM, st, H, ldh, (const uint16_t*)X, ldx,
                         n, C, alpha, beta, pl, (float*)workspace);
    int rc = mq_check_launch();
    if (rc != MQ_OK) return rc;
    if (pl.ntail) {
      hipLaunchKernelGGL(syrk_big_reduce_kernel, dim3(T2 * T2 / 4 / 256, pl.ntail), dim3(256), 0, st, H, ldh, C, alpha, beta,
                         pl, (const float*)workspace);
      if ((rc = mq_check_launch()) != MQ_OK) return rc;
    }
    return mirror ? mq_symmetrize_upper(H, ldh, C, stream) : MQ_OK;
  }
  pick_split(n > 0 ? n : 1, C, ntri, splits, tps);
  if (splits > 1) {
    const size_t need = (size_t)splits * ntri * T * T * sizeof(float);
    if (!workspace || workspace_bytes < need) return MQ_ERR_WORKSPACE;
  }
  if (f16)
    hipLaunchKernelGGL(syrk_bf16_kernel<true>, dim3(ntri * splits), dim3(256), SMEM_BYTES, st, H, ldh, (const uint16_t*)X,
                       ldx, n, C, alpha, beta, ntri, splits, tps, (float*)workspace, mirror);
  else
    hipLaunchKernelGGL(syrk_bf16_kernel<false>, dim3(ntri * splits), dim3(256), SMEM_BYTES, st, H, ldh, (const uint16_t*)X,
                       ldx, n, C, alpha, beta, ntri, splits, tps, (float*)workspace, mirror);
  int rc = mq_check_launch();
  if (rc != MQ_OK) return rc;
  if (splits > 1) {
    hipLaunchKernelGGL(syrk_reduce_kernel, dim3(ntri), dim3(256), SMEM_BYTES, st, H, ldh, C, alpha, beta, ntri, splits,
                       (const float*)workspace, mirror);
    rc = mq_check_launch();
  }
  return rc;
}

extern "C" int mq_hessian_syrk_bf16(float* H, long ldh, const void* X, long ldx, int n, int C, float beta, float alpha,
                                    int mirror, void* workspace, size_t workspace_bytes, void* stream) {
  return mq_hessian_syrk(H, ldh, X, MQ_DT_BF16, ldx, n, C, beta, alpha, mirror, workspace, workspace_bytes, stream);
}

// Host arrays of `groups` entries each.  Problems that the direct-load kernel cannot take (few tokens, unaligned
// rows, fp32 tokens) make the whole call fall back to one plain call per problem, so the result never depends on
// the path.
extern "C" size_t mq_hessian_syrk_grouped_workspace_bytes(int groups, const int* n, int C) {
  size_t need = 0, packed = 0;
  for (int g = 0; g < groups; ++g) {
    const size_t w = mq_hessian_syrk_workspace_bytes(n[g], C);
    if (w > need) need = w;
    packed += n[g] >= 4096 && C >= 4096 ? mq_packed_tokens_bytes(n[g], C) : 0;  // the packed route packs every problem first
  }
  return need > packed ? need : packed;
}

extern "C" int mq_hessian_syrk_grouped(int groups, float* const* H, const long* ldh, const void* const* X, int x_dtype,
                                       const long* ldx, const int* n, int C, const float* beta, const float* alpha,
                                       int mirror, void* workspace, size_t workspace_bytes, void* stream) {
  if (groups < 0 || C <= 0 || (groups > 0 && (!H || !ldh || !X || !ldx || !n || !beta || !alpha))) return MQ_ERR_ARG;
  if (x_dtype != MQ_DT_F32 && x_dtype != MQ_DT_BF16 && x_dtype != MQ_DT_F16) return MQ_ERR_ARG;
  bool fast = groups > 1 && x_dtype != MQ_DT_F32;
  for (int g = 0; g < groups; ++g) {
    if (!H[g] || n[g] < 0 || ldh[g] < C || (n[g] > 0 && (!X[g] || ldx[g] < C))) return MQ_ERR_ARG;
    if (n[g] <= 0 || !use_big(X[g], ldx[g], n[g], C)) fast = false;
  }
  hipStream_t st = (hipStream_t)stream;
  bool packed = groups > 1 && x_dtype != MQ_DT_F32 && groups <= 64;
  size_t pbytes = 0;
  for (int g = 0; g < groups && packed; ++g) {
    packed = route_packed(X[g], ldx[g], n[g], C);
    pbytes += packed ? mq_packed_tokens_bytes(n[g], C) : 0;
  }
  if (packed && workspace && workspace_bytes >= pbytes && !((uintptr_t)workspace & 15)) {
    const void* Xp[64];
    char* w = (char*)workspace;
    for (int g = 0; g < groups; ++g) {
      const int rc = mq_pack_tokens(X[g], x_dtype, ldx[g], nullptr, n[g], C, w, nullptr, 0, stream);
      if (rc != MQ_OK) return rc;
      Xp[g] = w;
      w += mq_packed_tokens_bytes(n[g], C);
    }
    return mq_hessian_syrk_packed_grouped(groups, H, ldh, Xp, x_dtype, n, C, beta, alpha, mirror, stream);
  }
  if (!fast) {
    for (int g = 0; g < groups; ++g) {
      const int rc = mq_hessian_syrk(H[g], ldh[g], X[g], x_dtype, ldx[g], n[g], C, beta[g], alpha[g], mirror, workspace,
                                     workspace_bytes, stream);
      if (rc != MQ_OK) return rc;
    }
    return MQ_OK;
  }
  static std::once_flag once;
  std::call_once(once, [] {
    (void)hipFuncSetAttribute((const void*)syrk_bf16_dma_grouped_kernel<false>, hipFuncAttributeMaxDynamicSharedMemorySize,
                              (int)DMA_SMEM);
    (void)hipFuncSetAttribute((const void*)syrk_bf16_dma_grouped_kernel<true>, hipFuncAttributeMaxDynamicSharedMemorySize,
                              (int)DMA_SMEM);
  });
  const int tiles = (C + T2 - 1) / T2, ntri = tiles * (tiles + 1) / 2;
  for (int g0 = 0; g0 < groups; g0 += SYRK_MAX_GROUP) {
    const int cnt = groups - g0 < SYRK_MAX_GROUP ? groups - g0 : SYRK_MAX_GROUP;
    SyrkGroupTable t;
    for (int i = 0; i < SYRK_MAX_GROUP; ++i) {
      const int g = g0 + (i < cnt ? i : 0);
      t.H[i] = H[g];
      t.X[i] = (const uint16_t*)X[g];
      t.ldh[i] = ldh[g];
      t.ldx[i] = ldx[g];
      t.n[i] = n[g];
      t.alpha[i] = alpha[g];
      t.beta[i] = beta[g];
    }
    if (x_dtype == MQ_DT_F16)
      hipLaunchKernelGGL(syrk_bf16_dma_grouped_kernel<true>, dim3(ntri, cnt), dim3(512), DMA_SMEM, st, t, C, ntri);
    else
      hipLaunchKernelGGL(syrk_bf16_dma_grouped_kernel<false>, dim3(ntri, cnt), dim3(512), DMA_SMEM, st, t, C, ntri);
    int rc = mq_check_launch();
    if (rc != MQ_OK) return rc;
    if (mirror)
      for (int i = 0; i < cnt; ++i)
        if ((rc = mq_symmetrize_upper(H[g0 + i], ldh[g0 + i], C, stream)) != MQ_OK) return rc;
  }
  return MQ_OK;
}

extern "C" int mq_hessian_syrk_bf16_grouped(int groups, float* const* H, const long* ldh, const void* const* X,
                                            const long* ldx, const int* n, int C, const float* beta, const float* alpha,
                                            int mirror, void* workspace, size_t workspace_bytes, void* stream) {
  return mq_hessian_syrk_grouped(groups, H, ldh, X, MQ_DT_BF16, ldx, n, C, beta, alpha, mirror, workspace, workspace_bytes,
                                 stream);
}

// ---- packed tokens ------------------------------------------------------------------------------------------------
extern "C" size_t mq_packed_tokens_bytes(int n, int C) {
  if (n <= 0 || C <= 0) return 0;
  return (size_t)pk_pad_tokens(n) * pk_pad_channels(C) * 2;
}

extern "C" int mq_pack_tokens(const void* X, int x_dtype, long ldx, const long* rows, int n, int C, void* Xp, void* Xg,
                              long ldg, void* stream) {
  if (n < 0 || C <= 0 || (n > 0 && (!X || !Xp || ldx < C))) return MQ_ERR_ARG;
  if (x_dtype != MQ_DT_BF16 && x_dtype != MQ_DT_F16) return MQ_ERR_ARG;
  if ((C & 7) || (ldx & 7) || ((uintptr_t)X & 15) || ((uintptr_t)Xp & 15)) return MQ_ERR_ARG;  // 16-byte loads and cells
  if (Xg && (ldg < C || (ldg & 7) || ((uintptr_t)Xg & 15))) return MQ_ERR_ARG;
  if (n == 0) return MQ_OK;
  const int Cp = pk_pad_channels(C), octets = pk_pad_tokens(n) / 8;
  hipLaunchKernelGGL(pack_tokens_kernel, dim3(Cp / 256, octets), dim3(256), 0, (hipStream_t)stream,
                     (const uint16_t*)X, ldx, rows, n, C, Cp, (uint16_t*)Xp, (uint16_t*)Xg, ldg);
  return mq_check_launch();
}

extern "C" size_t mq_hessian_syrk_packed_workspace_bytes(int n, int C) {
  if (n <= 0 || C <= 0) return 0;
  return plan_big_ws_bytes(plan_big(pk_pad_tokens(n), pk_pad_channels(C)));
}

extern "C" int mq_hessian_syrk_packed(float* H, long ldh, const void* Xp, int x_dtype, int n, int C, float beta, float alpha,
                                      int mirror, void* workspace, size_t workspace_bytes, void* stream) {
  if (!H || C <= 0 || n <= 0 || ldh < C || !Xp || ((uintptr_t)Xp & 15)) return MQ_ERR_ARG;
  if (x_dtype != MQ_DT_BF16 && x_dtype != MQ_DT_F16) return MQ_ERR_ARG;
  hipStream_t st = (hipStream_t)stream;
  static std::once_flag once;
  std::call_once(once, [] {
    (void)hipFuncSetAttribute((const void*)syrk_packed_kernel<false>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)PK_SMEM);
    (void)hipFuncSetAttribute((const void*)syrk_packed_kernel<true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)PK_SMEM);
  });
  const int n_pad = pk_pad_tokens(n), Cp = pk_pad_channels(C);
  const SyrkPlan pl = plan_big(n_pad, Cp);
  const size_t need = plan_big_ws_bytes(pl);
  if (need && (!workspace || workspace_bytes < need)) return MQ_ERR_WORKSPACE;
  const dim3 grid(pl.head > pl.ntail ? pl.head : pl.ntail, pl.ntail ? 1 + pl.splits : 1);
  if (x_dtype == MQ_DT_F16)
    hipLaunchKernelGGL(syrk_packed_kernel<true>, grid, dim3(512), PK_SMEM, st, H, ldh, (const uint16_t*)Xp, n_pad, Cp, C, alpha,
                       beta, pl, (float*)workspace);
  else
    hipLaunchKernelGGL(syrk_packed_kernel<false>, grid, dim3(512), PK_SMEM, st, H, ldh, (const uint16_t*)Xp, n_pad, Cp, C, alpha,
                       beta, pl, (float*)workspace);
  int rc = mq_check_launch();
  if (rc != MQ_OK) return rc;
  if (pl.ntail) {
    hipLaunchKernelGGL(syrk_big_reduce_kernel, dim3(T2 * T2 / 4 / 256, pl.ntail), dim3(256), 0, st, H, ldh, C, alpha, beta, pl,
                       (const float*)workspace);
    if ((rc = mq_check_launch()) != MQ_OK) return rc;
  }
  return mirror ? mq_symmetrize_upper(H, ldh, C, stream) : MQ_OK;
}

// Host arrays of `groups` entries each; every problem n >= 1.  Up to 16 problems share a launch.
extern "C" int mq_hessian_syrk_packed_grouped(int groups, float* const* H, const long* ldh, const void* const* Xp, int x_dtype,
                                              const int* n, int C, const float* beta, const float* alpha, int mirror,
                                              void* stream) {
  if (groups < 0 || C <= 0 || (groups > 0 && (!H || !ldh || !Xp || !n || !beta || !alpha))) return MQ_ERR_ARG;
  if (x_dtype != MQ_DT_BF16 && x_dtype != MQ_DT_F16) return MQ_ERR_ARG;
  for (int g = 0; g < groups; ++g)
    if (!H[g] || !Xp[g] || n[g] <= 0 || ldh[g] < C || ((uintptr_t)Xp[g] & 15)) return MQ_ERR_ARG;
  hipStream_t st = (hipStream_t)stream;
  static std::once_flag once;
  std::call_once(once, [] {
    (void)hipFuncSetAttribute((const void*)syrk_packed_grouped_kernel<false>, hipFuncAttributeMaxDynamicSharedMemorySize,
                              (int)PK_SMEM);
    (void)hipFuncSetAttribute((const void*)syrk_packed_grouped_kernel<true>, hipFuncAttributeMaxDynamicSharedMemorySize,
                              (int)PK_SMEM);
  });
  const int Cp = pk_pad_channels(C), tiles = Cp / T2, ntri = tiles * (tiles + 1) / 2;
  for (int g0 = 0; g0 < groups; g0 += SYRK_MAX_GROUP) {
    const int cnt = groups - g0 < SYRK_MAX_GROUP ? groups - g0 : SYRK_MAX_GROUP;
    // Within a launch the problems with the most tokens go first: a workgroup runs the whole token range of its tile, so
    // with token counts far apart (the experts of a MoE layer) the long tiles should start early and the short ones
    // fill the launch's last round.
    int order[SYRK_MAX_GROUP];
    for (int i = 0; i < cnt; ++i) order[i] = g0 + i;
    for (int i = 1; i < cnt; ++i)
      for (int k = i; k > 0 && n[order[k]] > n[order[k - 1]]; --k) {
        const int tmp = order[k];
        order[k] = order[k - 1];
        order[k - 1] = tmp;
      }
    SyrkPackedTable t;
    for (int i = 0; i < SYRK_MAX_GROUP; ++i) {
      const int g = order[i < cnt ? i : 0];
      t.H[i] = H[g];
      t.Xp[i] = (const uint16_t*)Xp[g];
      t.ldh[i] = ldh[g];
      t.n_pad[i] = pk_pad_tokens(n[g]);
      t.alpha[i] = alpha[g];
      t.beta[i] = beta[g];
    }
    if (x_dtype == MQ_DT_F16)
      hipLaunchKernelGGL(syrk_packed_grouped_kernel<true>, dim3(ntri, cnt), dim3(512), PK_SMEM, st, t, Cp, C, ntri);
    else
      hipLaunchKernelGGL(syrk_packed_grouped_kernel<false>, dim3(ntri, cnt), dim3(512), PK_SMEM, st, t, Cp, C, ntri);
    int rc = mq_check_launch();
    if (rc != MQ_OK) return rc;
    if (mirror)
      for (int i = 0; i < cnt; ++i)
        if ((rc = mq_symmetrize_upper(H[g0 + i], ldh[g0 + i], C, stream)) != MQ_OK) return rc;
  }
  return MQ_OK;
}
