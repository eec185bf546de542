// GPTQ column loop for gfx950: device code, launch plan and launcher (shared by the loop's own entry points and by
// the entry point that runs a loop beside a factorisation in the same launches).
//
// Layout follows the loop's natural access: Wt is the transposed weight (C x R, one weight column per
// memory row), so a wavefront that gives one lane to each output row reads and writes fully coalesced.
// Rows of W never interact, so there is no grid-wide synchronisation anywhere.
//
//   one launch per block b of <=128 columns [i1, i2), two kinds of workgroups:
//     column workgroups : 64 rows each.  They first bring their 128 columns up to date with the previous
//                         block's errors (a 128x64x128 product on the matrix cores), then walk the columns in
//                         order (quantize -> dequantize -> error -> fused-multiply-add of the error into the
//                         remaining block columns) and leave codes, dequantized weights and the error block.
//     trailing tiles    : Wt[i2:, :] += U[earlier blocks, i2:]^T * E, the lazy-batch update of the columns beyond
//                         block b with the errors of earlier blocks, as 128x128 tiles (gemm_f32_tile.hpp): the
//                         next block always, everything beyond once per batch of blocks (see run_loop).
//   The sequential walk of block b thus overlaps the bulk of the trailing updates; the error blocks live in a
//   ring.
//
// Arithmetic per column is the reference's: q = clamp(floor(x/s + z + 0.5), 0, maxq) with IEEE division,
// y = round_to(dtype)((q - z) * s), e = y - x, w_k = fma(U[j,k], e, w_k).
//
// Second mode (ZMODE, mq_gptq_loop_chol): the same recurrence written on the Cholesky factor of H itself instead of
// the factor of its inverse (see mq_factor_chol): the multipliers are F[j,k] = -R[j,k]/R[k,k] and what a column hands
// on is not its quantization error but its total change z = y - w_original.  Nothing else differs: same walk, same
// lazy batches; the original weights come from a second, read-only copy of the transposed weights.
#pragma once
#include <hip/hip_fp16.h>

#include <cstdlib>
#include <mutex>

#include "gemm_f32_tile.hpp"

// (internal linkage: each translation unit that includes this header gets its own kernels and tuning knobs)
namespace mqloop {
namespace {

constexpr int B = 128;
constexpr int LOOP_BATCH_MAX = 8;   // the caller's E holds a ring of 2 * LOOP_BATCH_MAX error blocks
// blocks of errors per trailing update of everything beyond: 8, or env MQ_LOOP_BATCH (1..8), read once (a function-local
// static: safe whichever host thread asks first).  1, 2, 3, 4, 6, 8: 0.99, 0.83, 0.77, 0.73, 0.71, 0.70 ms per 2048x7168
// linear in grouped calls of eight; a lone call: 2.05 ms at 4, 2.2 at 8.
inline int loop_batch() {
  static const int v = [] {
    if (const char* e = getenv("MQ_LOOP_BATCH")) {
      const int x = atoi(e);
      if (x >= 1 && x <= LOOP_BATCH_MAX) return x;
    }
    return 8;
  }();
  return v;
}

__device__ __forceinline__ float round_dtype(float x, int rd) {
  // branch-free so that the unrolled column steps stay one basic block
  const float b = round_to_bf16(x);
  const float h = __half2float(__float2half_rn(x));
  return rd == 1 ? b : (rd == 2 ? h : x);
}

// Several linears of one shape walked side by side: every launch carries the column workgroups and the trailing
// tiles of all of them.  Per linear its own buffers; everything else (sizes, pitches, block schedule) is shared.
constexpr int MAX_GROUP = 16;
struct LoopGroup {
  float* Wt[MAX_GROUP];
  const float* U[MAX_GROUP];
  const float* scale[MAX_GROUP];
  const int* scale_row[MAX_GROUP];
  const float* qzero[MAX_GROUP];
  uint8_t* Qt[MAX_GROUP];
  float* E[MAX_GROUP];
  const float* W0t[MAX_GROUP];  // ZMODE: the original weights, laid out like Wt
  int n;
};
// where this launch's pieces lie inside a linear's buffers (elements)
struct LoopOffsets {
  long e_cur, e_prev;       // error block written / folded in by the column workgroups (e_prev < 0: none)
  long g_a, g_b, g_c;       // trailing update: A inside U, B inside E, C inside Wt
};

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
  int rd;
  uint8_t* Qt;
  float* E;            // errors of this block (out)
  const float* Eprev;  // errors of the previous block (nullable), nbprev columns of them
  int nbprev;
};

constexpr int MB = 16;       // micro-block: columns walked with weights in registers
constexpr int WSTRIDE = 64;  // weight tile in LDS is [column][lane]

// The 128x128 block of U in LDS: only the 16x16 micro-blocks on or above the diagonal are kept (36 of 64,
// 36 KB), row-major inside a micro-block, so that this kernel and a 128x128 GEMM tile need the same LDS.
__device__ __forceinline__ int ut_off(int j, int k) {
  const int jb = j >> 4, kb = k >> 4;
  return ((jb * (17 - jb)) / 2 + (kb - jb)) * 256 + (j & 15) * 16 + (k & 15);
}
constexpr int UT_FLOATS = 36 * 256;

typedef const int __attribute__((address_space(4))) * cint_p;  // constant address space: scalar loads

// acc += rep[lane N of this lane's row of 16 lanes] * v in one instruction: the multiplier comes through a DPP row
// broadcast.  FIRST: the two wait states required between the instruction that wrote rep and a DPP read of it (the
// compiler cannot see that this statement is a DPP instruction).
template <int N, bool FIRST>
__device__ __forceinline__ void fmac_rowbcast(float& acc, float rep, float v) {
  if (FIRST)
    asm("s_nop 1\n\tv_fmac_f32_dpp %0, %1, %2 row_newbcast:%3 row_mask:0xf bank_mask:0xf"
        : "+v"(acc)
        : "v"(rep), "v"(v), "n"(N));
  else
    asm("v_fmac_f32_dpp %0, %1, %2 row_newbcast:%3 row_mask:0xf bank_mask:0xf" : "+v"(acc) : "v"(rep), "v"(v), "n"(N));
}
template <int T, int N>
struct RowFma {  // x[T..N-1] += u[lane T.. of the row] * e
  static __device__ __forceinline__ void run(float (&x)[MB], float u, float e) {
    if constexpr (T < N) {
      fmac_rowbcast<T, T == 0>(x[T], u, e);
      RowFma<T + 1, N>::run(x, u, e);
    }
  }
};

// x[t] += sum_J U[j0+J, k0+t] * e[J] for the 16 columns k0.. and the 16 errors of columns j0.. (ascending J, one
// fused multiply-add each).  The multipliers are the same for every lane.  Row J of the 16x16 block of U is read
// from LDS once, lane l taking element l%16 (so each row of 16 lanes holds the whole row of U), and every product
// takes its multiplier from there through a DPP row broadcast: 16 LDS reads per pass instead of 64, and nothing
// but the multiply-adds in between.  (Scalar loads of U from memory measured slower: they wait on L2.)
__device__ __forceinline__ void fold16(const float* ut, const float (&e)[MB], int j0, int k0, float (&x)[MB], int lane) {
  float u[MB];
#pragma unroll
  for (int J = 0; J < MB; ++J) u[J] = ut[ut_off(j0 + J, k0) + (lane & 15)];
#pragma unroll
  for (int J = 0; J < MB; ++J) RowFma<0, MB>::run(x, u[J], e[J]);
}

// The strictly sequential part: 16 columns of one row per lane, weights in w[].  Per column, the reference's
// arithmetic: q = clamp(floor(x/s + z + 0.5), 0, maxq) with IEEE division, y = round_to(dtype)((q - z) * s),
// e = y - x, then w[t] = fma(U[j,t], e, w[t]) for the columns t still to come.  RD: 0 fp32, 1 bf16, 2 fp16.
// The multipliers U[j,t] (same for every lane) come from u[j], which holds row j of the 16x16 block of U in every row
// of 16 lanes, through DPP row broadcasts: one instruction per update.
// Each column's updates are issued at once and the scheduler is kept from moving work between columns: left
// alone it postpones a column's updates until that column is walked, which puts up to 15 dependent multiply-adds
// in front of every division.
//
// x / s with IEEE rounding, three dependent operations instead of the division's eleven (RCP): with rcp = RN(1/s)
// (a true division, but off the chain: s is known beforehand), q0 = RN(x*rcp), the exact remainder x - q0*s
// (one fma) and q1 = RN(q0 + rem*rcp) is the correctly rounded quotient (Markstein).  Where that argument does
// not apply -- s = 0 or so small that rcp overflows, a quotient beyond the fp32 range -- q0 already is what the
// division gives (an infinity or NaN), and is kept.  Used when one reciprocal serves the whole block (rcp_blk =
// 1/s computed once by the caller); with a scale per column the 16 reciprocals would cost more than they save.
struct WalkCtx {
  float rcp_blk, maxq;
  int left;  // columns of the block from this micro-block's first on
  float* esh_lane;
  float* wout;
  long ldw;
  uint8_t* qout;
  float* eout;
  long R;
};

template <int T, int J>
struct WalkFma {  // w[T..15] += U[j, T..] * e
  static __device__ __forceinline__ void run(float (&w)[MB], float u, float e) {
    if constexpr (T < MB) {
      fmac_rowbcast<T, T == J + 1>(w[T], u, e);
      WalkFma<T + 1, J>::run(w, u, e);
    }
  }
};

template <bool FULL, int RD, bool RCP, bool ZMODE, int J>
struct WalkStep {
  static __device__ __forceinline__ void run(float (&w)[MB], const float (&sc)[MB], const float (&zz)[MB],
                                             const float (&u)[MB], const float (&w0)[MB], const WalkCtx& c) {
    if constexpr (J < MB) {
      const float s = sc[J], z = zz[J];
      const float x = w[J];
      float quot;
      if (RCP) {
        const float q0 = x * c.rcp_blk;
        const float q1 = fmaf(fmaf(-q0, s, x), c.rcp_blk, q0);
        quot = fabsf(q0) < 3.0e38f ? q1 : q0;
      } else {
        quot = x / s;
      }
      const float v = quot + z;
      float q = floorf(v + 0.5f);
      q = fminf(fmaxf(q, 0.f), c.maxq);
      const float d = (q - z) * s;
      float y = d;
      if (RD == 1) {
        y = (float)(__bf16)d;  // the hardware conversion rounds to nearest even like round_to_bf16; NaN stays NaN
      } else if (RD == 2) {
        y = __half2float(__float2half_rn(d));
      }
      const float e = (FULL || J < c.left) ? (y - (ZMODE ? w0[J] : x)) : 0.f;
      WalkFma<J + 1, J>::run(w, u[J], e);  // the next column first: it is the dependence chain
      c.esh_lane[J * WSTRIDE] = e;
      if (FULL || J < c.left) {
        c.wout[(long)J * c.ldw] = y;
        c.qout[(long)J * c.R] = (uint8_t)q;
        c.eout[(long)J * c.R] = e;
      }
      __builtin_amdgcn_sched_barrier(0);
      WalkStep<FULL, RD, RCP, ZMODE, J + 1>::run(w, sc, zz, u, w0, c);
    }
  }
};

template <bool FULL, int RD, bool RCP, bool ZMODE>
__device__ __forceinline__ void walk16(float (&w)[MB], const float (&sc)[MB], const float (&zz)[MB], const float* ut,
                                       int c0, int lane, const float (&w0)[MB], const WalkCtx& c) {
  float u[MB];  // row J of the micro-block of U: lane l holds U[c0+J, c0 + l%16]
#pragma unroll
  for (int J = 0; J < MB; ++J) u[J] = ut[ut_off(c0 + J, c0) + (lane & 15)];
  WalkStep<FULL, RD, RCP, ZMODE, 0>::run(w, sc, zz, u, w0, c);
}

// One workgroup (four wavefronts) owns 64 rows; lane l of every wavefront is row l.  The 128-column
// block of those rows sits in LDS ([column][lane], so every access is conflict-free) next to the
// 128x128 block of U.  16 columns at a time move to the registers of wavefront 0 for the strictly
// sequential part; their 16 errors are published in LDS.  All four wavefronts fold them into the next 16 columns
// at once; into the rest of the block the other three fold them while wavefront 0 walks those next 16 columns,
// each taking every third pass of 16 columns.
// For every weight the updates are applied in ascending j with one fma each, exactly the order of the
// sequential reference.
//
// Nothing else runs on the CU to hide latency, so every phase issues its loads in bulk before the first
// use: the kernel is built from branch-free unrolled blocks for that reason (ROWMAP / QZERO are template
// flags, the rounding mode is a select).
// The body of one workgroup of a block's launch; bid = its index among the launch's workgroups (column workgroups of
// every linear first: they decide how long the launch takes; then the trailing tiles).
template <bool FULL, bool ROWMAP, bool QZERO, bool ZMODE>
__device__ __forceinline__ void block_body(LoopArgs a, int i1, int nb, int col_wgs, GemmF32 g, int tiles, int tiles_n, int vecA,
                                           int vecB, const LoopGroup& grp, LoopOffsets off, int bid, unsigned char* smem) {
  const int ncol = grp.n * col_wgs;
  const int e = __builtin_amdgcn_readfirstlane(bid < ncol ? bid / col_wgs : (bid - ncol) / tiles);
  a.Wt = grp.Wt[e];
  a.U = grp.U[e];
  a.scale = grp.scale[e];
  a.scale_row = grp.scale_row[e];
  a.qzero = grp.qzero[e];
  a.Qt = grp.Qt[e];
  a.E = grp.E[e] + off.e_cur;
  a.Eprev = off.e_prev >= 0 ? grp.E[e] + off.e_prev : nullptr;
  if (bid >= ncol) {  // a tile of the trailing update due at this block
    // (tiles in plain row-major order: the round-robin of workgroups over the eight XCDs then gives each XCD two
    // of the sixteen column tiles of every row tile -- measured better, in time and in bytes fetched, than one
    // contiguous run of tiles per XCD, whose working set of error blocks overflows the L2)
    const int idx = (bid - ncol) % tiles;
    g.A = a.U + off.g_a;
    g.B = grp.E[e] + off.g_b;
    g.C = a.Wt + off.g_c;
    gemmf32::tile_body<false, false>(g, idx / tiles_n, idx % tiles_n, 0, reinterpret_cast<float*>(smem), vecA, vecB);
    return;
  }
  const int wg = bid % col_wgs;
  float* tile = reinterpret_cast<float*>(smem);  // [B][WSTRIDE]
  float* ut = tile + B * WSTRIDE;                // packed upper micro-blocks of the U block
  float* esh = ut + UT_FLOATS;                   // [2][MB][WSTRIDE] errors of the current and the previous micro-block
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // a scalar: row addresses below stay in scalar registers
  const int r0 = wg * 64;
  // Lanes past the last row shadow row R-1: they compute and store exactly what that row's own lane
  // does, so no branch in this kernel ever diverges.
  const int r = min(r0 + lane, a.R - 1);
  float* __restrict__ wp = a.Wt + (long)i1 * a.ldw + r;
  // Every load of the set-up -- this block's weights, the previous block's errors, the two pieces of U -- is issued
  // before the first of them is needed; nothing else runs on the CU to hide their latency.
  float t[32];  // each wavefront stages 32 of the 128 columns
  // (scalar row base + 32-bit lane offset: one address instruction per load instead of 64-bit vector arithmetic)
  const unsigned ru = (unsigned)r;
#pragma unroll
  for (int k = 0; k < 32; ++k) {
    const float* rowp = a.Wt + (long)(i1 + min(wave * 32 + k, nb - 1)) * a.ldw;
    const float v = rowp[ru];
    t[k] = (FULL || wave * 32 + k < nb) ? v : 0.f;
  }
  const bool pre = a.Eprev != nullptr;
  // The previous block's errors, folded into this block's columns:
  //   tile[c][row] += sum_k U[i1-nbprev+k, i1+c] * Eprev[k][row].
  // Wavefront w takes columns 32w..32w+31 and all 64 rows: two 32x32 accumulators.  The errors (shared by the
  // four wavefronts) are staged in the LDS area the U block will occupy afterwards; the U operand comes
  // straight from memory in MFMA layout (lane = column, the two k of an instruction in the two lane halves).
  float* es = ut;  // [nbprev][64]
  const int m = lane & 31, slot = lane >> 5;
  float4 ev[B * 16 / 256];
  float av[B / 2];
  if (pre) {
    const bool evec = (r0 + 63 < a.R) && ((a.R & 3) == 0);
#pragma unroll
    for (int it = 0; it < B * 16 / 256; ++it) {
      const int idx = tid + it * 256;
      const int k = min(idx >> 4, a.nbprev - 1), r4 = (idx & 15) << 2;
      const float* q = a.Eprev + (long)k * a.R;
      if (evec) {
        ev[it] = *reinterpret_cast<const float4*>(q + r0 + r4);
      } else {
        ev[it].x = q[min(r0 + r4 + 0, a.R - 1)];
        ev[it].y = q[min(r0 + r4 + 1, a.R - 1)];
        ev[it].z = q[min(r0 + r4 + 2, a.R - 1)];
        ev[it].w = q[min(r0 + r4 + 3, a.R - 1)];
      }
    }
    const int col = FULL ? (wave * 32 + m) : min(wave * 32 + m, a.C - 1 - i1);
    if (a.nbprev == B) {  // the usual case: scalar row base, the lane adds its column and its k slot
      const unsigned off = (unsigned)(slot * (int)a.ldu + col);
#pragma unroll
      for (int tt = 0; tt < B / 2; ++tt) {
        const float* rowp = a.U + (long)(i1 - B + 2 * tt) * a.ldu + i1;
        av[tt] = rowp[off];
      }
    } else {
      const float* __restrict__ Uo = a.U + (long)(i1 - a.nbprev) * a.ldu + i1 + col;
#pragma unroll
      for (int tt = 0; tt < B / 2; ++tt) {
        const int k = 2 * tt + slot;
        const float v = Uo[(long)min(k, a.nbprev - 1) * a.ldu];
        av[tt] = k < a.nbprev ? v : 0.f;
      }
    }
  }
  const float* __restrict__ Ub = a.U + (long)i1 * a.ldu + i1;
  const bool vec = FULL && ((a.ldu & 3) == 0) && ((((uintptr_t)Ub) & 15) == 0);
  float4 uv[16];
  if (vec) {
#pragma unroll
    for (int u = 0; u < 16; ++u) {
      const int idx = tid + u * 256;
      const int j = idx >> 5, k = (idx & 31) << 2;
      uv[u] = (k + 3 > j) ? *reinterpret_cast<const float4*>(Ub + (long)j * a.ldu + k) : make_float4(0, 0, 0, 0);
    }
  }
#pragma unroll
  for (int k = 0; k < 32; ++k) tile[(wave * 32 + k) * WSTRIDE + lane] = t[k];
  if (pre) {
#pragma unroll
    for (int it = 0; it < B * 16 / 256; ++it) {
      const int idx = tid + it * 256;
      if ((idx >> 4) < a.nbprev) *reinterpret_cast<float4*>(&es[(idx >> 4) * 64 + ((idx & 15) << 2)]) = ev[it];
    }
    floatx16 acc0, acc1;
#pragma unroll
    for (int v = 0; v < 16; ++v) acc0[v] = acc1[v] = 0.f;
    __syncthreads();
#pragma unroll
    for (int tt = 0; tt < B / 2; ++tt) {
      const int k = min(2 * tt + slot, a.nbprev - 1);  // rows past nbprev meet a zero multiplier
      acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(av[tt], es[k * 64 + m], acc0, 0, 0, 0);
      acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(av[tt], es[k * 64 + 32 + m], acc1, 0, 0, 0);
    }
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int c = wave * 32 + 8 * (v >> 2) + 4 * slot + (v & 3);
      tile[c * WSTRIDE + m] += acc0[v];
      tile[c * WSTRIDE + 32 + m] += acc1[v];
    }
    __syncthreads();  // es is about to be overwritten by the U block
  }
  if (vec) {
#pragma unroll
    for (int u = 0; u < 16; ++u) {
      const int idx = tid + u * 256;
      const int j = idx >> 5, k = (idx & 31) << 2;
      if ((k >> 4) >= (j >> 4)) *reinterpret_cast<float4*>(&ut[ut_off(j, k)]) = uv[u];
    }
  } else {
    for (int idx = tid; idx < B * B; idx += 256) {
      const int j = idx >> 7, k = idx & 127;
      if ((k >> 4) >= (j >> 4)) ut[ut_off(j, k)] = (j < nb && k < nb && k > j) ? Ub[(long)j * a.ldu + k] : 0.f;
    }
  }
  __syncthreads();
  const float maxq = a.maxq;
  const int rd = a.rd;
  const int cend = FULL ? B : nb;
  cint_p srp = (cint_p)(a.scale_row);
  // Micro-block m (columns 16m..16m+15) is walked by wavefront 0 while the other three fold the errors of
  // micro-block m-1 into the columns beyond m.  Then all four fold the errors of m into the 16 columns of m+1 (the
  // only fold the next walk has to wait for, a quarter each).  The error buffer alternates.
  // With one scale row for the whole block (grouped scales, a group at least as wide as the block) the scale and
  // zero point are read once instead of per micro-block.
  bool one_row = false;
  float sc_blk = 0.f, zz_blk = 0.f, rcp_blk = 0.f;
  if (ROWMAP) {
    const int s0 = srp[i1];
    const int sa = a.scale_row[i1 + min(lane, cend - 1)], sb = a.scale_row[i1 + min(64 + lane, cend - 1)];
    one_row = __ballot(sa != s0 || sb != s0) == 0;  // every wavefront looks at all 128 entries: same answer in each
    if (one_row) {
      sc_blk = a.scale[(long)s0 * a.lds + r];
      zz_blk = QZERO ? a.qzero[(long)s0 * a.lds + r] : a.qzero_const;
      rcp_blk = 1.0f / sc_blk;
    }
  }
  // ZMODE: the original weights of the micro-block about to be walked, fetched one micro-block ahead by wavefront 0
  // (the walk of a micro-block hides the round trip)
  float w0n[MB];
  const float* w0p = ZMODE ? grp.W0t[e] + (long)i1 * a.ldw + r : nullptr;
  if (ZMODE && wave == 0) {
#pragma unroll
    for (int t = 0; t < MB; ++t) w0n[t] = w0p[(long)min(t, nb - 1) * a.ldw];
  }
#pragma unroll 1
  for (int c0 = 0; c0 < cend; c0 += MB) {
    const float* eprev = esh + (((c0 / MB) + 1) & 1) * MB * WSTRIDE;
    float* ecur = esh + ((c0 / MB) & 1) * MB * WSTRIDE;
    if (wave == 0) {
      float w[MB], sc[MB], zz[MB], w0[MB];
      if (ZMODE) {
#pragma unroll
        for (int t = 0; t < MB; ++t) w0[t] = w0n[t];
#pragma unroll
        for (int t = 0; t < MB; ++t) w0n[t] = w0p[(long)min(c0 + MB + t, nb - 1) * a.ldw];
      } else {
#pragma unroll
        for (int t = 0; t < MB; ++t) w0[t] = 0.f;
      }
      if (one_row) {
#pragma unroll
        for (int t = 0; t < MB; ++t) {
          sc[t] = sc_blk;
          zz[t] = zz_blk;
        }
      } else {
#pragma unroll
        for (int t = 0; t < MB; ++t) {
          const int col = FULL ? (i1 + c0 + t) : min(i1 + c0 + t, a.C - 1);
          const int srow = ROWMAP ? srp[col] : col;
          sc[t] = a.scale[(long)srow * a.lds + r];
          zz[t] = QZERO ? a.qzero[(long)srow * a.lds + r] : a.qzero_const;
        }
      }
#pragma unroll
      for (int t = 0; t < MB; ++t) w[t] = tile[(c0 + t) * WSTRIDE + lane];
      const float* utd = ut;
      const WalkCtx wc{rcp_blk, maxq, nb - c0, ecur + lane, wp + (long)c0 * a.ldw, a.ldw,
                       a.Qt + (long)(i1 + c0) * a.R + r, a.E + (long)c0 * a.R + r, a.R};
#define MQ_WALK(RD_, RCP_) walk16<FULL, RD_, RCP_, ZMODE>(w, sc, zz, utd, c0, lane, w0, wc)
      if (one_row) {
        if (rd == 1) MQ_WALK(1, true);
        else if (rd == 2) MQ_WALK(2, true);
        else MQ_WALK(0, true);
      } else {
        if (rd == 1) MQ_WALK(1, false);
        else if (rd == 2) MQ_WALK(2, false);
        else MQ_WALK(0, false);
      }
#undef MQ_WALK
    } else if (c0 > 0 && c0 + MB * wave < cend) {
      // the previous micro-block's errors: passes of 16 columns beyond micro-block c0, dealt round-robin to
      // wavefronts 1..3
      float e[MB];
#pragma unroll
      for (int J = 0; J < MB; ++J) e[J] = eprev[J * WSTRIDE + lane];
#pragma unroll 1
      for (int k0 = c0 + MB * wave; k0 < cend; k0 += 3 * MB) {
        float x[MB];
#pragma unroll
        for (int t = 0; t < MB; ++t) x[t] = tile[(k0 + t) * WSTRIDE + lane];
        fold16(ut, e, c0 - MB, k0, x, lane);
#pragma unroll
        for (int t = 0; t < MB; ++t) tile[(k0 + t) * WSTRIDE + lane] = x[t];
      }
    }
    __syncthreads();
    // this micro-block's errors into the next micro-block's columns, the only ones the walk needs at once: four
    // columns per wavefront (they already hold the previous micro-block's contribution, ascending j as ever)
    if (c0 + MB < cend) {
      const int k0 = c0 + MB + 4 * wave;
      float x[4];
      float u[MB];  // row J of the block of U above the next micro-block, rotated so that lane 0..3 of a row of 16 hold
                    // this wavefront's four columns
      float ej[MB];
#pragma unroll
      for (int t = 0; t < 4; ++t) x[t] = tile[(k0 + t) * WSTRIDE + lane];
#pragma unroll
      for (int J = 0; J < MB; ++J) {
        u[J] = ut[ut_off(c0 + J, c0 + MB) + ((lane + 4 * wave) & 15)];
        ej[J] = ecur[J * WSTRIDE + lane];
      }
#pragma unroll
      for (int J = 0; J < MB; ++J) {
        fmac_rowbcast<0, true>(x[0], u[J], ej[J]);
        fmac_rowbcast<1, false>(x[1], u[J], ej[J]);
        fmac_rowbcast<2, false>(x[2], u[J], ej[J]);
        fmac_rowbcast<3, false>(x[3], u[J], ej[J]);
      }
#pragma unroll
      for (int t = 0; t < 4; ++t) tile[(k0 + t) * WSTRIDE + lane] = x[t];
    }
    __syncthreads();
  }
}


// everything one launch takes besides the group's pointer table
struct LoopLaunch {
  LoopArgs a;
  int i1, nb, col_wgs;
  GemmF32 g;
  int tiles, tiles_n, vecA, vecB;
  LoopOffsets off;
};

template <bool FULL, bool ROWMAP, bool QZERO, bool ZMODE>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2))) void gptq_block_kernel(LoopLaunch L, LoopGroup grp) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  block_body<FULL, ROWMAP, QZERO, ZMODE>(L.a, L.i1, L.nb, L.col_wgs, L.g, L.tiles, L.tiles_n, L.vecA, L.vecB, grp, L.off,
                                         (int)blockIdx.x, smem);
}

constexpr size_t COL_SMEM = (size_t)(B * WSTRIDE + UT_FLOATS + 2 * MB * WSTRIDE) * sizeof(float);
constexpr size_t BLOCK_SMEM = COL_SMEM > gemmf32::SMEM_BYTES ? COL_SMEM : gemmf32::SMEM_BYTES;

// The launch sequence of one call: block by block, what each launch carries.
struct LoopPlan {
  LoopArgs a;
  LoopGroup grp;
  int block;
  int launches() const { return (a.C + block - 1) / block; }
  int width(int blk) const { return (blk + 1) * block <= a.C ? block : a.C - blk * block; }
  // fills L for block blk; returns the number of workgroups of its launch
  int at(int blk, LoopLaunch& L) const {
    const int i1 = blk * block, nb = width(blk), i2 = i1 + nb, G = grp.n;
    const int nbprev = blk ? block : 0;
    const int grid = (a.R + 63) / 64;
    L.a = a;
    L.a.nbprev = nbprev;
    L.i1 = i1;
    L.nb = nb;
    L.col_wgs = grid;
    // Error blocks live in a ring of 2 * loop_batch(): this block's, the previous one (the column workgroups fold it
    // into their own columns) and the batches a trailing update may still be reading.
    const int RING = 2 * loop_batch();  // a multiple of the batch: an aligned batch never wraps
    LoopOffsets& off = L.off;
    off.e_cur = (long)(blk % RING) * B * a.R;
    off.e_prev = blk ? (long)((blk - 1) % RING) * B * a.R : -1;
    // Trailing updates, Wt[i2+m, r] += sum_j U[j0+j, i2+m] * E[j, r], run beside the column walk of this block.
    // A rank-128 update of everything beyond is bound by reading and writing those columns, so with 128-column
    // blocks the errors go in batches of D blocks (aligned: blocks [mD, mD+D), neighbours in the ring).  A block
    // must hold every update but the previous block's when its walk starts.  Hence, with r = blk % D: r == 0 and
    // blk >= D: the batch just completed into everything beyond (K = 128 D); otherwise the r errors of the batch
    // under way into the next block only (K = 128 r).
    // Other block widths: the previous block's errors into everything beyond, every time.
    // (the pointers of g are filled in by the kernel from the offsets: they differ from linear to linear)
    L.g = GemmF32{nullptr, nullptr, nullptr, 1, a.ldu, a.R, 1, a.ldw, a.C - i2, a.R, nbprev, 1.f, 1.f, 0, 0, 1, 0, 0, 0};
    GemmF32& g = L.g;
    off.g_a = off.g_b = off.g_c = 0;
    L.tiles = 0;
    L.tiles_n = 1;
    L.vecA = L.vecB = 0;
    if (blk && i2 < a.C) {
      long j0 = i1 - nbprev;
      off.g_b = off.e_prev;
      if (block == B) {
        const int D = loop_batch(), r = blk % D;
        const int first = r ? blk - r : blk - D;  // first block of the errors applied now
        if (r) g.M = (a.C - i2 < block) ? a.C - i2 : block;
        j0 = (long)first * B;
        off.g_b = (long)(first % RING) * B * a.R;
        g.K = (blk - first) * B;
      }
      off.g_a = j0 * a.ldu + i2;
      off.g_c = (long)i2 * a.ldw;
      L.tiles_n = (a.R + gemmf32::BN - 1) / gemmf32::BN;
      L.tiles = ((g.M + gemmf32::BM - 1) / gemmf32::BM) * L.tiles_n;
      L.vecA = L.vecB = 1;
      for (int e = 0; e < G; ++e) {
        L.vecA &= (int)mq_gemm_operand_aligned(grp.U[e] + off.g_a, g.sak, 0);
        L.vecB &= (int)mq_gemm_operand_aligned(grp.E[e] + off.g_b, g.sbk, 0);
      }
    }
    return G * (grid + L.tiles);
  }
};

// kernel attributes: once per template instance, whichever host thread comes first
template <bool ROWMAP, bool QZERO, bool ZMODE>
inline void init_loop_kernels() {
  static std::once_flag once;
  std::call_once(once, [] {
    (void)hipFuncSetAttribute((const void*)gptq_block_kernel<true, ROWMAP, QZERO, ZMODE>,
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)BLOCK_SMEM);
    (void)hipFuncSetAttribute((const void*)gptq_block_kernel<false, ROWMAP, QZERO, ZMODE>,
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)BLOCK_SMEM);
  });
}

template <bool ROWMAP, bool QZERO, bool ZMODE>
inline int launch_block(const LoopPlan& p, int blk, hipStream_t st) {
  LoopLaunch L;
  const int wgs = p.at(blk, L);
  if (L.nb == B)
    hipLaunchKernelGGL((gptq_block_kernel<true, ROWMAP, QZERO, ZMODE>), dim3(wgs), dim3(256), BLOCK_SMEM, st, L, p.grp);
  else
    hipLaunchKernelGGL((gptq_block_kernel<false, ROWMAP, QZERO, ZMODE>), dim3(wgs), dim3(256), BLOCK_SMEM, st, L, p.grp);
  return mq_check_launch();
}

// Argument checks and the plan of a call.  W0t == nullptr: the classical loop on U.  W0t[e] (original weights, laid out
// like Wt[e]): the loop on the Cholesky multipliers F, passed in U's place.
inline int make_plan(LoopPlan& p, int G, float* const* Wt, long ldw, int C, int R, const float* const* U, long ldu,
                     const float* const* scale, long ld_scale, const int* const* scale_row, const float* const* qzero,
                     float qzero_const, float maxq, int round_dtype, int block, uint8_t* const* Qt, float* const* E,
                     const float* const* W0t, bool& rowmap, bool& qz) {
  if (G <= 0 || G > MAX_GROUP || !Wt || !U || !scale || !Qt || !E || C <= 0 || R <= 0) return MQ_ERR_ARG;
  if (ldw < R || ldu < C || ld_scale < R) return MQ_ERR_ARG;
  if (round_dtype < 0 || round_dtype > 2) return MQ_ERR_ARG;
  if (block <= 0 || block > B) block = B;  // wider blocks only reassociate the trailing sums
  LoopGroup& grp = p.grp;
  grp.n = G;
  rowmap = scale_row && scale_row[0];
  qz = qzero && qzero[0];
  for (int e = 0; e < MAX_GROUP; ++e) {
    const int k = e < G ? e : 0;
    if (!Wt[k] || !U[k] || !scale[k] || !Qt[k] || !E[k]) return MQ_ERR_ARG;
    if (((scale_row && scale_row[k]) != rowmap) || ((qzero && qzero[k]) != qz)) return MQ_ERR_ARG;  // all or none
    grp.Wt[e] = Wt[k];
    grp.U[e] = U[k];
    grp.scale[e] = scale[k];
    grp.scale_row[e] = rowmap ? scale_row[k] : nullptr;
    grp.qzero[e] = qz ? qzero[k] : nullptr;
    grp.Qt[e] = Qt[k];
    grp.E[e] = E[k];
    if (W0t && (!W0t[k] || W0t[k] == Wt[k])) return MQ_ERR_ARG;
    grp.W0t[e] = W0t ? W0t[k] : nullptr;
  }
  p.a = LoopArgs{Wt[0], ldw, C, R, U[0], ldu, scale[0], ld_scale, grp.scale_row[0], grp.qzero[0], qzero_const, maxq,
                 round_dtype, Qt[0], E[0], nullptr, 0};
  p.block = block;
  return MQ_OK;
}

}  // namespace
}  // namespace mqloop
