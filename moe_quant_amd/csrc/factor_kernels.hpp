// Damped-Hessian factorisation for GPTQ (device code and launch plan; the C entry points are in factor.hip):  given SPD H (upper triangle read), produce in place the
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
//     panel GEMM   : R_ab = H_ab * (R_bb^-1)^T            for a < b
//     trailing GEMM: H_aa' -= R_ab R_a'b^T                for a <= a' < b  (upper tiles only; applied lazily:
//                    at once only to the block column the next panel needs, to the rest several panels at a
//                    time, see factor_impl)
//   triangular inverse, one block row at a time, bottom to top, riding along in the same launches:
//     row b:  T^T = U22^T R12^T   (U22 = finished inverse of everything below/right of b, R12 = R[b, b+1:];
//                                  written to the unused mirror position below the diagonal)
//             U[b, b+1:] = -U_bb T
//     Both products only touch rows >= b, the elimination at step b only rows < b, so the first runs as extra
//     workgroups of step b's trailing-update launch and the second as extra workgroups of step b-1's panel
//     launch: the (1/3)C^3 flop of the inverse fill the CUs the late elimination steps leave idle.
//   finalize: U[j, k] /= U[j, j], strictly lower part zeroed.
#pragma once
#include <cstdlib>
#include <mutex>

#include "gemm_f32_tile.hpp"

// (internal linkage: each translation unit that includes this header gets its own kernels and tuning knobs)
namespace mqfactor {
namespace {

constexpr int NB = 128;
constexpr int SB = 32;     // sub-block edge inside the diagonal-block kernel
constexpr int LDM = 132;   // LDS row pitch: rows 16-byte aligned, consecutive rows 4 banks apart (8 rows span the 32 banks)
constexpr int SOFF = 4;    // column shift of the S triangle inside a row (keeps both triangles 16-byte aligned)
// Tuning knobs, read from the environment once (function-local statics: safe whichever host thread asks first).
inline int env_knob(const char* name, int dflt) {
  if (const char* e = getenv(name)) {
    const int v = atoi(e);
    if (v > 0) return v;
  }
  return dflt;
}
// panels per trailing update of the whole matrix (env MQ_PANELS)
inline int trail_panels() {
  static const int v = env_knob("MQ_PANELS", 8);
  return v;
}
// the first inverse product is cut into K chunks of this many blocks (4 = 512 deep), one workgroup each (env MQ_INV_KC)
inline int inv_kc() {
  static const int v = env_knob("MQ_INV_KC", 4);
  return v;
}

// ---------------------------------------------------------------------------------------------
// Diagonal block: S (128x128, upper valid) -> R^-1 where S = R R^T, R upper.
//
// One LDS array holds two triangular matrices side by side: the upper triangle S(i,k), k >= i, at
// column k+4, and below it Xt(c,k) = X[k][c], k <= c, at column k, where X accumulates R^-1 (columns
// i+1..i+3 of row i belong to neither).  Stacking M = [S; Xt] makes the inverse fall out of the
// factorisation: every elimination step that scales column j of S by 1/R_jj and subtracts its outer product
// from the columns to its left does, applied unchanged to the rows of Xt (initialised to the identity),
// exactly the right-looking update of the triangular inverse.  Nothing extra is computed for the inverse
// except more rows.
//
// Sub-blocks of 32: the 32x32 diagonal sub-block is eliminated by one wavefront with a row per lane in
// registers -- lanes 0-31 carry S rows, lanes 32-63 the matching Xt rows, same instructions -- and the
// off-diagonal work (column scaling by the sub-block inverse, outer-product updates) runs as 32x32x32
// products on the fp32 matrix cores, one product per wavefront at a time.
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ float& Sv(float* buf, int i, int k) { return buf[i * LDM + k + SOFF]; }
__device__ __forceinline__ float& Xv(float* buf, int c, int k) { return buf[c * LDM + k]; }

__device__ __forceinline__ float bcast_lane(float v, int lane) {
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), lane));
}

typedef unsigned uintx2 __attribute__((ext_vector_type(2)));

// acc -= rep[lane N of this lane's row of 16 lanes] * v, one instruction (a DPP row broadcast feeds the multiplier)
template <int N, bool FIRST>
__device__ __forceinline__ void fmac_rowbcast(float& acc, float rep, float v) {
  // FIRST: two wait states, required between the instruction that wrote rep and a DPP read of it; the
  // compiler cannot see that this statement is a DPP instruction, so the first of a run carries them itself
  if (FIRST)
    asm("s_nop 1\n\tv_fmac_f32_dpp %0, -%1, %2 row_newbcast:%3 row_mask:0xf bank_mask:0xf"
        : "+v"(acc)
        : "v"(rep), "v"(v), "n"(N));
  else
    asm("v_fmac_f32_dpp %0, -%1, %2 row_newbcast:%3 row_mask:0xf bank_mask:0xf" : "+v"(acc) : "v"(rep), "v"(v), "n"(N));
}

// columns K..0 of the rank-one update of the step before: reg[k] -= v_k * v; nearest column first, it holds the
// next pivot
template <int K, int TOP>
struct RankOne {
  static __device__ __forceinline__ void run(float (&reg)[SB], float lo, float hi, float v) {
    if constexpr (K >= 0) {
      fmac_rowbcast<(K & 15), K == TOP>(reg[K], K < 16 ? lo : hi, v);
      RankOne<K - 1, TOP>::run(reg, lo, hi, v);
    }
  }
};

// One elimination step on column J of the 32x32 sub-block held one row per lane in reg[].
// The rank-one update of step J needs v_k (the value lane k holds) as a multiplier common to all lanes, for
// every column k < J.  The 32 multipliers are replicated into every row of 16 lanes (lo: v_0..v_15, hi:
// v_16..v_31; two lane swaps) and each column then costs one multiply-add whose multiplier operand is a DPP row
// broadcast; those updates are applied one step late (vprev/lo/hi carry step J+1's vector and multipliers into
// step J), which takes the lane swaps off the dependence chain from pivot to pivot.
// The chain itself runs on values every lane holds alike, so it needs no cross-lane read at all: with
// s = S(J-1,J) and e = S(J-1,J-1), both read across lanes before the pivot's reciprocal root y is known, the
// next pivot is e - (s*y)^2: rsq, multiply, multiply-add per step.  Only the next pivot column is updated at once.
// A pivot that is not positive turns everything after it into NaN; the caller checks the diagonal afterwards.
template <int J>
struct ElimStep {
  static __device__ __forceinline__ void run(float (&reg)[SB], float dv, float vprev, float lo, float hi) {
    if constexpr (J + 1 < SB) RankOne<J - 1, J - 1>::run(reg, lo, hi, vprev);  // step J+1's updates of the columns k < J
    const float y = __frsqrt_rn(dv);
    float dnext = 0.f;
    float c = 0.f;
    if constexpr (J >= 1) {
      c = bcast_lane(reg[J], J - 1) * y;
      dnext = fmaf(-c, c, bcast_lane(reg[J - 1], J - 1));
    }
    const float v = reg[J] * y;
    reg[J] = v;
    if constexpr (J >= 1) reg[J - 1] = fmaf(-c, v, reg[J - 1]);
    float nlo = 0.f, nhi = 0.f;
    if constexpr (J >= 2) {
      const unsigned vu = __float_as_uint(v);
      const uintx2 t = __builtin_amdgcn_permlane32_swap(vu, vu, false, false);      // t[0]: lanes 0..31 twice
      const uintx2 u = __builtin_amdgcn_permlane16_swap(t[0], t[0], false, false);  // lanes 0..15 / 16..31 four times
      nlo = __uint_as_float(u[0]);
      nhi = __uint_as_float(u[1]);
    }
    // the instruction scheduler must not carry work across steps: left alone it postpones every column's updates
    // to the step that needs the column, which keeps all multipliers of all steps alive and puts them on the chain
    __builtin_amdgcn_sched_barrier(0);
    ElimStep<J - 1>::run(reg, dnext, v, nlo, nhi);
  }
};
template <>
struct ElimStep<-1> {
  static __device__ __forceinline__ void run(float (&)[SB], float, float, float, float) {}
};

// 16 consecutive floats (16-byte aligned) from LDS
__device__ __forceinline__ void ld16(const float* p, float (&v)[16]) {
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const floatx4 t = *reinterpret_cast<const floatx4*>(p + 4 * q);
    v[4 * q + 0] = t[0];
    v[4 * q + 1] = t[1];
    v[4 * q + 2] = t[2];
    v[4 * q + 3] = t[3];
  }
}

// 32x32x32 products on LDS tiles (row pitch LDM, tile origins 16-byte aligned), one wavefront each.
// Lane (x = lane%32, h = lane/32) supplies k = 16h..16h+15 of row x of both operands -- 64 contiguous bytes --
// and the product is formed transposed (operands swapped), so that the lane ends up with row x of C as four
// runs of four consecutive columns: C too moves 16 bytes at a time.
//   tile_update:  C(m,n) -= sum_k A(m,k) * B(n,k)        A_LOWER: A(m,k) counts only for k <= m
template <bool A_LOWER>
__device__ __forceinline__ void tile_update(float* c, const float* a, const float* b, int lane) {
  int x = lane & 31;
  asm volatile("" : "+v"(x));  // keeps the masks below from being hoisted out of the caller's loops
  const int h = lane >> 5;
  float av[16], bv[16];
  ld16(a + x * LDM + 16 * h, av);
  ld16(b + x * LDM + 16 * h, bv);
  floatx16 acc;
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    const floatx4 t = *reinterpret_cast<const floatx4*>(c + x * LDM + 8 * g + 4 * h);
    acc[4 * g + 0] = t[0];
    acc[4 * g + 1] = t[1];
    acc[4 * g + 2] = t[2];
    acc[4 * g + 3] = t[3];
  }
#pragma unroll
  for (int t = 0; t < 16; ++t) {
    float an = -av[t];
    if (A_LOWER) an = (16 * h + t <= x) ? an : 0.f;
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(bv[t], an, acc, 0, 0, 0);
  }
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    floatx4 t;
    t[0] = acc[4 * g + 0];
    t[1] = acc[4 * g + 1];
    t[2] = acc[4 * g + 2];
    t[3] = acc[4 * g + 3];
    *reinterpret_cast<floatx4*>(c + x * LDM + 8 * g + 4 * h) = t;
  }
}
//   tile_scale:  A(m,n) <- sum_{k >= n} A(m,k) * Xi(k,n), Xi = the lower-triangular Xt tile of the sub-block (in place)
//   tr != nullptr: the result is final (an Xt tile of the inverse); its transpose is also stored at tr
//   rd != nullptr: the result (a 32x32 piece of R) is also copied to global memory at rd (row pitch NB)
template <bool COPY_T>
__device__ __forceinline__ void tile_scale(float* a, const float* xi, float* tr, int lane, float* rd = nullptr) {
  int x = lane & 31;
  asm volatile("" : "+v"(x));  // keeps the masks below from being hoisted out of the caller's loops
  const int h = lane >> 5;
  float av[16], bv[16];
  ld16(a + x * LDM + 16 * h, av);
#pragma unroll
  for (int t = 0; t < 16; ++t) {
    const float e = xi[(16 * h + t) * LDM + x];
    bv[t] = (16 * h + t >= x) ? e : 0.f;
  }
  floatx16 acc;
#pragma unroll
  for (int v = 0; v < 16; ++v) acc[v] = 0.f;
#pragma unroll
  for (int t = 0; t < 16; ++t) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(bv[t], av[t], acc, 0, 0, 0);
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    floatx4 t;
    t[0] = acc[4 * g + 0];
    t[1] = acc[4 * g + 1];
    t[2] = acc[4 * g + 2];
    t[3] = acc[4 * g + 3];
    *reinterpret_cast<floatx4*>(a + x * LDM + 8 * g + 4 * h) = t;
    if (rd) *reinterpret_cast<floatx4*>(rd + x * NB + 8 * g + 4 * h) = t;
  }
  if (COPY_T) {
#pragma unroll
    for (int v = 0; v < 16; ++v) tr[(8 * (v >> 2) + 4 * h + (v & 3)) * LDM + x] = acc[v];
  }
}

constexpr int LDI = 36;  // row pitch of the 32x32 identity kept behind the matrix (same bank spread as LDM)

// one wavefront: eliminate the diagonal sub-block at offset o; leaves the sub-block of the inverse in Xt and,
// transposed, in the S triangle
// rd != nullptr: rows of the 32x32 piece of R (valid from the diagonal on) are also copied to global memory at rd
// (row pitch NB)
__device__ __forceinline__ void eliminate_subblock(float* buf, int o, int lane, int gidx, int* info, float* rd) {
  float reg[SB];
  const int li = lane & 31;
  const bool up = lane >= 32;
  float* row = buf + (o + li) * LDM + o;
  // S rows start from S (what a row holds left of its diagonal is other data: it stays in that lane's registers,
  // no other lane ever reads it), Xt rows from the identity
  const float* src = up ? buf + NB * LDM + li * LDI : row + SOFF;
#pragma unroll
  for (int q = 0; q < SB / 4; ++q) {
    const floatx4 t = *reinterpret_cast<const floatx4*>(src + 4 * q);
    reg[4 * q + 0] = t[0];
    reg[4 * q + 1] = t[1];
    reg[4 * q + 2] = t[2];
    reg[4 * q + 3] = t[3];
  }
  ElimStep<SB - 1>::run(reg, bcast_lane(reg[SB - 1], SB - 1), 0.f, 0.f, 0.f);
  if (rd && !up) {
#pragma unroll
    for (int q = 0; q < SB / 4; ++q) {
      const floatx4 t = {reg[4 * q], reg[4 * q + 1], reg[4 * q + 2], reg[4 * q + 3]};
      *reinterpret_cast<floatx4*>(rd + li * NB + 4 * q) = t;
    }
  }
  // The S rows are not written back to LDS: R itself is never read again there.  The Xt rows hold the sub-block of the inverse.
  // First its transpose goes into the S triangle, where the finished inverse is collected row-major for the
  // write to memory (the zeros right of a row's diagonal land left of another row's: Xt or unused columns);
  // then the rows themselves, in place, for the products that follow (the quad that straddles the diagonal
  // spills zeros into the unused columns li+1..li+3 only).
  if (up) {
#pragma unroll
    for (int k = 0; k < SB; ++k) Sv(buf, o + k, o + li) = reg[k];
#pragma unroll
    for (int q = 0; q < SB / 4; ++q) {
      const floatx4 t = {reg[4 * q], reg[4 * q + 1], reg[4 * q + 2], reg[4 * q + 3]};
      if (q <= (li >> 2)) *reinterpret_cast<floatx4*>(row + 4 * q) = t;
    }
  }
  // 1/R_jj sits on the diagonal just written: positive and finite unless pivot j or one before it failed.
  // Reported: the first failure in walking order, i.e. the highest column.
  const float dg = up ? Sv(buf, o + li, o + li) : 1.f;
  const unsigned long long fail = __ballot(!(dg > 0.f && dg < 3.0e38f));
  if (fail != 0 && lane == 0) atomicCAS(info, 0, gidx + 32 - __builtin_clzll(fail));
}

// buf: LDS, NB*LDM floats followed by a 32 x LDI identity.  blk: global 128x128 block (row pitch ld).
// gidx0: global index of its first row.  preloaded: the caller already filled Sv (upper) and zeroed the 32x32 Xt
// tiles below the diagonal ones (a barrier here orders those writes).  blk rows must be 16-byte aligned.
// rd (nullable): where the block R_bb of the factor itself goes, 128 x 128 row-major (valid on and above the diagonal).
__device__ __forceinline__ void diag_block_invert(float* buf, float* blk, long ld, int gidx0, int* info,
                                                  bool preloaded, float* rd, const float* src = nullptr, long src_ld = 0) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  for (int idx = tid; idx < SB * LDI; idx += 256) buf[NB * LDM + idx] = (idx / LDI == idx % LDI) ? 1.f : 0.f;
  if (preloaded) __syncthreads();
  if (!preloaded) {
    float4 v[16];
#pragma unroll
    for (int it = 0; it < 16; ++it) {
      const int idx = tid + it * 256, r = idx >> 5, c = (idx & 31) << 2;
      v[it] = *reinterpret_cast<const float4*>(src + (long)r * src_ld + c);
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
    // ---- phase: outer-product updates owed by column block Jp = J+1:  M(rb,K) -= V(rb) * R(K,Jp)^T for K <= J,
    //      over the S row blocks rb <= K and the Xt row blocks rb >= Jp.  Wavefront 0 takes the one tile the
    //      next elimination needs, S(J,J), and goes straight on to eliminate it; the others share the rest.
    if (J + 1 < NB / SB) {
      const int Jp = J + 1, op = Jp * SB;
      const int per_k_x = NB / SB - Jp;
      int t = 0;
      for (int K = J; K >= 0; --K) {
        const int cnt = (K + 1) + per_k_x;
        for (int q = cnt - 1; q >= 0; --q) {
          const bool is_s = q <= K;
          const int rb = is_s ? q : (Jp + (q - K - 1));
          const bool critical = is_s && K == J && rb == J;
          if (critical ? (wave != 0) : (wave == 0 || (t++ % 3) != wave - 1)) continue;
          const int ro = rb * SB, ko = K * SB;
          const int sh = is_s ? SOFF : 0;
          float* c = buf + ro * LDM + ko + sh;
          const float* a = buf + ro * LDM + op + sh;
          const float* b = buf + ko * LDM + op + SOFF;  // R(K,Jp), rows n, columns k
          if (!is_s && rb == Jp) tile_update<true>(c, a, b, lane);  // V is the sub-block inverse: lower triangle only
          else tile_update<false>(c, a, b, lane);
        }
      }
    }
    // ---- phase: elimination of the diagonal sub-block
    if (wave == 0) eliminate_subblock(buf, o, lane, gidx0 + o, info, rd ? rd + o * NB + o : nullptr);
    __syncthreads();
    // ---- phase: column block J of M times the sub-block inverse: J row blocks of S above the diagonal,
    //      3-J row blocks of Xt below it (those are final: also copied, transposed, into the S triangle)
    for (int t = wave; t < 3; t += 4) {
      const bool is_s = t < J;
      const int ro = (is_s ? t : t + 1) * SB;
      if (is_s) tile_scale<false>(buf + ro * LDM + o + SOFF, buf + o * LDM + o, nullptr, lane, rd ? rd + ro * NB + o : nullptr);
      else tile_scale<true>(buf + ro * LDM + o, buf + o * LDM + o, buf + o * LDM + ro + SOFF, lane);
    }
    __syncthreads();
  }
  // ---- phase: the S triangle now holds R^-1 row-major; written row by row, zero below the diagonal
#pragma unroll 4
  for (int it = 0; it < 16; ++it) {
    const int idx = tid + it * 256, r = idx >> 5, c = (idx & 31) << 2;
    const floatx4 t = *reinterpret_cast<const floatx4*>(buf + r * LDM + SOFF + c);
    float4 o4;
    o4.x = (r <= c + 0) ? t[0] : 0.f;
    o4.y = (r <= c + 1) ? t[1] : 0.f;
    o4.z = (r <= c + 2) ? t[2] : 0.f;
    o4.w = (r <= c + 3) ? t[3] : 0.f;
    *reinterpret_cast<float4*>(blk + (long)r * ld + c) = o4;
  }
}

// Several matrices of one size factored side by side: every launch carries the work of all of them.  The launch
// sequence is written for matrix 0; a workgroup that serves matrix e shifts every pointer by the distance from
// matrix 0's buffers to matrix e's (bytes: dA for the output buffers, dS for the input matrices).
constexpr int MAX_GROUP = 16;
struct FactorGroup {
  long dA[MAX_GROUP], dS[MAX_GROUP], dW[MAX_GROUP];  // dW: the same for the workspaces of the Cholesky-only mode
  int* info[MAX_GROUP];
  int n;
};
template <typename P>
__device__ __forceinline__ P* shifted(P* p, long bytes) {
  return reinterpret_cast<P*>(reinterpret_cast<uintptr_t>(p) + bytes);
}
// smask: which pointers of g point into the input matrix (bit 0: A, 1: B, 2: C, 3: Csrc; bit 4, trailing launches:
// workgroup 0 reads its old tile there too); the others point into the
// output buffer
__device__ __forceinline__ void rebase(GemmF32& g, const FactorGroup& grp, int e, int smask) {
  const long dA = grp.dA[e], dS = grp.dS[e];
  g.A = shifted(g.A, (smask & 1) ? dS : dA);
  g.B = shifted(g.B, (smask & 2) ? dS : dA);
  g.C = shifted(g.C, (smask & 4) ? dS : dA);
  if (g.Csrc) g.Csrc = shifted(g.Csrc, (smask & 8) ? dS : dA);
}

__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2))) void revchol_diag_kernel(const float* S, long lds,
                                                                                                    float* A, long ld, int i1,
                                                                                                    FactorGroup grp, float* Rd) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int e = blockIdx.x;
  S = shifted(S, grp.dS[e]);
  A = shifted(A, grp.dA[e]);
  float* rd = Rd ? shifted(Rd, grp.dW[e]) + (long)i1 * NB : nullptr;  // block b = i1 / NB of the workspace
  diag_block_invert(reinterpret_cast<float*>(smem), A + (long)i1 * ld + i1, ld, i1, grp.info[e], false, rd,
                    S + (long)i1 * lds + i1, lds);
}

// The next diagonal tile, brought up to date by one workgroup on its own:  S(r,c) = H(r,c) - sum_k P(r,k) P(c,k)
// for the 128x128 tile at (i1-128, i1-128), P = A[i1-128 : i1, i1 : i1+128] (the panel rows of that block).
// It sits on the dependence chain of every step, so it is not run as a generic GEMM tile: all of P goes to LDS
// once (64 KB, one barrier instead of one per K slice), only the ten 32x32 sub-tiles on or above the diagonal are
// formed, dealt 3/3/2/2 to the four wavefronts (12k instead of 16k matrix-core cycles), operands and results
// move 16 bytes at a time (transposed accumulators, as in tile_update), and the old tile is added row-wise from
// registers loaded at the very start.  The result lands in the S position of buf; left of a row's diagonal is junk.
__device__ __forceinline__ void diag_tile_update(float* buf, const float* A, long ld, int i1, const float* Hsrc, long ldh) {
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const float* P = A + (long)(i1 - NB) * ld + i1;
  const float* H = Hsrc + (long)(i1 - NB) * ldh + (i1 - NB);  // the old tile: A itself, or the caller's matrix at the first step
  floatx4 pv[16], hv[16];
#pragma unroll
  for (int it = 0; it < 16; ++it) {
    const int idx = tid + it * 256;
    pv[it] = *reinterpret_cast<const floatx4*>(P + (long)(idx >> 5) * ld + ((idx & 31) << 2));
  }
#pragma unroll
  for (int it = 0; it < 16; ++it) {
    const int idx = tid + it * 256;
    hv[it] = *reinterpret_cast<const floatx4*>(H + (long)(idx >> 5) * ldh + ((idx & 31) << 2));
  }
#pragma unroll
  for (int it = 0; it < 16; ++it) {
    const int idx = tid + it * 256;
    *reinterpret_cast<floatx4*>(buf + (idx >> 5) * LDM + ((idx & 31) << 2)) = pv[it];
  }
  __syncthreads();
  const int x = lane & 31, h = lane >> 5;
  // sub-tile list (row block, column block): wavefront w takes entries w, w+4, w+8
  constexpr int TI = 0x21110000, TJ = 0x23213210;  // nibble n: entry n (entries 0..7); entries 8, 9 below
  floatx16 acc[3];
#pragma unroll
  for (int s3 = 0; s3 < 3; ++s3) {
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[s3][v] = 0.f;
    const int e = wave + 4 * s3;
    if (e < 10) {
      const int I = e < 8 ? ((TI >> (4 * e)) & 15) : (e == 8 ? 2 : 3), Jc = e < 8 ? ((TJ >> (4 * e)) & 15) : 3;
      const float* pa = buf + (SB * I + x) * LDM + 4 * h;
      const float* pb = buf + (SB * Jc + x) * LDM + 4 * h;
#pragma unroll
      for (int j = 0; j < NB / 8; ++j) {
        const floatx4 a4 = *reinterpret_cast<const floatx4*>(pa + 8 * j);
        const floatx4 b4 = *reinterpret_cast<const floatx4*>(pb + 8 * j);
#pragma unroll
        for (int t = 0; t < 4; ++t) acc[s3] = __builtin_amdgcn_mfma_f32_32x32x2f32(b4[t], a4[t], acc[s3], 0, 0, 0);
      }
    }
  }
  __syncthreads();  // every wavefront is done reading P: its place is taken by the result
#pragma unroll
  for (int s3 = 0; s3 < 3; ++s3) {
    const int e = wave + 4 * s3;
    if (e < 10) {
      const int I = e < 8 ? ((TI >> (4 * e)) & 15) : (e == 8 ? 2 : 3), Jc = e < 8 ? ((TJ >> (4 * e)) & 15) : 3;
      float* pc = buf + (SB * I + x) * LDM + SOFF + SB * Jc + 4 * h;
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const floatx4 t = {-acc[s3][4 * g], -acc[s3][4 * g + 1], -acc[s3][4 * g + 2], -acc[s3][4 * g + 3]};
        *reinterpret_cast<floatx4*>(pc + 8 * g) = t;
      }
    }
  }
  __syncthreads();
#pragma unroll
  for (int it = 0; it < 16; ++it) {
    const int idx = tid + it * 256;
    floatx4* q = reinterpret_cast<floatx4*>(buf + (idx >> 5) * LDM + SOFF + ((idx & 31) << 2));
    *q = *q + hv[it];
  }
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

__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2))) void inv_first_kernel(GemmF32 ginv, int kc,
                                                                                                 FactorGroup grp) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  rebase(ginv, grp, blockIdx.y, 0);
  inv_first_tile(ginv, kc, blockIdx.x, reinterpret_cast<float*>(smem));
}

// One launch per elimination step b (block at offset i1, panel P = A[0:i1, i1:i1+128] already solved):
//   workgroup 0          : updates the next diagonal tile (rows/cols [i1-128, i1)) with the panel, keeps the
//                          result in LDS and inverts it right away (the next step's critical path);
//   next inv_tiles ones  : T^T = U22^T R12^T for block row b of the inverse: row tile tm (k <= its last row, U22 is
//                          triangular) times K chunk s of 512; chunk s lands 128*s columns to the right of chunk
//                          0, in the mirror area of block column b+s, free since that row's inverse is complete;
//                          the second product sums the chunks while loading them;
//   the rest             : the other upper tiles of the trailing update  A[0:i1,0:i1] -= P P^T  -- all of
//                          them, or (column_only) just the block column the next panel needs; see factor_impl.
// The diagonal-block work is thereby hidden behind the bulk of the trailing update, and the inverse behind both.
struct TrailLaunch {  // everything one launch takes besides the group's table
  GemmF32 g;
  int total;
  GemmF32 ginv;
  int inv_tiles, kc;
  float* A;
  long ld;
  int i1, column_only, others, smask;
  float* Rd;
};

__device__ __forceinline__ void trail_diag_body(GemmF32 g, int total, GemmF32 ginv, int inv_tiles, int kc, float* A, long ld,
                                                int i1, const FactorGroup& grp, int column_only, int others, int smask,
                                                float* Rd, int bid, float* buf) {
  using namespace gemmf32;
  // Workgroup order (a one-dimensional grid, so that what decides the launch's duration is dispatched first): the
  // diagonal-block workgroups of all matrices, then the inverse tiles of all matrices, then the trailing tiles.
  const int G = grp.n;
  int kind, e, idx;
  if (bid < G) {
    kind = 0, e = bid, idx = 0;
  } else if (bid < G + G * inv_tiles) {
    kind = 1, e = (bid - G) / inv_tiles, idx = (bid - G) % inv_tiles;
  } else {
    const int r = bid - G - G * inv_tiles;
    kind = 2, e = r / others, idx = r % others;
  }
  e = __builtin_amdgcn_readfirstlane(e);
  // The workgroup on the dependence chain and the deep (K = 512) tiles of the inverse decide how long the launch
  // takes; each shares its CU with a stream of short K = 128 tiles.  Wave priority lets them have the matrix pipes
  // first: the short tiles lose what the long ones gain, the launch ends earlier.
  if (kind < 2) __builtin_amdgcn_s_setprio(3);
  if (kind == 0) {
    rebase(g, grp, e, smask);
    A = shifted(A, grp.dA[e]);
    // (the last tile of the trailing update's upper-triangle order: the other workgroups cover total-1 tiles)
    // the whole tile goes to the S position: what lies left of a row's diagonal lands in that row's Xt or unused
    // columns, and the Xt part is cleared next
    const bool from_s = g.Csrc && (smask & 16);  // nothing has written this tile yet
    diag_tile_update(buf, A, ld, i1, from_s ? g.Csrc : A, from_s ? g.ldcs : ld);
    __syncthreads();
    // Xt starts at zero in its 32x32 tiles below the diagonal ones (those are written whole by the elimination)
    for (int idx2 = threadIdx.x; idx2 < (NB - SB) * (NB / 4); idx2 += 256) {
      const int r = SB + idx2 / (NB / 4), q = idx2 % (NB / 4);
      if (q < (r / SB) * (SB / 4)) *reinterpret_cast<floatx4*>(buf + r * LDM + 4 * q) = floatx4{0.f, 0.f, 0.f, 0.f};
    }
    float* rd = Rd ? shifted(Rd, grp.dW[e]) + (long)(i1 - NB) * NB : nullptr;
    diag_block_invert(buf, A + (long)(i1 - NB) * ld + (i1 - NB), ld, i1 - NB, grp.info[e], true, rd);
  } else if (kind == 1) {
    rebase(ginv, grp, e, 0);
    inv_first_tile(ginv, kc, idx, buf);
  } else {
    rebase(g, grp, e, smask);
    int tm, tn;
    const int T = i1 / NB;
    if (column_only) {  // block column T-1 above its diagonal tile, then the diagonal tile after that one
      tm = idx < T - 1 ? idx : T - 2;
      tn = idx < T - 1 ? T - 1 : T - 2;
    } else {
      tri_decode(xcd_remap(idx, total - 1), tm, tn);
    }
    tile_body<true, true>(g, tm, tn, 0, buf, 1, 1);
  }
}

__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2))) void trail_diag_kernel(TrailLaunch T, FactorGroup grp) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  trail_diag_body(T.g, T.total, T.ginv, T.inv_tiles, T.kc, T.A, T.ld, T.i1, grp, T.column_only, T.others, T.smask, T.Rd,
                  (int)blockIdx.x, reinterpret_cast<float*>(smem));
}

// Panel product of step b (P = H_ab Dinv^T, 128 columns wide, in place: tiles of 64 rows x all 128 columns)
// together with the second product of the inverse's block row b+1 (U12 = -U11 T, 128 rows high: tiles of
// 64 x 64): two independent GEMMs with K = 128 in one launch.
__global__ __launch_bounds__(256) void panel_inv_kernel(GemmF32 gp, int panel_tiles, GemmF32 g2, int inv_tiles,
                                                        FactorGroup grp, int smask_p) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  float* buf = reinterpret_cast<float*>(smem);
  const int bid = blockIdx.x, e = blockIdx.y;
  if (bid < panel_tiles) {
    rebase(gp, grp, e, smask_p);
    gemmf32::tile_short<2>(gp, bid * 64, 0, buf);
  } else {
    rebase(g2, grp, e, 0);
    const int r = bid - panel_tiles;
    gemmf32::tile_short<1>(g2, (r & 1) * 64, (r >> 1) * 64, buf);
  }
}

// U[j,k] <- U[j,k] / U[j,j] for k > j, 1 on the diagonal, 0 for k < j (normalize == 0: only the zeroing).
// One workgroup per row.  The diagonal travels through LDS: the one thread that loads it publishes the
// value before the barrier (a data dependence the compiler cannot reorder), so the thread that later
// overwrites the diagonal cannot be observed by anyone.
// A failed factorisation (*info != 0) leaves the identity, the fallback GPTQ takes when Cholesky raises.
__global__ __launch_bounds__(256) void unit_diag_kernel(float* A, long ld, int C, int normalize, FactorGroup grp) {
  __shared__ float dsh;
  const int j = blockIdx.x;
  float* row = shifted(A, grp.dA[blockIdx.y]) + (long)j * ld;
  if (*grp.info[blockIdx.y] != 0) {
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

// Cholesky-only mode: the column loop can run on R itself (H = R R^T) instead of its inverse.  With z_j the total
// change of column j (dequantized minus ORIGINAL weight), the value column k has when its turn comes is
//   x_k = w_k - (1/R_kk) sum_{j<k} z_j R[j,k],
// the same recurrence as the classical  x_k = w_k + sum_{j<k} e_j U[j,k]  (U = R^-1 with rows divided by the
// diagonal, e_j the quantization error of column j): with y = x + e the classical form reads y = w + e D^-1 R^-1,
// i.e. (y - w) R = e D^-1, which row k solves to the line above.  So the loop takes the multipliers
//   F[j,k] = -R[j,k] / R[k,k]   (k > j)
// and the triangular inverse, half the flop of the factorisation, is never formed.
// One workgroup per upper 128x128 tile, in place: off-diagonal tiles hold R; a diagonal tile holds the inverse of
// its block (of which only the diagonal, 1/R_kk, is used here), its R block comes from the workspace.  The diagonal
// of F and everything below it is left as it is: the loop reads k > j only.
// A failed factorisation (*info != 0) leaves F = 0 above the diagonal: the identity fallback of the reference.
__global__ __launch_bounds__(256) void chol_finalize_kernel(float* A, long ld, int C, FactorGroup grp, const float* Rd) {
  __shared__ float dcol[NB];
  const int e = blockIdx.y;
  A = shifted(A, grp.dA[e]);
  Rd = shifted(Rd, grp.dW[e]);
  int tm, tn;
  gemmf32::tri_decode(blockIdx.x, tm, tn);
  const int m0 = tm * NB, n0 = tn * NB, tid = threadIdx.x;
  const bool failed = *grp.info[e] != 0;
  if (tid < NB) dcol[tid] = A[(long)(n0 + tid) * ld + n0 + tid];  // 1 / R_kk
  __syncthreads();
#pragma unroll 4
  for (int it = 0; it < 16; ++it) {
    const int idx = tid + it * 256, r = idx >> 5, c = (idx & 31) << 2;
    float* q = A + (long)(m0 + r) * ld + n0 + c;
    if (tm != tn) {
      floatx4 v = *reinterpret_cast<const floatx4*>(q);
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] = failed ? 0.f : -(v[i] * dcol[c + i]);
      *reinterpret_cast<floatx4*>(q) = v;
    } else if (c + 3 > r) {  // the quad holds at least one element right of the diagonal
      const floatx4 rv = *reinterpret_cast<const floatx4*>(Rd + (long)(m0 + r) * NB + c);
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (c + i > r) q[i] = failed ? 0.f : -(rv[i] * dcol[c + i]);
    }
  }
}

constexpr size_t DIAG_SMEM = (size_t)(NB * LDM + SB * LDI) * sizeof(float);
constexpr size_t FUSED_SMEM = DIAG_SMEM > gemmf32::SMEM_BYTES ? DIAG_SMEM : gemmf32::SMEM_BYTES;


// The launch sequence of one call (a group of matrices of one size factored side by side).
// S[e]: the matrices to factor (upper triangle read), A[e]: where the factors are built and left.  S[e] == A[e] for
// every e: in place.  All matrices share C and the two pitches.
// ws == nullptr: the inverse factor U.  ws[e] (C*128 floats each): Cholesky-only mode, the loop multipliers F.
struct FactorPlan {
  FactorGroup grp;
  const float* S0;
  float* A;
  long lds, ld;
  int C, normalize, B;
  bool in_place, chol;
  float* Rd;

  int init(int G, const float* const* S, long lds_, float* const* Aout, long ld_, int C_, int normalize_, int* const* infos,
           float* const* ws) {
    if (G <= 0 || G > MAX_GROUP || !S || !Aout || !infos || C_ <= 0 || ld_ < C_ || lds_ < C_) return MQ_ERR_ARG;
    if (C_ % NB != 0) return MQ_ERR_ARG;  // the host pads with an identity block
    grp.n = G;
    in_place = S[0] == Aout[0];
    for (int e = 0; e < MAX_GROUP; ++e) {
      const int k = e < G ? e : 0;
      if (!S[k] || !Aout[k] || !infos[k] || ((S[k] == Aout[k]) != in_place)) return MQ_ERR_ARG;
      if ((ld_ & 3) || ((uintptr_t)Aout[k] & 15) || (lds_ & 3) || ((uintptr_t)S[k] & 15)) return MQ_ERR_ARG;  // float4 rows
      grp.dA[e] = (long)((intptr_t)Aout[k] - (intptr_t)Aout[0]);
      grp.dS[e] = (long)((intptr_t)S[k] - (intptr_t)S[0]);
      grp.info[e] = infos[k];
      if (ws && (!ws[k] || ((uintptr_t)ws[k] & 15))) return MQ_ERR_WORKSPACE;
      grp.dW[e] = ws ? (long)((intptr_t)ws[k] - (intptr_t)ws[0]) : 0;
    }
    Rd = ws ? ws[0] : nullptr;
    chol = Rd != nullptr;
    S0 = S[0];
    A = Aout[0];
    lds = lds_;
    ld = ld_;
    C = C_;
    normalize = normalize_;
    B = C / NB;
    return MQ_OK;
  }

  // kernel attributes: set once, whichever host thread comes first
  static void init_kernels() {
    static std::once_flag once;
    std::call_once(once, [] {
      (void)hipFuncSetAttribute((const void*)revchol_diag_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)DIAG_SMEM);
      (void)hipFuncSetAttribute((const void*)trail_diag_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)FUSED_SMEM);
      (void)hipFuncSetAttribute((const void*)panel_inv_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)gemmf32::short_smem_bytes(2));
      (void)hipFuncSetAttribute((const void*)inv_first_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)gemmf32::SMEM_BYTES);
    });
  }

  int kc_of(int) const { return inv_kc(); }  // one depth for all block rows: 2, 3 for the short rows measured no faster
  // the two products of block row b of the inverse (w = columns to the right of b)
  GemmF32 inv_first(int b, int& tiles) const {  // T^T (w x 128) = U22^T (w x w) * R12^T (w x 128), in K chunks
    const long p = (long)b * NB;
    const int w = C - (int)p - NB;
    const int kc = kc_of(w);
    tiles = (w / NB) * ((w / NB + kc - 1) / kc);
    return GemmF32{A + (p + NB) * ld + (p + NB), A + p * ld + (p + NB), A + (p + NB) * ld + p, 1, ld, 1, ld, ld,
                   w, NB, w, 1.f, 0.f, 0, 1, 1, 0, 0, 0};
  }
  GemmF32 inv_second(int b, int& tiles) const {  // U12 (128 x w) = -U11 (128 x 128) * T,  T(k,n) = Tt[n][k]
    const long p = (long)b * NB;
    const int w = C - (int)p - NB;
    tiles = w / NB;
    return GemmF32{A + p * ld + p, A + (p + NB) * ld + p, A + p * ld + (p + NB), ld, 1, 1, ld, ld,
                   NB, w, NB, -1.f, 0.f, 0, 0, 1, 0, 0, 0, (w / NB + kc_of(w) - 1) / kc_of(w), kc_of(w), NB};
  }

  int steps() const { return B - 1; }  // elimination steps; step s eliminates block b = B - 1 - s

  int first(hipStream_t st) const {  // the last diagonal block
    hipLaunchKernelGGL(revchol_diag_kernel, dim3(grp.n), dim3(256), DIAG_SMEM, st, S0, lds, A, ld, C - NB, grp, Rd);
    return mq_check_launch();
  }

  // the panel of step s (with, in the inverse mode, the second product of an earlier block row)
  int panel(int s, hipStream_t st) const {
    const int b = B - 1 - s, i1 = b * NB, G = grp.n;
    float* P = A + i1;  // panel: rows [0,i1), cols [i1, i1+NB)
    const float* Dinv = A + (long)i1 * ld + i1;
    // the first step reads what no earlier step has touched: from S (every later read finds its data in A)
    const bool first = (b == B - 1) && !in_place;
    GemmF32 panel{first ? S0 + i1 : P, Dinv, P, first ? lds : ld, 1, 1, ld, ld, i1, NB, NB, 1.f, 0.f, 0, 0, 1, 0, 0, 0};
    int t2 = 0;
    GemmF32 g2 = panel;
    if (!chol && b + 1 <= B - 2) g2 = inv_second(b + 1, t2);  // row b+1: its T was produced in the previous launch
    static_assert(NB == gemmf32::SHORT_K, "the panel kernel's tiles take K = 128");
    hipLaunchKernelGGL(panel_inv_kernel, dim3(2 * b + 4 * t2, G), dim3(256), gemmf32::short_smem_bytes(2), st, panel, 2 * b,
                       g2, 4 * t2, grp, first ? 1 : 0);
    return mq_check_launch();
  }

  // The trailing launch of step s: fills T, returns its number of workgroups.
  // The trailing update A[0:i1,0:i1] -= P P^T with one 128-wide panel is bound by reading and writing the
  // trailing matrix, so the panels go in trail_panels() at a time.  Only block column b-1 has to be complete for the
  // next panel, and workgroup 0 owns its diagonal tile.  Steps in between (column_only): the j panels block column
  // b-1 still lacks -- this one and the j-1 before it, neighbours in memory, A[:, i1 : i1+128j], one product with
  // K = 128j -- into that block column alone, and already into the diagonal tile after the next one, (b-2, b-2).
  // Every trail_panels()-th step: the last trail_panels() panels into every tile but (b-1, b-1), which had all but
  // this panel one step early and takes this one from workgroup 0 as always.
  // Out of place, no launch exists only to carry the matrix from S to A: through the first trail_panels() steps a tile
  // is written for the first time by whichever launch updates it, and that launch takes the old values from S -- the
  // block column and the early diagonal tile of a column-only step, every tile of the first full update; workgroup 0
  // reads S at step 0 alone (from step 1 on its tile is the one the step before wrote early).
  // (2, 3, 4, 6 panels: 306, 311, 314, 315 linears/s at four streams against 286 with one; a single
  // factorisation takes 3.21 -> 3.28 ms with four, the steps in between leave the chip idle.)
  int trail(int s, TrailLaunch& T) const {
    const int b = B - 1 - s, i1 = b * NB, G = grp.n;
    float* P = A + i1;
    const int TP = trail_panels();
    const int j = s % TP + 1;  // panels owed to block column b-1
    const int column_only = j < TP;
    const bool fresh = !in_place && s < TP;  // the tiles of this launch (workgroup 0's aside) hold nothing yet
    GemmF32 trail{P, P, A, ld, 1, 1, ld, ld, i1, i1, j * NB, -1.f, 1.f, 1, 0, 1, 0, 0, 0};
    if (fresh) {
      trail.Csrc = S0;
      trail.ldcs = lds;
    }
    const int tiles = i1 / NB, total = tiles * (tiles + 1) / 2;
    const int others = column_only ? (b - 1) + (b >= 2 ? 1 : 0) : total - 1;  // tiles besides workgroup 0's
    int t1 = 0;
    GemmF32 g1 = trail;
    if (!chol && b <= B - 2) g1 = inv_first(b, t1);  // rows > b of the inverse are complete
    T = TrailLaunch{trail, total, g1, t1, kc_of(C - i1 - NB), A, ld, i1, column_only, others,
                    (fresh ? 8 : 0) | (fresh && s == 0 ? 16 : 0), Rd};
    return G * (1 + t1 + others);
  }

  int launch_trail(int s, hipStream_t st) const {
    TrailLaunch T;
    const int wgs = trail(s, T);
    hipLaunchKernelGGL(trail_diag_kernel, dim3(wgs), dim3(256), FUSED_SMEM, st, T, grp);
    return mq_check_launch();
  }

  // after the last step: the multipliers F (Cholesky-only mode), or what is left of the inverse and its scaling
  int finish(hipStream_t st) const {
    const int G = grp.n;
    int rc;
    if (chol) {
      hipLaunchKernelGGL(chol_finalize_kernel, dim3(B * (B + 1) / 2, G), dim3(256), 0, st, A, ld, C, grp, (const float*)Rd);
      return mq_check_launch();
    }
    // what is left of the inverse once the elimination has reached the top: second product of row 1, both of row 0
    if (B >= 3) {
      int t2;
      GemmF32 g2 = inv_second(1, t2);
      hipLaunchKernelGGL(panel_inv_kernel, dim3(4 * t2, G), dim3(256), gemmf32::short_smem_bytes(2), st, g2, 0, g2, 4 * t2,
                         grp, 0);
      if ((rc = mq_check_launch()) != MQ_OK) return rc;
    }
    if (B >= 2) {
      int t;
      GemmF32 g1 = inv_first(0, t);
      hipLaunchKernelGGL(inv_first_kernel, dim3(t, G), dim3(256), gemmf32::SMEM_BYTES, st, g1, kc_of(C - NB), grp);
      if ((rc = mq_check_launch()) != MQ_OK) return rc;
      GemmF32 g2 = inv_second(0, t);
      hipLaunchKernelGGL(panel_inv_kernel, dim3(4 * t, G), dim3(256), gemmf32::short_smem_bytes(2), st, g2, 0, g2, 4 * t, grp,
                         0);
      if ((rc = mq_check_launch()) != MQ_OK) return rc;
    }
    hipLaunchKernelGGL(unit_diag_kernel, dim3(C, G), dim3(256), 0, st, A, ld, C, normalize, grp);
    return mq_check_launch();
  }
};

}  // namespace
}  // namespace mqfactor
