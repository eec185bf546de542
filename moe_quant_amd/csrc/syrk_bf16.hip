// Hessian accumulation  H <- beta*H + alpha * X^T X  for bf16 activations X (n x C, row-major) and an
// fp32 Hessian, on the bf16 matrix cores of gfx950 (v_mfma_f32_32x32x16_bf16).
//
// bf16*bf16 products are exact in fp32, so reading the bf16 tokens directly gives the same terms as
// up-casting X to fp32 first; only the summation order differs.
//
// Only tiles of the upper block triangle are computed.  X is token-major, the matrix cores want the
// reduction index (tokens) contiguous per lane, so every thread loads a 2-channel x 8-token patch with
// eight coalesced 4-byte loads, transposes it in registers and writes two 16-byte rows into an LDS
// tile laid out [channel][token].  With too few tiles to fill 256 CUs the token range is split; the
// partial tiles go to a caller-provided workspace and are reduced in a fixed order (deterministic).
#include "common.hpp"

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
      acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a0, b0, acc[0][0], 0, 0, 0);
      acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a0, b1, acc[0][1], 0, 0, 0);
      acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a1, b0, acc[1][0], 0, 0, 0);
      acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a1, b1, acc[1][1], 0, 0, 0);
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

extern "C" size_t mq_hessian_syrk_workspace_bytes(int n, int C) {
  if (n <= 0 || C <= 0) return 0;
  int ntri, splits, tps;
  pick_split(n, C, ntri, splits, tps);
  return splits > 1 ? (size_t)splits * ntri * T * T * sizeof(float) : 0;
}

extern "C" int mq_hessian_syrk_bf16(float* H, long ldh, const void* X, long ldx, int n, int C, float beta, float alpha,
                                    int mirror, void* workspace, size_t workspace_bytes, void* stream) {
  if (!H || C <= 0 || n < 0 || ldh < C || (n > 0 && (!X || ldx < C))) return MQ_ERR_ARG;
  if ((C & 1) || (ldx & 1) || ((uintptr_t)X & 3)) return MQ_ERR_ARG;  // 4-byte channel-pair loads
  int ntri, splits, tps;
  pick_split(n > 0 ? n : 1, C, ntri, splits, tps);
  hipStream_t st = (hipStream_t)stream;
  static bool attr_done = false;
  if (!attr_done) {
    (void)hipFuncSetAttribute((const void*)syrk_bf16_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)SMEM_BYTES);
    (void)hipFuncSetAttribute((const void*)syrk_reduce_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)SMEM_BYTES);
    attr_done = true;
  }
  if (splits > 1) {
    const size_t need = (size_t)splits * ntri * T * T * sizeof(float);
    if (!workspace || workspace_bytes < need) return MQ_ERR_WORKSPACE;
  }
  hipLaunchKernelGGL(syrk_bf16_kernel, dim3(ntri * splits), dim3(256), SMEM_BYTES, st, H, ldh, (const uint16_t*)X, ldx,
                     n, C, alpha, beta, ntri, splits, tps, (float*)workspace, mirror);
  int rc = mq_check_launch();
  if (rc != MQ_OK) return rc;
  if (splits > 1) {
    hipLaunchKernelGGL(syrk_reduce_kernel, dim3(ntri), dim3(256), SMEM_BYTES, st, H, ldh, C, alpha, beta, ntri, splits,
                       (const float*)workspace, mirror);
    rc = mq_check_launch();
  }
  return rc;
}
