// Hessian hygiene of the GPTQ pre-step, entirely on the device: no value travels to the host, so a
// caller can queue many linears on several streams without a single synchronisation.
//
//   mq_hessian_prestep : (mirror the upper triangle) + NaN scan -> identity on NaN, zero diagonal entries
//                        ("pruned" input channels) set to 1 and reported as a byte mask.
//   mq_hessian_damp    : input channels whose weight column is entirely zero get their Hessian row and
//                        column cleared and a unit diagonal; then rel_damp * mean(diag) is added to the
//                        diagonal.
//
// flags (int32[4], device): [0] NaN found (H was replaced by the identity), [1] number of pruned channels,
// [2] number of cleared channels (pruned or all-zero weights), [3] unused.
#include <mutex>

#include "common.hpp"

namespace {

enum { DT_F32 = 0, DT_BF16 = 1, DT_F16 = 2 };
constexpr int STRIPS = 16;  // row strips of W scanned by separate workgroups

__device__ __forceinline__ void tri_decode64(int L, int& tm, int& tn) {
  int c = (int)((__fsqrt_rn(8.0f * (float)L + 1.0f) - 1.0f) * 0.5f);
  while (c * (c + 1) / 2 > L) --c;
  while ((c + 1) * (c + 2) / 2 <= L) ++c;
  tn = c;
  tm = L - c * (c + 1) / 2;
}

__global__ void init_flags_kernel(int* flags) {
  if (threadIdx.x < 4) flags[threadIdx.x] = 0;
}

// One workgroup per 64x64 tile pair (bi <= bj).  mirror != 0: the upper tile is copied, transposed, onto
// the lower one (only the upper triangle, diagonal included, is scanned for NaN: the rest is about to be
// overwritten).  mirror == 0: both tiles are scanned, nothing is written.
__global__ __launch_bounds__(256) void scan_mirror_kernel(float* __restrict__ H, long ldh, int C, int mirror, int* flags) {
  __shared__ float t[64][65];
  int bi, bj;
  tri_decode64(blockIdx.x, bi, bj);
  bool nan = false;
  for (int idx = threadIdx.x; idx < 64 * 64; idx += 256) {
    const int r = idx >> 6, c = idx & 63;
    const int gr = bi * 64 + r, gc = bj * 64 + c;
    if (gr < C && gc < C && (bi != bj || c >= r)) {
      const float v = H[(long)gr * ldh + gc];
      nan |= (v != v);
      t[r][c] = v;
    }
    if (!mirror) {  // lower tile: row bj*64+r, column bi*64+c (lanes along the column index)
      const int lr = bj * 64 + r, lc = bi * 64 + c;
      if (lr < C && lc < C && (bi != bj || c < r)) {
        const float w = H[(long)lr * ldh + lc];
        nan |= (w != w);
      }
    }
  }
  if (nan) atomicOr(&flags[0], 1);
  if (!mirror) return;
  __syncthreads();
  for (int idx = threadIdx.x; idx < 64 * 64; idx += 256) {
    const int r = idx >> 6, c = idx & 63;  // destination row bj*64+r, column bi*64+c
    const int gr = bj * 64 + r, gc = bi * 64 + c;
    if (gr < C && gc < C && (bi != bj || c < r)) H[(long)gr * ldh + gc] = t[c][r];
  }
}

// One workgroup per row: identity row when a NaN was found; zero diagonal -> 1 and pruned[r] = 1.
__global__ __launch_bounds__(256) void prestep_fix_kernel(float* __restrict__ H, long ldh, int C, uint8_t* __restrict__ pruned,
                                                          int* flags) {
  const int r = blockIdx.x;
  float* row = H + (long)r * ldh;
  const int nan = flags[0];
  if (nan) {
    for (int k = threadIdx.x; k < C; k += 256) row[k] = (k == r) ? 1.f : 0.f;
    if (threadIdx.x == 0) pruned[r] = 0;
    return;
  }
  if (threadIdx.x == 0) {
    const bool z = (row[r] == 0.f);
    if (z) {
      row[r] = 1.f;
      atomicAdd(&flags[1], 1);
    }
    pruned[r] = z ? 1 : 0;
  }
}

// nonzero[s][c] = 1 when rows [s*rows_per, (s+1)*rows_per) of W hold a nonzero value in column c.
// Vector path: 2-byte elements, 16-byte aligned rows; a thread scans 8 columns, 8 threads share them.
__global__ __launch_bounds__(256) void wcol_scan_vec_kernel(const uint16_t* __restrict__ W, long ldw, int R, int C,
                                                            int rows_per, uint8_t* __restrict__ nonzero) {
  __shared__ uint32_t part[8][32][4];
  const int chunk = threadIdx.x & 31, rl = threadIdx.x >> 5;
  const int c0 = (blockIdx.x * 32 + chunk) * 8;
  const int r0 = blockIdx.y * rows_per, r1 = min(R, r0 + rows_per);
  uint4 acc = make_uint4(0, 0, 0, 0);
  if (c0 < C) {
    for (int r = r0 + rl; r < r1; r += 8) {
      const uint4 v = *reinterpret_cast<const uint4*>(W + (long)r * ldw + c0);
      acc.x |= v.x; acc.y |= v.y; acc.z |= v.z; acc.w |= v.w;
    }
  }
  part[rl][chunk][0] = acc.x & 0x7fff7fffu;  // sign bits dropped: -0 counts as zero
  part[rl][chunk][1] = acc.y & 0x7fff7fffu;
  part[rl][chunk][2] = acc.z & 0x7fff7fffu;
  part[rl][chunk][3] = acc.w & 0x7fff7fffu;
  __syncthreads();
  // thread t < 256 owns column 8*(t/8) + t%8 of the workgroup's 256 columns
  const int col = threadIdx.x, ch = col >> 3, e = col & 7;
  uint32_t any = 0;
#pragma unroll
  for (int q = 0; q < 8; ++q) any |= part[q][ch][e >> 1];
  const uint32_t mine = (e & 1) ? (any >> 16) : (any & 0xffffu);
  const int c = blockIdx.x * 256 + col;
  if (c < C) nonzero[(long)blockIdx.y * C + c] = mine ? 1 : 0;
}

__global__ __launch_bounds__(256) void wcol_scan_kernel(const void* __restrict__ W, int wdt, long ldw, int R, int C,
                                                        int rows_per, uint8_t* __restrict__ nonzero) {
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= C) return;
  const int r0 = blockIdx.y * rows_per, r1 = min(R, r0 + rows_per);
  uint32_t any = 0;
  if (wdt == DT_F32) {
    const uint32_t* p = reinterpret_cast<const uint32_t*>(W);
    for (int r = r0; r < r1; ++r) any |= p[(long)r * ldw + c] & 0x7fffffffu;
  } else {
    const uint16_t* p = reinterpret_cast<const uint16_t*>(W);
    for (int r = r0; r < r1; ++r) any |= p[(long)r * ldw + c] & 0x7fffu;
  }
  nonzero[(long)blockIdx.y * C + c] = any ? 1 : 0;
}

// One workgroup: dead[c] = pruned[c] || no strip saw a nonzero weight; damp = rel_damp * mean(diag after the
// fix); sums run in a fixed order (thread-strided partials, then a tree), so the result is reproducible.
__global__ __launch_bounds__(1024) void damp_scalar_kernel(const float* __restrict__ H, long ldh, int C,
                                                           const uint8_t* __restrict__ pruned,
                                                           const uint8_t* __restrict__ nonzero, float rel_damp,
                                                           uint8_t* __restrict__ dead, float* __restrict__ damp_out, int* flags) {
  __shared__ float ssum[1024];
  __shared__ int scnt[1024];
  float s = 0.f;
  int n = 0;
  // (1024 threads and an unrolled loop: every diagonal element is its own cache line, the loads must overlap)
#pragma unroll 4
  for (int c = threadIdx.x; c < C; c += 1024) {
    uint32_t nz = 0;
#pragma unroll
    for (int q = 0; q < STRIPS; ++q) nz |= nonzero[(long)q * C + c];
    const bool d = (pruned && pruned[c]) || !nz;
    dead[c] = d ? 1 : 0;
    n += d ? 1 : 0;
    s += d ? 1.f : H[(long)c * ldh + c];
  }
  ssum[threadIdx.x] = s;
  scnt[threadIdx.x] = n;
  __syncthreads();
  for (int w = 512; w > 0; w >>= 1) {
    if (threadIdx.x < w) {
      ssum[threadIdx.x] += ssum[threadIdx.x + w];
      scnt[threadIdx.x] += scnt[threadIdx.x + w];
    }
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    damp_out[0] = rel_damp * (ssum[0] / (float)C);
    flags[2] = scnt[0];
  }
}

// One workgroup per row: clear row/column entries of dead channels, then diagonal = (dead ? 1 : d) + damp.
__global__ __launch_bounds__(256) void damp_apply_kernel(float* __restrict__ H, long ldh, int C,
                                                         const uint8_t* __restrict__ dead, const float* __restrict__ damp_in,
                                                         const int* flags) {
  const int r = blockIdx.x;
  float* row = H + (long)r * ldh;
  const int n_dead = flags[2];
  const bool rdead = dead[r] != 0;
  if (n_dead) {
    for (int k = threadIdx.x; k < C; k += 256)
      if (rdead || dead[k]) row[k] = 0.f;
    __syncthreads();
  }
  if (threadIdx.x == 0) row[r] = (rdead ? 1.f : row[r]) + damp_in[0];
}

// Hp[i, j] = H[perm[i], perm[j]]: one workgroup per output row.  The source row travels to LDS with coalesced
// loads, the column gather happens there, the output row leaves coalesced: C^2 floats read, C^2 written, no
// second intermediate (torch's H[perm][:, perm] builds two).
__global__ __launch_bounds__(256) void permute_sym_kernel(const float* __restrict__ H, long ldh, const int* __restrict__ perm,
                                                          float* __restrict__ Hp, long ldp, int C) {
  extern __shared__ __attribute__((aligned(16))) float prow[];
  const int i = blockIdx.x;
  const float* src = H + (long)perm[i] * ldh;
  for (int k = threadIdx.x; k < C; k += 256) prow[k] = src[k];
  __syncthreads();
  float* dst = Hp + (long)i * ldp;
  for (int j = threadIdx.x; j < C; j += 256) dst[j] = prow[perm[j]];
}

}  // namespace

extern "C" int mq_permute_symmetric(const float* H, long ldh, const int* perm, float* Hp, long ldp, int C, void* stream) {
  if (!H || !perm || !Hp || H == Hp || C <= 0 || ldh < C || ldp < C) return MQ_ERR_ARG;
  const size_t smem = (size_t)C * sizeof(float);
  if (smem > 160 * 1024) return MQ_ERR_TOO_LARGE;  // one source row must fit the 160 KB of LDS
  static std::mutex mu;
  static size_t allowed = 48 * 1024;
  {
    std::lock_guard<std::mutex> lock(mu);
    if (smem > allowed) {
      if (hipFuncSetAttribute((const void*)permute_sym_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) !=
          hipSuccess)
        return MQ_ERR_LAUNCH;
      allowed = smem;
    }
  }
  hipLaunchKernelGGL(permute_sym_kernel, dim3(C), dim3(256), smem, (hipStream_t)stream, H, ldh, perm, Hp, ldp, C);
  return mq_check_launch();
}

extern "C" int mq_hessian_prestep(float* H, long ldh, int C, int upper_only, uint8_t* pruned, int* flags, void* stream) {
  if (!H || !pruned || !flags || C <= 0 || ldh < C) return MQ_ERR_ARG;
  hipStream_t st = (hipStream_t)stream;
  hipLaunchKernelGGL(init_flags_kernel, dim3(1), dim3(64), 0, st, flags);
  const int t = (C + 63) / 64;
  hipLaunchKernelGGL(scan_mirror_kernel, dim3(t * (t + 1) / 2), dim3(256), 0, st, H, ldh, C, upper_only, flags);
  hipLaunchKernelGGL(prestep_fix_kernel, dim3(C), dim3(256), 0, st, H, ldh, C, pruned, flags);
  return mq_check_launch();
}

extern "C" size_t mq_hessian_damp_workspace_bytes(int C) {
  if (C <= 0) return 0;
  const size_t c = ((size_t)C + 15) / 16 * 16;
  return (STRIPS + 1) * c + 16;  // per-strip nonzero bytes, the dead mask, the damping scalar
}

extern "C" int mq_hessian_damp(float* H, long ldh, int C, const void* W, int w_dtype, long ldw, int R,
                               const uint8_t* pruned, float rel_damp, int* flags, void* workspace, size_t workspace_bytes,
                               void* stream) {
  if (!H || !W || !flags || C <= 0 || R <= 0 || ldh < C || ldw < C) return MQ_ERR_ARG;
  if (w_dtype != DT_F32 && w_dtype != DT_BF16 && w_dtype != DT_F16) return MQ_ERR_ARG;
  if (!workspace || workspace_bytes < mq_hessian_damp_workspace_bytes(C)) return MQ_ERR_WORKSPACE;
  hipStream_t st = (hipStream_t)stream;
  const size_t c = ((size_t)C + 15) / 16 * 16;
  uint8_t* nonzero = reinterpret_cast<uint8_t*>(workspace);
  uint8_t* dead = nonzero + STRIPS * c;
  float* damp = reinterpret_cast<float*>(dead + c);
  const int rows_per = (R + STRIPS - 1) / STRIPS;
  const bool vec = w_dtype != DT_F32 && (ldw % 8 == 0) && (C % 8 == 0) && (((uintptr_t)W & 15) == 0);
  if (vec) {
    hipLaunchKernelGGL(wcol_scan_vec_kernel, dim3((C + 255) / 256, STRIPS), dim3(256), 0, st, (const uint16_t*)W, ldw, R, C,
                       rows_per, nonzero);
  } else {
    hipLaunchKernelGGL(wcol_scan_kernel, dim3((C + 255) / 256, STRIPS), dim3(256), 0, st, W, w_dtype, ldw, R, C, rows_per,
                       nonzero);
  }
  // the strips are laid out with pitch C (not the padded c) inside the first STRIPS*c bytes
  hipLaunchKernelGGL(damp_scalar_kernel, dim3(1), dim3(1024), 0, st, H, ldh, C, pruned, nonzero, rel_damp, dead, damp, flags);
  hipLaunchKernelGGL(damp_apply_kernel, dim3(C), dim3(256), 0, st, H, ldh, C, dead, damp, flags);
  return mq_check_launch();
}

// ---------------------------------------------------------------------------------------------
// mq_hessian_damp for callers that cannot hand over (or allocate) a workspace: code under HIP graph capture,
// tight serving loops, harnesses that forbid allocation.  The strip masks, the dead-channel mask and the damping
// scalar live in a device array that is part of the library image: every GPU the library runs on holds its own copy
// (MQ_DAMP_NOALLOC_BYTES, about 0.53 MiB) until the process ends.
// ---------------------------------------------------------------------------------------------
namespace {
constexpr int DAMP_NOALLOC_MAX_C = 32768;
constexpr size_t DAMP_NOALLOC_BYTES = (size_t)(STRIPS + 1) * DAMP_NOALLOC_MAX_C + 16;
constexpr int MAX_DEVICES = 64;
}  // namespace

static __device__ __align__(256) unsigned char scratch[DAMP_NOALLOC_BYTES];

extern "C" int mq_hessian_damp_noalloc(float* H, long ldh, int C, const void* W, int w_dtype, long ldw, int R,
                                       const uint8_t* pruned, float rel_damp, int* flags, void* stream) {
  if (C > DAMP_NOALLOC_MAX_C) return MQ_ERR_TOO_LARGE;
  // `scratch` in host code is only a handle for the symbol: the array's device address is looked up once per
  // device (each GPU has its own copy at its own address) and that pointer is what the kernels get.
  static std::mutex mu;
  static void* dev_ptr[MAX_DEVICES] = {};
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) return MQ_ERR_LAUNCH;
  void* ptr;
  {
    std::lock_guard<std::mutex> lock(mu);
    if (!dev_ptr[dev]) {
      void* p = nullptr;
      if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) return MQ_ERR_LAUNCH;
      dev_ptr[dev] = p;
    }
    ptr = dev_ptr[dev];
  }
  // Nothing in the scratch area has to start at zero: the strip masks, the dead mask and the scalar are written in
  // full by the first two kernels before the third reads them, so the previous call's contents do not matter.
  return mq_hessian_damp(H, ldh, C, W, w_dtype, ldw, R, pruned, rel_damp, flags, ptr, DAMP_NOALLOC_BYTES, stream);
}
