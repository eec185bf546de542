/* Plain-C restatement of the GPTQ column loop and the int4 packer.  TEST INFRASTRUCTURE ONLY: it is a
 * second, independently written checker beside oracle/gptq_oracle.py (exact fmaf, IEEE division) and is
 * never linked into or called by the shipped library.
 *
 * Follows MoE-Quant src/gptq_loop.py:141-148 (loop), :28-40 (quantize_error kernel), :77-88 (addvv kernel)
 * and src/quant_utils.py:30-49 (tl_round = floor(x+0.5), tl_quantize, tl_dequantize); packing follows
 * pack_quantized_model.py:66-67 with compressed_tensors.pack_to_int32's published layout.
 * Pinned by tests/test_oracle_loop.py (closed forms, fp64 textbook GPTQ, agreement with the torch oracle).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

static float round_bf16(float x) {
  uint32_t u;
  memcpy(&u, &x, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return x;
  u += 0x7fffu + ((u >> 16) & 1u);
  u &= 0xffff0000u;
  memcpy(&x, &u, 4);
  return x;
}

/* Wt: C x R (in/out), U: C x C, scale/qzero: C x R, Q: C x R out (codes as float, like the reference).
 * round_dtype: 0 none, 1 bf16.  Returns 0. */
int mq_ref_gptq_loop(float* Wt, int C, int R, const float* U, const float* scale, const float* qzero, float maxq,
                     int round_dtype, int block, float* Q) {
  if (block <= 0) block = C; /* src/gptq_loop.py:212-213 */
  float* E = (float*)malloc((size_t)block * R * sizeof(float));
  float* acc = (float*)malloc((size_t)R * sizeof(float));
  if (!E || !acc) return -1;
  for (int i1 = 0; i1 < C; i1 += block) {
    const int i2 = i1 + block < C ? i1 + block : C;
    for (int j = i1; j < i2; ++j) {
      float* x = Wt + (size_t)j * R;
      float* e = E + (size_t)(j - i1) * R;
      for (int r = 0; r < R; ++r) {
        const float s = scale[(size_t)j * R + r], z = qzero[(size_t)j * R + r];
        float q = floorf(x[r] / s + z + 0.5f); /* tl_round(x / scale + qzero) */
        q = fminf(fmaxf(q, 0.0f), maxq);       /* tl.clamp */
        float y = (q - z) * s;
        if (round_dtype == 1) y = round_bf16(y);
        e[r] = y - x[r];
        x[r] = y;
        Q[(size_t)j * R + r] = q;
      }
      for (int k = j + 1; k < i2; ++k) { /* addvv: C[a,:] = fma(va[a], vb[:], C[a,:]) */
        const float h = U[(size_t)j * C + k];
        float* wk = Wt + (size_t)k * R;
        for (int r = 0; r < R; ++r) wk[r] = fmaf(h, e[r], wk[r]);
      }
    }
    for (int k = i2; k < C; ++k) { /* weight[i2:] += U[i1:i2, i2:]^T @ E, zero-initialised fp32 accumulator */
      float* wk = Wt + (size_t)k * R;
      memset(acc, 0, (size_t)R * sizeof(float));
      for (int j = i1; j < i2; ++j) {
        const float h = U[(size_t)j * C + k];
        const float* e = E + (size_t)(j - i1) * R;
        for (int r = 0; r < R; ++r) acc[r] = fmaf(h, e[r], acc[r]);
      }
      for (int r = 0; r < R; ++r) wk[r] += acc[r];
    }
  }
  free(E);
  free(acc);
  return 0;
}

/* word[r,k] = sum_i ((codes[r,8k+i] - zero + 8) & 15) << 4i with zero = 8 (symmetric); columns past C are 0 */
void mq_ref_pack_int4(const uint8_t* codes, int R, int C, int32_t* out) {
  const int words = (C + 7) / 8;
  for (int r = 0; r < R; ++r)
    for (int k = 0; k < words; ++k) {
      uint32_t w = 0;
      for (int i = 0; i < 8; ++i) {
        const int c = 8 * k + i;
        if (c < C) w |= (uint32_t)(((int)codes[(size_t)r * C + c] - 8 + 8) & 15) << (4 * i);
      }
      out[(size_t)r * words + k] = (int32_t)w;
    }
}
