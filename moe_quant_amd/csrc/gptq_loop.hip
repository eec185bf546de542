// GPTQ column loop for gfx950: the C entry points (device code and launch plan: loop_kernels.hpp).
#include "loop_kernels.hpp"

namespace {

using namespace mqloop;

template <bool ROWMAP, bool QZERO, bool ZMODE>
int run_loop(const LoopPlan& p, hipStream_t st) {
  init_loop_kernels<ROWMAP, QZERO, ZMODE>();
  for (int blk = 0, n = p.launches(); blk < n; ++blk) {
    const int rc = launch_block<ROWMAP, QZERO, ZMODE>(p, blk, st);
    if (rc != MQ_OK) return rc;
  }
  return MQ_OK;
}

int loop_impl(int G, float* const* Wt, long ldw, int C, int R, const float* const* U, long ldu, const float* const* scale,
              long ld_scale, const int* const* scale_row, const float* const* qzero, float qzero_const, float maxq,
              int round_dtype, int block, uint8_t* const* Qt, float* const* E, const float* const* W0t, void* stream) {
  LoopPlan p;
  bool rowmap, qz;
  const int rc = make_plan(p, G, Wt, ldw, C, R, U, ldu, scale, ld_scale, scale_row, qzero, qzero_const, maxq, round_dtype,
                           block, Qt, E, W0t, rowmap, qz);
  if (rc != MQ_OK) return rc;
  hipStream_t st = (hipStream_t)stream;
  if (W0t) {
    if (rowmap) return qz ? run_loop<true, true, true>(p, st) : run_loop<true, false, true>(p, st);
    return qz ? run_loop<false, true, true>(p, st) : run_loop<false, false, true>(p, st);
  }
  if (rowmap) return qz ? run_loop<true, true, false>(p, st) : run_loop<true, false, false>(p, st);
  return qz ? run_loop<false, true, false>(p, st) : run_loop<false, false, false>(p, st);
}

}  // namespace

extern "C" size_t mq_gptq_loop_scratch_bytes(int R) {
  return R > 0 ? (size_t)2 * LOOP_BATCH_MAX * B * R * sizeof(float) : 0;
}

extern "C" int mq_gptq_loop(float* Wt, long ldw, int C, int R, const float* U, long ldu, const float* scale,
                            long ld_scale, const int* scale_row, const float* qzero, float qzero_const, float maxq,
                            int round_dtype, int block, uint8_t* Qt, float* E, void* stream) {
  return loop_impl(1, &Wt, ldw, C, R, &U, ldu, &scale, ld_scale, &scale_row, &qzero, qzero_const, maxq, round_dtype, block,
                   &Qt, &E, nullptr, stream);
}

// `groups` linears of one shape in one sequence of launches (host arrays of device pointers; scale_row / qzero: NULL,
// or arrays whose entries are all NULL or all set).  More than MAX_GROUP linears run as consecutive batches.
extern "C" int mq_gptq_loop_grouped(int groups, float* const* Wt, long ldw, int C, int R, const float* const* U, long ldu,
                                    const float* const* scale, long ld_scale, const int* const* scale_row,
                                    const float* const* qzero, float qzero_const, float maxq, int round_dtype, int block,
                                    uint8_t* const* Qt, float* const* E, void* stream) {
  if (groups < 0 || (groups > 0 && (!Wt || !U || !scale || !Qt || !E))) return MQ_ERR_ARG;
  for (int g0 = 0; g0 < groups; g0 += MAX_GROUP) {
    const int cnt = groups - g0 < MAX_GROUP ? groups - g0 : MAX_GROUP;
    const int rc = loop_impl(cnt, Wt + g0, ldw, C, R, U + g0, ldu, scale + g0, ld_scale, scale_row ? scale_row + g0 : nullptr,
                             qzero ? qzero + g0 : nullptr, qzero_const, maxq, round_dtype, block, Qt + g0, E + g0, nullptr,
                             stream);
    if (rc != MQ_OK) return rc;
  }
  return MQ_OK;
}

// The loop on the Cholesky multipliers F of mq_factor_chol (in U's place) and the original weights W0t (laid out
// like Wt, read only): same outputs as the classical loop on U up to fp32 rounding.
extern "C" int mq_gptq_loop_chol_grouped(int groups, float* const* Wt, const float* const* W0t, long ldw, int C, int R,
                                         const float* const* F, long ldf, const float* const* scale, long ld_scale,
                                         const int* const* scale_row, const float* const* qzero, float qzero_const,
                                         float maxq, int round_dtype, int block, uint8_t* const* Qt, float* const* E,
                                         void* stream) {
  if (groups < 0 || (groups > 0 && (!Wt || !W0t || !F || !scale || !Qt || !E))) return MQ_ERR_ARG;
  for (int g0 = 0; g0 < groups; g0 += MAX_GROUP) {
    const int cnt = groups - g0 < MAX_GROUP ? groups - g0 : MAX_GROUP;
    const int rc = loop_impl(cnt, Wt + g0, ldw, C, R, F + g0, ldf, scale + g0, ld_scale, scale_row ? scale_row + g0 : nullptr,
                             qzero ? qzero + g0 : nullptr, qzero_const, maxq, round_dtype, block, Qt + g0, E + g0, W0t + g0,
                             stream);
    if (rc != MQ_OK) return rc;
  }
  return MQ_OK;
}

extern "C" int mq_gptq_loop_chol(float* Wt, const float* W0t, long ldw, int C, int R, const float* F, long ldf,
                                 const float* scale, long ld_scale, const int* scale_row, const float* qzero,
                                 float qzero_const, float maxq, int round_dtype, int block, uint8_t* Qt, float* E,
                                 void* stream) {
  return mq_gptq_loop_chol_grouped(1, &Wt, &W0t, ldw, C, R, &F, ldf, &scale, ld_scale, &scale_row, &qzero, qzero_const, maxq,
                                   round_dtype, block, &Qt, &E, stream);
}
