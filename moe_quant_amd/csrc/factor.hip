// Damped-Hessian factorisation for GPTQ: the C entry points (device code and launch plan: factor_kernels.hpp).
#include "factor_kernels.hpp"

using namespace mqfactor;

static int factor_impl(int G, const float* const* S, long lds, float* const* Aout, long ld, int C, int normalize,
                       int* const* infos, float* const* ws, void* stream) {
  FactorPlan p;
  int rc = p.init(G, S, lds, Aout, ld, C, normalize, infos, ws);
  if (rc != MQ_OK) return rc;
  FactorPlan::init_kernels();
  hipStream_t st = (hipStream_t)stream;
  if ((rc = p.first(st)) != MQ_OK) return rc;
  for (int s = 0, n = p.steps(); s < n; ++s) {
    if ((rc = p.panel(s, st)) != MQ_OK) return rc;
    if ((rc = p.launch_trail(s, st)) != MQ_OK) return rc;
  }
  return p.finish(st);
}

extern "C" int mq_factor_upper_inverse(float* A, long ld, int C, int normalize, int* info, void* stream) {
  const float* S = A;
  return factor_impl(1, &S, ld, &A, ld, C, normalize, &info, nullptr, stream);
}

extern "C" int mq_factor_upper_inverse_from(const float* H, long ldh, float* A, long lda, int C, int normalize, int* info,
                                            void* stream) {
  if (H == A) return MQ_ERR_ARG;
  return factor_impl(1, &H, ldh, &A, lda, C, normalize, &info, nullptr, stream);
}

// `groups` matrices of one size in one sequence of launches (host arrays of device pointers).  More than MAX_GROUP
// matrices run as consecutive batches.
extern "C" int mq_factor_upper_inverse_grouped(int groups, const float* const* H, long ldh, float* const* A, long lda, int C,
                                               int normalize, int* const* info, void* stream) {
  if (groups < 0 || (groups > 0 && (!H || !A || !info))) return MQ_ERR_ARG;
  for (int g0 = 0; g0 < groups; g0 += MAX_GROUP) {
    const int cnt = groups - g0 < MAX_GROUP ? groups - g0 : MAX_GROUP;
    const int rc = factor_impl(cnt, H + g0, ldh, A + g0, lda, C, normalize, info + g0, nullptr, stream);
    if (rc != MQ_OK) return rc;
  }
  return MQ_OK;
}

// Cholesky-only mode (see chol_finalize_kernel): F[j,k] = -R[j,k] / R[k,k] for k > j, H = R R^T, in F's upper
// triangle; the diagonal and the lower triangle of F hold no defined values.
extern "C" size_t mq_factor_chol_workspace_bytes(int C) { return C > 0 ? (size_t)C * NB * sizeof(float) : 0; }

extern "C" int mq_factor_chol_grouped(int groups, const float* const* H, long ldh, float* const* F, long ldf, int C,
                                      int* const* info, void* const* workspace, size_t workspace_bytes, void* stream) {
  if (groups < 0 || (groups > 0 && (!H || !F || !info || !workspace))) return MQ_ERR_ARG;
  if (workspace_bytes < mq_factor_chol_workspace_bytes(C)) return MQ_ERR_WORKSPACE;
  for (int g0 = 0; g0 < groups; g0 += MAX_GROUP) {
    const int cnt = groups - g0 < MAX_GROUP ? groups - g0 : MAX_GROUP;
    const int rc = factor_impl(cnt, H + g0, ldh, F + g0, ldf, C, 1, info + g0, (float* const*)(workspace + g0), stream);
    if (rc != MQ_OK) return rc;
  }
  return MQ_OK;
}

extern "C" int mq_factor_chol(const float* H, long ldh, float* F, long ldf, int C, int* info, void* workspace,
                              size_t workspace_bytes, void* stream) {
  return mq_factor_chol_grouped(1, &H, ldh, &F, ldf, C, &info, &workspace, workspace_bytes, stream);
}
