// Launch parameter blocks shared by the C-ABI entry points and the kernel launchers.
#pragma once
#include <hip/hip_runtime.h>
#include "common.hpp"

namespace DA_NS {

struct FwdParams {
  const half_t* q1; const half_t* q2; const half_t* k1; const half_t* k2; const half_t* v;
  const half_t* lambda_scale;   // 1-element device tensor
  half_t* y;                    // [B,H,N,2D]
  half_t* u2;                   // [B,H,N,2D]  softmax(S2) V, saved for backward (may be null)
  float* lse1; float* lse2;     // [B,H,N] natural-log row logsumexp of the scaled scores (may be null)
  float* rinv;                  // [B,H,N] rsqrt(mean(X^2)+eps), only written when rms_norm (may be null)
  int BH, N;
  float sm_scale, lambda_init;
  int rms_norm;
  int causal;                   // query i sees keys 0..i only
  int n_keys;                   // keys n_keys..N-1 are padding and are ignored (N when there is none)
};

struct BwdParams {
  const half_t* q1; const half_t* q2; const half_t* k1; const half_t* k2; const half_t* v;
  const half_t* lambda_scale;
  const half_t* y; const half_t* u2;
  const float* lse1; const float* lse2; const float* rinv;
  const half_t* dy;
  half_t* dq1; half_t* dq2; half_t* dk1; half_t* dk2; half_t* dv;
  half_t* dlambda;              // 1 element
  // workspace carve-up
  half_t* dx;                   // [BH,N,2D] gradient w.r.t. the pre-norm rows, fp16
  float* stat;                  // [4][BH*N]: -lse1*log2(e), -lse2*log2(e), -delta1, -(lambda*delta1 + delta2)
  float* dlam_part;             // [n_part] per-workgroup partial sums of d(lambda)
  int n_part;
  int BH, N;
  float sm_scale, lambda_init;
  int rms_norm;
  int causal;
  unsigned stages;              // bit 0 row preprocess, 1 d(lambda) reduce, 2 dK/dV, 3 dQ
};

hipError_t launch_fwd(const FwdParams& p, int D, hipStream_t stream);
hipError_t launch_bwd(const BwdParams& p, int D, hipStream_t stream);
int bwd_num_partials(int BH, int N, int D);

}  // namespace DA_NS
