// Launch parameter blocks shared by the C-ABI entry points and the kernel launchers.
#pragma once
#include <hip/hip_runtime.h>
#include "common.hpp"

// One definition serves both builds of the kernels: T is the 16-bit element type of the tensors.
namespace da_abi {

// Element strides of a [B,H,N,C] tensor whose last dimension is contiguous.
struct Strides { long long b, h, n; };

template <class T>
struct FwdParamsT {
  const T* q1; const T* q2; const T* k1; const T* k2; const T* v;
  const T* lambda_scale;        // device memory: one value, or one per head (lambda_stride = 1)
  T* y;                         // [B,H,N,2D]
  T* u2;                        // [B,H,N,2D]  softmax(S2) V, saved for backward (may be null)
  float* lse1; float* lse2;     // [B,H,N] natural-log row logsumexp of the scaled scores (may be null)
  float* rinv;                  // [B,H,N] rsqrt(mean(X^2)+eps), only written when rms_norm (may be null)
  int BH, N;
  float sm_scale, lambda_init;
  int rms_norm;
  int causal;                   // query i sees keys 0..i only
  int n_keys;                   // rows n_keys..N-1 are padding: ignored as keys, never read from q1..v, never written to y (N when there is none)
  int H;                        // heads per batch entry: unit bh belongs to head bh % H
  int lambda_stride;            // 0: lambda_scale[0] for every head; 1: lambda_scale[head]
  int lambda_fp32;              // lambda_scale points to fp32 values instead of the tensors' 16-bit type
  Strides sqk, sv, sy;          // layouts of q1,q2,k1,k2 / v / y; u2 and the row statistics are dense
  DropoutCfg drop;               // threshold 0: no dropout
};

template <class T>
struct BwdParamsT {
  const T* q1; const T* q2; const T* k1; const T* k2; const T* v;
  const T* lambda_scale;        // one value, or one per head (lambda_stride = 1)
  const T* y; const T* u2;
  const float* lse1; const float* lse2; const float* rinv;
  const T* dy;
  T* dq1; T* dq2; T* dk1; T* dk2; T* dv;
  T* dlambda;                   // 1 element, or H elements with lambda_stride = 1
  // workspace carve-up
  T* dx;                        // [BH,N,2D] gradient w.r.t. the pre-norm rows, 16-bit
  float* stat;                  // [4][BH*N]: -lse1*log2(e), -lse2*log2(e), -delta1, -(lambda*delta1 + delta2)
  float* dlam_part;             // [n_part] per-workgroup partial sums of d(lambda)
  int n_part;
  int BH, N;
  float sm_scale, lambda_init;
  int rms_norm;
  int causal;
  int n_keys;                   // rows n_keys..N-1 are padding: ignored as keys, never read from q1..v, y, dy, never written to the gradients
  unsigned stages;              // bit 0 row preprocess, 1 d(lambda) reduce, 2 dK/dV, 3 dQ
  int dlam_fold;                // set by the launcher: extra workgroups at the end of a dK/dV or dQ grid that do the d(lambda) reduce
  int H;                        // heads per batch entry: unit bh belongs to head bh % H
  int lambda_stride;            // 0: one lambda; 1: one per head
  int lambda_fp32;              // lambda_scale and dlambda are fp32 instead of the tensors' 16-bit type
  Strides sqk, sv, sy, sdy;     // layouts of q1,q2,k1,k2 / v / y / dy
  Strides sdqk, sdv;            // layouts of dq1,dq2,dk1,dk2 / dv; the workspace, u2 and the row statistics are dense [BH,N,.]
  DropoutCfg drop;               // threshold 0: no dropout
};

// lambda of the (batch, head) unit bh
template <class P>
__device__ __forceinline__ float lambda_of_unit(const P& p, int bh) {
  const int idx = (bh % p.H) * p.lambda_stride;
  if (p.lambda_fp32) return reinterpret_cast<const float*>(p.lambda_scale)[idx];
  return (float)p.lambda_scale[idx];
}

// offset in elements of the first row of the (batch, head) unit bh
template <class P>
__device__ __forceinline__ size_t unit_base(const P& p, const Strides& s, int bh) {
  return (size_t)(bh / p.H) * (size_t)s.b + (size_t)(bh % p.H) * (size_t)s.h;
}

}  // namespace da_abi

namespace DA_NS {

using FwdParams = da_abi::FwdParamsT<half_t>;
using BwdParams = da_abi::BwdParamsT<half_t>;

hipError_t launch_fwd(const FwdParams& p, int D, hipStream_t stream);
hipError_t launch_bwd(const BwdParams& p, int D, hipStream_t stream);
int bwd_num_partials(int BH, int N, int D);

}  // namespace DA_NS
