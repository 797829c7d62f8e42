// C-ABI entry points of libdiffattn (declared in include/diffattn.h): argument validation,
// workspace carve-up and kernel launches.  Nothing here allocates or synchronises; the only state
// is the per-device address of the built-in scratch array of diffattn_backward_static.
#include <atomic>
#include <cstring>

#include "../../include/diffattn.h"
#include "params.hpp"

// Scratch of diffattn_backward_static: one copy per GPU, at an address that differs per GPU.  In
// host code the name is only a handle for hipGetSymbolAddress, never a device address.
static __device__ __align__(256) unsigned char scratch[DIFFATTN_STATIC_SCRATCH_BYTES];

using namespace da;

// The bf16 build of the kernels (the same sources compiled with -DDA_BF16) lives in namespace da_bf16.
namespace da_bf16 {
using FwdParams = da_abi::FwdParamsT<__bf16>;
using BwdParams = da_abi::BwdParamsT<__bf16>;
hipError_t launch_fwd(const FwdParams& p, int D, hipStream_t stream);
hipError_t launch_bwd(const BwdParams& p, int D, hipStream_t stream);
}  // namespace da_bf16

namespace {

constexpr int kKnownFlags = DIFFATTN_RMS_NORM | DIFFATTN_CAUSAL | DIFFATTN_BF16 | DIFFATTN_LAMBDA_PER_HEAD | DIFFATTN_LAMBDA_FP32 |
                            DIFFATTN_UNPADDED;

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

int check_dims(int B, int H, int N, int D) {
  if (B <= 0 || H <= 0 || N <= 0) return DIFFATTN_EINVAL_DIM;
  if (D != 32 && D != 64 && D != 128) return DIFFATTN_EINVAL_DIM;
  if ((long long)B * H > 0x7fffffffLL / 64) return DIFFATTN_EINVAL_DIM;
  // grid sizes are ints and the statistics copy of the dK/dV kernel uses 32-bit byte offsets
  // (up to 3*B*H*N floats): keep B*H*N below 2^28 rows (a 68 GiB v tensor at D = 64)
  if ((long long)B * H * N > (1LL << 28)) return DIFFATTN_EINVAL_DIM;
  if (N % 128 != 0) return DIFFATTN_EINVAL_SEQ;
  return DIFFATTN_OK;
}

constexpr int kMaxDevices = 64;
std::atomic<void*> g_scratch_ptr[kMaxDevices];

// Device address of `scratch` on the current device, looked up once per device.
int static_scratch(void** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  if (dev < 0 || dev >= kMaxDevices) return DIFFATTN_EINVAL_DIM;
  void* ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (!ptr) {
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return (int)e;
    if (!ptr) return (int)hipErrorInvalidSymbol;
    g_scratch_ptr[dev].store(ptr, std::memory_order_release);   // every thread finds the same address
  }
  *out = ptr;
  return DIFFATTN_OK;
}

// Layout of the caller's tensors: the given strides, or dense [B,H,rows,C] where none are given; `rows` is
// N, or n_valid with DIFFATTN_UNPADDED.
struct Layouts { da_abi::Strides qk, v, y, dy, dqk, dv; };

inline da_abi::Strides dense(int H, int N, int C) { return {(long long)H * N * C, (long long)N * C, (long long)C}; }

inline bool stride_ok(long long b, long long h, long long n, int C) {
  // rows are contiguous and at least C apart; every row starts on a 16-byte boundary; the kernels
  // form 32-bit byte offsets of up to 16 rows
  return n >= C && n % 8 == 0 && n <= (1LL << 26) && b >= 0 && h >= 0 && b % 8 == 0 && h % 8 == 0;
}

// a tensor that is written must not lie on top of itself (an input may be broadcast with a zero stride)
inline bool no_overlap(long long b, long long h, int B, int H) { return (B == 1 || b != 0) && (H == 1 || h != 0); }

// `backward`: the backward reads dy and writes the gradients through their strides; the forward ignores those
// fields, so a caller of the forward may leave them zero.  Gradient strides that are all zero mean dense.
int resolve_layout(const diffattn_layout* l, int B, int H, int rows, int D, bool backward, Layouts* out) {
  out->qk = out->dqk = dense(H, rows, D);
  out->v = out->y = out->dy = out->dv = dense(H, rows, 2 * D);
  if (!l) return DIFFATTN_OK;
  if (!stride_ok(l->qk_b, l->qk_h, l->qk_n, D) || !stride_ok(l->v_b, l->v_h, l->v_n, 2 * D) ||
      !stride_ok(l->y_b, l->y_h, l->y_n, 2 * D))
    return DIFFATTN_EINVAL_LAYOUT;
  out->qk = {l->qk_b, l->qk_h, l->qk_n};
  out->v = {l->v_b, l->v_h, l->v_n};
  out->y = {l->y_b, l->y_h, l->y_n};
  if (!backward) return no_overlap(l->y_b, l->y_h, B, H) ? DIFFATTN_OK : DIFFATTN_EINVAL_LAYOUT;
  if (!stride_ok(l->dy_b, l->dy_h, l->dy_n, 2 * D)) return DIFFATTN_EINVAL_LAYOUT;
  out->dy = {l->dy_b, l->dy_h, l->dy_n};
  if (l->dqk_b || l->dqk_h || l->dqk_n) {
    if (!stride_ok(l->dqk_b, l->dqk_h, l->dqk_n, D) || !no_overlap(l->dqk_b, l->dqk_h, B, H)) return DIFFATTN_EINVAL_LAYOUT;
    out->dqk = {l->dqk_b, l->dqk_h, l->dqk_n};
  }
  if (l->dv_b || l->dv_h || l->dv_n) {
    if (!stride_ok(l->dv_b, l->dv_h, l->dv_n, 2 * D) || !no_overlap(l->dv_b, l->dv_h, B, H)) return DIFFATTN_EINVAL_LAYOUT;
    out->dv = {l->dv_b, l->dv_h, l->dv_n};
  }
  return DIFFATTN_OK;
}

// Dropout parameters as the kernels want them; none (threshold 0) without a request or with p = 0.
int resolve_dropout(const diffattn_dropout* d, da_abi::DropoutCfg* out) {
  *out = {0u, 0u, 0u, 1.0f};
  if (!d) return DIFFATTN_OK;
  // the range test is done on the bit pattern: this file is built with -fno-honor-nans, under which a
  // floating-point comparison does not reject a NaN
  unsigned bits;
  memcpy(&bits, &d->p, sizeof bits);
  if (bits > 0x3f7f0000u) return DIFFATTN_EINVAL_DROPOUT;      // negative, NaN, or above 255/256 = 0x3f7f0000
  const unsigned thr = (unsigned)(d->p * 256.0f + 0.5f);
  if (thr > 255u) return DIFFATTN_EINVAL_DROPOUT;
  out->seed_lo = (unsigned)(d->seed & 0xffffffffull);
  out->seed_hi = (unsigned)(d->seed >> 32);
  out->threshold = thr;
  out->keep_scale = 256.0f / (float)(256u - thr);
  return DIFFATTN_OK;
}

// keep[bh][q][k] = 1 if the pair survives dropout in softmax stream `stream`, else 0
__global__ __launch_bounds__(256) void dropout_mask_kernel(unsigned char* keep, da_abi::DropoutCfg cfg, int N, int stream) {
  const int bh = blockIdx.y;
  const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (size_t)N * N) return;
  const unsigned q = (unsigned)(idx / N), k = (unsigned)(idx % N);
  const unsigned word = dropout_word(dropout_key(cfg, 2u * bh + stream), (unsigned)N / 2, q >> 1, k >> 1);
  keep[(size_t)bh * N * N + idx] = dropout_keep(word, q, k, cfg.threshold) ? 1 : 0;
}

inline size_t round_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

struct WsLayout {
  size_t dx, stat, part, total;
};

WsLayout ws_layout(int BH, int N, int D) {
  WsLayout w;
  size_t rows = (size_t)BH * N;
  size_t off = 0;
  w.dx = off;      off = round_up(off + rows * 2 * D * sizeof(half_t), 256);
  w.stat = off;    off = round_up(off + 4 * rows * sizeof(float), 256);
  w.part = off;    off = round_up(off + (size_t)bwd_num_partials(BH, N, D) * sizeof(float), 256);
  w.total = off;
  return w;
}

template <class T>
void fill_fwd(da_abi::FwdParamsT<T>& p, const void* q1, const void* q2, const void* k1, const void* k2,
              const void* v, const void* lambda_scale, void* y, void* u2, float* lse1, float* lse2, float* rinv,
              int BH, int H, int N, int n_valid, float sm_scale, float lambda_init, int flags, const Layouts& lay,
              const da_abi::DropoutCfg& drop) {
  p.drop = drop;
  p.sqk = lay.qk; p.sv = lay.v; p.sy = lay.y;
  p.q1 = (const T*)q1; p.q2 = (const T*)q2; p.k1 = (const T*)k1; p.k2 = (const T*)k2;
  p.v = (const T*)v; p.lambda_scale = (const T*)lambda_scale;
  p.y = (T*)y; p.u2 = (T*)u2; p.lse1 = lse1; p.lse2 = lse2; p.rinv = rinv;
  p.BH = BH; p.N = N; p.sm_scale = sm_scale; p.lambda_init = lambda_init;
  p.rms_norm = (flags & DIFFATTN_RMS_NORM) ? 1 : 0;
  p.causal = (flags & DIFFATTN_CAUSAL) ? 1 : 0;
  p.n_keys = n_valid;
  p.H = H; p.lambda_stride = (flags & DIFFATTN_LAMBDA_PER_HEAD) ? 1 : 0;
  p.lambda_fp32 = (flags & DIFFATTN_LAMBDA_FP32) ? 1 : 0;
}

template <class T>
void fill_bwd(da_abi::BwdParamsT<T>& p, const void* q1, const void* q2, const void* k1, const void* k2,
              const void* v, const void* lambda_scale, const void* y, const void* u2,
              const float* lse1, const float* lse2, const float* rinv, const void* dy,
              void* dq1, void* dq2, void* dk1, void* dk2, void* dv, void* dlambda,
              void* ws_dx, void* ws_stat, void* ws_part, int n_part,
              int BH, int H, int N, int n_valid, float sm_scale, float lambda_init, int flags, unsigned stage_mask,
              const Layouts& lay, const da_abi::DropoutCfg& drop) {
  p.drop = drop;
  p.sqk = lay.qk; p.sv = lay.v; p.sy = lay.y; p.sdy = lay.dy; p.sdqk = lay.dqk; p.sdv = lay.dv;
  p.q1 = (const T*)q1; p.q2 = (const T*)q2; p.k1 = (const T*)k1; p.k2 = (const T*)k2;
  p.v = (const T*)v; p.lambda_scale = (const T*)lambda_scale;
  p.y = (const T*)y; p.u2 = (const T*)u2; p.lse1 = lse1; p.lse2 = lse2; p.rinv = rinv;
  p.dy = (const T*)dy;
  p.dq1 = (T*)dq1; p.dq2 = (T*)dq2; p.dk1 = (T*)dk1; p.dk2 = (T*)dk2; p.dv = (T*)dv;
  p.dlambda = (T*)dlambda;
  p.dx = (T*)ws_dx; p.stat = (float*)ws_stat; p.dlam_part = (float*)ws_part; p.n_part = n_part;
  p.BH = BH; p.N = N; p.sm_scale = sm_scale; p.lambda_init = lambda_init;
  p.rms_norm = (flags & DIFFATTN_RMS_NORM) ? 1 : 0;
  p.causal = (flags & DIFFATTN_CAUSAL) ? 1 : 0;
  p.n_keys = n_valid;
  p.stages = stage_mask & DIFFATTN_STAGE_ALL;
  p.H = H; p.lambda_stride = (flags & DIFFATTN_LAMBDA_PER_HEAD) ? 1 : 0;
  p.lambda_fp32 = (flags & DIFFATTN_LAMBDA_FP32) ? 1 : 0;
}

}  // namespace

extern "C" {

int diffattn_abi_version(void) { return 7; }

const char* diffattn_strerror(int code) {
  switch (code) {
    case DIFFATTN_OK: return "success";
    case DIFFATTN_EINVAL_NULL: return "a required pointer is null";
    case DIFFATTN_EINVAL_DIM: return "unsupported sizes: D must be 32, 64 or 128 and B, H, N positive";
    case DIFFATTN_EINVAL_SEQ: return "N must be a multiple of 128 (and 1 <= n_valid <= N)";
    case DIFFATTN_EINVAL_WS: return "workspace too small or misaligned";
    case DIFFATTN_EINVAL_ALIGN: return "tensor pointers must be 16-byte aligned";
    case DIFFATTN_EINVAL_SCRATCH: return "problem too large for the built-in scratch of diffattn_backward_static (DIFFATTN_STATIC_SCRATCH_BYTES): use diffattn_backward with a caller workspace";
    case DIFFATTN_EINVAL_LAYOUT: return "bad strides in diffattn_layout: every stride must be a non-negative multiple of 8 elements, a row stride at least the row width, and the batch and head strides of a tensor that is written non-zero";
    case DIFFATTN_EINVAL_DROPOUT: return "dropout probability must lie in [0, 255/256]";
    case DIFFATTN_EINVAL_FLAGS: return "unknown bits in flags (known: DIFFATTN_RMS_NORM, DIFFATTN_CAUSAL, DIFFATTN_BF16, DIFFATTN_LAMBDA_PER_HEAD, DIFFATTN_LAMBDA_FP32, DIFFATTN_UNPADDED)";
    default: break;
  }
  if (code > 0) return hipGetErrorString(static_cast<hipError_t>(code));
  return "unknown diffattn error";
}

int diffattn_forward(const void* q1, const void* q2, const void* k1, const void* k2, const void* v,
                     const void* lambda_scale, void* y, void* u2, float* lse1, float* lse2, float* rinv,
                     int B, int H, int N, int D, float sm_scale, float lambda_init, int flags,
                     void* stream) {
  return diffattn_forward_padded(q1, q2, k1, k2, v, lambda_scale, y, u2, lse1, lse2, rinv,
                                 B, H, N, N, D, sm_scale, lambda_init, flags, nullptr, nullptr, stream);
}

int diffattn_forward_padded(const void* q1, const void* q2, const void* k1, const void* k2, const void* v,
                            const void* lambda_scale, void* y, void* u2, float* lse1, float* lse2, float* rinv,
                            int B, int H, int N, int n_valid, int D, float sm_scale, float lambda_init, int flags,
                            const diffattn_layout* layout, const diffattn_dropout* dropout, void* stream) {
  if (!q1 || !q2 || !k1 || !k2 || !v || !lambda_scale || !y) return DIFFATTN_EINVAL_NULL;
  if (flags & ~kKnownFlags) return DIFFATTN_EINVAL_FLAGS;
  if (int e = check_dims(B, H, N, D)) return e;
  if (n_valid < 1 || n_valid > N) return DIFFATTN_EINVAL_SEQ;
  if (!aligned16(q1) || !aligned16(q2) || !aligned16(k1) || !aligned16(k2) || !aligned16(v) ||
      !aligned16(y) || !aligned16(u2))
    return DIFFATTN_EINVAL_ALIGN;
  Layouts lay;
  if (int e = resolve_layout(layout, B, H, (flags & DIFFATTN_UNPADDED) ? n_valid : N, D, false, &lay)) return e;
  da_abi::DropoutCfg drop;
  if (int e = resolve_dropout(dropout, &drop)) return e;
  if (flags & DIFFATTN_BF16) {
    da_bf16::FwdParams p;
    fill_fwd(p, q1, q2, k1, k2, v, lambda_scale, y, u2, lse1, lse2, rinv, B * H, H, N, n_valid, sm_scale, lambda_init, flags, lay, drop);
    return (int)da_bf16::launch_fwd(p, D, (hipStream_t)stream);
  }
  FwdParams p;
  fill_fwd(p, q1, q2, k1, k2, v, lambda_scale, y, u2, lse1, lse2, rinv, B * H, H, N, n_valid, sm_scale, lambda_init, flags, lay, drop);
  return (int)launch_fwd(p, D, (hipStream_t)stream);
}

size_t diffattn_backward_workspace_bytes(int B, int H, int N, int D, int flags) {
  if (check_dims(B, H, N, D) || (flags & ~kKnownFlags)) return 0;
  return ws_layout(B * H, N, D).total;
}

int diffattn_backward_stages(const void* q1, const void* q2, const void* k1, const void* k2, const void* v,
                             const void* lambda_scale, const void* y, const void* u2,
                             const float* lse1, const float* lse2, const float* rinv, const void* dy,
                             void* dq1, void* dq2, void* dk1, void* dk2, void* dv, void* dlambda,
                             void* workspace, size_t workspace_bytes,
                             int B, int H, int N, int n_valid, int D, float sm_scale, float lambda_init, int flags,
                             unsigned stage_mask, const diffattn_layout* layout, const diffattn_dropout* dropout,
                             void* stream) {
  if (!q1 || !q2 || !k1 || !k2 || !v || !lambda_scale || !y || !u2 || !lse1 || !lse2 || !dy || !workspace)
    return DIFFATTN_EINVAL_NULL;
  // outputs are required by the stages that write them
  if ((stage_mask & DIFFATTN_STAGE_DLAMBDA) && !dlambda) return DIFFATTN_EINVAL_NULL;
  if ((stage_mask & DIFFATTN_STAGE_DKDV) && (!dk1 || !dk2 || !dv)) return DIFFATTN_EINVAL_NULL;
  if ((stage_mask & DIFFATTN_STAGE_DQ) && (!dq1 || !dq2)) return DIFFATTN_EINVAL_NULL;
  if (flags & ~kKnownFlags) return DIFFATTN_EINVAL_FLAGS;
  if ((flags & DIFFATTN_RMS_NORM) && !rinv) return DIFFATTN_EINVAL_NULL;
  if (int e = check_dims(B, H, N, D)) return e;
  if (n_valid < 1 || n_valid > N) return DIFFATTN_EINVAL_SEQ;
  const void* ptrs[] = {q1, q2, k1, k2, v, y, u2, dy, dq1, dq2, dk1, dk2, dv};
  for (const void* q : ptrs)
    if (!aligned16(q)) return DIFFATTN_EINVAL_ALIGN;
  Layouts lay;
  if (int e = resolve_layout(layout, B, H, (flags & DIFFATTN_UNPADDED) ? n_valid : N, D, true, &lay)) return e;
  da_abi::DropoutCfg drop;
  if (int e = resolve_dropout(dropout, &drop)) return e;
  const WsLayout w = ws_layout(B * H, N, D);
  if (workspace_bytes < w.total || (reinterpret_cast<uintptr_t>(workspace) & 255u)) return DIFFATTN_EINVAL_WS;
  char* ws = (char*)workspace;
  const int n_part = bwd_num_partials(B * H, N, D);
  if (flags & DIFFATTN_BF16) {
    da_bf16::BwdParams p;
    fill_bwd(p, q1, q2, k1, k2, v, lambda_scale, y, u2, lse1, lse2, rinv, dy, dq1, dq2, dk1, dk2, dv, dlambda,
             ws + w.dx, ws + w.stat, ws + w.part, n_part, B * H, H, N, n_valid, sm_scale, lambda_init, flags, stage_mask, lay, drop);
    return (int)da_bf16::launch_bwd(p, D, (hipStream_t)stream);
  }
  BwdParams p;
  fill_bwd(p, q1, q2, k1, k2, v, lambda_scale, y, u2, lse1, lse2, rinv, dy, dq1, dq2, dk1, dk2, dv, dlambda,
           ws + w.dx, ws + w.stat, ws + w.part, n_part, B * H, H, N, n_valid, sm_scale, lambda_init, flags, stage_mask, lay, drop);
  return (int)launch_bwd(p, D, (hipStream_t)stream);
}

int diffattn_backward(const void* q1, const void* q2, const void* k1, const void* k2, const void* v,
                      const void* lambda_scale, const void* y, const void* u2,
                      const float* lse1, const float* lse2, const float* rinv, const void* dy,
                      void* dq1, void* dq2, void* dk1, void* dk2, void* dv, void* dlambda,
                      void* workspace, size_t workspace_bytes,
                      int B, int H, int N, int D, float sm_scale, float lambda_init, int flags,
                      void* stream) {
  return diffattn_backward_stages(q1, q2, k1, k2, v, lambda_scale, y, u2, lse1, lse2, rinv, dy,
                                  dq1, dq2, dk1, dk2, dv, dlambda, workspace, workspace_bytes,
                                  B, H, N, N, D, sm_scale, lambda_init, flags, DIFFATTN_STAGE_ALL, nullptr, nullptr, stream);
}

int diffattn_backward_static(const void* q1, const void* q2, const void* k1, const void* k2, const void* v,
                             const void* lambda_scale, const void* y, const void* u2,
                             const float* lse1, const float* lse2, const float* rinv, const void* dy,
                             void* dq1, void* dq2, void* dk1, void* dk2, void* dv, void* dlambda,
                             int B, int H, int N, int D, float sm_scale, float lambda_init, int flags,
                             void* stream) {
  if (flags & ~kKnownFlags) return DIFFATTN_EINVAL_FLAGS;
  if (int e = check_dims(B, H, N, D)) return e;
  const size_t need = ws_layout(B * H, N, D).total;
  if (need > (size_t)DIFFATTN_STATIC_SCRATCH_BYTES) return DIFFATTN_EINVAL_SCRATCH;
  void* ws = nullptr;
  if (int e = static_scratch(&ws)) return e;
  // every byte of the workspace that a kernel reads was written earlier in the same call: nothing
  // has to be cleared, whatever an earlier call left behind
  return diffattn_backward_stages(q1, q2, k1, k2, v, lambda_scale, y, u2, lse1, lse2, rinv, dy,
                                  dq1, dq2, dk1, dk2, dv, dlambda, ws, need,
                                  B, H, N, N, D, sm_scale, lambda_init, flags, DIFFATTN_STAGE_ALL, nullptr, nullptr, stream);
}

int diffattn_dropout_mask(unsigned char* keep, int B, int H, int N, int softmax_stream, const diffattn_dropout* dropout,
                          void* stream) {
  if (!keep || !dropout) return DIFFATTN_EINVAL_NULL;
  if (B <= 0 || H <= 0 || N <= 0 || N % 2 != 0 || (long long)B * H > 65535 || (softmax_stream != 0 && softmax_stream != 1))
    return DIFFATTN_EINVAL_DIM;
  da_abi::DropoutCfg drop;
  if (int e = resolve_dropout(dropout, &drop)) return e;
  const dim3 grid((unsigned)(((size_t)N * N + 255) / 256), (unsigned)(B * H));
  hipLaunchKernelGGL(dropout_mask_kernel, grid, dim3(256), 0, (hipStream_t)stream, keep, drop, N, softmax_stream);
  return (int)hipGetLastError();
}

}  // extern "C"
