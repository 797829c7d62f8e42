// Stand-alone use of libdiffattn from C++ through its C ABI, without PyTorch: device buffers from
// hipMalloc, a stream of its own, forward and backward of one problem read from a file.  It is the
// example that goes with include/diffattn.h and the program tests/test_gpu_c_abi.py drives.
//
//   abi_example <in.bin> <out.bin> [token-major]
//
// With a third argument the tensors q1, q2, k1, k2, v, dy of in.bin and y of out.bin are stored
// [B,N,H,C] (the layout a projection writes) and are handed to the library as they are, through the
// strides of diffattn_layout; the gradient strides of the layout are left zero, so the gradients come
// back dense [B,H,N,C].
//
// in.bin : int32 B, H, N, D, flags; float32 lambda_init, sm_scale; then the 16-bit tensors q1, q2, k1,
//          k2 [B,H,N,D], v, dy [B,H,N,2D] and lambda (1 or H values), all in the dtype the flags name
// out.bin: the 16-bit tensors y [B,H,N,2D], dq1, dq2, dk1, dk2 [B,H,N,D], dv [B,H,N,2D], dlambda
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "../../include/diffattn.h"

#define HIP_OK(x)                                                                           \
  do {                                                                                      \
    hipError_t e_ = (x);                                                                    \
    if (e_ != hipSuccess) { fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_)); return 2; } \
  } while (0)
#define DA_OK(x)                                                                       \
  do {                                                                                 \
    int c_ = (x);                                                                      \
    if (c_ != 0) { fprintf(stderr, "%s: %s\n", #x, diffattn_strerror(c_)); return 3; } \
  } while (0)

int main(int argc, char** argv) {
  if (argc != 3 && argc != 4) { fprintf(stderr, "usage: %s in.bin out.bin [token-major]\n", argv[0]); return 1; }
  const bool token_major = (argc == 4);
  FILE* f = fopen(argv[1], "rb");
  if (!f) { perror(argv[1]); return 1; }
  int32_t hdr[5];
  float scal[2];
  if (fread(hdr, 4, 5, f) != 5 || fread(scal, 4, 2, f) != 2) { fprintf(stderr, "short header\n"); return 1; }
  const int B = hdr[0], H = hdr[1], N = hdr[2], D = hdr[3], flags = hdr[4];
  const float lambda_init = scal[0], sm_scale = scal[1];
  const size_t qk = (size_t)B * H * N * D, vv = 2 * qk, rows = (size_t)B * H * N;
  const size_t n_lambda = (flags & DIFFATTN_LAMBDA_PER_HEAD) ? H : 1;
  // host staging: q1 q2 k1 k2 v dy lambda
  const size_t in_elems[7] = {qk, qk, qk, qk, vv, vv, n_lambda};
  std::vector<std::vector<uint16_t>> host(7);
  for (int i = 0; i < 7; ++i) {
    host[i].resize(in_elems[i]);
    if (fread(host[i].data(), 2, in_elems[i], f) != in_elems[i]) { fprintf(stderr, "short input\n"); return 1; }
  }
  fclose(f);

  hipStream_t stream;
  HIP_OK(hipStreamCreate(&stream));
  void* in[7];
  for (int i = 0; i < 7; ++i) {
    HIP_OK(hipMalloc(&in[i], in_elems[i] * 2));
    HIP_OK(hipMemcpyAsync(in[i], host[i].data(), in_elems[i] * 2, hipMemcpyHostToDevice, stream));
  }
  // outputs of the forward, inputs of the backward
  void *y, *u2;
  float *lse1, *lse2, *rinv;
  HIP_OK(hipMalloc(&y, vv * 2)); HIP_OK(hipMalloc(&u2, vv * 2));
  HIP_OK(hipMalloc((void**)&lse1, rows * 4)); HIP_OK(hipMalloc((void**)&lse2, rows * 4)); HIP_OK(hipMalloc((void**)&rinv, rows * 4));
  // gradients: dq1 dq2 dk1 dk2 dv dlambda
  const size_t out_elems[6] = {qk, qk, qk, qk, vv, n_lambda};
  void* grad[6];
  for (int i = 0; i < 6; ++i) HIP_OK(hipMalloc(&grad[i], out_elems[i] * 2));
  const size_t ws_bytes = diffattn_backward_workspace_bytes(B, H, N, D, flags);
  if (ws_bytes == 0) { fprintf(stderr, "sizes rejected\n"); return 3; }
  void* ws;
  HIP_OK(hipMalloc(&ws, ws_bytes));      // hipMalloc returns 256-byte aligned memory

  if (token_major) {
    // a [B,N,H,C] buffer seen as [B,H,N,C]: batch stride N*H*C, head stride C, row stride H*C
    const long long d = D, dv = 2 * D;
    const diffattn_layout lay = {(long long)N * H * d, d, H * d, (long long)N * H * dv, dv, H * dv,
                                 (long long)N * H * dv, dv, H * dv, (long long)N * H * dv, dv, H * dv};
    DA_OK(diffattn_forward_padded(in[0], in[1], in[2], in[3], in[4], in[6], y, u2, lse1, lse2, rinv,
                                  B, H, N, N, D, sm_scale, lambda_init, flags, &lay, nullptr, stream));
    DA_OK(diffattn_backward_stages(in[0], in[1], in[2], in[3], in[4], in[6], y, u2, lse1, lse2, rinv, in[5],
                                   grad[0], grad[1], grad[2], grad[3], grad[4], grad[5], ws, ws_bytes,
                                   B, H, N, N, D, sm_scale, lambda_init, flags, DIFFATTN_STAGE_ALL, &lay, nullptr, stream));
  } else {
    DA_OK(diffattn_forward(in[0], in[1], in[2], in[3], in[4], in[6], y, u2, lse1, lse2, rinv,
                           B, H, N, D, sm_scale, lambda_init, flags, stream));
    DA_OK(diffattn_backward(in[0], in[1], in[2], in[3], in[4], in[6], y, u2, lse1, lse2, rinv, in[5],
                            grad[0], grad[1], grad[2], grad[3], grad[4], grad[5], ws, ws_bytes,
                            B, H, N, D, sm_scale, lambda_init, flags, stream));
  }
  HIP_OK(hipStreamSynchronize(stream));

  FILE* o = fopen(argv[2], "wb");
  if (!o) { perror(argv[2]); return 1; }
  std::vector<uint16_t> buf(vv);
  HIP_OK(hipMemcpy(buf.data(), y, vv * 2, hipMemcpyDeviceToHost));
  fwrite(buf.data(), 2, vv, o);
  for (int i = 0; i < 6; ++i) {
    HIP_OK(hipMemcpy(buf.data(), grad[i], out_elems[i] * 2, hipMemcpyDeviceToHost));
    fwrite(buf.data(), 2, out_elems[i], o);
  }
  fclose(o);
  printf("abi_example: B=%d H=%d N=%d D=%d flags=%d ok\n", B, H, N, D, flags);
  return 0;
}
