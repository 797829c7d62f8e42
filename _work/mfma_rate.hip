// Diagnostic, not part of libdiffattn: the fp16 (and bf16) MFMA rate this GPU sustains when every SIMD
// issues v_mfma_f32_32x32x16_f16 (_bf16) back to back and nothing else, for three kinds of operand data.  The
// matrix pipes are 100 % busy in every case (32 shader cycles per instruction and wave slot); what
// changes with the data is the clock the power management lets the chip hold.  The numbers put
// the published peak (which assumes the maximum clock) next to what a kernel with realistic
// operands can at most reach on the same machine.
//
// Build: hipcc --offload-arch=gfx950 -O3 -o mfma_rate mfma_rate.hip     Run: ./mfma_rate
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <vector>

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef __bf16 b8 __attribute__((ext_vector_type(8)));
typedef float f16v __attribute__((ext_vector_type(16)));

#define CHECK(x)                                                                          \
  do {                                                                                    \
    hipError_t e_ = (x);                                                                  \
    if (e_ != hipSuccess) { fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_)); exit(1); } \
  } while (0)

// Four independent accumulation chains per wave; four operand sets are rotated so that consecutive
// instructions see different inputs.
__device__ inline f16v mfma(h8 a, h8 b, f16v c) { return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0); }
__device__ inline f16v mfma(b8 a, b8 b, f16v c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0); }

// V8 is h8 or b8; src holds 16-bit elements of that type
template <class V8>
__global__ void mfma_loop(const unsigned short* src, float* out, long long* stamps, int iters) {
  V8 a[4], b[4];
  for (int i = 0; i < 4; ++i) {
    a[i] = *reinterpret_cast<const V8*>(src + ((i * 1024 + threadIdx.x) % 4096) * 8);
    b[i] = *reinterpret_cast<const V8*>(src + ((i * 1024 + 512 + threadIdx.x) % 4096) * 8);
  }
  f16v c0 = {0}, c1 = {0}, c2 = {0}, c3 = {0};
  const long long cyc0 = __builtin_readcyclecounter(), wall0 = wall_clock64();
  for (int it = 0; it < iters; ++it) {
    c0 = mfma(a[0], b[0], c0);
    c1 = mfma(a[1], b[1], c1);
    c2 = mfma(a[2], b[2], c2);
    c3 = mfma(a[3], b[3], c3);
  }
  float s = 0;
  for (int r = 0; r < 16; ++r) s += c0[r] + c1[r] + c2[r] + c3[r];
  const long long cyc1 = __builtin_readcyclecounter(), wall1 = wall_clock64();
  out[blockIdx.x * blockDim.x + threadIdx.x] = s;
  if (threadIdx.x == 0 && blockIdx.x == 0) { stamps[0] = cyc1 - cyc0; stamps[1] = wall1 - wall0; }
}

int main() {
  hipDeviceProp_t prop;
  CHECK(hipGetDeviceProperties(&prop, 0));
  const int cus = prop.multiProcessorCount;
  const int n = 4096 * 8, iters = 200000;
  std::vector<_Float16> zeros(n), halves(n), normal(n);
  std::vector<__bf16> normal_bf(n);
  srand(1);
  for (int i = 0; i < n; ++i) {
    const float u1 = (rand() + 1.0f) / (RAND_MAX + 2.0f), u2 = (rand() + 1.0f) / (RAND_MAX + 2.0f);
    const float x = sqrtf(-2.f * logf(u1)) * cosf(6.2831853f * u2);   // Box-Muller
    normal[i] = (_Float16)x;
    normal_bf[i] = (__bf16)x;
    halves[i] = (_Float16)0.5f;
    zeros[i] = (_Float16)0.f;
  }
  unsigned short* d_src; float* d_out; long long* d_stamps;
  CHECK(hipMalloc(&d_src, n * 2));
  CHECK(hipMalloc(&d_out, (size_t)cus * 1024 * sizeof(float)));
  CHECK(hipMalloc(&d_stamps, 2 * sizeof(long long)));
  hipEvent_t e0, e1;
  CHECK(hipEventCreate(&e0)); CHECK(hipEventCreate(&e1));
  struct Case { const char* name; const void* data; bool bf16; } cases[] = {
      {"fp16 all zero", zeros.data(), false}, {"fp16 all 0.5", halves.data(), false},
      {"fp16 N(0,1)", normal.data(), false}, {"bf16 N(0,1)", normal_bf.data(), true}};
  printf("%s, %d CUs; %d x 4 MFMAs per wave; clock = shader cycles / 100 MHz wall clock of one wave\n",
         prop.gcnArchName, cus, iters);
  printf("%-14s %14s %10s %12s %12s\n", "operands", "waves per SIMD", "ms", "clock GHz", "TFLOP/s");
  for (int rep = 0; rep < 2; ++rep)        // the first pass also warms the clocks up
    for (const Case& cs : cases)
      for (int waves : {1, 2, 4}) {
        CHECK(hipMemcpy(d_src, cs.data, n * 2, hipMemcpyHostToDevice));
        CHECK(hipEventRecord(e0));
        if (cs.bf16) hipLaunchKernelGGL(mfma_loop<b8>, dim3(cus), dim3(256 * waves), 0, 0, d_src, d_out, d_stamps, iters);
        else         hipLaunchKernelGGL(mfma_loop<h8>, dim3(cus), dim3(256 * waves), 0, 0, d_src, d_out, d_stamps, iters);
        CHECK(hipGetLastError());
        CHECK(hipEventRecord(e1));
        CHECK(hipEventSynchronize(e1));
        float ms;
        long long st[2];
        CHECK(hipEventElapsedTime(&ms, e0, e1));
        CHECK(hipMemcpy(st, d_stamps, sizeof(st), hipMemcpyDeviceToHost));
        if (rep == 0) continue;
        const double flop = 4.0 * iters * 32768.0 * cus * 4 * waves;
        printf("%-14s %14d %10.2f %12.3f %12.1f\n", cs.name, waves, ms, st[0] / (st[1] * 10.0), flop / (ms * 1e-3) / 1e12);
      }
  return 0;
}
