// Register-only probes of what the matrix pipe of gfx950 sustains, for judging the attention
// kernels: no memory access inside the timed loops, every operand lives in registers.
//   1. rate      v_mfma_f32_32x32x16_bf16 with constant and with random operands (3 wavefronts per
//                SIMD, four accumulator chains): the difference is the power limit.
//   2. per-XCD   the same loop timed per workgroup with the wall clock, grouped by XCD.
//   3. co-issue  per loop iteration 8 MFMAs with NF v_fma_f32 spread evenly between them, 2 and 3
//                wavefronts per SIMD, constant operands (so that the clock stays put): how much
//                VALU work hides behind an MFMA.  The same with v_exp_f32 and with the MFMA-free loop.
// Build: hipcc --offload-arch=gfx950 -O3 mfma_ceiling.hip -o mfma_ceiling ; run without arguments.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#define CK(x)                                                                      \
  do {                                                                             \
    hipError_t e_ = (x);                                                           \
    if (e_ != hipSuccess) {                                                        \
      printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__);        \
      exit(1);                                                                     \
    }                                                                              \
  } while (0)

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;

constexpr int kCUs = 256;

// ---- 1, 2: MFMA rate, operands from memory once (constant: all 1.0; random: uniform in +-0.01) ----
__global__ __launch_bounds__(768, 3) void mfma_rate_kernel(const bf16x8* in, float* out, unsigned long long* t, int iters) {
  bf16x8 a[4], b[4];
#pragma unroll
  for (int j = 0; j < 4; j++) {
    a[j] = in[(2 * j) * 768 + threadIdx.x];
    b[j] = in[(2 * j + 1) * 768 + threadIdx.x];
  }
  f32x16 c0 = {}, c1 = {}, c2 = {}, c3 = {};
  __syncthreads();
  const unsigned long long t0 = wall_clock64();
  for (int i = 0; i < iters; i++) {
    c0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[0], b[0], c0, 0, 0, 0);
    c1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[1], b[1], c1, 0, 0, 0);
    c2 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[2], b[2], c2, 0, 0, 0);
    c3 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[3], b[3], c3, 0, 0, 0);
  }
  __syncthreads();
  const unsigned long long t1 = wall_clock64();
  float s = 0;
  for (int i = 0; i < 16; i++) s += c0[i] + c1[i] + c2[i] + c3[i];
  out[blockIdx.x * 768 + threadIdx.x] = s;
  if (threadIdx.x == 0) {
    unsigned xcc;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc));
    t[blockIdx.x * 2] = t1 - t0;
    t[blockIdx.x * 2 + 1] = xcc & 0xf;
  }
}

// ---- 3: NM MFMAs per iteration, round robin over four accumulators, NF VALU instructions between them ----
// KIND 0: v_fma_f32, 1: v_exp_f32.  Inline assembly, so the order in the binary is the order here.
template <int NM, int NF, int KIND>
__global__ __launch_bounds__(256) void coissue_kernel(float* out, int iters) {
  bf16x8 a, b;
  for (int e = 0; e < 8; e++) { a[e] = (__bf16)1.0f; b[e] = (__bf16)1.0f; }
  f32x16 c[4];
  for (int i = 0; i < 4; i++) for (int e = 0; e < 16; e++) c[i][e] = 0.f;
  float x[16];
  for (int i = 0; i < 16; i++) x[i] = threadIdx.x * 1e-3f + i;
  const float m = 1.0001f, ad = 0.5f;
  constexpr int G = NM > 0 ? NM : 8;
  for (int i = 0; i < iters; i++) {
#pragma unroll
    for (int g = 0; g < G; g++) {
      if (NM > 0) asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(c[g & 3]) : "v"(a), "v"(b));
#pragma unroll
      for (int j = 0; j < NF / G; j++) {
        const int r = (g * (NF / G) + j) & 15;
        if (KIND == 0) asm volatile("v_fma_f32 %0, %0, %1, %2" : "+v"(x[r]) : "v"(m), "v"(ad));
        else asm volatile("v_exp_f32 %0, %0" : "+v"(x[r]));
      }
    }
  }
  float s = 0;
  for (int i = 0; i < 16; i++) s += x[i];
  for (int i = 0; i < 4; i++) for (int e = 0; e < 16; e++) s += c[i][e];
  if (s == 12345.f) out[0] = s;
}

template <int NM, int NF, int KIND>
static double coissue(float* d_out, int waves_per_simd) {
  const int iters = 20000;
  hipEvent_t e0, e1;
  CK(hipEventCreate(&e0));
  CK(hipEventCreate(&e1));
  hipLaunchKernelGGL((coissue_kernel<NM, NF, KIND>), dim3(kCUs * waves_per_simd), dim3(256), 0, 0, d_out, iters);
  CK(hipDeviceSynchronize());
  CK(hipEventRecord(e0));
  hipLaunchKernelGGL((coissue_kernel<NM, NF, KIND>), dim3(kCUs * waves_per_simd), dim3(256), 0, 0, d_out, iters);
  CK(hipEventRecord(e1));
  CK(hipEventSynchronize(e1));
  float ms;
  CK(hipEventElapsedTime(&ms, e0, e1));
  return ms * 1e6 / iters;  // ns per iteration of every wavefront
}

static void coissue_table(float* d_out, int w) {
  const double mf = coissue<8, 0, 0>(d_out, w);
  const double f48 = coissue<0, 48, 0>(d_out, w), f96 = coissue<0, 96, 0>(d_out, w), x32 = coissue<0, 32, 1>(d_out, w);
  const double b48 = coissue<8, 48, 0>(d_out, w), b96 = coissue<8, 96, 0>(d_out, w), bx = coissue<8, 32, 1>(d_out, w);
  printf("co-issue, %d wavefronts/SIMD, ns per iteration (8 MFMAs per wavefront):\n", w);
  printf("  8 MFMA alone %.1f (%.0f TFLOP/s) | 48 fma alone %.1f | 96 fma alone %.1f | 32 exp alone %.1f\n", mf,
         8 * 32768.0 * kCUs * 4 * w / mf / 1e3, f48, f96, x32);
  printf("  8 MFMA + 48 fma %.1f (hidden %.1f of %.1f) | + 96 fma %.1f (hidden %.1f) | + 32 exp %.1f (hidden %.1f of %.1f)\n", b48,
         mf + f48 - b48, f48, b96, mf + f96 - b96, bx, mf + x32 - bx, x32);
  printf("  -> VALU time hidden per MFMA time: %.2f (fma), %.2f (exp)\n", (mf + f96 - b96) / mf, (mf + x32 - bx) / mf);
}

int main() {
  const int G = kCUs, iters = 40000;
  std::vector<unsigned short> h(8 * 768 * 8);
  void* in;
  float* out;
  unsigned long long* t;
  CK(hipMalloc(&in, h.size() * 2));
  CK(hipMalloc(&out, G * 768 * 4));
  CK(hipMalloc(&t, G * 16));
  for (int mode = 0; mode < 2; mode++) {
    srand(3);
    for (auto& x : h) {
      float f = mode ? (rand() / (float)RAND_MAX - 0.5f) * 0.02f : 1.0f;
      unsigned u;
      memcpy(&u, &f, 4);
      x = (unsigned short)(u >> 16);
    }
    CK(hipMemcpy(in, h.data(), h.size() * 2, hipMemcpyHostToDevice));
    for (int rep = 0; rep < 3; rep++) {
      hipEvent_t e0, e1;
      CK(hipEventCreate(&e0));
      CK(hipEventCreate(&e1));
      CK(hipEventRecord(e0));
      hipLaunchKernelGGL(mfma_rate_kernel, dim3(G), dim3(768), 0, 0, (const bf16x8*)in, out, t, iters);
      CK(hipEventRecord(e1));
      CK(hipEventSynchronize(e1));
      float ms;
      CK(hipEventElapsedTime(&ms, e0, e1));
      std::vector<unsigned long long> ht(G * 2);
      CK(hipMemcpy(ht.data(), t, G * 16, hipMemcpyDeviceToHost));
      double sum[16] = {0};
      int cnt[16] = {0};
      for (int i = 0; i < G; i++) { sum[ht[2 * i + 1] & 15] += (double)ht[2 * i]; cnt[ht[2 * i + 1] & 15]++; }
      const double flops = 4.0 * iters * 32768.0 * 12 * G;
      printf("rate, %s operands, rep %d: %.3f ms = %.0f TFLOP/s; per-XCD mean loop time (us, 100 MHz wall clock):", mode ? "random" : "constant", rep, ms, flops / ms / 1e9);
      for (int x = 0; x < 8; x++) printf(" %.0f", cnt[x] ? sum[x] / cnt[x] / 100.0 : 0.0);
      printf("\n");
    }
  }
  coissue_table(out, 2);
  coissue_table(out, 3);
  fflush(stdout);
  return 0;
}
