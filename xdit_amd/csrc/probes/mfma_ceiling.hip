// Register-only probes of what the matrix pipe of gfx950 sustains, for judging the attention
// kernels: no memory access inside the timed loops, every operand lives in registers.
//   1. rate      v_mfma_f32_32x32x16_bf16 with constant and with random operands (3 wavefronts per
//                SIMD, four accumulator chains): the difference is the power limit.
//   2. per-XCD   the same loop timed per workgroup with the wall clock, grouped by XCD.
//   3. co-issue  per loop iteration 8 MFMAs with NF v_fma_f32 spread evenly between them, 2 and 3
//                wavefronts per SIMD, constant operands (so that the clock stays put): how much
//                VALU work hides behind an MFMA.  The same with v_exp_f32, with the MFMA-free loop,
//                and with the fp8 MFMA (v_mfma_f32_32x32x64_f8f6f4, 4 per iteration).
//   4. loop models  the instruction mix of the attention loops per wavefront and KV tile, from
//                registers only: bf16 32 MFMAs (32x32x16) + 112 fma-type + 32 exp; fp8 8 MFMAs
//                (32x32x64) + 104 fma-type + 32 exp.  "phased": half the MFMAs, all the VALU work, the
//                other half, as a wavefront of the kernels runs them; "interleaved": every MFMA
//                followed by its share of the VALU work.  Constant and random operands, 8 and 12
//                wavefronts per compute unit.  What the kernels add to this is LDS fragment reads,
//                tile loads, barriers and waits.
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
// KIND 0: v_fma_f32, 1: v_exp_f32.  FP8: v_mfma_f32_32x32x64_f8f6f4 (fp8 operands, 64 cycles) instead
// of v_mfma_f32_32x32x16_bf16 (32 cycles).  Inline assembly, so the order in the binary is the order here.
typedef __attribute__((ext_vector_type(8))) int i32x8;
template <int NM, int NF, int KIND, bool FP8 = false>
__global__ __launch_bounds__(256) void coissue_kernel(float* out, int iters) {
  bf16x8 a, b;
  for (int e = 0; e < 8; e++) { a[e] = (__bf16)1.0f; b[e] = (__bf16)1.0f; }
  i32x8 a8, b8;
  for (int e = 0; e < 8; e++) { a8[e] = 0x38383838; b8[e] = 0x38383838; }  // 1.0 in e4m3
  f32x16 c[4];
  for (int i = 0; i < 4; i++) for (int e = 0; e < 16; e++) c[i][e] = 0.f;
  float x[16];
  for (int i = 0; i < 16; i++) x[i] = threadIdx.x * 1e-3f + i;
  const float m = 1.0001f, ad = 0.5f;
  constexpr int G = NM > 0 ? NM : 8;
  for (int i = 0; i < iters; i++) {
#pragma unroll
    for (int g = 0; g < G; g++) {
      if (NM > 0) {
        if (FP8) asm volatile("v_mfma_f32_32x32x64_f8f6f4 %0, %1, %2, %0" : "+v"(c[g & 3]) : "v"(a8), "v"(b8));
        else asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(c[g & 3]) : "v"(a), "v"(b));
      }
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

template <int NM, int NF, int KIND, bool FP8 = false>
static double coissue(float* d_out, int waves_per_simd) {
  const int iters = 20000;
  hipEvent_t e0, e1;
  CK(hipEventCreate(&e0));
  CK(hipEventCreate(&e1));
  hipLaunchKernelGGL((coissue_kernel<NM, NF, KIND, FP8>), dim3(kCUs * waves_per_simd), dim3(256), 0, 0, d_out, iters);
  CK(hipDeviceSynchronize());
  CK(hipEventRecord(e0));
  hipLaunchKernelGGL((coissue_kernel<NM, NF, KIND, FP8>), dim3(kCUs * waves_per_simd), dim3(256), 0, 0, d_out, iters);
  CK(hipEventRecord(e1));
  CK(hipEventSynchronize(e1));
  float ms;
  CK(hipEventElapsedTime(&ms, e0, e1));
  return ms * 1e6 / iters;  // ns per iteration of every wavefront
}

static void coissue_table_fp8(float* d_out, int w) {
  const double mf = coissue<4, 0, 0, true>(d_out, w);
  const double f48 = coissue<0, 48, 0>(d_out, w), f96 = coissue<0, 96, 0>(d_out, w), x32 = coissue<0, 32, 1>(d_out, w);
  const double b48 = coissue<4, 48, 0, true>(d_out, w), b96 = coissue<4, 96, 0, true>(d_out, w), bx = coissue<4, 32, 1, true>(d_out, w);
  printf("co-issue with the fp8 MFMA (32x32x64), %d wavefronts/SIMD, ns per iteration (4 MFMAs per wavefront):\n", w);
  printf("  4 MFMA alone %.1f (%.0f TFLOP/s) | 4 MFMA + 48 fma %.1f (hidden %.1f of %.1f) | + 96 fma %.1f (hidden %.1f of %.1f) | + 32 exp %.1f (hidden %.1f of %.1f)\n",
         mf, 4 * 131072.0 * kCUs * 4 * w / mf / 1e3, b48, mf + f48 - b48, f48, b96, mf + f96 - b96, f96, bx, mf + x32 - bx, x32);
  printf("  -> VALU time hidden per MFMA time: %.2f (fma), %.2f (exp)\n", (mf + f96 - b96) / mf, (mf + x32 - bx) / mf);
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

// ---- 4: loop models --------------------------------------------------------------------------
#define XDIT_PROBE_FMA(r) asm volatile("v_fma_f32 %0, %0, %1, %2" : "+v"(x[(r) & 15]) : "v"(m), "v"(ad))
#define XDIT_PROBE_EXP(r) asm volatile("v_exp_f32 %0, %0" : "+v"(x[(r) & 15]))
// the softmax of four logits: scale-and-shift, exponential, row sum, half a conversion, half a max
#define XDIT_PROBE_SOFTMAX4(j)                                                              \
  _Pragma("unroll") for (int q_ = 0; q_ < 4; q_++) {                                         \
    XDIT_PROBE_FMA(4 * (j) + q_); XDIT_PROBE_EXP(4 * (j) + q_ + 5); XDIT_PROBE_FMA(4 * (j) + q_ + 9); \
  }                                                                                         \
  XDIT_PROBE_FMA((j) + 3); XDIT_PROBE_FMA((j) + 7); XDIT_PROBE_FMA((j) + 11); XDIT_PROBE_FMA((j) + 13);

template <bool FP8, bool INTERLEAVED, int NW>
__global__ __launch_bounds__(64 * NW) void loop_model_kernel(const i32x8* in, float* out, int iters) {
  i32x8 a[4], b[4];
  for (int j = 0; j < 4; j++) { a[j] = in[(2 * j) * 768 + threadIdx.x]; b[j] = in[(2 * j + 1) * 768 + threadIdx.x]; }
  f32x16 c[4];
  for (int i = 0; i < 4; i++) for (int e = 0; e < 16; e++) c[i][e] = 0.f;
  float x[16];
  for (int i = 0; i < 16; i++) x[i] = threadIdx.x * 1e-3f + i;
  const float m = 1.0001f, ad = 0.5f;
  constexpr int NM = FP8 ? 8 : 32;   // MFMAs per tile; the softmax of 32 logits is 8 groups of four
  auto mfma = [&](int g) {
    if (FP8) asm volatile("v_mfma_f32_32x32x64_f8f6f4 %0, %1, %2, %0" : "+v"(c[g & 3]) : "v"(a[g & 3]), "v"(b[(g >> 2) & 3]));
    else asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(c[g & 3]) : "v"(__builtin_shufflevector(a[g & 3], a[g & 3], 0, 1, 2, 3)), "v"(__builtin_shufflevector(b[(g >> 2) & 3], b[(g >> 2) & 3], 0, 1, 2, 3)));
  };
  for (int it = 0; it < iters; it++) {
    if (!INTERLEAVED) {
#pragma unroll
      for (int g = 0; g < NM / 2; g++) mfma(g);
#pragma unroll
      for (int j = 0; j < 8; j++) { XDIT_PROBE_SOFTMAX4(j) }
#pragma unroll
      for (int g = NM / 2; g < NM; g++) mfma(g);
    } else {
#pragma unroll
      for (int j = 0; j < 8; j++) {
#pragma unroll
        for (int g = 0; g < NM / 8; g++) mfma(j * (NM / 8) + g);
        XDIT_PROBE_SOFTMAX4(j)
      }
    }
  }
  float s = 0;
  for (int i = 0; i < 16; i++) s += x[i];
  for (int i = 0; i < 4; i++) for (int e = 0; e < 16; e++) s += c[i][e];
  if (s == 12345.f) out[0] = s;
}

template <bool FP8, bool INTERLEAVED, int NW>
static void loop_model(const void* in, float* out, const char* operands) {
  const int iters = FP8 ? 6000 : 3000;
  hipEvent_t e0, e1;
  CK(hipEventCreate(&e0));
  CK(hipEventCreate(&e1));
  float ms = 0;
  for (int rep = 0; rep < 3; rep++) {  // the third run is reported: the clock has settled
    CK(hipEventRecord(e0));
    hipLaunchKernelGGL((loop_model_kernel<FP8, INTERLEAVED, NW>), dim3(kCUs), dim3(64 * NW), 0, 0, (const i32x8*)in, out, iters);
    CK(hipEventRecord(e1));
    CK(hipEventSynchronize(e1));
    CK(hipEventElapsedTime(&ms, e0, e1));
  }
  const double flop = (FP8 ? 8 * 131072.0 : 32 * 32768.0) * NW * kCUs * iters;
  printf("loop model %s, %s operands, %s, %d wavefronts/CU: %.3f ms = %.0f TFLOP/s of MFMA work\n", FP8 ? "fp8" : "bf16", operands,
         INTERLEAVED ? "interleaved" : "phased", NW, ms, flop / ms / 1e9);
}

template <bool FP8>
static void loop_models(float* out) {
  std::vector<unsigned char> h(8 * 768 * 32);
  void* in;
  CK(hipMalloc(&in, h.size()));
  for (int mode = 0; mode < 2; mode++) {
    srand(5);
    if (FP8) {
      // e4m3: constant 1.0, or random sign and mantissa with exponent fields 5..10 (finite, normal)
      for (auto& x : h) x = mode ? (unsigned char)((rand() & 0x87) | ((rand() % 6 + 5) << 3)) : 0x38;
    } else {
      for (size_t i = 0; i + 1 < h.size(); i += 2) {
        float f = mode ? (rand() / (float)RAND_MAX - 0.5f) * 0.02f : 1.0f;
        unsigned u;
        memcpy(&u, &f, 4);
        h[i] = (unsigned char)(u >> 16);
        h[i + 1] = (unsigned char)(u >> 24);
      }
    }
    CK(hipMemcpy(in, h.data(), h.size(), hipMemcpyHostToDevice));
    const char* w = mode ? "random" : "constant";
    loop_model<FP8, false, 8>(in, out, w);
    loop_model<FP8, true, 8>(in, out, w);
    loop_model<FP8, false, 12>(in, out, w);
    loop_model<FP8, true, 12>(in, out, w);
  }
  CK(hipFree(in));
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
  coissue_table_fp8(out, 2);
  coissue_table_fp8(out, 3);
  loop_models<false>(out);
  loop_models<true>(out);
  fflush(stdout);
  return 0;
}
