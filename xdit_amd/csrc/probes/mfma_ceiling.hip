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
//   5. LDS reads    throughput per compute unit of the fragment reads of the 16-bit kernel, 12
//                wavefronts reading and nothing else: ds_read_b128 and ds_read_b64_tr_b16 on
//                contiguous addresses and on the kernel's K and V^T fragment address patterns.
//   7. VALU rates   clocks per wavefront instruction and SIMD of the softmax's instructions (3 wavefronts
//                per SIMD, four independent chains each).
//   6. structure   the loop of the 16-bit kernel with its LDS reads and barrier (12 wavefronts of 32
//                rows) against a pair structure (8 wavefronts of 64 rows) that reads 2.7 times less LDS.
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

// ---- 5: LDS read throughput.  KIND 0: ds_read_b128, 16 B per lane contiguous; 1: ds_read_b64_tr_b16,
// 8 B per lane contiguous; 2: ds_read_b128 on the K fragment pattern of the 16-bit kernel (head_dim
// 128: key row r lives in piece r % 16 of 1040 B at slot r / 16 of 256 B; lane = (row, 16-byte half));
// 3: ds_read_b64_tr_b16 on its V^T fragment pattern (pieces of 1088 B).
typedef __attribute__((ext_vector_type(4))) int i32x4;
typedef __attribute__((ext_vector_type(2))) int i32x2;
template <int KIND>
__global__ __launch_bounds__(768) void lds_read_kernel(int* out, int iters) {
  __shared__ __attribute__((aligned(16))) unsigned char smem[65536];
  for (int i = threadIdx.x; i < 65536 / 4; i += 768) ((int*)smem)[i] = i;
  __syncthreads();
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  unsigned addr = (unsigned)(size_t)(__attribute__((address_space(3))) unsigned char*)smem;
  if (KIND == 0) addr += wave * 1024 + lane * 16;
  else if (KIND == 1) addr += wave * 1024 + lane * 8;
  else if (KIND == 2) addr += ((lane & 31) % 16) * 1040 + ((lane & 31) / 16) * 256 + (lane >> 5) * 16;
  else addr += ((4 * (lane >> 5) + ((lane & 15) >> 2)) % 16) * 1088 + (16 * ((lane >> 4) & 1) + 4 * (lane & 3)) * 2;
  i32x4 acc = {0, 0, 0, 0};
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int j = 0; j < 8; j++) {
      if (KIND == 0 || KIND == 2) {
        i32x4 v;
        asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(j * 32));
        asm volatile("s_waitcnt lgkmcnt(4)" : "+v"(v));
        acc += v;
      } else {
        i32x2 v;
        asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(KIND == 3 ? (j & 3) * 64 + (j >> 2) * 8 * 1088 : j * 512));
        asm volatile("s_waitcnt lgkmcnt(4)" : "+v"(v));
        acc[0] += v[0];
        acc[1] += v[1];
      }
    }
  }
  asm volatile("s_waitcnt lgkmcnt(0)");
  out[blockIdx.x * 768 + threadIdx.x] = acc[0] + acc[1] + acc[2] + acc[3];
}
template <int KIND>
static void lds_read_rate(int* out, const char* name, int bytes_per_lane) {
  const int iters = 20000;
  hipEvent_t e0, e1;
  CK(hipEventCreate(&e0));
  CK(hipEventCreate(&e1));
  for (int w = 0; w < 3; w++) hipLaunchKernelGGL(lds_read_kernel<KIND>, dim3(kCUs), dim3(768), 0, 0, out, iters);
  CK(hipEventRecord(e0));
  hipLaunchKernelGGL(lds_read_kernel<KIND>, dim3(kCUs), dim3(768), 0, 0, out, iters);
  CK(hipEventRecord(e1));
  CK(hipEventSynchronize(e1));
  float ms;
  CK(hipEventElapsedTime(&ms, e0, e1));
  const double bytes = 8.0 * iters * 12 * 64 * bytes_per_lane;  // per compute unit
  printf("LDS reads, %s: %.0f bytes/ns per compute unit (%.0f bytes/clock at 2.4 GHz)\n", name, bytes / (ms * 1e6), bytes / (ms * 1e6) / 2.4);
}

// ---- 6: structure models WITH LDS traffic and barriers (values are meaningless, the instruction
// streams are the kernels').  "present": 12 wavefronts x 32 query rows, every wavefront reads the
// whole K tile (16 ds_read_b128) and V tile (32 ds_read_b64_tr_b16) of 64 keys, one barrier per
// tile, the softmax of the attention kernel on its 32 values per lane.  "pair": 8 wavefronts x 64
// query rows; the two wavefronts of a pair each compute S^T for 32 of the 64 keys, exchange their
// P fragments through LDS (second barrier) and each accumulate 64 of the 128 head_dim columns, so
// a wavefront reads 24 KiB of LDS per tile for 64 rows instead of 32 KiB for 32.
typedef bf16x8 vec8;
typedef __attribute__((ext_vector_type(4))) __bf16 vec4;
typedef __attribute__((ext_vector_type(2))) __bf16 vec2;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(8))) short s16x8;
#define LDS __attribute__((address_space(3)))
__device__ __forceinline__ vec8 mma_in(s16x4 a, s16x4 b) { s16x8 v = __builtin_shufflevector(a, b, 0, 1, 2, 3, 4, 5, 6, 7); return __builtin_bit_cast(vec8, v); }
__device__ __forceinline__ s16x4 read_tr(LDS unsigned char* p) { return __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS s16x4*)p); }
__device__ __forceinline__ float max_of_halves(float x) { float y = __shfl_xor(x, 32); return fmaxf(x, y); }

// softmax of one tile's 32 values per lane (as in the attention kernel): lazy max, exp2, row sum, bf16 P
__device__ __forceinline__ void softmax32(const f32x16 (&s)[2], float& m_used, float& l, f32x16* o, int no, vec8 (&pf)[4], float c) {
  float mx = s[0][0];
#pragma unroll
  for (int e = 1; e < 16; e++) mx = fmaxf(mx, s[0][e]);
#pragma unroll
  for (int e = 0; e < 16; e++) mx = fmaxf(mx, s[1][e]);
  mx = max_of_halves(mx);
  const float m_new = fmaxf(m_used, mx);
  if (__builtin_amdgcn_ballot_w64((m_new - m_used) * c > 8.0f) != 0) {
    const float alpha = __builtin_amdgcn_exp2f((m_used - m_new) * c);
    m_used = m_new; l *= alpha;
    for (int d = 0; d < no; d++)
#pragma unroll
      for (int e = 0; e < 16; e++) o[d][e] *= alpha;
  }
  const float mc = m_used * c;
#pragma unroll
  for (int kb = 0; kb < 2; kb++)
#pragma unroll
    for (int e = 0; e < 16; e += 2) {
      float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[kb][e], c, -mc));
      float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[kb][e + 1], c, -mc));
      l += p0 + p1;
      f32x2 pp = {p0, p1};
      vec2 pk = __builtin_convertvector(pp, vec2);
      pf[2 * kb + (e >> 3)][e & 7] = pk[0];
      pf[2 * kb + (e >> 3)][(e & 7) + 1] = pk[1];
    }
}

constexpr int TILE = 32768;  // K 16 KiB + V 16 KiB per buffer

__global__ __launch_bounds__(768) void present_structure_kernel(const vec8* in, float* out, int iters) {
  extern __shared__ unsigned char smem_[];
  LDS unsigned char* smem = (LDS unsigned char*)smem_;
  const int lane = threadIdx.x & 63;
  for (int i = threadIdx.x; i < 2 * TILE / 16; i += 768) ((LDS vec8*)smem)[i] = in[i & 4095];
  vec8 qf[8];
#pragma unroll
  for (int k = 0; k < 8; k++) qf[k] = in[4096 + k * 768 + threadIdx.x];
  f32x16 oacc[4] = {};
  float m_used = -INFINITY, l = 0.f;
  for (int it = 0; it < iters; it++) {
    __syncthreads();
    LDS unsigned char* kb_ = smem + (it & 1) * TILE;
    LDS unsigned char* vb_ = kb_ + 16384;
    f32x16 sacc[2] = {};
    vec8 kf; s16x4 v0, v1;
#pragma unroll
    for (int i = 0; i < 16; i++) {
      kf = *(LDS vec8*)(kb_ + i * 1024 + lane * 16);
      sacc[i % 2] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[i / 2], sacc[i % 2], 0, 0, 0);
    }
    vec8 pf[4];
    softmax32(sacc, m_used, l, oacc, 4, pf, 0.1275f);
#pragma unroll
    for (int i = 0; i < 16; i++) {
      v0 = read_tr(vb_ + i * 1024 + lane * 8);
      v1 = read_tr(vb_ + i * 1024 + 512 + lane * 8);
      oacc[i % 4] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(mma_in(v0, v1), pf[i / 4], oacc[i % 4], 0, 0, 0);
    }
  }
  float s = l;
  for (int d = 0; d < 4; d++) for (int e = 0; e < 16; e++) s += oacc[d][e];
  out[blockIdx.x * 768 + threadIdx.x] = s;
}

__global__ __launch_bounds__(512) void pair_structure_kernel(const vec8* in, float* out, int iters) {
  extern __shared__ unsigned char smem_[];
  LDS unsigned char* smem = (LDS unsigned char*)smem_;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, role = wave & 1;
  for (int i = threadIdx.x; i < 2 * TILE / 16; i += 512) ((LDS vec8*)smem)[i] = in[i & 4095];
  LDS unsigned char* pbase = smem + 2 * TILE;  // 2 buffers x 8 wavefronts x 4 KiB of P
  vec8 qf[2][8];
#pragma unroll
  for (int r = 0; r < 2; r++)
#pragma unroll
    for (int k = 0; k < 8; k++) qf[r][k] = in[4096 + (r * 8 + k) * 512 + threadIdx.x];
  f32x16 oacc[4] = {};  // [db * 2 + rb]
  float m_used[2] = {-INFINITY, -INFINITY}, l[2] = {0.f, 0.f};
  for (int it = 0; it < iters; it++) {
    __syncthreads();
    LDS unsigned char* kb_ = smem + (it & 1) * TILE + role * 8192;           // this wavefront's 32 keys
    LDS unsigned char* vb_ = smem + (it & 1) * TILE + 16384 + role * 8192;   // this wavefront's 64 head_dim columns
    f32x16 sacc[2] = {};
#pragma unroll
    for (int ks = 0; ks < 8; ks++) {
      vec8 kf = *(LDS vec8*)(kb_ + ks * 1024 + lane * 16);
      sacc[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[0][ks], sacc[0], 0, 0, 0);
      sacc[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[1][ks], sacc[1], 0, 0, 0);
    }
    // per row block: 16 values per lane of this wavefront's 32 keys -> 2 P fragments each
    vec8 pown[2][2];
#pragma unroll
    for (int rb = 0; rb < 2; rb++) {
      float mx = sacc[rb][0];
#pragma unroll
      for (int e = 1; e < 16; e++) mx = fmaxf(mx, sacc[rb][e]);
      mx = max_of_halves(mx);
      const float m_new = fmaxf(m_used[rb], mx);
      const float c = 0.1275f;
      if (__builtin_amdgcn_ballot_w64((m_new - m_used[rb]) * c > 8.0f) != 0) {
        const float alpha = __builtin_amdgcn_exp2f((m_used[rb] - m_new) * c);
        m_used[rb] = m_new; l[rb] *= alpha;
#pragma unroll
        for (int e = 0; e < 16; e++) { oacc[rb][e] *= alpha; oacc[2 + rb][e] *= alpha; }
      }
      const float mc = m_used[rb] * c;
#pragma unroll
      for (int e = 0; e < 16; e += 2) {
        float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[rb][e], c, -mc));
        float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[rb][e + 1], c, -mc));
        l[rb] += p0 + p1;
        f32x2 pp = {p0, p1};
        vec2 pk = __builtin_convertvector(pp, vec2);
        pown[rb][e >> 3][e & 7] = pk[0];
        pown[rb][e >> 3][(e & 7) + 1] = pk[1];
      }
    }
    LDS unsigned char* pw = pbase + (it & 1) * 32768 + wave * 4096;
    LDS unsigned char* pr = pbase + (it & 1) * 32768 + (wave ^ 1) * 4096;
#pragma unroll
    for (int j = 0; j < 4; j++) *(LDS vec8*)(pw + j * 1024 + lane * 16) = pown[j >> 1][j & 1];
    __syncthreads();
    vec8 pother[2][2];
#pragma unroll
    for (int j = 0; j < 4; j++) pother[j >> 1][j & 1] = *(LDS vec8*)(pr + j * 1024 + lane * 16);
#pragma unroll
    for (int kk = 0; kk < 4; kk++)   // 16-key blocks: two of this wavefront's keys, two of the partner's
#pragma unroll
      for (int db = 0; db < 2; db++) {
        const int i = kk * 2 + db;
        s16x4 v0 = read_tr(vb_ + i * 1024 + lane * 8), v1 = read_tr(vb_ + i * 1024 + 512 + lane * 8);
        const vec8 vf = mma_in(v0, v1);
        oacc[db * 2 + 0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, kk < 2 ? pown[0][kk] : pother[0][kk - 2], oacc[db * 2 + 0], 0, 0, 0);
        oacc[db * 2 + 1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, kk < 2 ? pown[1][kk] : pother[1][kk - 2], oacc[db * 2 + 1], 0, 0, 0);
      }
  }
  float s = l[0] + l[1];
  for (int d = 0; d < 4; d++) for (int e = 0; e < 16; e++) s += oacc[d][e];
  out[blockIdx.x * 512 + threadIdx.x] = s;
}


template <typename K>
static double structure_time(K kern, int threads, size_t lds, const vec8* in, float* out, int iters) {
  hipEvent_t e0, e1;
  CK(hipEventCreate(&e0));
  CK(hipEventCreate(&e1));
  for (int w = 0; w < 8; w++) hipLaunchKernelGGL(kern, dim3(kCUs), dim3(threads), lds, 0, in, out, iters);
  float best = 1e30f;
  for (int r = 0; r < 5; r++) {
    CK(hipEventRecord(e0));
    hipLaunchKernelGGL(kern, dim3(kCUs), dim3(threads), lds, 0, in, out, iters);
    CK(hipEventRecord(e1));
    CK(hipEventSynchronize(e1));
    float ms;
    CK(hipEventElapsedTime(&ms, e0, e1));
    if (ms < best) best = ms;
  }
  return best;
}
static void structure_models(float* out) {
  const int iters = 4000;
  const size_t n = 4096 + 16 * 768;
  std::vector<unsigned short> h(n * 8);
  vec8* d;
  CK(hipMalloc(&d, n * 16));
  CK(hipFuncSetAttribute((const void*)present_structure_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 2 * TILE));
  CK(hipFuncSetAttribute((const void*)pair_structure_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 2 * TILE + 65536));
  for (int mode = 0; mode < 2; mode++) {
    srand(1);
    for (auto& x : h) {
      float f = mode ? (rand() / (float)RAND_MAX - 0.5f) * 2.0f : 0.0078125f;
      unsigned u;
      memcpy(&u, &f, 4);
      x = (unsigned short)(u >> 16);
    }
    CK(hipMemcpy(d, h.data(), n * 16, hipMemcpyHostToDevice));
    const double tc = structure_time(present_structure_kernel, 768, 2 * TILE, d, out, iters);
    const double tp = structure_time(pair_structure_kernel, 512, 2 * TILE + 65536, d, out, iters);
    printf("structure model with LDS reads and barriers, %s operands: present (12 x 32 rows) %.0f TFLOP/s | pair (8 x 64 rows) %.0f TFLOP/s of MFMA work\n",
           mode ? "random" : "constant", kCUs * 12.0 * 32 * 32768.0 * iters / tc / 1e9, kCUs * 8.0 * 32 * 32768.0 * iters / tp / 1e9);
  }
  CK(hipFree(d));
}

// ---- 7: issue rate of the VALU instructions of the softmax (inline assembly, four independent chains)
#define XDIT_REP8(X) X X X X X X X X
template <int KIND>
__global__ __launch_bounds__(768) void valu_rate_kernel(float* out, int iters) {
  float a0 = threadIdx.x * 1e-3f, a1 = a0 + 1, a2 = a0 + 2, a3 = a0 + 3;
  for (int i = 0; i < iters; i++) {
    if (KIND == 0) { XDIT_REP8(asm volatile("v_exp_f32 %0, %0\n v_exp_f32 %1, %1\n v_exp_f32 %2, %2\n v_exp_f32 %3, %3" : "+v"(a0), "+v"(a1), "+v"(a2), "+v"(a3));) }
    if (KIND == 1) { XDIT_REP8(asm volatile("v_fma_f32 %0, %0, %1, %2\n v_fma_f32 %1, %1, %2, %3\n v_fma_f32 %2, %2, %3, %0\n v_fma_f32 %3, %3, %0, %1" : "+v"(a0), "+v"(a1), "+v"(a2), "+v"(a3));) }
    if (KIND == 2) { XDIT_REP8(asm volatile("v_add_f32 %0, %0, %1\n v_add_f32 %1, %1, %2\n v_add_f32 %2, %2, %3\n v_add_f32 %3, %3, %0" : "+v"(a0), "+v"(a1), "+v"(a2), "+v"(a3));) }
    if (KIND == 3) { XDIT_REP8(asm volatile("v_max3_f32 %0, %0, %1, %2\n v_max3_f32 %1, %1, %2, %3\n v_max3_f32 %2, %2, %3, %0\n v_max3_f32 %3, %3, %0, %1" : "+v"(a0), "+v"(a1), "+v"(a2), "+v"(a3));) }
    if (KIND == 4) { XDIT_REP8(asm volatile("v_cvt_pk_bf16_f32 %0, %1, %2\n v_cvt_pk_bf16_f32 %1, %2, %3\n v_cvt_pk_bf16_f32 %2, %3, %0\n v_cvt_pk_bf16_f32 %3, %0, %1" : "+v"(a0), "+v"(a1), "+v"(a2), "+v"(a3));) }
    if (KIND == 5) { XDIT_REP8(asm volatile("v_cvt_pk_fp8_f32 %0, %1, %2\n v_cvt_pk_fp8_f32 %1, %2, %3\n v_cvt_pk_fp8_f32 %2, %3, %0\n v_cvt_pk_fp8_f32 %3, %0, %1" : "+v"(a0), "+v"(a1), "+v"(a2), "+v"(a3));) }
  }
  out[blockIdx.x * 768 + threadIdx.x] = a0 + a1 + a2 + a3;
}
template <int KIND>
static void valu_rate(float* out, const char* name) {
  const int iters = 20000;
  hipEvent_t e0, e1;
  CK(hipEventCreate(&e0));
  CK(hipEventCreate(&e1));
  for (int w = 0; w < 3; w++) hipLaunchKernelGGL(valu_rate_kernel<KIND>, dim3(kCUs), dim3(768), 0, 0, out, iters);
  CK(hipEventRecord(e0));
  hipLaunchKernelGGL(valu_rate_kernel<KIND>, dim3(kCUs), dim3(768), 0, 0, out, iters);
  CK(hipEventRecord(e1));
  CK(hipEventSynchronize(e1));
  float ms;
  CK(hipEventElapsedTime(&ms, e0, e1));
  const double per_simd = 32.0 * iters * 3;  // wavefront instructions per SIMD
  printf("VALU rate, %s: %.2f ns per wavefront instruction and SIMD (%.1f clocks at 2.4 GHz)\n", name, ms * 1e6 / per_simd, ms * 1e6 / per_simd * 2.4);
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
  lds_read_rate<0>((int*)out, "ds_read_b128, 16 bytes per lane contiguous", 16);
  lds_read_rate<1>((int*)out, "ds_read_b64_tr_b16, 8 bytes per lane contiguous", 8);
  lds_read_rate<2>((int*)out, "ds_read_b128 on the kernel's K fragment pattern", 16);
  lds_read_rate<3>((int*)out, "ds_read_b64_tr_b16 on the kernel's V^T fragment pattern", 8);
  structure_models(out);
  valu_rate<0>(out, "v_exp_f32");
  valu_rate<1>(out, "v_fma_f32");
  valu_rate<2>(out, "v_add_f32");
  valu_rate<3>(out, "v_max3_f32");
  valu_rate<4>(out, "v_cvt_pk_bf16_f32");
  valu_rate<5>(out, "v_cvt_pk_fp8_f32");
  fflush(stdout);
  return 0;
}
