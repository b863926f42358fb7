// Stand-alone microbenchmark (not part of the library): how vector instructions and 16x16x32 matrix-core
// instructions share one SIMD of gfx950.  It backs the issue model the kernels were tuned against:
//
//   part 1  a stream of m MFMAs and a independent vector instructions per loop iteration, interleaved evenly, with
//           1..4 waves per SIMD, against the same MFMAs alone and the same vector instructions alone;
//   part 2  the inner loop of the state kernels in isolation -- per operand fragment 8 DPP multiplies and 4
//           v_cvt_pk_bf16_f32 feeding 4 MFMAs that depend on them -- in the order a compiler emits it (a burst of
//           vector work, then a burst of MFMAs) and software-pipelined by one fragment (vector work of fragment x+1
//           between the MFMAs of fragment x).
//
// Build and run:  python retention_integration_amd/csrc/build.py --probe && ./retention_integration_amd/probe_issue
// Every instruction under test is volatile inline assembly, so the order written is the order issued.
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
#define CK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__); exit(1); } } while (0)
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) unsigned u32x4;

#define MUL(d, a, b) asm volatile("v_mul_f32 %0, %1, %2" : "=v"(d) : "v"(a), "v"(b))
#define FMA(d, a, b) asm volatile("v_fma_f32 %0, %1, %2, %0" : "+v"(d) : "v"(a), "v"(b))
#define MULDPP(d, a, b) asm volatile("v_mul_f32_dpp %0, %1, %2 row_newbcast:5 row_mask:0xf bank_mask:0xf bound_ctrl:1" : "=v"(d) : "v"(a), "v"(b))
#define CVT(d, a, b) asm volatile("v_cvt_pk_bf16_f32 %0, %1, %2" : "=v"(d) : "v"(a), "v"(b))
#define MFMA(acc, a, b) asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+v"(acc) : "v"(a), "v"(b))

// ---- part 1: NM MFMAs and NV vector instructions of one KIND per iteration, evenly interleaved ----
// KIND 0 v_mul_f32, 1 v_fma_f32, 2 v_cvt_pk_bf16_f32, 3 v_mul_f32_dpp
template <int NM, int NV, int KIND>
__global__ __launch_bounds__(1024) void mix_kernel(float* out, int iters) {
  const int l = threadIdx.x;
  float x[16], y[16];
  for (int i = 0; i < 16; i++) { x[i] = 1.0f + 1e-6f * (l + i); y[i] = 0; }
  u32x4 a = {0x3f803f80u + l, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u}, b = {0x3f803f80u, 0x3f803f80u + l, 0, 0};
  f32x4 acc[8];
  for (int i = 0; i < 8; i++) acc[i] = (f32x4){0, 0, 0, 0};
  for (int it = 0; it < iters; it++) {
    constexpr int STEPS = NM > 0 ? NM : 1, VPS = NV / STEPS;
#pragma unroll
    for (int s = 0; s < STEPS; s++) {
      if (NM > 0) MFMA(acc[s & 7], a, b);
#pragma unroll
      for (int v = 0; v < VPS; v++) {
        const int i = (s * VPS + v) & 15;
        if (KIND == 0) MUL(y[i], x[i], x[(i + 3) & 15]);
        if (KIND == 1) FMA(y[i], x[i], x[(i + 3) & 15]);
        if (KIND == 2) { unsigned u; CVT(u, x[i], x[(i + 3) & 15]); y[i] = __uint_as_float(u); }
        if (KIND == 3) MULDPP(y[i], x[i], x[(i + 3) & 15]);
      }
    }
  }
  float s = 0;
  for (int i = 0; i < 16; i++) s += y[i];
  for (int i = 0; i < 8; i++) for (int v = 0; v < 4; v++) s += acc[i][v];
  out[blockIdx.x * blockDim.x + l] = s;
}

// ---- part 2: the fragment pattern.  MODE 0 burst, 1 pipelined (MFMA, 2 mul, 1 cvt, ...), 2 MFMAs only, 3 vector only ----
template <int MODE>
__global__ __launch_bounds__(256) void frag_kernel(float* out, int iters) {
  constexpr int NX = 8;
  const int l = threadIdx.x;
  float rowf[8], srcf[8], p[8];
  for (int i = 0; i < 8; i++) { rowf[i] = 1.0f + 1e-3f * (l + i); srcf[i] = 1.0f - 1e-3f * (l + i); }
  u32x4 bfr[4];
  for (int i = 0; i < 4; i++) bfr[i] = (u32x4){0x3f803f80u + l, 0x3f803f80u, 0x3f803f80u + i, 0x3f803f80u};
  f32x4 acc[NX][4];
  for (int x = 0; x < NX; x++) for (int i = 0; i < 4; i++) acc[x][i] = (f32x4){0, 0, 0, 0};
  unsigned A[2][4] = {{0, 0, 0, 0}, {0, 0, 0, 0}};
  auto build = [&](unsigned (&An)[4]) {
    for (int j = 0; j < 4; j++) { MULDPP(p[2 * j], srcf[2 * j], rowf[2 * j]); MULDPP(p[2 * j + 1], srcf[2 * j + 1], rowf[2 * j + 1]); CVT(An[j], p[2 * j], p[2 * j + 1]); }
  };
  if (MODE == 1) build(A[0]);
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int x = 0; x < NX; x++) {
      unsigned (&Ac)[4] = A[MODE == 1 ? (x & 1) : 0];
      unsigned (&An)[4] = A[MODE == 1 ? ((x + 1) & 1) : 0];
      if (MODE == 0 || MODE == 3) build(Ac);
      if (MODE == 0) asm volatile("s_nop 1");
      const u32x4 a = {Ac[0], Ac[1], Ac[2], Ac[3]};
      if (MODE != 3) {
#pragma unroll
        for (int nt = 0; nt < 4; nt++) {
          MFMA(acc[x][nt], a, bfr[nt]);
          if (MODE == 1) { MULDPP(p[2 * nt], srcf[2 * nt], rowf[2 * nt]); MULDPP(p[2 * nt + 1], srcf[2 * nt + 1], rowf[2 * nt + 1]); CVT(An[nt], p[2 * nt], p[2 * nt + 1]); }
        }
      }
    }
  }
  float s = 0;
  for (int x = 0; x < NX; x++) for (int i = 0; i < 4; i++) for (int v = 0; v < 4; v++) s += acc[x][i][v];
  s += __uint_as_float(A[0][0]) + __uint_as_float(A[1][1]);
  out[blockIdx.x * blockDim.x + l] = s;
}

template <typename K> static float time_ms(K launch) {
  hipEvent_t e0, e1;
  CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
  launch(); CK(hipDeviceSynchronize());
  float best = 1e9;
  for (int rep = 0; rep < 3; rep++) {
    CK(hipEventRecord(e0)); launch(); CK(hipEventRecord(e1)); CK(hipDeviceSynchronize());
    float m; CK(hipEventElapsedTime(&m, e0, e1));
    if (m < best) best = m;
  }
  return best;
}

template <int NM, int NV, int KIND> static void run_mix(const char* name, float* d, int cus) {
  const int iters = 4000;
  printf("%-26s", name);
  for (int wps = 1; wps <= 4; wps++) {   // one workgroup per compute unit, 4 * wps waves = wps per SIMD
    const float ms = time_ms([&] { hipLaunchKernelGGL((mix_kernel<NM, NV, KIND>), dim3(cus), dim3(256 * wps), 0, 0, d, iters); });
    printf("  %dw %7.1f", wps, ms * 1e6 / iters);
  }
  printf("   ns per iteration\n");
}
template <int MODE> static void run_frag(const char* name, float* d, int cus) {
  const int iters = 2000;
  printf("%-44s", name);
  int maxb = 0;
  CK(hipOccupancyMaxActiveBlocksPerMultiprocessor(&maxb, frag_kernel<MODE>, 256, 0));
  for (int wps = 1; wps <= 2; wps++) {   // wps workgroups of 4 waves per compute unit
    if (wps > maxb) { printf("  %dw (does not fit)", wps); continue; }
    const float ms = time_ms([&] { hipLaunchKernelGGL((frag_kernel<MODE>), dim3(cus * wps), dim3(256), 0, 0, d, iters); });
    printf("  %dw %6.2f", wps, ms * 1e6 / iters / 8 / wps);
  }
  printf("   ns per fragment (12 vector + 4 MFMA) per SIMD\n");
}

int main() {
  hipDeviceProp_t prop;
  CK(hipGetDeviceProperties(&prop, 0));
  const int cus = prop.multiProcessorCount;
  printf("%s, %d compute units; columns: waves per SIMD\n", prop.gcnArchName, cus);
  float* d;
  CK(hipMalloc(&d, (size_t)cus * 2 * 1024 * sizeof(float)));
  printf("part 1: 8 MFMA (16x16x32 bf16) and N independent vector instructions per iteration\n");
  run_mix<8, 0, 0>("8 mfma", d, cus);
  run_mix<0, 32, 0>("32 v_mul_f32", d, cus);
  run_mix<0, 32, 1>("32 v_fma_f32", d, cus);
  run_mix<0, 32, 2>("32 v_cvt_pk_bf16_f32", d, cus);
  run_mix<0, 32, 3>("32 v_mul_f32_dpp", d, cus);
  run_mix<8, 8, 0>("8 mfma + 8 v_mul", d, cus);
  run_mix<8, 16, 0>("8 mfma + 16 v_mul", d, cus);
  run_mix<8, 24, 0>("8 mfma + 24 v_mul", d, cus);
  run_mix<8, 32, 0>("8 mfma + 32 v_mul", d, cus);
  run_mix<8, 48, 0>("8 mfma + 48 v_mul", d, cus);
  run_mix<8, 32, 1>("8 mfma + 32 v_fma", d, cus);
  run_mix<8, 32, 2>("8 mfma + 32 v_cvt_pk", d, cus);
  run_mix<8, 32, 3>("8 mfma + 32 v_mul_dpp", d, cus);
  printf("part 2: the state kernels' fragment pattern (8 v_mul_f32_dpp + 4 v_cvt_pk_bf16_f32 -> 4 dependent MFMAs)\n");
  run_frag<2>("4 mfma only", d, cus);
  run_frag<3>("8 dpp + 4 cvt only", d, cus);
  run_frag<0>("burst: 12 vector, then 4 mfma", d, cus);
  run_frag<1>("pipelined: mfma, 2 mul, cvt, mfma, ...", d, cus);
  return 0;
}
