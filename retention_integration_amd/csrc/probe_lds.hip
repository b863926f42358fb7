// Stand-alone microbenchmark (not part of the library): throughput of wave-wide LDS reads for the address patterns the
// MFMA kernels use, under the candidate swizzles of an unpadded row-major tile with 64-, 128- and 256-byte rows
// (CPR = 4, 8, 16 chunks of 16 bytes per row; chunk c of row r is stored at slot c ^ swizzle(r)).  It backs the two
// swizzle kinds of common.h (SWZ_K8, SWZ_ROW).
//
// Patterns (lane l, g = l / 16, c = l % 16):
//   row operand    ds_read_b128     row c, chunk 4*ks + g         (attention K/V/Q/dO tiles, sympow_grad's state tile)
//   transposed 4g  ds_read_b64_tr   row 4g + (c >> 2), columns 16*nt + 4*(c & 3)      (attention V^T, K^T, Q^T, dO^T)
//   transposed 8g  ds_read_b64_tr   row 8g + 4*hf + (c >> 2), same columns            (sympow_tn / sympow_nn operands)
//   row scalar     ds_read_b32      row c, one column, the same for the four lane groups (X tile of sympow_nn / _grad)
//
// Every read is volatile inline assembly; a lane's address comes from a table computed on the host, so any pattern can
// be timed.  256 workgroups of 8 waves, 8 reads per loop iteration; printed: ns per wave-wide read per CU (best of 3).
//
// Build and run:  python retention_integration_amd/csrc/build.py --probe && ./retention_integration_amd/probe_lds
#include <hip/hip_runtime.h>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <functional>

#define CK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__); exit(1); } } while (0)

typedef __attribute__((ext_vector_type(4))) unsigned u32x4;
typedef __attribute__((ext_vector_type(2))) unsigned u32x2;

enum { K_B128 = 1, K_TR = 2, K_B32 = 3 };

template <int KIND>
__global__ __launch_bounds__(512) void read_kernel(float* out, const unsigned* tab, int iters) {
  extern __shared__ char smem[];
  const int t = threadIdx.x;
  for (int i = t; i < 16384; i += blockDim.x) ((unsigned*)smem)[i] = 0x3f803f80u;
  __syncthreads();
  const unsigned addr = (unsigned)(uintptr_t)(__attribute__((address_space(3))) char*)smem + tab[t & 63];
  u32x4 d4[8];
  u32x2 d2[8];
  unsigned d1[8];
  for (int i = 0; i < 8; i++) { d4[i] = (u32x4){0, 0, 0, 0}; d2[i] = (u32x2){0, 0}; d1[i] = 0; }
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int s = 0; s < 8; s++) {   // the 4 KB steps keep every read inside the 64 KB and on the same banks
      if (KIND == K_B128) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(d4[s]) : "v"(addr), "n"(s * 4096));
      if (KIND == K_TR) asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(d2[s]) : "v"(addr), "n"(s * 4096));
      if (KIND == K_B32) asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(d1[s]) : "v"(addr), "n"(s * 4096));
    }
    asm volatile("s_waitcnt lgkmcnt(0)");
  }
  float sm = 0;
  for (int i = 0; i < 8; i++) {
    for (int v = 0; v < 4; v++) sm += __uint_as_float(d4[i][v]);
    sm += __uint_as_float(d2[i][0]) + __uint_as_float(d2[i][1]) + __uint_as_float(d1[i]);
  }
  out[blockIdx.x * blockDim.x + t] = sm;
}

static float* out;
static unsigned* dtab;

static float run(int kind, const std::function<unsigned(int)>& f) {
  unsigned h[64];
  for (int l = 0; l < 64; l++) {
    h[l] = f(l);
    if (h[l] + 7 * 4096 + 16 > 65536) { printf("pattern leaves the 64 KB\n"); exit(1); }
  }
  CK(hipMemcpy(dtab, h, sizeof(h), hipMemcpyHostToDevice));
  hipEvent_t e0, e1;
  CK(hipEventCreate(&e0));
  CK(hipEventCreate(&e1));
  const int iters = 1000, waves = 8;
  float best = 1e9;
  for (int rep = 0; rep < 3; rep++) {
    CK(hipEventRecord(e0));
    if (kind == K_B128) hipLaunchKernelGGL(read_kernel<K_B128>, dim3(256), dim3(64 * waves), 65536, 0, out, dtab, iters);
    if (kind == K_TR) hipLaunchKernelGGL(read_kernel<K_TR>, dim3(256), dim3(64 * waves), 65536, 0, out, dtab, iters);
    if (kind == K_B32) hipLaunchKernelGGL(read_kernel<K_B32>, dim3(256), dim3(64 * waves), 65536, 0, out, dtab, iters);
    CK(hipGetLastError());
    CK(hipEventRecord(e1));
    CK(hipDeviceSynchronize());
    float ms;
    CK(hipEventElapsedTime(&ms, e0, e1));
    if (ms < best) best = ms;
  }
  CK(hipEventDestroy(e0));
  CK(hipEventDestroy(e1));
  return best * 1e6f / iters / 8 / waves;
}

// the candidate swizzles
static int swz_k8(int CPR, int row) {   // SWZ_K8 of common.h
  if (CPR == 8) { const int k = (row >> 1) & 7; return ((k & 1) << 2) | (k >> 1); }
  if (CPR == 16) { const int k = row & 15; return ((k & 3) << 2) | (k >> 2); }
  return (row >> 2) & 3;
}
static int swz_row(int CPR, int row) { return ((row * CPR) >> 3) & (CPR - 1); }   // SWZ_ROW of common.h
static int swz_low(int CPR, int row) { return row & (CPR - 1); }
static int swz_none(int, int) { return 0; }

int main() {
  CK(hipMalloc(&out, 256 * 512 * 4));
  CK(hipMalloc(&dtab, 256));
  CK(hipFuncSetAttribute((const void*)read_kernel<K_B128>, hipFuncAttributeMaxDynamicSharedMemorySize, 65536));
  CK(hipFuncSetAttribute((const void*)read_kernel<K_TR>, hipFuncAttributeMaxDynamicSharedMemorySize, 65536));
  CK(hipFuncSetAttribute((const void*)read_kernel<K_B32>, hipFuncAttributeMaxDynamicSharedMemorySize, 65536));
  printf("consecutive addresses (no conflicts): ds_read_b128 %.2f, ds_read_b64_tr_b16 %.2f, ds_read_b32 %.2f ns per wave-wide read\n",
         run(K_B128, [](int l) { return 16u * l; }), run(K_TR, [](int l) { return 8u * l; }), run(K_B32, [](int l) { return 4u * l; }));
  struct Cand { const char* name; int (*f)(int, int); };
  const Cand cands[] = {{"SWZ_K8", swz_k8}, {"SWZ_ROW", swz_row}, {"row % CPR", swz_low}, {"none", swz_none}};
  printf("%-9s %-10s  %11s  %13s  %13s  %10s   (ns per wave-wide read)\n", "row bytes", "swizzle", "row operand", "transposed 4g", "transposed 8g", "row scalar");
  for (int CPR : {4, 8, 16}) {
    const int RB = CPR * 16;
    for (const Cand& cd : cands) {
      auto S = [&](int row) { return cd.f(CPR, row); };
      // worst of the instances a kernel issues (ks = 0, 1; nt = 0, 1; hf = 0, 1)
      float a = 0, t4 = 0, t8 = 0;
      for (int ks = 0; ks < (CPR >= 8 ? 2 : 1); ks++)
        a = fmaxf(a, run(K_B128, [&](int l) { const int g = l >> 4, c = l & 15; return (unsigned)(c * RB + ((((4 * ks + g) % CPR) ^ S(c)) * 16)); }));
      for (int nt = 0; nt < 2; nt++) {
        t4 = fmaxf(t4, run(K_TR, [&](int l) {
               const int g = l >> 4, c = l & 15, row = 4 * g + (c >> 2), col = 16 * nt + 4 * (c & 3);
               return (unsigned)(row * RB + (((col / 8) ^ S(row)) * 16) + (col % 8) * 2); }));
        for (int hf = 0; hf < 2; hf++)
          t8 = fmaxf(t8, run(K_TR, [&](int l) {
                 const int g = l >> 4, c = l & 15, row = 8 * g + 4 * hf + (c >> 2), col = 16 * nt + 4 * (c & 3);
                 return (unsigned)(row * RB + (((col / 8) ^ S(row)) * 16) + (col % 8) * 2); }));
      }
      const float x = run(K_B32, [&](int l) { const int c = l & 15; return (unsigned)(c * RB + (S(c) * 16)); });
      printf("%-9d %-10s  %11.2f  %13.2f  %13.2f  %10.2f\n", RB, cd.name, a, t4, t8, x);
    }
  }
  return 0;
}
