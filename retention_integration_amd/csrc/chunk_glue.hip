// Per-chunk gate arithmetic of the chunked algorithm, fused into two HBM-bound kernels
// (ref: retention/power_retention_maker.py:143-186 and its autograd):
//
// forward  : A = cumsum_c(log_G),  lcs = A[c-1],  Kd = K * exp((A[c-1] - A)/deg),  Qg = Q * exp(A/deg)
// backward : dK = dK_attn + dKd * w,  dQ = dQ_attn + dQg * u,  dV = dV_attn + dV_state,
//            dA_t = dG_attn_t + (sum_d dQg.Qg - sum_d dKd.Kd)_t / deg,
//            dA_{c-1} += (sum_{t,d} dKd.Kd)/deg + dlcs,   dlog_G = reverse-cumsum_c(dA)
//
// One workgroup per (chunk, kv head); the chunk's gate vector lives in LDS.
#include "common.h"
#include "kernels.h"

namespace pr {

constexpr int GLUE_MAX_C = 8192;

// In-place inclusive scan of a[0..c) in LDS by 256 threads (reverse = suffix sums).
__device__ inline void block_scan(float* a, float* tot, int c, bool reverse) {
  const int tid = threadIdx.x;
  const int seg = (c + 255) / 256;
  const int lo = min(tid * seg, c), hi = min(lo + seg, c);
  float run = 0.f;
  for (int i = lo; i < hi; i++) {
    const int j = reverse ? c - 1 - i : i;
    run += a[j];
    a[j] = run;
  }
  tot[tid] = run;
  __syncthreads();
  for (int off = 1; off < 256; off <<= 1) {
    const float add = tid >= off ? tot[tid - off] : 0.f;
    __syncthreads();
    tot[tid] += add;
    __syncthreads();
  }
  const float base = tid > 0 ? tot[tid - 1] : 0.f;
  for (int i = lo; i < hi; i++) a[reverse ? c - 1 - i : i] += base;
  __syncthreads();
}

template <typename T, int DH>
__global__ __launch_bounds__(256) void chunk_prep_fwd_kernel(const float* __restrict__ logG, const T* __restrict__ K,
                                                             const T* __restrict__ Q, float* __restrict__ A,
                                                             float* __restrict__ lcs, T* __restrict__ Kd,
                                                             T* __restrict__ Qg, int c, int h, int r, float inv_deg) {
  typedef typename VecOf<T>::v8 v8;
  extern __shared__ __attribute__((aligned(16))) char smem[];
  float* a = (float*)smem;     // [c]
  float* tot = a + c;          // [256]
  const int tid = threadIdx.x, bn = blockIdx.x / h, hh = blockIdx.x % h, hq = h * r;
  const float* lg = logG + (long)bn * c * h + hh;
  for (int i = tid; i < c; i += 256) a[i] = lg[(long)i * h];
  __syncthreads();
  block_scan(a, tot, c, false);
  float* Ao = A + (long)bn * c * h + hh;
  for (int i = tid; i < c; i += 256) Ao[(long)i * h] = a[i];
  const float a_last = a[c - 1];
  if (tid == 0) lcs[(long)bn * h + hh] = a_last;

  constexpr int LPR = DH / 8;          // threads per row
  const int sub = tid % LPR, col = sub * 8;
  for (int t = tid / LPR; t < c; t += 256 / LPR) {
    const float w = __expf((a_last - a[t]) * inv_deg), u = __expf(a[t] * inv_deg);
    {
      const long o = (((long)bn * c + t) * h + hh) * DH + col;
      float f[8];
      unpack8(*(const v8*)(K + o), f);
#pragma unroll
      for (int i = 0; i < 8; i++) f[i] *= w;
      *(v8*)(Kd + o) = pack8<T>(f);
    }
    for (int rr = 0; rr < r; rr++) {
      const long o = (((long)bn * c + t) * hq + hh * r + rr) * DH + col;
      float f[8];
      unpack8(*(const v8*)(Q + o), f);
#pragma unroll
      for (int i = 0; i < 8; i++) f[i] *= u;
      *(v8*)(Qg + o) = pack8<T>(f);
    }
  }
}

struct GlueBwdArgs {
  const float* A;       // [BN, c, h] or null (ungated)
  const void* Kd;       // [BN, c, h, d]
  const void* dKd;      // [BN, c, h, d]
  const void* Qg;       // [BN, c, hq, d]
  const void* dQg;      // [BN, c, hq, d]
  const void* dK_attn;  // [BN, c, h, d]
  const void* dQ_attn;  // [BN, c, hq, d]
  const void* dV_attn;  // [BN, c, h, d]
  const void* dV_state; // [BN, c, h, d]
  const float* dG_attn; // [BN, c, h]
  const float* dlcs_a;  // [BN, h]
  const float* dlcs_b;  // [BN, h]
  void* dK;
  void* dQ;
  void* dV;
  float* dlogG;         // [BN, c, h]
  int c, h, r;
  float inv_deg;
};

template <typename T, int DH> __global__ __launch_bounds__(256) void chunk_glue_bwd_kernel(GlueBwdArgs g) {
  typedef typename VecOf<T>::v8 v8;
  extern __shared__ __attribute__((aligned(16))) char smem[];
  float* da = (float*)smem;       // [c]
  float* tot = da + g.c;          // [256]
  const int tid = threadIdx.x, c = g.c, h = g.h, r = g.r, hq = h * r;
  const int bn = blockIdx.x / h, hh = blockIdx.x % h;
  const bool gated = g.A != nullptr;
  const float* Ai = gated ? g.A + (long)bn * c * h + hh : nullptr;
  const float a_last = gated ? Ai[(long)(c - 1) * h] : 0.f;

  constexpr int LPR = DH / 8;
  const int sub = tid % LPR, col = sub * 8;
  float ksum = 0.f;   // this thread's share of sum_{t,d} dKd.Kd
  for (int t = tid / LPR; t < c; t += 256 / LPR) {
    const float at = gated ? Ai[(long)t * h] : 0.f;
    const float w = gated ? __expf((a_last - at) * g.inv_deg) : 1.f, u = gated ? __expf(at * g.inv_deg) : 1.f;
    float dotk = 0.f, dotq = 0.f;
    {
      const long o = (((long)bn * c + t) * h + hh) * DH + col;
      float kd[8], dkd[8], dka[8], dva[8], dvs[8], ok[8], ov[8];
      unpack8(*(const v8*)((const T*)g.Kd + o), kd);
      unpack8(*(const v8*)((const T*)g.dKd + o), dkd);
      unpack8(*(const v8*)((const T*)g.dK_attn + o), dka);
      unpack8(*(const v8*)((const T*)g.dV_attn + o), dva);
      unpack8(*(const v8*)((const T*)g.dV_state + o), dvs);
#pragma unroll
      for (int i = 0; i < 8; i++) {
        dotk += kd[i] * dkd[i];
        ok[i] = dka[i] + dkd[i] * w;
        ov[i] = dva[i] + dvs[i];
      }
      *(v8*)((T*)g.dK + o) = pack8<T>(ok);
      *(v8*)((T*)g.dV + o) = pack8<T>(ov);
    }
    for (int rr = 0; rr < r; rr++) {
      const long o = (((long)bn * c + t) * hq + hh * r + rr) * DH + col;
      float qg[8], dqg[8], dqa[8], oq[8];
      unpack8(*(const v8*)((const T*)g.Qg + o), qg);
      unpack8(*(const v8*)((const T*)g.dQg + o), dqg);
      unpack8(*(const v8*)((const T*)g.dQ_attn + o), dqa);
#pragma unroll
      for (int i = 0; i < 8; i++) {
        dotq += qg[i] * dqg[i];
        oq[i] = dqa[i] + dqg[i] * u;
      }
      *(v8*)((T*)g.dQ + o) = pack8<T>(oq);
    }
    if (gated) {
#pragma unroll
      for (int m = 1; m < LPR; m <<= 1) {
        dotk += __shfl_xor(dotk, m);
        dotq += __shfl_xor(dotq, m);
      }
      if (sub == 0) {
        da[t] = g.dG_attn[((long)bn * c + t) * h + hh] + (dotq - dotk) * g.inv_deg;
        ksum += dotk;
      }
    }
  }
  if (!gated) return;
  // total of dKd.Kd over the chunk
  tot[tid] = ksum;
  __syncthreads();
  for (int off = 128; off > 0; off >>= 1) {
    if (tid < off) tot[tid] += tot[tid + off];
    __syncthreads();
  }
  if (tid == 0) da[c - 1] += tot[0] * g.inv_deg + g.dlcs_a[(long)bn * h + hh] + g.dlcs_b[(long)bn * h + hh];
  __syncthreads();
  block_scan(da, tot, c, true);
  float* out = g.dlogG + (long)bn * c * h + hh;
  for (int i = tid; i < c; i += 256) out[(long)i * h] = da[i];
}

template <typename T>
static int prep_launch(const float* logG, const void* K, const void* Q, float* A, float* lcs, void* Kd, void* Qg, int BN,
                       int c, int h, int r, int d, int deg, hipStream_t st) {
  const size_t smem = (size_t)(c + 256) * sizeof(float);
  dim3 grid((unsigned)(BN * h));
#define PR_CP(DD)                                                                                                      \
  case DD:                                                                                                             \
    hipLaunchKernelGGL((chunk_prep_fwd_kernel<T, DD>), grid, dim3(256), smem, st, logG, (const T*)K, (const T*)Q, A,   \
                       lcs, (T*)Kd, (T*)Qg, c, h, r, 1.f / deg);                                                       \
    break;
  switch (d) { PR_CP(32) PR_CP(64) PR_CP(128) default: return -2; }
#undef PR_CP
  return (int)hipGetLastError();
}

int chunk_prep_fwd(const float* logG, const void* K, const void* Q, float* A, float* lcs, void* Kd, void* Qg, int BN,
                   int c, int h, int r, int d, int deg, int dtype, hipStream_t st) {
  if (c > GLUE_MAX_C) return -5;
  if (dtype == DT_BF16) return prep_launch<bf16_t>(logG, K, Q, A, lcs, Kd, Qg, BN, c, h, r, d, deg, st);
  if (dtype == DT_F16) return prep_launch<f16_t>(logG, K, Q, A, lcs, Kd, Qg, BN, c, h, r, d, deg, st);
  return -1;
}

int chunk_glue_bwd(const float* A, const void* Kd, const void* dKd, const void* Qg, const void* dQg,
                   const void* dK_attn, const void* dQ_attn, const void* dV_attn, const void* dV_state,
                   const float* dG_attn, const float* dlcs_a, const float* dlcs_b, void* dK, void* dQ, void* dV,
                   float* dlogG, int BN, int c, int h, int r, int d, int deg, int dtype, hipStream_t st) {
  if (c > GLUE_MAX_C) return -5;
  GlueBwdArgs g{A, Kd, dKd, Qg, dQg, dK_attn, dQ_attn, dV_attn, dV_state, dG_attn, dlcs_a, dlcs_b,
                dK, dQ, dV, dlogG, c, h, r, 1.f / deg};
  const size_t smem = (size_t)(c + 256) * sizeof(float);
  dim3 grid((unsigned)(BN * h));
#define PR_GB(T, DD)                                                                                                   \
  case DD: hipLaunchKernelGGL((chunk_glue_bwd_kernel<T, DD>), grid, dim3(256), smem, st, g); break;
#define PR_GBT(T)                                                                                                      \
  switch (d) { PR_GB(T, 32) PR_GB(T, 64) PR_GB(T, 128) default: return -2; }                                           \
  return (int)hipGetLastError();
  if (dtype == DT_BF16) { PR_GBT(bf16_t) }
  if (dtype == DT_F16) { PR_GBT(f16_t) }
#undef PR_GBT
#undef PR_GB
  return -1;
}

}  // namespace pr
