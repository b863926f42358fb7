// Per-chunk gate arithmetic of the chunked algorithm, as HBM-bound kernels
// (ref: retention/power_retention_maker.py:143-186 and its autograd):
//
// forward  : A = cumsum_c(log_G),  lcs = A[c-1],  Kd = K * exp((A[c-1] - A)/deg),  Qg = Q * exp(A/deg)
// backward : dK = dK_attn + dKd * w,  dQ = dQ_attn + dQg * u,  dV = dV_attn + dV_state,
//            dA_t = dG_attn_t + (sum_d dQg.Qg - sum_d dKd.Kd)_t / deg,
//            dA_{c-1} += (sum_{t,d} dKd.Kd)/deg + dlcs,   dlog_G = reverse-cumsum_c(dA)
//
// The scans over the chunk (one workgroup per (chunk, head), gate vector in LDS) are separate tiny kernels;
// the row-wise parts are fully parallel over (chunk, position, head) with 16 bytes per lane.
#include "common.h"
#include "kernels.h"

namespace pr {

constexpr int GLUE_MAX_C = 8192;

// Workgroups go to the 8 XCDs (each with its own L2) round-robin by linear id.  The h workgroups of a chunk read
// interleaved elements of the same cache lines ([.., position, head] arrays), so ids are permuted to put them on one
// XCD: XCD x takes the x-th eighth of the (chunk, head) pairs.  Otherwise every line is fetched by up to 8 L2s.
__device__ __forceinline__ int xcd_contiguous(int id, int total) {
  return total % 8 == 0 ? (id % 8) * (total / 8) + id / 8 : id;
}

// In-place inclusive scan of a[0..c) in LDS by 256 threads (reverse = suffix sums): every thread scans its own run of
// elements, the run totals are scanned inside each wave with lane shifts and across the four waves through tot[0..4).
__device__ inline void block_scan(float* a, float* tot, int c, bool reverse) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int seg = (c + 255) / 256;
  const int lo = min(tid * seg, c), hi = min(lo + seg, c);
  float run = 0.f;
  for (int i = lo; i < hi; i++) {
    const int j = reverse ? c - 1 - i : i;
    run += a[j];
    a[j] = run;
  }
  float x = run;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const float y = __shfl_up(x, off);
    if (lane >= off) x += y;
  }
  if (lane == 63) tot[wave] = x;   // (callers that used tot before have synchronised since)
  __syncthreads();
  float base = x - run;
  for (int w = 0; w < wave; w++) base += tot[w];
  for (int i = lo; i < hi; i++) a[reverse ? c - 1 - i : i] += base;
  __syncthreads();
}

// A[bn, :, hh] = cumsum(log_G[bn, :, hh]);  lcs[bn, hh] = A[bn, c-1, hh]
// live[bn, hh] = {first t whose key factor exp((A[c-1] - A[t]) / deg) is not zero (the expression of gate_apply_fwd),
//                 one past the last t with exp(A[t]) != 0}: outside them the discounted keys, resp. everything that
// carries the factor exp(A[t]) of a query's state part, are exact zeros, and the kernels that contract over the chunk's
// rows leave those rows out.
__global__ __launch_bounds__(256) void gate_scan_fwd_kernel(const float* __restrict__ logG, float* __restrict__ A,
                                                            float* __restrict__ lcs, int* __restrict__ live, int c, int h,
                                                            float inv_deg) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  float* a = (float*)smem;
  float* tot = a + c;
  const int tid = threadIdx.x, wg = xcd_contiguous(blockIdx.x, gridDim.x), bn = wg / h, hh = wg % h;
  const long base = (long)bn * c * h + hh;
  for (int i = tid; i < c; i += 256) a[i] = logG[base + (long)i * h];
  __syncthreads();
  block_scan(a, tot, c, false);
  for (int i = tid; i < c; i += 256) A[base + (long)i * h] = a[i];
  if (tid == 0 && lcs) lcs[(long)bn * h + hh] = a[c - 1];
  if (live) {
    const float al = a[c - 1];
    int lo = c, hi = 0;
    for (int i = tid; i < c; i += 256) {
      if (__expf((al - a[i]) * inv_deg) != 0.f) lo = min(lo, i);
      if (__expf(a[i]) != 0.f) hi = max(hi, i + 1);
    }
#pragma unroll
    for (int m = 32; m > 0; m >>= 1) {
      lo = min(lo, __shfl_xor(lo, m));
      hi = max(hi, __shfl_xor(hi, m));
    }
    int* red = (int*)(tot + 8);   // (tot[0..4) may still be read by a slower wave of the scan)
    if ((tid & 63) == 0) {
      red[2 * (tid >> 6)] = lo;
      red[2 * (tid >> 6) + 1] = hi;
    }
    __syncthreads();
    if (tid == 0) {
      live[((long)bn * h + hh) * 2] = min(min(red[0], red[2]), min(red[4], red[6]));
      live[((long)bn * h + hh) * 2 + 1] = max(max(red[1], red[3]), max(red[5], red[7]));
    }
  }
}

// one group of DH/8 lanes per (chunk, position, kv head)
template <typename T, int DH>
__global__ __launch_bounds__(256) void gate_apply_fwd_kernel(const float* __restrict__ A, const float* __restrict__ lcs,
                                                             const T* __restrict__ K, const T* __restrict__ Q,
                                                             T* __restrict__ Kd, T* __restrict__ Qg, long groups,
                                                             int c, int h, int r, float inv_deg,
                                                             const int* __restrict__ live) {
  typedef typename VecOf<T>::v8 v8;
  constexpr int LPR = DH / 8;
  const long gid = ((long)blockIdx.x * 256 + threadIdx.x) / LPR;
  if (gid >= groups) return;
  const int col = (threadIdx.x % LPR) * 8;
  const int hh = (int)(gid % h);
  const long bn = gid / ((long)c * h);
  const float at = A[gid], al = lcs[bn * h + hh];
  const float w = __expf((al - at) * inv_deg), u = __expf(at * inv_deg);
  float f[8];
  // (live: the readers of Kd leave out the time steps before live[bn, hh, 0], whose factor w is zero, in whole row
  // blocks of theirs -- 64, 128 or 256 rows: the rows before the block of 256 that holds the first live one are neither
  // read nor written here)
  if (!live || (int)((gid / h) % c) >= (live[(bn * h + hh) * 2] & ~255)) {
    unpack8(*(const v8*)(K + gid * DH + col), f);
#pragma unroll
    for (int i = 0; i < 8; i++) f[i] *= w;
    *(v8*)(Kd + gid * DH + col) = pack8<T>(f);
  }
  for (int rr = 0; Qg && rr < r; rr++) {
    const long o = (gid * r + rr) * DH + col;
    unpack8(*(const v8*)(Q + o), f);
#pragma unroll
    for (int i = 0; i < 8; i++) f[i] *= u;
    *(v8*)(Qg + o) = pack8<T>(f);
  }
}

// dA += sum over the r query heads of dGq (when given); dA[c-1] += (sum_t dotk)/deg + dlcs_a + dlcs_b, then
// dlog_G = reverse cumsum of dA (in place)
__global__ __launch_bounds__(256) void gate_scan_bwd_kernel(float* __restrict__ dA, const float* __restrict__ dGq,
                                                            const float* __restrict__ dotk,
                                                            const float* __restrict__ dlcs_a,
                                                            const float* __restrict__ dlcs_b, int c, int h, int r,
                                                            float inv_deg) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  float* a = (float*)smem;
  float* tot = a + c;
  const int tid = threadIdx.x, wg = xcd_contiguous(blockIdx.x, gridDim.x), bn = wg / h, hh = wg % h;
  const long base = (long)bn * c * h + hh;
  float ks = 0.f;
  for (int i = tid; i < c; i += 256) {
    float v = dA[base + (long)i * h];
    if (dGq)
      for (int rr = 0; rr < r; rr++) v += dGq[(base + (long)i * h) * r + rr];
    a[i] = v;
    ks += dotk[base + (long)i * h];
  }
#pragma unroll
  for (int m = 32; m > 0; m >>= 1) ks += __shfl_xor(ks, m);
  if ((tid & 63) == 0) tot[tid >> 6] = ks;
  __syncthreads();
  if (tid == 0)
    a[c - 1] += (tot[0] + tot[1] + tot[2] + tot[3]) * inv_deg + dlcs_a[(long)bn * h + hh] +
                (dlcs_b ? dlcs_b[(long)bn * h + hh] : 0.f);
  __syncthreads();
  block_scan(a, tot, c, true);
  for (int i = tid; i < c; i += 256) dA[base + (long)i * h] = a[i];
}

template <typename T>
static int prep_launch(const float* logG, const void* K, const void* Q, float* A, float* lcs, void* Kd, void* Qg, int* live,
                       int BN, int c, int h, int r, int d, int deg, hipStream_t st) {
  const size_t smem = (size_t)(c + 256) * sizeof(float);
  // (either half on its own: no log_G = A and lcs are already there; no Kd = only the sums are wanted)
  if (logG) PR_LAUNCH("gate_scan_fwd", gate_scan_fwd_kernel, dim3((unsigned)(BN * h)), dim3(256), smem, st, logG, A, lcs, live, c, h, 1.f / deg);
  if (!Kd) return (int)hipGetLastError();
  const long groups = (long)BN * c * h;
#define PR_CP(DD)                                                                                                      \
  case DD:                                                                                                             \
    PR_LAUNCH("gate_apply_fwd", (gate_apply_fwd_kernel<T, DD>), dim3((unsigned)((groups * (DD / 8) + 255) / 256)), dim3(256), 0, \
                       st, A, lcs, (const T*)K, (const T*)Q, (T*)Kd, (T*)Qg, groups, c, h, r, 1.f / deg,               \
                       (!logG && g_gate_skip) ? live : nullptr);                                                      \
    break;
  switch (d) { PR_CP(32) PR_CP(64) PR_CP(128) default: return -2; }
#undef PR_CP
  return (int)hipGetLastError();
}

int gate_cumsum(const float* logG, float* A, int B, int t, int h, hipStream_t st) {
  if (t > GLUE_MAX_C) return -5;
  const size_t smem = (size_t)(t + 256) * sizeof(float);
  PR_LAUNCH("gate_scan_fwd", gate_scan_fwd_kernel, dim3((unsigned)(B * h)), dim3(256), smem, st, logG, A, (float*)nullptr, (int*)nullptr, t, h, 1.f);
  return (int)hipGetLastError();
}

int chunk_prep_fwd(const float* logG, const void* K, const void* Q, float* A, float* lcs, void* Kd, void* Qg, int* live,
                   int BN, int c, int h, int r, int d, int deg, int dtype, hipStream_t st) {
  if (c > GLUE_MAX_C) return -5;
  if (dtype == DT_BF16) return prep_launch<bf16_t>(logG, K, Q, A, lcs, Kd, Qg, live, BN, c, h, r, d, deg, st);
  if (dtype == DT_F16) return prep_launch<f16_t>(logG, K, Q, A, lcs, Kd, Qg, live, BN, c, h, r, d, deg, st);
  return -1;
}

int chunk_gate_scan_bwd(float* dA, const float* dGq, const float* dotk, const float* dlcs_a, const float* dlcs_b, int BN,
                        int c, int h, int r, int deg, hipStream_t st) {
  if (c > GLUE_MAX_C) return -5;
  const size_t smem = (size_t)(c + 256) * sizeof(float);
  PR_LAUNCH("gate_scan_bwd", gate_scan_bwd_kernel, dim3((unsigned)(BN * h)), dim3(256), smem, st, dA, dGq, dotk, dlcs_a, dlcs_b,
                     c, h, r, 1.f / deg);
  return (int)hipGetLastError();
}

}  // namespace pr
