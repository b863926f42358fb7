// Gated exclusive scan over the chunk axis (HBM-bound).
//
//   Y[0] = 0,  Y[k+1] = Y[k] * exp(log_G[k]) + X[k]
//
// X: [B, n, H, F], log_G: [B, n, H] fp32, Y: [B, n_out, H, F] with n_out = n + 1 (the reference
// operator, retention/_discumsum/reference.py:3-15) or n (the composed path keeps only the first
// n entries, retention/power_retention_maker.py:167-170).  Every thread owns 16 bytes of the
// feature axis and walks the chunks in order with an fp32 running state; loads for the next
// chunks are issued ahead of the dependent multiply-add so the walk is bandwidth bound.
#include "common.h"
#include "kernels.h"

namespace pr {

template <typename T, int BYTES = 16> struct Pack16 { enum { N = BYTES / sizeof(T) }; typedef __attribute__((ext_vector_type(BYTES / sizeof(T)))) T type; };
template <typename T> struct Pack16<T, 4> { enum { N = 1 }; struct type { T v; __device__ T& operator[](int) { return v; } __device__ const T& operator[](int) const { return v; } }; };

// Sum over the 64 lanes of a wave without LDS traffic inside a row: four rotate-adds (DPP) give every lane its
// row total, two cross-row exchanges finish.
__device__ __forceinline__ float wave_sum_dpp(float x) {
#define PR_ROR(n) __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x120 + n, 0xf, 0xf, true))
  x += PR_ROR(8);
  x += PR_ROR(4);
  x += PR_ROR(2);
  x += PR_ROR(1);
#undef PR_ROR
  return sum_over_rows(x);
}

// Streaming accesses.  The scans' inputs are not read again, and the forward scan's result is first read two kernels
// later: marked non-temporal they do not displace what the kernels around the scans re-read from the caches (7-9 us of
// a training step at the headline shape; the backward scan's result is read by the next kernel and is stored normally).
template <typename V> __device__ __forceinline__ V load_streaming(const V* p) {
  if constexpr (sizeof(V) == 16) return __builtin_nontemporal_load(p); else return *p;
}
template <typename V> __device__ __forceinline__ void store_streaming(const V& v, V* p) {
  if constexpr (sizeof(V) == 16) __builtin_nontemporal_store(v, p); else *p = v;
}

// Y0 [B, H, F] or null: the scan starts from it instead of zero (Y[0] = Y0).  Yfin [B, H, F] or null: receives entry n
// of the scan when the tensor itself keeps only n entries (n_out == n).
// The gate factors exp(log_G[k]) of the block's (batch, head) for all chunks, staged in LDS once per block, so that
// the walk has no global load of its own besides the streams (and no exponential per step).
constexpr int SCAN_MAXN = 2048;   // chunks whose gates fit the LDS table (longer scans read the gates as they go)
__device__ __forceinline__ const float* stage_gates(float* gsh, const float* __restrict__ logG, int n, int H) {
  if (n > SCAN_MAXN) return nullptr;
  const int bh = blockIdx.y, b = bh / H, hh = bh % H;
  const float* lg = logG + (long)b * n * H + hh;
  for (int k = threadIdx.x; k < n; k += blockDim.x) gsh[k] = __expf(lg[(long)k * H]);
  __syncthreads();
  return gsh;
}

// True for the whole block when every factor exp(log_G[k]), k >= 1, of the block's (batch, head) is an exact zero: each
// entry of the scan is then a copy of the input entry next to it (gsh: the staged factors).
__device__ __forceinline__ bool all_carries_zero(const float* gsh, int n) {
  bool nz = false;
  for (int k = 1 + (int)threadIdx.x; k < n; k += blockDim.x) nz |= gsh[k] != 0.f;
  return __syncthreads_or(nz ? 1 : 0) == 0;
}

template <typename T, int AHEAD, int BYTES>
__device__ __forceinline__ void discumsum_fwd_body(const T* __restrict__ X, const float* __restrict__ logG,
                                                   T* __restrict__ Y, int n, int n_out, int H, long F, int block,
                                                   const float* gsh, const T* __restrict__ Y0 = nullptr,
                                                   T* __restrict__ Yfin = nullptr) {
  constexpr int N = Pack16<T, BYTES>::N;
  typedef typename Pack16<T, BYTES>::type vec;
  const long per_bh = F / N;
  const long idx = (long)block * blockDim.x + threadIdx.x;
  const int bh = blockIdx.y;
  if (idx >= per_bh) return;
  const int b = bh / H, hh = bh % H;
  const vec* x = (const vec*)(X + ((long)b * n * H + hh) * F) + idx;
  vec* y = (vec*)(Y + ((long)b * n_out * H + hh) * F) + idx;
  const long xs = (long)H * F / N;  // stride between chunks, in vectors
  const float* lg = logG + (long)b * n * H + hh;

  float st[N];
#pragma unroll
  for (int i = 0; i < N; i++) st[i] = 0.f;
  vec zero;
#pragma unroll
  for (int i = 0; i < N; i++) zero[i] = (T)0.f;
  if (Y0) {
    zero = *((const vec*)(Y0 + (long)bh * F) + idx);
#pragma unroll
    for (int i = 0; i < N; i++) st[i] = to_f32(zero[i]);
  }
  y[0] = zero;
  vec* yfin = Yfin ? (vec*)(Yfin + (long)bh * F) + idx : nullptr;

  const int steps = (Yfin && n_out == n) ? n : n_out - 1;  // chunks that are consumed
  if (steps <= 0) return;
  // One step of the walk.  No branches inside: the loads of later chunks stay in flight across the steps only while
  // the compiler can count them -- with a conditional load or store in the loop it waited for ALL of them at every step
  // (vmcnt(0)); counted, the forward walk is 8 % faster at the headline shape.  (The backward walk, two input streams,
  // measured 10 % SLOWER that way and keeps the simple loop.)
  auto walk = [&](int k, const vec& cur) __attribute__((always_inline)) {
    const float gk = gsh ? gsh[k] : __expf(lg[(long)k * H]);
    const float g = (k == 0 && !Y0) ? 0.f : gk;
    vec o;
#pragma unroll
    for (int i = 0; i < N; i++) {
      st[i] = st[i] * g + to_f32(cur[i]);
      o[i] = (T)st[i];
    }
    vec* dst = (k + 1 < n_out) ? &y[(long)(k + 1) * xs] : yfin;
    store_streaming(o, dst);
  };
  vec buf[AHEAD];
#pragma unroll
  for (int a = 0; a < AHEAD; a++) buf[a] = load_streaming(&x[(long)min(a, steps - 1) * xs]);
  int k0 = 0;
  for (; k0 + 2 * AHEAD <= steps; k0 += AHEAD) {   // whole batches whose successors exist
#pragma unroll
    for (int a = 0; a < AHEAD; a++) {
      const vec cur = buf[a];
      buf[a] = load_streaming(&x[(long)(k0 + a + AHEAD) * xs]);
      walk(k0 + a, cur);
    }
  }
  if (k0 + AHEAD <= steps) {   // a whole batch followed by a partial one (loads past the end repeat the last chunk)
#pragma unroll
    for (int a = 0; a < AHEAD; a++) {
      const vec cur = buf[a];
      buf[a] = load_streaming(&x[(long)min(k0 + a + AHEAD, steps - 1) * xs]);
      walk(k0 + a, cur);
    }
    k0 += AHEAD;
  }
#pragma unroll
  for (int a = 0; a < AHEAD; a++)
    if (k0 + a < steps) walk(k0 + a, buf[a]);
}

template <typename T, int AHEAD, int BYTES = 16>
__global__ __launch_bounds__(256) void discumsum_fwd_kernel(const T* __restrict__ X, const float* __restrict__ logG,
                                                            T* __restrict__ Y, int n, int n_out, int H, long F) {
  __shared__ float gsh[SCAN_MAXN];
  discumsum_fwd_body<T, AHEAD, BYTES>(X, logG, Y, n, n_out, H, F, blockIdx.x, stage_gates(gsh, logG, n, H));
}
// Two tensors that share their gates in one launch: a 16-bit one (16 bytes per lane) in the first nblk blocks of a
// row of the grid, a small fp32 one (one element per lane, every chunk in flight) in the rest.  The small scan is
// bound by latency; next to the big one it costs nothing.
template <typename T, int AHEAD>
__global__ __launch_bounds__(256) void discumsum_pair_fwd_kernel(const T* __restrict__ X, const float* __restrict__ X2,
                                                                 const float* __restrict__ logG, T* __restrict__ Y,
                                                                 float* __restrict__ Y2, int n, int n_out, int H,
                                                                 long F, long F2, int nblk, const T* __restrict__ Y0,
                                                                 const float* __restrict__ Y02, T* __restrict__ Yfin,
                                                                 float* __restrict__ Yfin2, int follow) {
  __shared__ float gsh[SCAN_MAXN];
  const float* gs = stage_gates(gsh, logG, n, H);
  // (the readers take the input wherever an entry equals it: nothing of this (batch, head) is read or written)
  if (follow && gs && all_carries_zero(gs, n)) return;
  if ((int)blockIdx.x < nblk) discumsum_fwd_body<T, AHEAD, 16>(X, logG, Y, n, n_out, H, F, blockIdx.x, gs, Y0, Yfin);
  else discumsum_fwd_body<float, 64, 4>(X2, logG, Y2, n, n_out, H, F2, blockIdx.x - nblk, gs, Y02, Yfin2);
}

// Reverse scan: r_k = dY[k+1] + exp(log_G[k+1]) * r_{k+1};  dX[k] = r_k;
// dlog_G[k] = exp(log_G[k]) * sum_F Y[k] * r_k, written as one partial per wave (summed by
// discumsum_reduce_kernel in a fixed order, so the result is deterministic).
// partial layout: [BH][n][waves_per_bh]
// dYfin [B, H, F] or null: the gradient of entry n when the tensors keep only n entries (the forward's Yfin).
// dY0 [B, H, F] or null: receives the gradient of the scan's starting value, dY[0] + exp(log_G[0]) * r_0.
template <typename T, int AHEAD, int BYTES>
__device__ __forceinline__ void discumsum_bwd_body(const T* __restrict__ dY, const T* __restrict__ Y,
                                                   const float* __restrict__ logG, T* __restrict__ dX,
                                                   float* __restrict__ partial, int n, int n_out, int H, long F,
                                                   int waves_per_bh, int block, int wave0, const float* gsh,
                                                   const T* __restrict__ dYfin = nullptr, T* __restrict__ dY0 = nullptr) {
  constexpr int N = Pack16<T, BYTES>::N;
  typedef typename Pack16<T, BYTES>::type vec;
  const long per_bh = F / N;
  const long idx = (long)block * blockDim.x + threadIdx.x;
  const int bh = blockIdx.y;
  const bool live = idx < per_bh;
  const int b = bh / H, hh = bh % H;
  const long safe = live ? idx : 0;
  const vec* dy = (const vec*)(dY + ((long)b * n_out * H + hh) * F) + safe;
  const vec* y = (const vec*)(Y + ((long)b * n_out * H + hh) * F) + safe;
  vec* dx = (vec*)(dX + ((long)b * n * H + hh) * F) + safe;
  const long xs = (long)H * F / N;
  const float* lg = logG + (long)b * n * H + hh;
  const int wave = wave0 + ((block * blockDim.x + threadIdx.x) >> 6);
  float* part = partial + (long)bh * n * waves_per_bh + wave;

  float r[N];
#pragma unroll
  for (int i = 0; i < N; i++) r[i] = 0.f;
  vec zero;
#pragma unroll
  for (int i = 0; i < N; i++) zero[i] = (T)0.f;
  if (dYfin) zero = *((const vec*)(dYfin + (long)bh * F) + safe);   // stands for dY[n] below
  // step j = 0 .. n-1 handles chunk k = n-1-j; dY[k+1] exists when k+1 < n_out
  vec bd[AHEAD], by[AHEAD];
#pragma unroll
  for (int a = 0; a < AHEAD; a++) {
    const int k = n - 1 - a;
    if (k >= 0) {
      bd[a] = (k + 1 < n_out) ? load_streaming(&dy[(long)(k + 1) * xs]) : zero;
      by[a] = load_streaming(&y[(long)k * xs]);
    }
  }
  float g_next = 0.f;  // exp(log_G[k+1]); r_n = 0 so its value at k = n-1 is irrelevant
  for (int j0 = 0; j0 < n; j0 += AHEAD) {
#pragma unroll
    for (int a = 0; a < AHEAD; a++) {
      const int k = n - 1 - (j0 + a);
      if (k >= 0) {
        const vec d = bd[a], yk = by[a];
        const int kn = k - AHEAD;
        if (kn >= 0) {
          bd[a] = load_streaming(&dy[(long)(kn + 1) * xs]);   // kn + 1 <= n - AHEAD < n_out
          by[a] = load_streaming(&y[(long)kn * xs]);
        }
        const float gk = gsh ? gsh[k] : __expf(lg[(long)k * H]);
        float dot = 0.f;
        vec o;
#pragma unroll
        for (int i = 0; i < N; i++) {
          r[i] = r[i] * g_next + to_f32(d[i]);
          o[i] = (T)r[i];
          dot += to_f32(yk[i]) * r[i];
        }
        if (live) dx[(long)k * xs] = o;
        dot = wave_sum_dpp(live ? dot : 0.f);
        if (lane_id() == 0) part[(long)k * waves_per_bh] = dot * gk;
        g_next = gk;
      }
    }
  }
  if (dY0 && live) {   // r = r_0, g_next = exp(log_G[0])
    const vec d0 = dy[0];
    vec o;
#pragma unroll
    for (int i = 0; i < N; i++) o[i] = (T)(to_f32(d0[i]) + g_next * r[i]);
    *((vec*)(dY0 + (long)bh * F) + safe) = o;
  }
}

template <typename T, int AHEAD, int BYTES = 16>
__global__ __launch_bounds__(256) void discumsum_bwd_kernel(const T* __restrict__ dY, const T* __restrict__ Y,
                                                            const float* __restrict__ logG, T* __restrict__ dX,
                                                            float* __restrict__ partial, int n, int n_out, int H,
                                                            long F, int waves_per_bh) {
  __shared__ float gsh[SCAN_MAXN];
  discumsum_bwd_body<T, AHEAD, BYTES>(dY, Y, logG, dX, partial, n, n_out, H, F, waves_per_bh, blockIdx.x, 0,
                                      stage_gates(gsh, logG, n, H));
}
// The pair of tensors of discumsum_pair_fwd_kernel; their gate gradients land in one set of partials, so dlog_G is
// the sum of both.
template <typename T, int AHEAD>
__global__ __launch_bounds__(256) void discumsum_pair_bwd_kernel(const T* __restrict__ dY, const T* __restrict__ Y,
                                                                 const float* __restrict__ dY2,
                                                                 const float* __restrict__ Y2,
                                                                 const float* __restrict__ logG, T* __restrict__ dX,
                                                                 float* __restrict__ dX2, float* __restrict__ partial,
                                                                 int n, int n_out, int H, long F, long F2, int nblk,
                                                                 int waves_per_bh, const T* __restrict__ dYfin,
                                                                 const float* __restrict__ dYfin2,
                                                                 T* __restrict__ dY0, float* __restrict__ dY02,
                                                                 int follow) {
  __shared__ float gsh[SCAN_MAXN];
  const float* gs = stage_gates(gsh, logG, n, H);
  if (follow && gs && all_carries_zero(gs, n)) {
    // the readers take dY[k + 1] for dX[k]; the gate gradient exp(log_G[k]) * (Y[k] . dX[k]) is zero for k >= 1 by the
    // factor and for k = 0 by Y[0] = 0: this block's partial sums are written as zeros and nothing else is touched
    const int wave = (int)((blockIdx.x * blockDim.x + threadIdx.x) >> 6);   // (as the bodies number their waves)
    float* part = partial + (long)blockIdx.y * n * waves_per_bh + wave;
    if (lane_id() == 0)
      for (int k = 0; k < n; k++) part[(long)k * waves_per_bh] = 0.f;
    return;
  }
  if ((int)blockIdx.x < nblk)
    discumsum_bwd_body<T, AHEAD, 16>(dY, Y, logG, dX, partial, n, n_out, H, F, waves_per_bh, blockIdx.x, 0, gs, dYfin,
                                     dY0);
  else
    discumsum_bwd_body<float, 64, 4>(dY2, Y2, logG, dX2, partial, n, n_out, H, F2, waves_per_bh, blockIdx.x - nblk,
                                     nblk * 4, gs, dYfin2, dY02);
}

// one wave per (bh, k): sums the waves_per_bh partials in a fixed order
__global__ __launch_bounds__(256) void discumsum_reduce_kernel(const float* __restrict__ partial, float* __restrict__ dlogG,
                                                               int n, int H, int waves_per_bh, int BH) {
  const int w = (blockIdx.x * blockDim.x + threadIdx.x) >> 6;  // over BH * n
  if (w >= BH * n) return;
  const int bh = w / n, k = w % n;
  const int b = bh / H, hh = bh % H;
  const float* p = partial + (long)w * waves_per_bh;
  float s = 0.f;
  for (int i = lane_id(); i < waves_per_bh; i += 64) s += p[i];
  s = wave_sum_dpp(s);
  if (lane_id() == 0) dlogG[((long)b * n + k) * H + hh] = s;
}

template <typename T>
static int launch_fwd(const void* X, const float* logG, void* Y, int B, int n, int n_out, int H, long F, hipStream_t st) {
  constexpr int N = Pack16<T>::N;
  const long per_bh = F / N;
  dim3 grid((unsigned)((per_bh + 255) / 256), (unsigned)(B * H));
  // very few elements (the fp32 key sums): one element per thread and every chunk's load in flight at once, so the
  // walk costs one memory round trip instead of n
  if (sizeof(T) == 4 && F * B * H < 256 * 1024) {
    dim3 g1((unsigned)((F + 255) / 256), (unsigned)(B * H));
    PR_LAUNCH("discumsum_fwd", (discumsum_fwd_kernel<T, 64, 4>), g1, dim3(256), 0, st, (const T*)X, logG, (T*)Y, n, n_out, H, F);
    return (int)hipGetLastError();
  }
  // few threads in flight (small F): keep many chunks' loads outstanding per thread instead
  if (per_bh * B * H < 256 * 1024)
    PR_LAUNCH("discumsum_fwd", (discumsum_fwd_kernel<T, 16>), grid, dim3(256), 0, st, (const T*)X, logG, (T*)Y, n, n_out, H, F);
  else
    PR_LAUNCH("discumsum_fwd", (discumsum_fwd_kernel<T, 4>), grid, dim3(256), 0, st, (const T*)X, logG, (T*)Y, n, n_out, H, F);
  return (int)hipGetLastError();
}
template <typename T>
static int launch_bwd(const void* dY, const void* Y, const float* logG, void* dX, float* dlogG, float* partial, int B,
                      int n, int n_out, int H, long F, hipStream_t st) {
  constexpr int N = Pack16<T>::N;
  const long per_bh = F / N;
  const int tot = B * H * n;
  if (sizeof(T) == 4 && F * B * H < 256 * 1024) {   // see launch_fwd: one element per thread, all chunks in flight
    const unsigned b1 = (unsigned)((F + 255) / 256);
    PR_LAUNCH("discumsum_bwd", (discumsum_bwd_kernel<T, 64, 4>), dim3(b1, (unsigned)(B * H)), dim3(256), 0, st, (const T*)dY,
                       (const T*)Y, logG, (T*)dX, partial, n, n_out, H, F, (int)b1 * 4);
    PR_LAUNCH("discumsum_reduce", discumsum_reduce_kernel, dim3((tot * 64 + 255) / 256), dim3(256), 0, st, partial, dlogG, n, H,
                       (int)b1 * 4, B * H);
    return (int)hipGetLastError();
  }
  const unsigned blocks = (unsigned)((per_bh + 255) / 256);
  const int waves = blocks * 4;
  dim3 grid(blocks, (unsigned)(B * H));
  if (per_bh * B * H < 256 * 1024)
    PR_LAUNCH("discumsum_bwd", (discumsum_bwd_kernel<T, 8>), grid, dim3(256), 0, st, (const T*)dY, (const T*)Y, logG, (T*)dX,
                       partial, n, n_out, H, F, waves);
  else
    PR_LAUNCH("discumsum_bwd", (discumsum_bwd_kernel<T, 2>), grid, dim3(256), 0, st, (const T*)dY, (const T*)Y, logG, (T*)dX,
                       partial, n, n_out, H, F, waves);
  PR_LAUNCH("discumsum_reduce", discumsum_reduce_kernel, dim3((tot * 64 + 255) / 256), dim3(256), 0, st, partial, dlogG, n, H,
                     waves, B * H);
  return (int)hipGetLastError();
}

template <typename T>
static int launch_pair_fwd(const void* X, const float* X2, const float* logG, void* Y, float* Y2, int B, int n,
                           int n_out, int H, long F, long F2, const ScanCarry& cy, int follow, hipStream_t st) {
  const int nblk = (int)((F / Pack16<T>::N + 255) / 256), nblk2 = (int)((F2 + 255) / 256);
  dim3 grid((unsigned)(nblk + nblk2), (unsigned)(B * H));
  if ((F / Pack16<T>::N) * B * H < 256 * 1024)
    PR_LAUNCH("discumsum_pair_fwd", (discumsum_pair_fwd_kernel<T, 16>), grid, dim3(256), 0, st, (const T*)X, X2, logG, (T*)Y, Y2, n,
              n_out, H, F, F2, nblk, (const T*)cy.in, cy.in2, (T*)cy.out, cy.out2, follow);
  else
    PR_LAUNCH("discumsum_pair_fwd", (discumsum_pair_fwd_kernel<T, 4>), grid, dim3(256), 0, st, (const T*)X, X2, logG, (T*)Y, Y2, n,
              n_out, H, F, F2, nblk, (const T*)cy.in, cy.in2, (T*)cy.out, cy.out2, follow);
  return (int)hipGetLastError();
}
template <typename T>
static int launch_pair_bwd(const void* dY, const void* Y, const float* dY2, const float* Y2, const float* logG,
                           void* dX, float* dX2, float* dlogG, float* partial, int B, int n, int n_out, int H, long F,
                           long F2, const ScanCarry& cy, int follow, hipStream_t st) {
  const int nblk = (int)((F / Pack16<T>::N + 255) / 256), nblk2 = (int)((F2 + 255) / 256);
  const int waves = (nblk + nblk2) * 4, tot = B * H * n;
  dim3 grid((unsigned)(nblk + nblk2), (unsigned)(B * H));
  if ((F / Pack16<T>::N) * B * H < 256 * 1024)
    PR_LAUNCH("discumsum_pair_bwd", (discumsum_pair_bwd_kernel<T, 8>), grid, dim3(256), 0, st, (const T*)dY, (const T*)Y, dY2, Y2,
              logG, (T*)dX, dX2, partial, n, n_out, H, F, F2, nblk, waves, (const T*)cy.in, cy.in2, (T*)cy.out, cy.out2, follow);
  else
    PR_LAUNCH("discumsum_pair_bwd", (discumsum_pair_bwd_kernel<T, 2>), grid, dim3(256), 0, st, (const T*)dY, (const T*)Y, dY2, Y2,
              logG, (T*)dX, dX2, partial, n, n_out, H, F, F2, nblk, waves, (const T*)cy.in, cy.in2, (T*)cy.out, cy.out2, follow);
  PR_LAUNCH("discumsum_reduce", discumsum_reduce_kernel, dim3((tot * 64 + 255) / 256), dim3(256), 0, st, partial, dlogG, n, H,
                     waves, B * H);
  return (int)hipGetLastError();
}

// (the promise is used only where the scan has no value to start from or to hand on, keeps n entries, and its factors fit
// the staged table)
static int follow_ok(int follow, const ScanCarry& cy, int n, int n_out) {
  return follow && g_gate_skip && !cy.in && !cy.out && n_out == n && n <= SCAN_MAXN;
}
int discumsum_pair_fwd(const void* X, const float* X2, const float* logG, void* Y, float* Y2, int B, int n, int n_out,
                       int H, long F, long F2, const ScanCarry& cy, int consumers_follow_gates, int dtype,
                       hipStream_t st) {
  const int fl = follow_ok(consumers_follow_gates, cy, n, n_out);
  if (dtype == DT_BF16) return launch_pair_fwd<bf16_t>(X, X2, logG, Y, Y2, B, n, n_out, H, F, F2, cy, fl, st);
  if (dtype == DT_F16) return launch_pair_fwd<f16_t>(X, X2, logG, Y, Y2, B, n, n_out, H, F, F2, cy, fl, st);
  return -1;
}
long discumsum_pair_bwd_workspace_floats(int B, int n, int H, long F, long F2) {
  return (long)B * H * ((F / 8 + 255) / 256 + (F2 + 255) / 256) * 4 * n;
}
int discumsum_pair_bwd(const void* dY, const void* Y, const float* dY2, const float* Y2, const float* logG, void* dX,
                       float* dX2, float* dlogG, float* partial, int B, int n, int n_out, int H, long F, long F2,
                       const ScanCarry& cy, int consumers_follow_gates, int dtype, hipStream_t st) {
  const int fl = follow_ok(consumers_follow_gates, cy, n, n_out);
  if (dtype == DT_BF16)
    return launch_pair_bwd<bf16_t>(dY, Y, dY2, Y2, logG, dX, dX2, dlogG, partial, B, n, n_out, H, F, F2, cy, fl, st);
  if (dtype == DT_F16)
    return launch_pair_bwd<f16_t>(dY, Y, dY2, Y2, logG, dX, dX2, dlogG, partial, B, n, n_out, H, F, F2, cy, fl, st);
  return -1;
}

// Gate gradient of a scan whose backward pass has already been formed elsewhere: given the scan Y and
// R[k] = dL/dX[k] (both [B, n, H, F], and the fp32 pair Y2, R2 [B, n, H, F2]),
//   dlog_G[k] = exp(log_G[k]) * (sum_F Y[k] R[k] + sum_F2 Y2[k] R2[k]).
// grid (blocks, B*H, n); a thread of the first nblk blocks owns four 16-byte vectors of the 16-bit tensors, a thread
// of the others four floats.  Partials as in discumsum_bwd_body.
template <typename T>
__global__ __launch_bounds__(256) void scan_gate_grad_kernel(const T* __restrict__ Y, const T* __restrict__ R,
                                                             const float* __restrict__ Y2, const float* __restrict__ R2,
                                                             const float* __restrict__ logG, float* __restrict__ partial,
                                                             int n, int H, long F, long F2, int nblk, int waves_per_bh) {
  typedef typename Pack16<T, 16>::type vec;
  const int bh = blockIdx.y, k = blockIdx.z, b = bh / H, hh = bh % H;
  const long row = ((long)b * n + k) * H + hh;
  float dot = 0.f;
  if ((int)blockIdx.x < nblk) {
    const vec* y = (const vec*)(Y + row * F);
    const vec* rr = (const vec*)(R + row * F);
    const long nv = F / 8, i0 = (long)blockIdx.x * 1024 + threadIdx.x;
    vec a[4], c4[4];
#pragma unroll
    for (int u = 0; u < 4; u++)
      if (i0 + 256 * u < nv) {
        a[u] = y[i0 + 256 * u];
        c4[u] = rr[i0 + 256 * u];
      }
#pragma unroll
    for (int u = 0; u < 4; u++)
      if (i0 + 256 * u < nv)
#pragma unroll
        for (int i = 0; i < 8; i++) dot += to_f32(a[u][i]) * to_f32(c4[u][i]);
  } else {
    const long i0 = (long)(blockIdx.x - nblk) * 1024 + threadIdx.x;
#pragma unroll
    for (int u = 0; u < 4; u++)
      if (i0 + 256 * u < F2) dot += Y2[row * F2 + i0 + 256 * u] * R2[row * F2 + i0 + 256 * u];
  }
  dot = wave_sum_dpp(dot);
  const int wave = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (lane_id() == 0) partial[((long)bh * n + k) * waves_per_bh + wave] = dot * __expf(logG[row]);
}
long scan_gate_grad_workspace_floats(int B, int n, int H, long F, long F2) {
  return (long)B * H * n * ((F / 8 + 1023) / 1024 + (F2 + 1023) / 1024) * 4;
}
int scan_gate_grad(const void* Y, const void* R, const float* Y2, const float* R2, const float* logG, float* dlogG,
                   float* partial, int B, int n, int H, long F, long F2, int dtype, hipStream_t st) {
  const int nblk = (int)((F / 8 + 1023) / 1024), nblk2 = (int)((F2 + 1023) / 1024);
  const int waves = (nblk + nblk2) * 4, tot = B * H * n;
  dim3 grid((unsigned)(nblk + nblk2), (unsigned)(B * H), (unsigned)n);
  if (dtype == DT_BF16)
    PR_LAUNCH("scan_gate_grad", scan_gate_grad_kernel<bf16_t>, grid, dim3(256), 0, st, (const bf16_t*)Y, (const bf16_t*)R, Y2, R2,
                       logG, partial, n, H, F, F2, nblk, waves);
  else if (dtype == DT_F16)
    PR_LAUNCH("scan_gate_grad", scan_gate_grad_kernel<f16_t>, grid, dim3(256), 0, st, (const f16_t*)Y, (const f16_t*)R, Y2, R2,
                       logG, partial, n, H, F, F2, nblk, waves);
  else
    return -1;
  PR_LAUNCH("discumsum_reduce", discumsum_reduce_kernel, dim3((tot * 64 + 255) / 256), dim3(256), 0, st, partial, dlogG, n, H,
                     waves, B * H);
  return (int)hipGetLastError();
}

int discumsum_fwd(const void* X, const float* logG, void* Y, int B, int n, int n_out, int H, long F, int dtype,
                  hipStream_t st) {
  switch (dtype) {
    case DT_BF16: return launch_fwd<bf16_t>(X, logG, Y, B, n, n_out, H, F, st);
    case DT_F16: return launch_fwd<f16_t>(X, logG, Y, B, n, n_out, H, F, st);
    case DT_F32: return launch_fwd<float>(X, logG, Y, B, n, n_out, H, F, st);
  }
  return -1;
}
long discumsum_bwd_workspace_floats(int B, int n, int H, long F, int dtype) {
  const int N = dtype == DT_F32 ? 1 : 8;   // fp32 may run one element per thread (small tensors)
  const long blocks = (F / N + 255) / 256;
  return (long)B * H * blocks * 4 * n;
}
int discumsum_bwd(const void* dY, const void* Y, const float* logG, void* dX, float* dlogG, float* partial, int B, int n,
                  int n_out, int H, long F, int dtype, hipStream_t st) {
  switch (dtype) {
    case DT_BF16: return launch_bwd<bf16_t>(dY, Y, logG, dX, dlogG, partial, B, n, n_out, H, F, st);
    case DT_F16: return launch_bwd<f16_t>(dY, Y, logG, dX, dlogG, partial, B, n, n_out, H, F, st);
    case DT_F32: return launch_bwd<float>(dY, Y, logG, dX, dlogG, partial, B, n, n_out, H, F, st);
  }
  return -1;
}

}  // namespace pr
