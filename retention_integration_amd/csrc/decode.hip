// Single-token inference step on the state (HBM-bound): query the state and, optionally, fold one new token into it
// in the same pass over S.
//
//   query  (ref: retention/_query_state/reference.py:36-96 with one query position; composed at
//           retention/power_retention_maker.py:358-363):
//       q' = Q * exp(G_last / deg) rounded to the input dtype,
//       y[e] = sum_f phi(q')[f] S[f, e],   lq = sum_f phi(q')[f] s[f],
//       merged with the attention result over the not-yet-folded cache (Y_attn, l_attn, rowmax) exactly as the
//       chunked kernel does;
//   update (ref: retention/power_retention_maker.py:366-382 with a single new key/value, and
//           retention/_update_state/reference.py:33-52):
//       S'[f, e] = decay * S[f, e] + m_f phi(k)[f] v[e],   s'[f] = decay * s[f] + m_f phi(k)[f].
//
// The query reads the OLD state, so one pass serves both (and the update may be in place: a state element is read and
// then written by the same thread, the key sum of a feature row by the lanes of one wave before its lane 0 writes it): every workgroup owns a slice of the features of one
// (batch, kv head), streams its rows of S once (16 bytes per lane, fully coalesced), accumulates the query partials
// in registers and writes the updated rows.  A second, tiny kernel adds the partials of the slices and merges; with
// many (batch, kv head) pairs and one or two query rows a single 1024-thread workgroup takes a whole pair and merges
// in the same kernel.
#include <mutex>

#include "common.h"
#include "kernels.h"

namespace pr {

// Partial query sums of decode_step_static() (below): device memory that belongs to the library, one copy per GPU,
// held until the process ends.  In host code this name is only a handle for hipGetSymbolAddress -- never a device
// address: kernels get the address that call returns.
constexpr long DEC_STATIC_FLOATS = 2L << 20;   // 8 MiB
static __device__ __align__(256) float scratch[DEC_STATIC_FLOATS];

constexpr int DEC_MAXROWS = 16;   // query rows (positions x query heads per kv head) handled per (batch, kv head)


__device__ __forceinline__ void feature_pair(int f, int& x, int& w, float& mult) {
  int y = 0;
  while (128 * (y + 1) * (y + 2) <= f) y++;
  const int rem = f - 128 * y * (y + 1);
  x = rem >> 4;
  w = 16 * y + (rem & 15);
  mult = (x < 16 * y) ? 2.f : 1.f;
}

struct DecodeArgs {
  const void* Q;        // [B, rows_t, h*r, d]   (rows_t positions)
  const float* gq;      // [B, h] accumulated log gate at the query position, or null
  const void* S;        // [B, h, D, d]
  const float* s;       // [B, h, D]
  const void* Knew;     // [B, h, d] or null (no update)
  const void* Vnew;     // [B, h, d]
  const float* decay;   // [B, h] log of the decay applied to the old state, or null (= 0)
  void* Sout;           // [B, h, D, d]
  float* sout;          // [B, h, D]
  float* part;          // [B*h, split, rows, d + 1] partial query sums (unused when one workgroup owns a pair)
  int h, r, tq, split, deg;
  // the merge with the attention part
  const void* Y_attn;   // [B, tq, h*r, d] or null
  const float* l_attn;  // [B, tq, h*r]
  const float* rowmax;  // [B, tq, h*r]
  void* out;            // [B, tq, h*r, d]
  float scale_p;
  int attend_new;       // the attention part is the one new token attending to itself
};

// out[row, e] = (Y_attn * wa + y * wq) / (l_attn * wa + lq * wq), the merge of the chunked kernel
// (sympow_nn.hip); without an attention part out = y / lq.  Run by one wave; y(e) gives the query sums.
// With Qn/Kn/Vn the attention part is that of the ONE new token attending to itself (tq = 1): one weight
// (scale q.k)^deg, so Y_attn = v, l_attn = 1 + 1e-6 and rowmax = log of the weight
// (ref: retention/_attention/reference.py:42-69 with a single key).
template <typename T, int DH, typename YF>
__device__ __forceinline__ void decode_merge_row(int lane, YF y, float lq, const T* __restrict__ Y_attn,
                                                 const float* __restrict__ l_attn, const float* __restrict__ rowmax,
                                                 const T* __restrict__ Qn, const T* __restrict__ Kn,
                                                 const T* __restrict__ Vn, T* __restrict__ out, long ro, int pair,
                                                 float scale_p, float deg) {
  constexpr int D = 128 * (DH / 16) * (DH / 16 + 1);
  float wa = 0.f, wq = 1.f, la = 0.f;
  const T* ya = Y_attn ? Y_attn + ro * DH : nullptr;
  if (Kn) {
    float dot = 0.f;
    for (int e = lane; e < DH; e += 64) dot += (float)Qn[ro * DH + e] * (float)Kn[(long)pair * DH + e];
    dot = sum_over_rows(sum_in_row(dot));
    const float scale = __expf(__logf(scale_p) / deg), eps = 1e-7f / scale;
    const float m = 0.5f * deg * __logf(dot * dot + eps * eps) + __logf(scale_p);
    const float beta = fmaxf(m, 0.5f * __logf((float)D));
    la = 1.f + 1e-6f;
    wa = __expf(m - beta);
    wq = scale_p * __expf(-beta);
    ya = Vn + (long)pair * DH;
  } else if (Y_attn) {
    const float m = rowmax[ro], beta = fmaxf(m, 0.5f * __logf((float)D));
    la = l_attn[ro];
    wa = __expf(m - beta);
    wq = scale_p * __expf(-beta);
  }
  const float inv = 1.f / (la * wa + lq * wq);
  for (int e = lane; e < DH; e += 64) {
    float num = y(e) * wq;
    if (ya) num += (float)ya[e] * wa;
    out[ro * DH + e] = (T)(num * inv);
  }
}

// One workgroup of NTHR threads streams the feature rows [f_lo, f_hi) of one (batch, kv head).
// WHOLE: the workgroup owns every feature of its pair and merges the result itself; otherwise it writes the
// partial sums of its slice for decode_merge_kernel.
template <typename T, int DH, int MAXR, int NTHR, bool WHOLE>
__global__ __launch_bounds__(NTHR) void decode_step_kernel(DecodeArgs a) {
  typedef typename VecOf<T>::v8 v8;
  constexpr int LPR = DH / 8, FPP = NTHR / LPR;            // lanes per feature row, feature rows per pass
  constexpr int NW = NTHR / 64;                            // waves (each holds 64 / LPR feature rows per pass)
  constexpr int D = 128 * (DH / 16) * (DH / 16 + 1);
  __shared__ float qs[MAXR][DH];
  __shared__ float ks[DH];
  __shared__ float red[NW][DH + 1];
  __shared__ float tot[DH + 1];

  const int pair = blockIdx.x, sp = blockIdx.y;
  const int b = pair / a.h, hh = pair % a.h;
  const int rows = a.tq * a.r, hq = a.h * a.r;
  const int tid = threadIdx.x, sub = tid % LPR, fr = tid / LPR;
  const bool upd = a.Knew != nullptr;

  // gated, rounded query rows and the new key in LDS as floats
  const float qg = a.gq ? __expf(a.gq[b * a.h + hh] / (float)a.deg) : 1.f;
  for (int i = tid; i < rows * DH; i += NTHR) {
    const int row = i / DH, e = i % DH, t = row / a.r, rr = row % a.r;
    const float q = (float)((const T*)a.Q)[(((long)b * a.tq + t) * hq + hh * a.r + rr) * DH + e];
    qs[row][e] = (float)(T)(q * qg);
  }
  if (upd)
    for (int i = tid; i < DH; i += NTHR) ks[i] = (float)((const T*)a.Knew)[((long)b * a.h + hh) * DH + i];
  __syncthreads();

  const float dec = (upd && a.decay) ? __expf(a.decay[b * a.h + hh]) : 1.f;
  float vnew[8];
  if (upd) unpack8(*(const v8*)((const T*)a.Vnew + ((long)b * a.h + hh) * DH + 8 * sub), vnew);

  const int per = WHOLE ? D : (D + a.split - 1) / a.split;
  const int f_lo = WHOLE ? 0 : sp * per, f_hi = min(D, f_lo + per);
  const T* Sg = (const T*)a.S + (long)pair * D * DH;
  T* So = upd ? (T*)a.Sout + (long)pair * D * DH : nullptr;
  const float* sg = a.s + (long)pair * D;
  float* so = upd ? a.sout + (long)pair * D : nullptr;

  float acc[MAXR][8], lq[MAXR];
#pragma unroll
  for (int r_ = 0; r_ < MAXR; r_++) {
    lq[r_] = 0.f;
#pragma unroll
    for (int i = 0; i < 8; i++) acc[r_][i] = 0.f;
  }
  // four feature rows per lane in flight: the loop is bound by memory latency otherwise
  constexpr int UN = 4;
  for (int f0 = f_lo + fr; f0 < f_hi; f0 += UN * FPP) {
    v8 raw[UN];
    float sf[UN];
#pragma unroll
    for (int u = 0; u < UN; u++) {
      const int f = min(f0 + u * FPP, f_hi - 1);
      raw[u] = *(const v8*)(Sg + (long)f * DH + 8 * sub);
      sf[u] = sg[f];
    }
#pragma unroll
    for (int u = 0; u < UN; u++) {
      const int f = f0 + u * FPP;
      if (f >= f_hi) break;
      int x, w;
      float mult;
      feature_pair(f, x, w, mult);
      float sv[8];
      unpack8(raw[u], sv);
#pragma unroll
      for (int r_ = 0; r_ < MAXR; r_++) {
        if (r_ < rows) {
          const float ph = qs[r_][x] * qs[r_][w];
#pragma unroll
          for (int i = 0; i < 8; i++) acc[r_][i] = __builtin_fmaf(ph, sv[i], acc[r_][i]);
          lq[r_] = __builtin_fmaf(ph, sf[u], lq[r_]);
        }
      }
      if (upd) {
        const float pk = mult * ks[x] * ks[w];
        float o8[8];
#pragma unroll
        for (int i = 0; i < 8; i++) o8[i] = __builtin_fmaf(dec, sv[i], pk * vnew[i]);
        *(v8*)(So + (long)f * DH + 8 * sub) = pack8<T>(o8);
        if (sub == 0) so[f] = __builtin_fmaf(dec, sf[u], pk);
      }
    }
  }

  // Sum over the feature rows: first over the 64 / LPR rows a wave holds (lanes LPR apart), then over the waves through
  // LDS, one query row at a time.
  // (compile-time row index: a run-time index would put the accumulators in scratch memory for the whole kernel)
  const int wave = tid >> 6, lane = tid & 63;
  float* part = WHOLE ? nullptr : a.part + ((long)pair * a.split + sp) * rows * (DH + 1);
#pragma unroll
  for (int r_ = 0; r_ < MAXR; r_++) {
    if (r_ < rows) {
      float v[9];
#pragma unroll
      for (int i = 0; i < 8; i++) v[i] = acc[r_][i];
      v[8] = lq[r_];
#pragma unroll
      for (int off = LPR; off < 64; off <<= 1)
#pragma unroll
        for (int i = 0; i < 9; i++) v[i] += __shfl_xor(v[i], off);
      __syncthreads();   // red and tot of the previous row have been read
      if (lane < LPR) {
#pragma unroll
        for (int i = 0; i < 8; i++) red[wave][8 * lane + i] = v[i];
        if (lane == 0) red[wave][DH] = v[8];
      }
      __syncthreads();
      if (tid <= DH) {
        float t = 0.f;
#pragma unroll
        for (int k = 0; k < NW; k++) t += red[k][tid];
        if (WHOLE) tot[tid] = t;
        else part[r_ * (DH + 1) + tid] = t;
      }
      if (WHOLE) {
        __syncthreads();
        if (wave == 0) {
          const int t = r_ / a.r, rr = r_ % a.r;
          const long ro = ((long)b * a.tq + t) * hq + hh * a.r + rr;
          const bool an = a.attend_new != 0;
          decode_merge_row<T, DH>(lane, [&](int e) { return tot[e]; }, tot[DH], (const T*)a.Y_attn, a.l_attn,
                                  a.rowmax, an ? (const T*)a.Q : nullptr, an ? (const T*)a.Knew : nullptr,
                                  an ? (const T*)a.Vnew : nullptr, (T*)a.out, ro, pair, a.scale_p, (float)a.deg);
        }
      }
    }
  }
}

// Adds the partial sums of the feature slices of a (batch, kv head) and merges: one wave per query row.
template <typename T, int DH>
__global__ __launch_bounds__(64) void decode_merge_kernel(DecodeArgs a) {
  const int pair = blockIdx.x, row = blockIdx.y, rows = a.tq * a.r, hq = a.h * a.r;
  const int b = pair / a.h, hh = pair % a.h, t = row / a.r, rr = row % a.r;
  const long ro = ((long)b * a.tq + t) * hq + hh * a.r + rr;
  const int split = a.split;
  const float* p = a.part + (long)pair * split * rows * (DH + 1) + row * (DH + 1);
  float lq = 0.f;
  for (int k = 0; k < split; k++) lq += p[(long)k * rows * (DH + 1) + DH];
  const bool an = a.attend_new != 0;
  decode_merge_row<T, DH>(
      threadIdx.x,
      [&](int e) {
        float y = 0.f;
        for (int k = 0; k < split; k++) y += p[(long)k * rows * (DH + 1) + e];
        return y;
      },
      lq, (const T*)a.Y_attn, a.l_attn, a.rowmax, an ? (const T*)a.Q : nullptr, an ? (const T*)a.Knew : nullptr,
      an ? (const T*)a.Vnew : nullptr, (T*)a.out, ro, pair, a.scale_p, (float)a.deg);
}

int decode_split(int B, int h) {
  // about a thousand workgroups of 256 threads (four per compute unit, resident together); at most 16 slices per
  // (batch, kv head)
  const int pairs = B * h;
  const int split = (1024 + pairs - 1) / pairs;
  return split < 1 ? 1 : (split > 16 ? 16 : split);
}
long decode_workspace_floats(int B, int h, int r, int tq, int d) {
  return (long)B * h * decode_split(B, h) * tq * r * (d + 1);
}

// With at least one (batch, kv head) per compute unit and few query rows, one workgroup of 1024 threads takes a whole
// pair and merges in the same kernel (no partial sums, no second launch).
static bool decode_whole_pair(int B, int h, int rows) { return B * h >= 256 && rows <= 2; }

template <typename T, int DH>
static int decode_launch(const DecodeArgs& a0, int B, hipStream_t st) {
  DecodeArgs a = a0;
  const int rows = a.tq * a.r;
  // the accumulators of all query rows live in registers: a kernel per power of two keeps the common single-row
  // step small
  if (decode_whole_pair(B, a.h, rows)) {
    a.split = 1;
    const dim3 grid((unsigned)(B * a.h));
    if (rows <= 1) PR_LAUNCH("decode_step", (decode_step_kernel<T, DH, 1, 1024, true>), grid, dim3(1024), 0, st, a);
    else PR_LAUNCH("decode_step", (decode_step_kernel<T, DH, 2, 1024, true>), grid, dim3(1024), 0, st, a);
    return (int)hipGetLastError();
  }
  a.split = decode_split(B, a.h);
  const dim3 grid((unsigned)(B * a.h), (unsigned)a.split);
  if (rows <= 1) PR_LAUNCH("decode_step", (decode_step_kernel<T, DH, 1, 256, false>), grid, dim3(256), 0, st, a);
  else if (rows <= 2) PR_LAUNCH("decode_step", (decode_step_kernel<T, DH, 2, 256, false>), grid, dim3(256), 0, st, a);
  else if (rows <= 4) PR_LAUNCH("decode_step", (decode_step_kernel<T, DH, 4, 256, false>), grid, dim3(256), 0, st, a);
  else if (rows <= 8) PR_LAUNCH("decode_step", (decode_step_kernel<T, DH, 8, 256, false>), grid, dim3(256), 0, st, a);
  else PR_LAUNCH("decode_step", (decode_step_kernel<T, DH, DEC_MAXROWS, 256, false>), grid, dim3(256), 0, st, a);
  PR_LAUNCH("decode_merge", (decode_merge_kernel<T, DH>), dim3((unsigned)(B * a.h), (unsigned)rows), dim3(64), 0, st, a);
  return (int)hipGetLastError();
}

int decode_step(const void* Q, const float* gq, const void* S, const float* s, const void* Y_attn, const float* l_attn,
                const float* rowmax, const void* Knew, const void* Vnew, const float* decay, void* Sout, float* sout,
                void* out, float* workspace, int B, int tq, int h, int r, int d, int deg, float scale_p, int dtype,
                int attend_new, hipStream_t st) {
  if (tq * r > DEC_MAXROWS) return -3;
  DecodeArgs a{Q, gq, S, s, Knew, Vnew, decay, Sout, sout, workspace, h, r, tq, 1, deg,
               Y_attn, l_attn, rowmax, out, scale_p, attend_new};
#define PR_DEC(T)                                                                                                      \
  switch (d) {                                                                                                         \
    case 32: return decode_launch<T, 32>(a, B, st);                                                                    \
    case 64: return decode_launch<T, 64>(a, B, st);                                                                    \
    case 128: return decode_launch<T, 128>(a, B, st);                                                                  \
    default: return -2;                                                                                                \
  }
  if (dtype == DT_BF16) { PR_DEC(bf16_t) }
  if (dtype == DT_F16) { PR_DEC(f16_t) }
#undef PR_DEC
  return -1;
}

long decode_static_floats() { return DEC_STATIC_FLOATS; }

// The address of the library's per-GPU array on the current device, taken once per device with
// hipGetSymbolAddress (a runtime call that is not stream work: it must not happen for the first time while a stream
// is being captured, so decode_static_prepare() lets a caller do it ahead of time).  Returns 0 or a hipError_t.
namespace {
constexpr int MAX_DEVICES = 64;
std::mutex static_mu;
float* static_ptr[MAX_DEVICES] = {};   // the array's address on each GPU (each holds its own copy)
int static_array(int dev, float** out) {
  if (dev < 0 || dev >= MAX_DEVICES) return (int)hipErrorInvalidDevice;
  std::lock_guard<std::mutex> lock(static_mu);
  if (!static_ptr[dev]) {   // first use on this GPU, which is the current one
    float* p = nullptr;
    if (hipError_t e = hipGetSymbolAddress((void**)&p, HIP_SYMBOL(scratch))) return (int)e;
    if (!p) return (int)hipErrorInvalidSymbol;
    static_ptr[dev] = p;
  }
  *out = static_ptr[dev];
  return 0;
}
}  // namespace

int decode_static_prepare() {
  int dev = -1;
  if (hipError_t e = hipGetDevice(&dev)) return (int)e;
  float* p;
  return static_array(dev, &p);
}

// decode_step with the partial sums in the library's own per-GPU array instead of a caller's workspace: nothing is
// allocated here or below.  Every slice of every (batch, kv head) writes all of its partial sums before the merge
// kernel reads them, so nothing has to be cleared between calls; two calls in flight on one GPU at the same time
// would share the array and race.  The array used is that of the GPU the stream belongs to, which must be the
// current one (-7 otherwise: each GPU has its own copy, and the kernels run where the stream lives).  Returns -6 when
// the step needs more than the array holds, or a positive hipError_t if the array's address cannot be obtained.
int decode_step_static(const void* Q, const float* gq, const void* S, const float* s, const void* Y_attn,
                       const float* l_attn, const float* rowmax, const void* Knew, const void* Vnew,
                       const float* decay, void* Sout, float* sout, void* out, int B, int tq, int h, int r, int d,
                       int deg, float scale_p, int dtype, int attend_new, hipStream_t st) {
  if (decode_workspace_floats(B, h, r, tq, d) > DEC_STATIC_FLOATS) return -6;
  int dev = -1;
  if (hipError_t e = hipGetDevice(&dev)) return (int)e;
  if (st != nullptr) {   // (the null stream is the current device's by definition)
    hipDevice_t sdev = -1;
    if (hipError_t e = hipStreamGetDevice(st, &sdev)) return (int)e;
    if ((int)sdev != dev) return -7;
  }
  float* part;
  if (int rc = static_array(dev, &part)) return rc;
  return decode_step(Q, gq, S, s, Y_attn, l_attn, rowmax, Knew, Vnew, decay, Sout, sout, out, part, B, tq, h, r, d, deg,
                     scale_p, dtype, attend_new, st);
}

}  // namespace pr
