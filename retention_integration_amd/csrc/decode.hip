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
// in registers and writes the updated rows.  A second, tiny kernel adds the partials of the slices and merges.
#include "common.h"
#include "kernels.h"

namespace pr {

constexpr int DEC_MAXROWS = 8;   // query rows (positions x query heads per kv head) handled per (batch, kv head)


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
  float* part;          // [B*h, split, rows, d + 1] partial query sums
  int h, r, tq, split, deg;
};

template <typename T, int DH>
__global__ __launch_bounds__(256) void decode_step_kernel(DecodeArgs a) {
  typedef typename VecOf<T>::v8 v8;
  constexpr int LPR = DH / 8, FPP = 256 / LPR;            // lanes per feature row, feature rows per pass
  constexpr int D = 128 * (DH / 16) * (DH / 16 + 1);
  __shared__ float qs[DEC_MAXROWS][DH];
  __shared__ float ks[DH];
  __shared__ float red[FPP][DH + 1];

  const int pair = blockIdx.x, sp = blockIdx.y;
  const int b = pair / a.h, hh = pair % a.h;
  const int rows = a.tq * a.r, hq = a.h * a.r;
  const int tid = threadIdx.x, sub = tid % LPR, fr = tid / LPR;
  const bool upd = a.Knew != nullptr;

  // gated, rounded query rows and the new key in LDS as floats
  const float qg = a.gq ? __expf(a.gq[b * a.h + hh] / (float)a.deg) : 1.f;
  for (int i = tid; i < rows * DH; i += 256) {
    const int row = i / DH, e = i % DH, t = row / a.r, rr = row % a.r;
    const float q = (float)((const T*)a.Q)[(((long)b * a.tq + t) * hq + hh * a.r + rr) * DH + e];
    qs[row][e] = (float)(T)(q * qg);
  }
  if (upd)
    for (int i = tid; i < DH; i += 256) ks[i] = (float)((const T*)a.Knew)[((long)b * a.h + hh) * DH + i];
  __syncthreads();

  const float dec = (upd && a.decay) ? __expf(a.decay[b * a.h + hh]) : 1.f;
  float vnew[8];
  if (upd) unpack8(*(const v8*)((const T*)a.Vnew + ((long)b * a.h + hh) * DH + 8 * sub), vnew);

  const int per = (D + a.split - 1) / a.split;
  const int f_lo = sp * per, f_hi = min(D, f_lo + per);
  const T* Sg = (const T*)a.S + (long)pair * D * DH;
  T* So = upd ? (T*)a.Sout + (long)pair * D * DH : nullptr;
  const float* sg = a.s + (long)pair * D;
  float* so = upd ? a.sout + (long)pair * D : nullptr;

  float acc[DEC_MAXROWS][8], lq[DEC_MAXROWS];
#pragma unroll
  for (int r_ = 0; r_ < DEC_MAXROWS; r_++) {
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
      for (int r_ = 0; r_ < DEC_MAXROWS; r_++) {
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

  // reduce over the FPP feature-row groups of the workgroup, one query row at a time
  float* part = a.part + ((long)pair * a.split + sp) * rows * (DH + 1);
  // (compile-time row index: a run-time index would put the accumulators in scratch memory for the whole kernel)
#pragma unroll
  for (int r_ = 0; r_ < DEC_MAXROWS; r_++) {
    if (r_ < rows) {
      __syncthreads();
#pragma unroll
      for (int i = 0; i < 8; i++) red[fr][8 * sub + i] = acc[r_][i];
      if (sub == 0) red[fr][DH] = lq[r_];
      __syncthreads();
      if (tid <= DH) {
        float t = 0.f;
        for (int k = 0; k < FPP; k++) t += red[k][tid];
        part[r_ * (DH + 1) + tid] = t;
      }
    }
  }
}

// out[row, e] = (Y_attn * wa + y * wq) / (l_attn * wa + lq * wq), the merge of the chunked kernel
// (sympow_nn.hip); without an attention part out = y / lq.
// With Qn/Kn/Vn the attention part is that of the ONE new token attending to itself (tq = 1): one weight
// (scale q.k)^deg, so Y_attn = v, l_attn = 1 + 1e-6 and rowmax = log of the weight
// (ref: retention/_attention/reference.py:42-69 with a single key).
template <typename T, int DH>
__global__ __launch_bounds__(64) void decode_merge_kernel(const float* __restrict__ part, const T* __restrict__ Y_attn,
                                                          const float* __restrict__ l_attn,
                                                          const float* __restrict__ rowmax, const T* __restrict__ Qn,
                                                          const T* __restrict__ Kn, const T* __restrict__ Vn,
                                                          T* __restrict__ out, int h, int r, int tq, int split,
                                                          float scale_p, float deg) {
  constexpr int D = 128 * (DH / 16) * (DH / 16 + 1);
  const int pair = blockIdx.x, row = blockIdx.y, rows = tq * r, hq = h * r;
  const int b = pair / h, hh = pair % h, t = row / r, rr = row % r;
  const long ro = ((long)b * tq + t) * hq + hh * r + rr;
  const float* p = part + (long)pair * split * rows * (DH + 1) + row * (DH + 1);
  float lq = 0.f;
  for (int k = 0; k < split; k++) lq += p[(long)k * rows * (DH + 1) + DH];
  float wa = 0.f, wq = 1.f, la = 0.f;
  const T* ya = Y_attn ? Y_attn + ro * DH : nullptr;
  if (Kn) {
    float dot = 0.f;
    for (int e = threadIdx.x; e < DH; e += 64) dot += (float)Qn[ro * DH + e] * (float)Kn[(long)pair * DH + e];
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
  for (int e = threadIdx.x; e < DH; e += 64) {
    float y = 0.f;
    for (int k = 0; k < split; k++) y += p[(long)k * rows * (DH + 1) + e];
    float num = y * wq;
    if (ya) num += (float)ya[e] * wa;
    out[ro * DH + e] = (T)(num * inv);
  }
}

int decode_split(int B, int h) {
  // enough workgroups to fill the chip a few times over, at most 16 slices per (batch, kv head)
  const int pairs = B * h;
  int split = (2048 + pairs - 1) / pairs;
  return split < 1 ? 1 : (split > 16 ? 16 : split);
}
long decode_workspace_floats(int B, int h, int r, int tq, int d) {
  return (long)B * h * decode_split(B, h) * tq * r * (d + 1);
}

template <typename T, int DH>
static int decode_launch(const DecodeArgs& a0, const void* Y_attn, const float* l_attn, const float* rowmax, void* out,
                         int B, float scale_p, int attend_new, hipStream_t st) {
  DecodeArgs a = a0;
  a.split = decode_split(B, a.h);
  hipLaunchKernelGGL((decode_step_kernel<T, DH>), dim3((unsigned)(B * a.h), (unsigned)a.split), dim3(256), 0, st, a);
  hipLaunchKernelGGL((decode_merge_kernel<T, DH>), dim3((unsigned)(B * a.h), (unsigned)(a.tq * a.r)), dim3(64), 0, st,
                     a.part, (const T*)Y_attn, l_attn, rowmax, attend_new ? (const T*)a.Q : nullptr,
                     attend_new ? (const T*)a.Knew : nullptr, attend_new ? (const T*)a.Vnew : nullptr, (T*)out, a.h,
                     a.r, a.tq, a.split, scale_p, (float)a.deg);
  return (int)hipGetLastError();
}

int decode_step(const void* Q, const float* gq, const void* S, const float* s, const void* Y_attn, const float* l_attn,
                const float* rowmax, const void* Knew, const void* Vnew, const float* decay, void* Sout, float* sout,
                void* out, float* workspace, int B, int tq, int h, int r, int d, int deg, float scale_p, int dtype,
                int attend_new, hipStream_t st) {
  if (tq * r > DEC_MAXROWS) return -3;
  DecodeArgs a{Q, gq, S, s, Knew, Vnew, decay, Sout, sout, workspace, h, r, tq, 1, deg};
#define PR_DEC(T)                                                                                                      \
  switch (d) {                                                                                                         \
    case 32: return decode_launch<T, 32>(a, Y_attn, l_attn, rowmax, out, B, scale_p, attend_new, st);                              \
    case 64: return decode_launch<T, 64>(a, Y_attn, l_attn, rowmax, out, B, scale_p, attend_new, st);                              \
    case 128: return decode_launch<T, 128>(a, Y_attn, l_attn, rowmax, out, B, scale_p, attend_new, st);                            \
    default: return -2;                                                                                                \
  }
  if (dtype == DT_BF16) { PR_DEC(bf16_t) }
  if (dtype == DT_F16) { PR_DEC(f16_t) }
#undef PR_DEC
  return -1;
}

}  // namespace pr
