// Row-wise preparation for the query_state backward (formulas: retention/_query_state/triton.py:546-553):
//   delta = sum_e O*dO,  beta = max(rowmax, log sqrt(D)),  f = 1/den,
//   w_attn = exp(rowmax - beta),  w_qs = scale^p * exp(-beta)       (w_attn = 0, w_qs = 1 without attention part)
//   dOs = w_qs f dO,  cvec = -w_qs f delta,  dY_attn = w_attn f dO,  dl_attn = -w_attn f delta.
#include "common.h"
#include "kernels.h"

namespace pr {

template <typename T, int DH>
__global__ __launch_bounds__(256) void qs_bwd_prep_kernel(const T* __restrict__ O, const T* __restrict__ dO,
                                                          const float* __restrict__ den,
                                                          const float* __restrict__ rowmax,
                                                          const float* __restrict__ qgate, T* __restrict__ dOs,
                                                          float* __restrict__ cvec, T* __restrict__ dYa,
                                                          float* __restrict__ dla, float* __restrict__ dYscale,
                                                          long rows, int h, int rr, float scale_p,
                                                          const int* __restrict__ live_rows, int c) {
  typedef typename VecOf<T>::v8 v8;
  constexpr int LPR = DH / 8;  // lanes per row
  // Two rows per thread, half the rows apart, with the loads of both in flight before anything is computed; the row
  // arithmetic in 32 bits (the host refuses 2^31 rows or more).
  constexpr int RPT = 2;
  const unsigned nrows = (unsigned)rows, half = (nrows + RPT - 1) / RPT;
  const unsigned gid = blockIdx.x * 256u + threadIdx.x;
  const unsigned row0 = gid / LPR;
  const int col = (int)(gid % LPR) * 8;
  const unsigned hr = (unsigned)h * (unsigned)rr;
  bool live[RPT];
  unsigned r[RPT];
  v8 ov[RPT], gv[RPT];
  float dn[RPT], mv[RPT], qg[RPT];
  int lv[RPT];
#pragma unroll
  for (int j = 0; j < RPT; j++) {
    const unsigned row = row0 + j * half;
    live[j] = row0 < half && row < nrows;
    r[j] = live[j] ? row : 0u;
    ov[j] = *(const v8*)(O + (long)r[j] * DH + col);
    gv[j] = *(const v8*)(dO + (long)r[j] * DH + col);
    dn[j] = den[r[j]];
    mv[j] = rowmax ? rowmax[r[j]] : 0.f;
    // the forward's log factor on the state part of this row: rows are (.., position, kv head, query head of it)
    const unsigned pos = r[j] / hr, hh = (r[j] - pos * hr) / (unsigned)rr;
    qg[j] = qgate ? qgate[(long)pos * h + hh] : 0.f;
    // (live_rows: per (chunk, kv head) the end of the positions whose state part is not an exact zero)
    lv[j] = live_rows ? live_rows[((long)(pos / (unsigned)c) * h + hh) * 2 + 1] : 0;
  }
#pragma unroll
  for (int j = 0; j < RPT; j++) {
    float o[8], g[8];
    unpack8(ov[j], o);
    unpack8(gv[j], g);
    float delta = 0.f;
#pragma unroll
    for (int i = 0; i < 8; i++) delta += o[i] * g[i];
#pragma unroll
    for (int m = 1; m < LPR; m <<= 1) delta += __shfl_xor(delta, m);
    const float f = 1.f / dn[j];
    float wa = 0.f, wq = 1.f;
    if (rowmax) {
      constexpr int D = 128 * (DH / 16) * (DH / 16 + 1);
      const float m = mv[j], beta = fmaxf(m, 0.5f * __logf((float)D));
      wa = __expf(m - beta);
      wq = scale_p * __expf(qg[j] - beta);
    }
    if (!live[j]) continue;
    // Row factors of the two parts.  They are ~1e-3..1 unless the row's total weight is ~0 (a zero query: 1/den is
    // then ~1e14 and multiplies a feature vector that is exactly zero).  fp16 cannot hold dO times such a factor, so
    // there it is capped far above any regular value; the products with the zero features stay zero instead of NaN.
    float cq = wq * f, ca = wa * f;
    if (!__is_same(T, bf16_t)) {
      cq = fminf(cq, 4096.f);
      ca = fminf(ca, 4096.f);
    }
    float a[8], b[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
      a[i] = g[i] * cq;
      b[i] = g[i] * ca;
    }
    // (the reader of dOs walks the chunk's rows in stages of at most 256 positions and stops after the one that holds
    // the last position whose state part counts, so the rows of the stages after it are not written)
    bool wanted = true;
    if (live_rows) {
      const unsigned pos = r[j] / hr;
      wanted = (int)(pos % (unsigned)c) < ((lv[j] + 255) & ~255);
    }
    const long ro = (long)r[j] * DH + col;
    if (wanted) *(v8*)(dOs + ro) = pack8<T>(a);
    if (dYa) *(v8*)(dYa + ro) = pack8<T>(b);
    if (col == 0) {
      cvec[r[j]] = -cq * delta;
      if (dla) dla[r[j]] = -ca * delta;
      // dY_attn = dO * dYscale[row], for consumers that scale on the fly.  The factor is <= 1/l_attn, i.e. <= ~1
      // unless every weight of the row underflowed (a zero query, e.g. a padded row, in fp16: l_attn = 1e-6); it is
      // capped so that weight * factor stays inside the fp16 range there too.
      if (dYscale) dYscale[r[j]] = fminf(ca, 3.0e4f);
    }
  }
}

template <typename T>
static int prep_launch(const void* O, const void* dO, const float* den, const float* rowmax, const float* qgate, void* dOs,
                       float* cvec, void* dYa, float* dla, float* dYscale, long rows, int h, int r, int d, float scale_p,
                       const int* live, int c, hipStream_t st) {
  if (rows >= (1L << 31)) return -4;
  const long threads = ((rows + 1) / 2) * (d / 8);   // two rows per thread
  dim3 grid((unsigned)((threads + 255) / 256));
#define PR_PREP(DD)                                                                                                    \
  case DD:                                                                                                             \
    PR_LAUNCH("qs_bwd_prep", (qs_bwd_prep_kernel<T, DD>), grid, dim3(256), 0, st, (const T*)O, (const T*)dO, den, rowmax,    \
                       qgate, (T*)dOs, cvec, (T*)dYa, dla, dYscale, rows, h, r, scale_p, live, c);                     \
    break;
  switch (d) { PR_PREP(32) PR_PREP(64) PR_PREP(128) default: return -2; }
#undef PR_PREP
  return (int)hipGetLastError();
}

int qs_bwd_prep(const void* O, const void* dO, const float* den, const float* rowmax, const float* qgate, void* dOs,
                float* cvec, void* dY_attn, float* dl_attn, float* dY_scale, long rows, int h, int r, int d, float scale_p,
                const int* live_rows, int c, int dtype, hipStream_t st) {
  if (qgate && !rowmax) return -3;   // the gate enters through the merge weights
  if (live_rows && (!qgate || c <= 0)) return -3;   // live_rows describes the gate factor of the state part
  if (!g_gate_skip) live_rows = nullptr;
  if (dtype == DT_BF16)
    return prep_launch<bf16_t>(O, dO, den, rowmax, qgate, dOs, cvec, dY_attn, dl_attn, dY_scale, rows, h, r, d, scale_p, live_rows, c, st);
  if (dtype == DT_F16)
    return prep_launch<f16_t>(O, dO, den, rowmax, qgate, dOs, cvec, dY_attn, dl_attn, dY_scale, rows, h, r, d, scale_p, live_rows, c, st);
  return -1;
}

}  // namespace pr
