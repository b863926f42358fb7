// Causal power attention, forward (ref: retention/_attention/reference.py:10-69).
//
//   s = scale * q.k,  z = deg*log(|s| + 1e-7) + G_q - G_k  (masked to keys j <= i + tk - tq),
//   m = max_j z,  P = exp(z - m),  l = sum_j P + 1e-6,  o = P V
//   norm: returns o / l;  otherwise (o, l, m).
//
// Query rows of the r query heads that share a kv head are folded into one row axis of length tq*r.
// A workgroup = 4 waves owns 64*MT folded rows of one (batch, kv head); keys stream through LDS 64 at
// a time.  All products are formed transposed (S^T = K Q^T, O^T = V^T P^T) so that the accumulator
// layout of S^T is directly the operand layout of the second contraction and no data moves between
// lanes; row statistics live one row per lane column.
//
// The weights are evaluated without logarithms: w = exp(z) = (|s| + 1e-7)^deg * exp(G_q - G_k) is
// accumulated unnormalised (w <= (|s|+eps)^deg because gates only decay), its running maximum is
// tracked, and the row is divided by max_j w at the end, which gives exactly exp(z - m) sums.  For
// key tiles entirely in a row's past the gate factor is split as exp(G_q - R) * exp(R - G_k) with R
// the gate at the tile's last key, so the exponentials are per row and per key, not per pair; only
// the tiles that touch the diagonal evaluate exp(G_q - G_k) per pair.
#include "common.h"
#include "kernels.h"

namespace pr {

constexpr int AT_BN = 64;
constexpr float AT_LOG_EPS = 1e-7f, AT_SUM_EPS = 1e-6f, AT_EXP_CLAMP = 80.f;

template <bool DEG2> __device__ __forceinline__ float pow_even(float a, int half_deg) {  // a^(2*half_deg)
  const float a2 = a * a;
  float p = a2;
  if (!DEG2)
    for (int k = 1; k < half_deg; k++) p *= a2;
  return p;
}

template <typename T, int DH, int MT, bool DEG2>
__global__ __launch_bounds__(256) void attention_fwd_kernel(AttnFwdArgs a) {
  typedef typename VecOf<T>::v8 v8;
  typedef typename VecOf<T>::v4 v4;
  constexpr int LD = DH + 8, KS = DH / 32, NT = DH / 16, KT = AT_BN / 16, ROWS = 64 * MT;
  constexpr int CH = AT_BN * DH / 8, PT = (CH + 255) / 256;
  extern __shared__ __attribute__((aligned(16))) char smem[];
  T* Kt = (T*)smem;                           // [2][BN][LD]
  T* Vt = Kt + 2 * AT_BN * LD;                // [2][BN][LD]
  constexpr int GS = 2 * AT_BN + 4;
  float* gk = (float*)(Vt + 2 * AT_BN * LD);  // [2][GS]: raw gate [BN], exp(R - gate) [BN], R

  const int tid = threadIdx.x, l = tid & 63, g = l >> 4, wave = tid >> 6, tcol = l & 15;
  const int b = blockIdx.y / a.h, hh = blockIdx.y % a.h;
  const int hq = a.h * a.r, rows = a.tq * a.r, shift = a.tk - a.tq;
  const int row0 = blockIdx.x * ROWS;
  const T* Qg = (const T*)a.Q + (long)b * a.tq * hq * DH;
  const T* Kg = (const T*)a.K + (long)b * a.tk * a.h * DH + hh * DH;
  const T* Vg = (const T*)a.V + (long)b * a.tk * a.h * DH + hh * DH;
  const float* Gg = a.G ? a.G + (long)b * a.tk * a.h + hh : nullptr;
  const long kstride = (long)a.h * DH;
  const int half_deg = (int)a.deg / 2;
  const float eps_s = AT_LOG_EPS / a.scale;          // |scale*x| + eps = scale * (|x| + eps/scale)
  const float scale_p = __powf(a.scale, a.deg);

  v8 Qf[MT][KS];
  int ti[MT];
  long qoff[MT];
  bool live[MT];
  float Gq[MT], mx[MT], lsum[MT];
#pragma unroll
  for (int mi = 0; mi < MT; mi++) {
    const int row = row0 + wave * 16 * MT + 16 * mi + tcol;
    live[mi] = row < rows;
    const int rr = live[mi] ? row : 0;
    const int t = rr / a.r;
    ti[mi] = t + shift;
    qoff[mi] = (long)t * hq + hh * a.r + (rr - t * a.r);
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      u32x4 z = {0, 0, 0, 0};
      if (live[mi]) z = *(const u32x4*)(Qg + qoff[mi] * DH + 32 * ks + 8 * g);
      Qf[mi][ks] = __builtin_bit_cast(v8, z);
    }
    Gq[mi] = Gg ? Gg[(long)ti[mi] * a.h] : 0.f;
    mx[mi] = 0.f;
    lsum[mi] = 0.f;
  }
  f32x4 acc[MT][NT];
#pragma unroll
  for (int mi = 0; mi < MT; mi++)
#pragma unroll
    for (int nt = 0; nt < NT; nt++) acc[mi][nt] = (f32x4){0, 0, 0, 0};

  const int last_row = min(row0 + ROWS, rows) - 1;
  const int kmax = min(a.tk, last_row / a.r + shift + 1);   // keys any row of the workgroup can see
  const int first_ti = row0 / a.r + shift;                   // smallest time index in the workgroup
  const int ntiles = (kmax + AT_BN - 1) / AT_BN;

  u32x4 rk[PT], rv[PT];
  float rg = 0.f, rR = 0.f;
  auto fetch = [&](int j0) {
#pragma unroll
    for (int i = 0; i < PT; i++) {
      const int ch = tid + 256 * i;
      const int key = j0 + ch / (DH / 8), col = (ch % (DH / 8)) * 8;
      rk[i] = (u32x4){0, 0, 0, 0};
      rv[i] = (u32x4){0, 0, 0, 0};
      if (ch < CH && key < a.tk) {
        rk[i] = *(const u32x4*)(Kg + key * kstride + col);
        rv[i] = *(const u32x4*)(Vg + key * kstride + col);
      }
    }
    if (tid < AT_BN && Gg) {
      rg = Gg[(long)min(j0 + tid, a.tk - 1) * a.h];
      rR = Gg[(long)min(j0 + AT_BN - 1, a.tk - 1) * a.h];
    }
  };
  auto stash = [&](int stage) {
#pragma unroll
    for (int i = 0; i < PT; i++) {
      const int ch = tid + 256 * i;
      if (ch < CH) {
        const int o = stage * AT_BN * LD + (ch / (DH / 8)) * LD + (ch % (DH / 8)) * 8;
        *(u32x4*)(Kt + o) = rk[i];
        *(u32x4*)(Vt + o) = rv[i];
      }
    }
    if (tid < AT_BN) {
      gk[stage * GS + tid] = rg;
      gk[stage * GS + AT_BN + tid] = __expf(fminf(rR - rg, AT_EXP_CLAMP));
      if (tid == 0) gk[stage * GS + 2 * AT_BN] = rR;
    }
  };

  fetch(0);
  for (int it = 0; it < ntiles; it++) {
    const int j0 = it * AT_BN, stage = it & 1;
    stash(stage);
    __syncthreads();
    if (it + 1 < ntiles) fetch(j0 + AT_BN);
    const T* kt_ = Kt + stage * AT_BN * LD;
    const T* vt_ = Vt + stage * AT_BN * LD;
    const float* gk_ = gk + stage * GS;
    const bool diag = (j0 + AT_BN - 1 > first_ti) || (j0 + AT_BN > a.tk);   // some pair of the tile is masked
    const float R = gk_[2 * AT_BN];

    v8 kf[KT][KS];
#pragma unroll
    for (int kt = 0; kt < KT; kt++)
#pragma unroll
      for (int ks = 0; ks < KS; ks++) kf[kt][ks] = lds_frag<T>(kt_, LD, 16 * kt, 32 * ks);
    f32x4 gkv[KT];
#pragma unroll
    for (int kt = 0; kt < KT; kt++) gkv[kt] = *(const f32x4*)(gk_ + (diag ? 0 : AT_BN) + 16 * kt + 4 * g);

    v8 pf[MT][KT / 2];
#pragma unroll
    for (int mi = 0; mi < MT; mi++) {
      const float eu = scale_p * (diag ? 1.f : __expf(fminf(Gq[mi] - R, AT_EXP_CLAMP)));
      float p[KT][4];
#pragma unroll
      for (int kt = 0; kt < KT; kt++) {
        f32x4 s = {0, 0, 0, 0};
#pragma unroll
        for (int ks = 0; ks < KS; ks++) s = mfma16(kf[kt][ks], Qf[mi][ks], s);
#pragma unroll
        for (int v = 0; v < 4; v++) {
          const float pw = pow_even<DEG2>(fabsf(s[v]) + eps_s, half_deg);
          float w;
          if (diag) {
            const int key = j0 + 16 * kt + 4 * g + v;
            w = pw * eu * __expf(fminf(Gq[mi] - gkv[kt][v], AT_EXP_CLAMP));
            if (key > ti[mi] || key >= a.tk) w = 0.f;
          } else {
            w = pw * gkv[kt][v] * eu;
          }
          p[kt][v] = w;
          mx[mi] = fmaxf(mx[mi], w);
        }
      }
      // the row sum is taken over the weights as the matrix cores will see them (rounded to 16 bit), so that
      // o / l is an exact average (ref rounds p before summing: retention/_attention/reference.py:52-55)
#pragma unroll
      for (int kp = 0; kp < KT / 2; kp++) {
        float q8[8];
#pragma unroll
        for (int v = 0; v < 4; v++) {
          q8[v] = p[2 * kp][v];
          q8[4 + v] = p[2 * kp + 1][v];
        }
        pf[mi][kp] = pack8<T>(q8);
        unpack8(pf[mi][kp], q8);
#pragma unroll
        for (int v = 0; v < 8; v++) lsum[mi] += q8[v];
      }
    }
    // O^T += V^T P^T, 32 keys per step: elements 0-3 are keys 4g.. of the first 16, 4-7 of the second 16
#pragma unroll
    for (int kp = 0; kp < KT / 2; kp++) {
#pragma unroll
      for (int nt = 0; nt < NT; nt++) {
        v4 lo = lds_frag_tr4<T>(vt_, LD, 32 * kp + 4 * g, 16 * nt);
        v4 hi = lds_frag_tr4<T>(vt_, LD, 32 * kp + 16 + 4 * g, 16 * nt);
        v8 vf = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
#pragma unroll
        for (int mi = 0; mi < MT; mi++) acc[mi][nt] = mfma16(vf, pf[mi][kp], acc[mi][nt]);
      }
    }
  }

  T* Og = (T*)a.O + (long)b * a.tq * hq * DH;
#pragma unroll
  for (int mi = 0; mi < MT; mi++) {
    const float wmax = max_over_rows(mx[mi]);          // = exp(rowmax)
    const float wsum = sum_over_rows(lsum[mi]);
    if (!live[mi]) continue;
    const float inv = 1.f / wmax;
    const float lrow = wsum * inv + AT_SUM_EPS;
    const float f = a.norm ? inv / lrow : inv;
#pragma unroll
    for (int nt = 0; nt < NT; nt++) {
      float o4[4];
#pragma unroll
      for (int v = 0; v < 4; v++) o4[v] = acc[mi][nt][v] * f;
      *(v4*)(Og + qoff[mi] * DH + 16 * nt + 4 * g) = pack4<T>(o4);
    }
    if (g == 0) {
      const long o = (long)b * a.tq * hq + qoff[mi];
      if (a.l) a.l[o] = lrow;
      if (a.rowmax) a.rowmax[o] = __logf(wmax);
    }
  }
}

template <typename T, int DH> static int attn_fwd_launch(const AttnFwdArgs& a, int B, hipStream_t st) {
  constexpr int MT = DH <= 64 ? 2 : 1;
  constexpr size_t smem = 2 * 2 * AT_BN * (DH + 8) * sizeof(T) + 2 * (2 * AT_BN + 4) * sizeof(float);
  const int rows = a.tq * a.r;
  dim3 grid((rows + 64 * MT - 1) / (64 * MT), (unsigned)(B * a.h));
  if (a.deg == 2.f) {
    auto kern = attention_fwd_kernel<T, DH, MT, true>;
    allow_big_lds((const void*)kern, smem);
    hipLaunchKernelGGL(kern, grid, dim3(256), smem, st, a);
  } else {
    auto kern = attention_fwd_kernel<T, DH, MT, false>;
    allow_big_lds((const void*)kern, smem);
    hipLaunchKernelGGL(kern, grid, dim3(256), smem, st, a);
  }
  return (int)hipGetLastError();
}

int attention_fwd(const AttnFwdArgs& a, int B, int d, int dtype, hipStream_t st) {
#define PR_AF(T)                                                                                                       \
  switch (d) {                                                                                                         \
    case 32: return attn_fwd_launch<T, 32>(a, B, st);                                                                  \
    case 64: return attn_fwd_launch<T, 64>(a, B, st);                                                                  \
    case 128: return attn_fwd_launch<T, 128>(a, B, st);                                                                \
    default: return -2;                                                                                                \
  }
  if (dtype == DT_BF16) { PR_AF(bf16_t) }
  if (dtype == DT_F16) { PR_AF(f16_t) }
#undef PR_AF
  return -1;
}

}  // namespace pr
