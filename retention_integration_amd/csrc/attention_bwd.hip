// Causal power attention, backward (formulas: autograd of retention/_attention/reference.py:42-69;
// cross-check retention/_attention/triton.py:248-387).  Inputs are the forward's operands, its row
// maximum m, and the gradients dO (of the unnormalised o) and dl (of the row sum l):
//
//   P = exp(z - m),  dP = dO V^T + dl,  dz = P * dP,  dV = P^T dO,
//   dGq_i = sum_j dz_ij,  dGk_j = -sum_i dz_ij,
//   d(q.k) = dz * deg * sign(s) / (|q.k| + 1e-7/scale),  dQ = d(q.k) K,  dK = d(q.k)^T Q.
//
// Two kernels, each recomputing P: one owns query rows and walks the keys (dQ, dGq), the other owns keys
// and walks the query rows (dK, dV, dGk).  Products are oriented so that every accumulator layout is
// already the operand layout of the next contraction (see attention_fwd.hip).
//
// No logarithm or division per pair: with a = |q.k| + eps/scale,
//   P = a^deg * E,  E = scale^deg * exp(G_q - m - G_k),  d(q.k)/deg = sign(s) * a^(deg-1) * E * dP,
// and away from the diagonal E factors into a per-row and a per-key exponential around a reference
// gate R (the gate at the last key of the key tile, so both exponents are <= 0 for decaying gates).
#include "common.h"
#include "kernels.h"

namespace pr {

constexpr int AB_BN = 64;   // keys per step in the dQ kernel
constexpr int AB_BM = 32;   // query rows per step in the dK/dV kernel
constexpr float AB_LOG_EPS = 1e-7f, AB_EXP_CLAMP = 80.f;

// a^(deg-2) for even deg
template <bool DEG2> __device__ __forceinline__ float pow_m2(float a, int half_deg) {
  if (DEG2) return 1.f;
  const float a2 = a * a;
  float p = 1.f;
  for (int k = 1; k < half_deg; k++) p *= a2;
  return p;
}

// One pair: s = raw q.k, E as above, dpl = dP (incl. dl).  Returns P, dz and d(q.k)/deg.
template <bool DEG2>
__device__ __forceinline__ void pair_grad(float s, float E, float dpl, float eps_s, int half_deg, float& p, float& dz,
                                          float& dsr) {
  const float as = fabsf(s) + eps_s;
  const float t1 = pow_m2<DEG2>(as, half_deg) * as * E;   // a^(deg-1) E
  p = t1 * as;
  dz = p * dpl;
  dsr = copysignf(t1, s) * dpl;
}

// ------------------------------------------------------------------ dQ, dGq
template <typename T, int DH, int MT, bool DEG2>
__global__ __launch_bounds__(256, 2) void attention_bwd_dq_kernel(AttnBwdArgs a, int nblocks, int npairs) {
  typedef typename VecOf<T>::v8 v8;
  typedef typename VecOf<T>::v4 v4;
  constexpr int LD = DH + 8, KS = DH / 32, NT = DH / 16, KT = AB_BN / 16, ROWS = 64 * MT;
  constexpr int CH = AB_BN * DH / 8, PT = (CH + 255) / 256;
  constexpr int GS = 2 * AB_BN + 4;
  extern __shared__ __attribute__((aligned(16))) char smem[];
  T* Kt = (T*)smem;
  T* Vt = Kt + 2 * AB_BN * LD;
  float* gk = (float*)(Vt + 2 * AB_BN * LD);   // [2][GS]: raw gate [BN], exp(R - gate) [BN], R

  // Workgroups are dealt round-robin by their linear index to the 8 XCDs and then to the 4 shader engines of an
  // XCD; only the CU inside a shader engine is chosen by load.  Blocks differ in length (causal), so each of the 32
  // (XCD, shader engine) groups gets whole (batch, kv head) pairs, the longest blocks of all its pairs first.
  const int grp = blockIdx.x % 32, u = blockIdx.x / 32, ppg = (npairs + 31) / 32;
  const int pair = (u % ppg) * 32 + grp;
  if (pair >= npairs) return;
  const int tid = threadIdx.x, l = tid & 63, g = l >> 4, wave = tid >> 6, tcol = l & 15;
  const int b = pair / a.h, hh = pair % a.h;
  const int hq = a.h * a.r, rows = a.tq * a.r, shift = a.tk - a.tq;
  const int row0 = (nblocks - 1 - u / ppg) * ROWS;   // late rows see the most keys
  const T* Qg = (const T*)a.Q + (long)b * a.tq * hq * DH;
  const T* dOg = (const T*)a.dO + (long)b * a.tq * hq * DH;
  const T* Kg = (const T*)a.K + (long)b * a.tk * a.h * DH + hh * DH;
  const T* Vg = (const T*)a.V + (long)b * a.tk * a.h * DH + hh * DH;
  const float* Gg = a.G ? a.G + (long)b * a.tk * a.h + hh : nullptr;
  const long kstride = (long)a.h * DH;
  const int half_deg = (int)a.deg / 2;
  const float eps_s = AB_LOG_EPS / a.scale;
  const float scale_p = __expf(a.deg * __logf(a.scale));

  v8 Qf[MT][KS], dOf[MT][KS];
  int ti[MT];
  long qoff[MT];
  bool live[MT];
  float base[MT], dlr[MT], dgq[MT], osc[MT];   // base = G_q - m
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
      u32x4 z = {0, 0, 0, 0}, z2 = {0, 0, 0, 0};
      if (live[mi]) {
        z = *(const u32x4*)(Qg + qoff[mi] * DH + 32 * ks + 8 * g);
        z2 = *(const u32x4*)(dOg + qoff[mi] * DH + 32 * ks + 8 * g);
      }
      Qf[mi][ks] = __builtin_bit_cast(v8, z);
      dOf[mi][ks] = __builtin_bit_cast(v8, z2);
    }
    const long so = (long)b * a.tq * hq + qoff[mi];
    base[mi] = (Gg ? Gg[(long)ti[mi] * a.h] : 0.f) - a.rowmax[so];
    dlr[mi] = a.dl ? a.dl[so] : 0.f;
    osc[mi] = a.dO_scale ? a.dO_scale[so] : 1.f;
    dgq[mi] = 0.f;
  }
  f32x4 acc[MT][NT];
#pragma unroll
  for (int mi = 0; mi < MT; mi++)
#pragma unroll
    for (int nt = 0; nt < NT; nt++) acc[mi][nt] = (f32x4){0, 0, 0, 0};

  const int last_row = min(row0 + ROWS, rows) - 1;
  const int kmax = min(a.tk, last_row / a.r + shift + 1);
  const int first_ti = row0 / a.r + shift;
  const int ntiles = (kmax + AB_BN - 1) / AB_BN;

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
    if (tid < AB_BN && Gg) {
      rg = Gg[(long)min(j0 + tid, a.tk - 1) * a.h];
      rR = Gg[(long)min(j0 + AB_BN - 1, a.tk - 1) * a.h];
    }
  };
  auto stash = [&](int stage) {
#pragma unroll
    for (int i = 0; i < PT; i++) {
      const int ch = tid + 256 * i;
      if (ch < CH) {
        const int o = stage * AB_BN * LD + (ch / (DH / 8)) * LD + (ch % (DH / 8)) * 8;
        *(u32x4*)(Kt + o) = rk[i];
        *(u32x4*)(Vt + o) = rv[i];
      }
    }
    if (tid < AB_BN) {
      gk[stage * GS + tid] = rg;
      gk[stage * GS + AB_BN + tid] = __expf(fminf(rR - rg, AB_EXP_CLAMP));
      if (tid == 0) gk[stage * GS + 2 * AB_BN] = rR;
    }
  };

  fetch(0);
  for (int it = 0; it < ntiles; it++) {
    const int j0 = it * AB_BN, stage = it & 1;
    stash(stage);
    lds_barrier();
    if (it + 1 < ntiles) fetch(j0 + AB_BN);
    const T* kt_ = Kt + stage * AB_BN * LD;
    const T* vt_ = Vt + stage * AB_BN * LD;
    const float* gk_ = gk + stage * GS;
    const bool diag = (j0 + AB_BN - 1 > first_ti) || (j0 + AB_BN > a.tk);
    const float R = gk_[2 * AB_BN];
    float eu[MT];
#pragma unroll
    for (int mi = 0; mi < MT; mi++) eu[mi] = scale_p * (diag ? 1.f : __expf(fminf(base[mi] - R, AB_EXP_CLAMP)));

    v8 dsf[MT][KT / 2];
#pragma unroll
    for (int kp = 0; kp < KT / 2; kp++) {
      float d8[MT][8];
#pragma unroll
      for (int half = 0; half < 2; half++) {
        const int kt = 2 * kp + half;
        v8 kf[KS], vf[KS];
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
          kf[ks] = lds_frag<T>(kt_, LD, 16 * kt, 32 * ks);
          vf[ks] = lds_frag<T>(vt_, LD, 16 * kt, 32 * ks);
        }
        const f32x4 gkv = *(const f32x4*)(gk_ + (diag ? 0 : AB_BN) + 16 * kt + 4 * g);
#pragma unroll
        for (int mi = 0; mi < MT; mi++) {
          f32x4 s = {0, 0, 0, 0}, dp = {0, 0, 0, 0};
#pragma unroll
          for (int ks = 0; ks < KS; ks++) {
            s = mfma16(kf[ks], Qf[mi][ks], s);
            dp = mfma16(vf[ks], dOf[mi][ks], dp);
          }
#pragma unroll
          for (int v = 0; v < 4; v++) {
            float E;
            if (diag) {
              const int key = j0 + 16 * kt + 4 * g + v;
              E = eu[mi] * __expf(fminf(base[mi] - gkv[v], AB_EXP_CLAMP));
              if (key > ti[mi] || key >= a.tk) E = 0.f;
            } else {
              E = eu[mi] * gkv[v];
            }
            float p, dz, dsr;
            pair_grad<DEG2>(s[v], E, dp[v] * osc[mi] + dlr[mi], eps_s, half_deg, p, dz, dsr);
            dgq[mi] += dz;
            d8[mi][4 * half + v] = dsr;
          }
        }
      }
#pragma unroll
      for (int mi = 0; mi < MT; mi++) dsf[mi][kp] = pack8<T>(d8[mi]);
    }
    // dQ^T[d, row] += K^T[d, key] dsr^T[key, row]
#pragma unroll
    for (int kp = 0; kp < KT / 2; kp++) {
#pragma unroll
      for (int nt = 0; nt < NT; nt++) {
        v4 lo = lds_frag_tr4<T>(kt_, LD, 32 * kp + 4 * g, 16 * nt);
        v4 hi = lds_frag_tr4<T>(kt_, LD, 32 * kp + 16 + 4 * g, 16 * nt);
        v8 kT = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
#pragma unroll
        for (int mi = 0; mi < MT; mi++) acc[mi][nt] = mfma16(kT, dsf[mi][kp], acc[mi][nt]);
      }
    }
  }

  T* dQg = (T*)a.dQ + (long)b * a.tq * hq * DH;
#pragma unroll
  for (int mi = 0; mi < MT; mi++) {
    const float tot = sum_over_rows(dgq[mi]);
    if (!live[mi]) continue;
#pragma unroll
    for (int nt = 0; nt < NT; nt++) {
      float o4[4];
#pragma unroll
      for (int v = 0; v < 4; v++) o4[v] = acc[mi][nt][v] * a.deg;
      *(v4*)(dQg + qoff[mi] * DH + 16 * nt + 4 * g) = pack4<T>(o4);
    }
    if (g == 0 && a.dGq) a.dGq[(long)b * a.tq * hq + qoff[mi]] = tot;
  }
}

// ------------------------------------------------------------------ dK, dV, dGk
template <typename T, int DH, int MK, bool DEG2>
__global__ __launch_bounds__(256, 2) void attention_bwd_dkv_kernel(AttnBwdArgs a, int nblocks, int npairs) {
  typedef typename VecOf<T>::v8 v8;
  typedef typename VecOf<T>::v4 v4;
  constexpr int LD = DH + 8, KS = DH / 32, NT = DH / 16, QT = AB_BM / 16, KEYS = 64 * MK;
  constexpr int CH = AB_BM * DH / 8, PT = (CH + 255) / 256;
  extern __shared__ __attribute__((aligned(16))) char smem[];
  T* Qt = (T*)smem;                       // [2][BM][LD]
  T* dOt = Qt + 2 * AB_BM * LD;           // [2][BM][LD]
  float* rowv = (float*)(dOt + 2 * AB_BM * LD);  // [2][5][BM]: G_q - m, dl, time index, scale^deg exp(G_q - m - R), dO scale

  // Workgroups are dealt round-robin by their linear index to the 8 XCDs and then to the 4 shader engines of an
  // XCD; only the CU inside a shader engine is chosen by load.  Blocks differ in length (causal), so each of the 32
  // (XCD, shader engine) groups gets whole (batch, kv head) pairs, the longest blocks of all its pairs first.
  const int grp = blockIdx.x % 32, u = blockIdx.x / 32, ppg = (npairs + 31) / 32;
  const int pair = (u % ppg) * 32 + grp;
  if (pair >= npairs) return;
  const int tid = threadIdx.x, l = tid & 63, g = l >> 4, wave = tid >> 6, kcol = l & 15;
  const int b = pair / a.h, hh = pair % a.h;
  const int hq = a.h * a.r, rows = a.tq * a.r, shift = a.tk - a.tq;
  const int key0 = (u / ppg) * KEYS;                 // early keys are seen by the most rows
  const T* Qg = (const T*)a.Q + (long)b * a.tq * hq * DH;
  const T* dOg = (const T*)a.dO + (long)b * a.tq * hq * DH;
  const T* Kg = (const T*)a.K + (long)b * a.tk * a.h * DH + hh * DH;
  const T* Vg = (const T*)a.V + (long)b * a.tk * a.h * DH + hh * DH;
  const float* Gg = a.G ? a.G + (long)b * a.tk * a.h + hh : nullptr;
  const long kstride = (long)a.h * DH;
  const int half_deg = (int)a.deg / 2;
  const float eps_s = AB_LOG_EPS / a.scale;
  const float scale_p = __expf(a.deg * __logf(a.scale));
  const int last_key = min(key0 + KEYS, a.tk) - 1;
  const float R = Gg ? Gg[(long)last_key * a.h] : 0.f;   // reference gate of this key block

  v8 Kf[MK][KS], Vf[MK][KS];
  int key[MK];
  bool live[MK];
  float Gk[MK], ev[MK], dgk[MK];
#pragma unroll
  for (int kj = 0; kj < MK; kj++) {
    key[kj] = key0 + wave * 16 * MK + 16 * kj + kcol;
    live[kj] = key[kj] < a.tk;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      u32x4 z = {0, 0, 0, 0}, z2 = {0, 0, 0, 0};
      if (live[kj]) {
        z = *(const u32x4*)(Kg + key[kj] * kstride + 32 * ks + 8 * g);
        z2 = *(const u32x4*)(Vg + key[kj] * kstride + 32 * ks + 8 * g);
      }
      Kf[kj][ks] = __builtin_bit_cast(v8, z);
      Vf[kj][ks] = __builtin_bit_cast(v8, z2);
    }
    Gk[kj] = (Gg && live[kj]) ? Gg[(long)key[kj] * a.h] : 0.f;
    ev[kj] = __expf(fminf(R - Gk[kj], AB_EXP_CLAMP));
    dgk[kj] = 0.f;
  }
  f32x4 accK[MK][NT], accV[MK][NT];
#pragma unroll
  for (int kj = 0; kj < MK; kj++)
#pragma unroll
    for (int nt = 0; nt < NT; nt++) {
      accK[kj][nt] = (f32x4){0, 0, 0, 0};
      accV[kj][nt] = (f32x4){0, 0, 0, 0};
    }

  // folded rows that can see any key of this workgroup: time index >= key0
  const int row_begin = max(0, (key0 - shift) * a.r) / AB_BM * AB_BM;
  const int nsteps = (rows - row_begin + AB_BM - 1) / AB_BM;

  u32x4 rq[PT], rdo[PT];
  float r0 = 0.f, r1 = 0.f, r2 = 0.f, r3 = 1.f;
  auto fetch = [&](int rbase) {
#pragma unroll
    for (int i = 0; i < PT; i++) {
      const int ch = tid + 256 * i;
      const int row = rbase + ch / (DH / 8), col = (ch % (DH / 8)) * 8;
      rq[i] = (u32x4){0, 0, 0, 0};
      rdo[i] = (u32x4){0, 0, 0, 0};
      if (ch < CH && row < rows) {
        const int t = row / a.r;
        const long qo = (long)t * hq + hh * a.r + (row - t * a.r);
        rq[i] = *(const u32x4*)(Qg + qo * DH + col);
        rdo[i] = *(const u32x4*)(dOg + qo * DH + col);
      }
    }
    if (tid < AB_BM) {
      const int row = rbase + tid;
      r0 = 0.f; r1 = 0.f; r2 = -1.f; r3 = 1.f;  // time index -1: sees no key
      if (row < rows) {
        const int t = row / a.r;
        const long so = (long)b * a.tq * hq + (long)t * hq + hh * a.r + (row - t * a.r);
        r0 = (Gg ? Gg[(long)(t + shift) * a.h] : 0.f) - a.rowmax[so];
        r1 = a.dl ? a.dl[so] : 0.f;
        r2 = (float)(t + shift);
        r3 = a.dO_scale ? a.dO_scale[so] : 1.f;
      }
    }
  };
  auto stash = [&](int stage) {
#pragma unroll
    for (int i = 0; i < PT; i++) {
      const int ch = tid + 256 * i;
      if (ch < CH) {
        const int o = stage * AB_BM * LD + (ch / (DH / 8)) * LD + (ch % (DH / 8)) * 8;
        *(u32x4*)(Qt + o) = rq[i];
        *(u32x4*)(dOt + o) = rdo[i];
      }
    }
    if (tid < AB_BM) {
      float* rv = rowv + stage * 5 * AB_BM;
      rv[tid] = r0;
      rv[AB_BM + tid] = r1;
      rv[2 * AB_BM + tid] = r2;
      rv[3 * AB_BM + tid] = scale_p * __expf(fminf(r0 - R, AB_EXP_CLAMP));
      rv[4 * AB_BM + tid] = r3;
    }
  };

  if (nsteps > 0) fetch(row_begin);
  for (int it = 0; it < nsteps; it++) {
    const int rbase = row_begin + it * AB_BM, stage = it & 1;
    stash(stage);
    lds_barrier();
    if (it + 1 < nsteps) fetch(rbase + AB_BM);
    const T* qt_ = Qt + stage * AB_BM * LD;
    const T* dot_ = dOt + stage * AB_BM * LD;
    const float* rv = rowv + stage * 5 * AB_BM;
    // exact per-pair path unless every row of the step is real and sees every (real) key of the workgroup
    const bool diag = (rbase / a.r + shift < last_key) || (rbase + AB_BM > rows) || (key0 + KEYS > a.tk);

    v8 pf[MK], dsf[MK];
    {
      float p8[MK][8], d8[MK][8];
#pragma unroll
      for (int qt = 0; qt < QT; qt++) {
        v8 qf[KS], dof[KS];
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
          qf[ks] = lds_frag<T>(qt_, LD, 16 * qt, 32 * ks);
          dof[ks] = lds_frag<T>(dot_, LD, 16 * qt, 32 * ks);
        }
        const f32x4 gm = *(const f32x4*)(rv + (diag ? 0 : 3 * AB_BM) + 16 * qt + 4 * g);
        const f32x4 dlv = *(const f32x4*)(rv + AB_BM + 16 * qt + 4 * g);
        const f32x4 tiv = *(const f32x4*)(rv + 2 * AB_BM + 16 * qt + 4 * g);
        const f32x4 osv = *(const f32x4*)(rv + 4 * AB_BM + 16 * qt + 4 * g);
#pragma unroll
        for (int kj = 0; kj < MK; kj++) {
          f32x4 s = {0, 0, 0, 0}, dp = {0, 0, 0, 0};
#pragma unroll
          for (int ks = 0; ks < KS; ks++) {
            s = mfma16(qf[ks], Kf[kj][ks], s);
            dp = mfma16(dof[ks], Vf[kj][ks], dp);
          }
#pragma unroll
          for (int v = 0; v < 4; v++) {
            float E;
            if (diag) {
              E = scale_p * __expf(fminf(gm[v] - Gk[kj], AB_EXP_CLAMP));
              if ((float)key[kj] > tiv[v] || !live[kj]) E = 0.f;
            } else {
              E = gm[v] * ev[kj];
            }
            float p, dz, dsr;
            pair_grad<DEG2>(s[v], E, dp[v] * osv[v] + dlv[v], eps_s, half_deg, p, dz, dsr);
            dgk[kj] -= dz;
            p8[kj][4 * qt + v] = p * osv[v];
            d8[kj][4 * qt + v] = dsr;
          }
        }
      }
#pragma unroll
      for (int kj = 0; kj < MK; kj++) {
        pf[kj] = pack8<T>(p8[kj]);
        dsf[kj] = pack8<T>(d8[kj]);
      }
    }
    // dV^T[e, key] += dO^T[e, row] P[row, key];  dK^T[d, key] += Q^T[d, row] dsr[row, key]
#pragma unroll
    for (int nt = 0; nt < NT; nt++) {
      v4 lo = lds_frag_tr4<T>(dot_, LD, 4 * g, 16 * nt);
      v4 hi = lds_frag_tr4<T>(dot_, LD, 16 + 4 * g, 16 * nt);
      v8 doT = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
      lo = lds_frag_tr4<T>(qt_, LD, 4 * g, 16 * nt);
      hi = lds_frag_tr4<T>(qt_, LD, 16 + 4 * g, 16 * nt);
      v8 qT = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
#pragma unroll
      for (int kj = 0; kj < MK; kj++) {
        accV[kj][nt] = mfma16(doT, pf[kj], accV[kj][nt]);
        accK[kj][nt] = mfma16(qT, dsf[kj], accK[kj][nt]);
      }
    }
  }

  T* dKg = (T*)a.dK + (long)b * a.tk * a.h * DH + hh * DH;
  T* dVg = (T*)a.dV + (long)b * a.tk * a.h * DH + hh * DH;
#pragma unroll
  for (int kj = 0; kj < MK; kj++) {
    const float tot = sum_over_rows(dgk[kj]);
    if (!live[kj]) continue;
#pragma unroll
    for (int nt = 0; nt < NT; nt++) {
      float k4[4], v4f[4];
#pragma unroll
      for (int v = 0; v < 4; v++) {
        k4[v] = accK[kj][nt][v] * a.deg;
        v4f[v] = accV[kj][nt][v];
      }
      *(v4*)(dKg + key[kj] * kstride + 16 * nt + 4 * g) = pack4<T>(k4);
      *(v4*)(dVg + key[kj] * kstride + 16 * nt + 4 * g) = pack4<T>(v4f);
    }
    if (g == 0 && a.dGk) a.dGk[((long)b * a.tk + key[kj]) * a.h + hh] = tot;
  }
}

template <typename T, int DH, bool DEG2> static int attn_bwd_launch(const AttnBwdArgs& a, int B, hipStream_t st) {
  {
    constexpr int MT = DH <= 64 ? 2 : 1;
    constexpr size_t smem = 2 * 2 * AB_BN * (DH + 8) * sizeof(T) + 2 * (2 * AB_BN + 4) * sizeof(float);
    const int rows = a.tq * a.r;
    const int nblocks = (rows + 64 * MT - 1) / (64 * MT), npairs = B * a.h;
    dim3 grid((unsigned)((npairs + 31) / 32 * 32 * nblocks));
    auto kern = attention_bwd_dq_kernel<T, DH, MT, DEG2>;
    allow_big_lds((const void*)kern, smem);
    hipLaunchKernelGGL(kern, grid, dim3(256), smem, st, a, nblocks, npairs);
  }
  {
    constexpr int MK = DH <= 64 ? 2 : 1;
    constexpr size_t smem = 2 * 2 * AB_BM * (DH + 8) * sizeof(T) + 2 * 5 * AB_BM * sizeof(float);
    const int nblocks = (a.tk + 64 * MK - 1) / (64 * MK), npairs = B * a.h;
    dim3 grid((unsigned)((npairs + 31) / 32 * 32 * nblocks));
    auto kern = attention_bwd_dkv_kernel<T, DH, MK, DEG2>;
    allow_big_lds((const void*)kern, smem);
    hipLaunchKernelGGL(kern, grid, dim3(256), smem, st, a, nblocks, npairs);
  }
  return (int)hipGetLastError();
}

int attention_bwd(const AttnBwdArgs& a, int B, int d, int dtype, hipStream_t st) {
#define PR_AB(T)                                                                                                       \
  switch (d) {                                                                                                         \
    case 32: return a.deg == 2.f ? attn_bwd_launch<T, 32, true>(a, B, st) : attn_bwd_launch<T, 32, false>(a, B, st);   \
    case 64: return a.deg == 2.f ? attn_bwd_launch<T, 64, true>(a, B, st) : attn_bwd_launch<T, 64, false>(a, B, st);   \
    case 128: return a.deg == 2.f ? attn_bwd_launch<T, 128, true>(a, B, st) : attn_bwd_launch<T, 128, false>(a, B, st);\
    default: return -2;                                                                                                \
  }
  if (dtype == DT_BF16) { PR_AB(bf16_t) }
  if (dtype == DT_F16) { PR_AB(f16_t) }
#undef PR_AB
  return -1;
}

}  // namespace pr
