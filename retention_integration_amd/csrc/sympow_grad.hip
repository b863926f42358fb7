// Gradient of the degree-2 feature map through a state contraction:
//
//   dphi[row, f] = sum_e G[row, e] * B[f, e] + cvec[row] * sB[f]
//   dX[row, x_f] += m_f * X[row, w_f] * dphi[row, f]
//   dX[row, w_f] += m_f * X[row, x_f] * dphi[row, f]          (f = (x_f, w_f) in the tiled layout)
//
// Two callers:
//   * query_state backward, dQ: X = gated Q, G = scaled dO, cvec = -scaled delta, B = S, sB = s, m = 1
//                                                  (ref: retention/_query_state/triton.py:546-553)
//   * update_state backward, dK: X = K, G = V, cvec = 1, B = dS, sB = ds, m = 2 below the block diagonal
//                                                  (ref: retention/_update_state/reference.py:55-83)
//
// dphi is never stored.  A workgroup = 4 waves owns 64*MT rows (16*MT per wave).  For one x column X and
// one 16-wide strip y the wave forms the 16x16 tile dphi^T[i, row] (i = feature within the strip) on the
// matrix cores, B rows straight from LDS as the A operand and G^T from registers as the B operand,
// then folds it twice on the VALU: into dX[row, 16y+i] (times X[row, X]) kept in registers, and into
// dX[row, X] (dot with X[row, 16y+i] over i) reduced across the wave and parked in LDS.
#include "common.h"
#include "kernels.h"

namespace pr {

template <typename T, int DK, int DV, int MT, int XS, bool MULT>
__global__ __launch_bounds__(256) void sympow_grad_kernel(GradArgs a) {
  typedef typename VecOf<T>::v8 v8;
  typedef typename VecOf<T>::v4 v4;
  constexpr int TT = DK / 16, KS = DV / 32, LDB = DV + 8, ROWS = 64 * MT;
  constexpr int D = 128 * TT * (TT + 1);
  constexpr int SROWS = 16 * XS;                     // B rows per strip per stage
  constexpr int CH_PER_Y = SROWS * DV / 8;           // 16-byte chunks per strip
  constexpr int MAX_PT = (TT * CH_PER_Y + 255) / 256;
  constexpr int NSTAGE = TT * (16 / XS);
  extern __shared__ __attribute__((aligned(16))) char smem[];
  T* bt = (T*)smem;                                   // [2][TT][SROWS][LDB]
  float* st = (float*)(bt + 2 * TT * SROWS * LDB);    // [2][TT][SROWS]
  float* dxb = st + 2 * TT * SROWS;                   // [ROWS][DK + 1]
  constexpr int LDD = DK + 1;

  const int tid = threadIdx.x, l = tid & 63, g = l >> 4, wave = tid >> 6, tcol = l & 15;
  const int bn = blockIdx.y / a.h, hh = blockIdx.y % a.h;
  const int hA = a.h * a.r, rows = a.c * a.r;
  const int row0 = blockIdx.x * ROWS;
  const T* Xg = (const T*)a.X + (long)bn * a.c * hA * DK;
  const T* Gg = (const T*)a.G + (long)bn * a.c * hA * DV;
  const T* Bg = (const T*)a.B + ((long)bn * a.h + hh) * D * DV;
  const float* sBg = a.sB + ((long)bn * a.h + hh) * D;
  T* dXg = (T*)a.dX + (long)bn * a.c * hA * DK;
  auto row_off = [&](int row) -> long {
    const int t = row / a.r, rr = row - t * a.r;
    return (long)t * hA + hh * a.r + rr;
  };

  if (a.skip_first && (bn % a.n == 0)) {
    for (int i = tid; i < ROWS * DK / 8; i += 256) {
      const int rl = i / (DK / 8), col = (i % (DK / 8)) * 8;
      if (row0 + rl < rows) *(u32x4*)(dXg + row_off(row0 + rl) * DK + col) = (u32x4){0, 0, 0, 0};
    }
    return;
  }

  // per-lane row data (row = this lane's column of the dphi^T tiles)
  v8 Gf[MT][KS];
  float xr[MT][TT][4];
  float cv[MT];
  long roff[MT];
  bool rlive[MT];
#pragma unroll
  for (int mi = 0; mi < MT; mi++) {
    const int row = row0 + wave * 16 * MT + 16 * mi + tcol;
    rlive[mi] = row < rows;
    roff[mi] = row_off(rlive[mi] ? row : 0);
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      u32x4 z = {0, 0, 0, 0};
      if (rlive[mi]) z = *(const u32x4*)(Gg + roff[mi] * DV + 32 * ks + 8 * g);
      Gf[mi][ks] = __builtin_bit_cast(v8, z);
    }
#pragma unroll
    for (int y = 0; y < TT; y++) {
      u32x2 z = {0, 0};
      if (rlive[mi]) z = *(const u32x2*)(Xg + roff[mi] * DK + 16 * y + 4 * g);
      v4 h4 = __builtin_bit_cast(v4, z);
#pragma unroll
      for (int v = 0; v < 4; v++) xr[mi][y][v] = (float)h4[v];
    }
    cv[mi] = rlive[mi] ? (a.cvec ? a.cvec[(long)bn * a.c * hA + roff[mi]] : 1.f) : 0.f;
  }
  f32x4 accA[MT][TT];
#pragma unroll
  for (int mi = 0; mi < MT; mi++)
#pragma unroll
    for (int y = 0; y < TT; y++) accA[mi][y] = (f32x4){0, 0, 0, 0};

  // stage s covers x columns Xbase .. Xbase+XS-1 of block column xb, strips y = xb .. TT-1
  u32x4 rb[MAX_PT];
  float rs[(TT * SROWS + 255) / 256];
  T xnext[MT][XS];  // X[row, Xbase + xx] of the stage being fetched
  auto fetch = [&](int s) {
    const int xb = s / (16 / XS), Xbase = 16 * xb + XS * (s % (16 / XS));
    const int ny = TT - xb;
#pragma unroll
    for (int mi = 0; mi < MT; mi++)
#pragma unroll
      for (int xx = 0; xx < XS; xx++) xnext[mi][xx] = rlive[mi] ? Xg[roff[mi] * DK + Xbase + xx] : (T)0.f;
#pragma unroll
    for (int i = 0; i < MAX_PT; i++) {
      const int ch = tid + 256 * i;
      if (ch < ny * CH_PER_Y) {
        const int yy = ch / CH_PER_Y, rem = ch % CH_PER_Y, y = xb + yy;
        const int rl = rem / (DV / 8), col = (rem % (DV / 8)) * 8;
        rb[i] = *(const u32x4*)(Bg + (long)(128 * y * (y + 1) + 16 * Xbase + rl) * DV + col);
      }
    }
#pragma unroll
    for (int i = 0; i < (TT * SROWS + 255) / 256; i++) {
      const int j = tid + 256 * i;
      if (j < ny * SROWS) {
        const int yy = j / SROWS, y = xb + yy;
        rs[i] = sBg[128 * y * (y + 1) + 16 * Xbase + j % SROWS];
      }
    }
  };
  auto stash = [&](int s, int stage) {
    const int xb = s / (16 / XS);
    const int ny = TT - xb;
    T* b = bt + stage * TT * SROWS * LDB;
#pragma unroll
    for (int i = 0; i < MAX_PT; i++) {
      const int ch = tid + 256 * i;
      if (ch < ny * CH_PER_Y) {
        const int yy = ch / CH_PER_Y, rem = ch % CH_PER_Y;
        *(u32x4*)(b + (yy * SROWS + rem / (DV / 8)) * LDB + (rem % (DV / 8)) * 8) = rb[i];
      }
    }
#pragma unroll
    for (int i = 0; i < (TT * SROWS + 255) / 256; i++) {
      const int j = tid + 256 * i;
      if (j < ny * SROWS) st[stage * TT * SROWS + j] = rs[i];
    }
  };

  fetch(0);
  for (int s = 0; s < NSTAGE; s++) {
    const int stage = s & 1;
    stash(s, stage);
    float xcur[MT][XS];
#pragma unroll
    for (int mi = 0; mi < MT; mi++)
#pragma unroll
      for (int xx = 0; xx < XS; xx++) xcur[mi][xx] = (float)xnext[mi][xx];
    __syncthreads();
    if (s + 1 < NSTAGE) fetch(s + 1);
    const int xb = s / (16 / XS), Xbase = 16 * xb + XS * (s % (16 / XS));
    const T* b = bt + stage * TT * SROWS * LDB;
    const float* sv = st + stage * TT * SROWS;
#pragma unroll
    for (int xx = 0; xx < XS; xx++) {
      const int X = Xbase + xx;
      float xX[MT], pd[MT], po[MT];
#pragma unroll
      for (int mi = 0; mi < MT; mi++) {
        xX[mi] = xcur[mi][xx];
        pd[mi] = 0.f;
        po[mi] = 0.f;
      }
#pragma unroll
      for (int yy = 0; yy < TT; yy++) {
        const int y = xb + yy;
        if (y < TT) {
          v8 af[KS];
#pragma unroll
          for (int ks = 0; ks < KS; ks++) af[ks] = lds_frag<T>(b + yy * SROWS * LDB, LDB, 16 * xx, 32 * ks);
          const f32x4 s4 = *(const f32x4*)(sv + yy * SROWS + 16 * xx + 4 * g);
          const bool off = MULT && (yy > 0);
#pragma unroll
          for (int mi = 0; mi < MT; mi++) {
            f32x4 dphi = s4 * cv[mi];
#pragma unroll
            for (int ks = 0; ks < KS; ks++) dphi = mfma16(af[ks], Gf[mi][ks], dphi);
            const float xs = off ? 2.f * xX[mi] : xX[mi];
            // xr is indexed by the runtime strip y: select with a compile-time loop
            float dot = 0.f;
#pragma unroll
            for (int yc = 0; yc < TT; yc++) {
              if (yc == y) {
                accA[mi][yc] += dphi * xs;
#pragma unroll
                for (int v = 0; v < 4; v++) dot += xr[mi][yc][v] * dphi[v];
              }
            }
            if (off) po[mi] += dot; else pd[mi] += dot;
          }
        }
      }
#pragma unroll
      for (int mi = 0; mi < MT; mi++) {
        const float tot = sum_over_rows(pd[mi] + 2.f * po[mi]);
        if (g == (X & 3)) dxb[(wave * 16 * MT + 16 * mi + tcol) * LDD + X] = tot;
      }
    }
  }
  __syncthreads();
#pragma unroll
  for (int mi = 0; mi < MT; mi++)
#pragma unroll
    for (int y = 0; y < TT; y++)
#pragma unroll
      for (int v = 0; v < 4; v++) dxb[(wave * 16 * MT + 16 * mi + tcol) * LDD + 16 * y + 4 * g + v] += accA[mi][y][v];
  __syncthreads();
  for (int i = tid; i < ROWS * DK / 8; i += 256) {
    const int rl = i / (DK / 8), col = (i % (DK / 8)) * 8;
    if (row0 + rl < rows) {
      float f[8];
#pragma unroll
      for (int j = 0; j < 8; j++) f[j] = dxb[rl * LDD + col + j];
      *(v8*)(dXg + row_off(row0 + rl) * DK + col) = pack8<T>(f);
    }
  }
}

template <typename T, int DK, int DV, bool MULT> static int grad_launch(const GradArgs& a, int BN, hipStream_t st) {
  constexpr int MT = 2, XS = DK <= 64 ? 2 : 1, TT = DK / 16;
  constexpr size_t smem = 2 * TT * 16 * XS * (DV + 8) * sizeof(T) + 2 * TT * 16 * XS * sizeof(float) +
                          64 * MT * (DK + 1) * sizeof(float);
  const int rows = a.c * a.r;
  dim3 grid((rows + 64 * MT - 1) / (64 * MT), (unsigned)(BN * a.h));
  auto kern = sympow_grad_kernel<T, DK, DV, MT, XS, MULT>;
  allow_big_lds((const void*)kern, smem);
  hipLaunchKernelGGL(kern, grid, dim3(256), smem, st, a);
  return (int)hipGetLastError();
}

int sympow_grad(const GradArgs& a, int BN, int d, int mult, int dtype, hipStream_t st) {
#define PR_G_D(T, DD)                                                                                                  \
  case DD: return mult ? grad_launch<T, DD, DD, true>(a, BN, st) : grad_launch<T, DD, DD, false>(a, BN, st);
#define PR_G_T(T)                                                                                                      \
  switch (d) { PR_G_D(T, 32) PR_G_D(T, 64) PR_G_D(T, 128) default: return -2; }
  if (dtype == DT_BF16) { PR_G_T(bf16_t) }
  if (dtype == DT_F16) { PR_G_T(f16_t) }
#undef PR_G_T
#undef PR_G_D
  return -1;
}

}  // namespace pr
