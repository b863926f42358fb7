// State query contraction  out[row, e] = sum_f m_f * phi(X_row)[f] * B[f, e],
//                           aux[row]    = sum_f m_f * phi(X_row)[f] * sB[f]
// over the tiled degree-2 feature layout, phi(x)[f] = x[x_f] * x[w_f].
//
// Two callers:
//   * query_state forward (m = 1): X = gated Q, B = S, sB = sum of keys, followed by the merge with
//     the intra-chunk attention result           (ref: retention/_query_state/reference.py:36-96)
//   * update_state backward, dV (m = 2 below the block diagonal): X = K, B = dS
//                                                (ref: retention/_update_state/reference.py:61)
//
// A workgroup = 4 waves owns 64*MT rows; each wave 16*MT rows and all DV columns.  B is streamed
// through LDS in its memory order, 32 features (two x columns of one 16-wide y strip) per step, and
// read with the transposing LDS load; the phi operand is built in registers from the wave's own rows
// (one scalar x[X] times eight x[16y+..] values per lane).  sB rides along as two extra bf16/fp16
// columns (high and low part of the fp32 value) of the B tile.
#include "common.h"
#include "kernels.h"

namespace pr {

constexpr int NN_KF = 32;

template <bool MULT> struct FeatIter {
  int y, X0, phase, T;
  __device__ void init(int T_) {
    T = T_;
    if (MULT && T > 1) { phase = 0; y = 1; X0 = 0; } else { phase = MULT ? 1 : 2; y = 0; X0 = 0; }
  }
  __device__ bool done() const { return y >= T; }
  __device__ int f0() const { return 128 * y * (y + 1) + 16 * X0; }
  // returns true when the step just consumed was the last one below the diagonal
  __device__ bool next() {
    X0 += 2;
    if (phase == 0) {
      if (X0 == 16 * y) { y++; X0 = 0; }
      if (y == T) { phase = 1; y = 0; X0 = 0; return true; }
    } else if (phase == 1) {
      if (X0 == 16 * (y + 1)) { y++; X0 = 16 * y; }
    } else {
      if (X0 == 16 * (y + 1)) { y++; X0 = 0; }
    }
    return false;
  }
};

template <typename T> struct ScaleS;  // keeps sB inside the 16-bit range
template <> struct ScaleS<bf16_t> { static constexpr float down = 1.f, up = 1.f; };
template <> struct ScaleS<f16_t> { static constexpr float down = 1.f / 256.f, up = 256.f; };

template <typename T> struct PhiRow;
template <> struct PhiRow<bf16_t> {
  float row[8];
  __device__ __forceinline__ void load(const bf16_t* p) { unpack8(*(const bf16x8*)p, row); }
  __device__ __forceinline__ bf16x8 make(bf16_t x) const {
    const float xs = (float)x;
    float p[8];
#pragma unroll
    for (int i = 0; i < 8; i++) p[i] = xs * row[i];
    return pack8<bf16_t>(p);
  }
};
template <> struct PhiRow<f16_t> {
  f16x8 row;
  __device__ __forceinline__ void load(const f16_t* p) { row = *(const f16x8*)p; }
  __device__ __forceinline__ f16x8 make(f16_t x) const { return row * x; }
};

template <typename T, int DK, int DV, int MT, bool MULT, int EPI>
__global__ __launch_bounds__(256) void sympow_nn_kernel(NNArgs a) {
  typedef typename VecOf<T>::v8 v8;
  constexpr int LDX = DK + 8, LDB = DV + 16 + 8, NT = DV / 16, TT = DK / 16;
  constexpr int D = 128 * TT * (TT + 1);
  constexpr int ROWS = 64 * MT;
  constexpr int B_CH = NN_KF * DV / 8, B_PT = (B_CH + 255) / 256;
  constexpr int X_CH = ROWS * DK / 8, X_PT = (X_CH + 255) / 256;
  extern __shared__ __attribute__((aligned(16))) char smem[];
  T* xt = (T*)smem;                 // [ROWS][LDX]
  T* bt = xt + ROWS * LDX;          // [2][KF][LDB]

  const int tid = threadIdx.x, l = tid & 63, g = l >> 4, wave = tid >> 6;
  const int bn = blockIdx.y / a.h, hh = blockIdx.y % a.h;
  const int hA = a.h * a.r, rows = a.c * a.r;
  const int row0 = blockIdx.x * ROWS;
  const T* X = (const T*)a.X + (long)bn * a.c * hA * DK;
  const T* Bg = (const T*)a.B + ((long)bn * a.h + hh) * D * DV;
  const float* sBg = a.sB ? a.sB + ((long)bn * a.h + hh) * D : nullptr;
  auto row_off = [&](int row) -> long {  // element offset of a folded row, per unit of the last dim
    const int t = row / a.r, rr = row - t * a.r;
    return (long)t * hA + hh * a.r + rr;
  };

  // stage the X rows and clear the B tiles (the unused aux columns must stay zero)
#pragma unroll
  for (int i = 0; i < X_PT; i++) {
    const int ch = tid + 256 * i;
    if (ch < X_CH) {
      const int rl = ch / (DK / 8), col = (ch % (DK / 8)) * 8;
      u32x4 v = {0, 0, 0, 0};
      if (row0 + rl < rows) v = *(const u32x4*)(X + row_off(row0 + rl) * DK + col);
      *(u32x4*)(xt + rl * LDX + col) = v;
    }
  }
  for (int i = tid; i < 2 * NN_KF * LDB / 2; i += 256) ((uint32_t*)bt)[i] = 0;

  const bool skip = (EPI == NN_EPI_MERGE) && a.skip_first && (bn % a.n == 0);
  f32x4 acc[MT][NT + 1];
#pragma unroll
  for (int i = 0; i < MT; i++)
#pragma unroll
    for (int j = 0; j <= NT; j++) acc[i][j] = (f32x4){0, 0, 0, 0};

  if (!skip) {
    u32x4 rb[B_PT];
    float rs = 0.f;
    auto fetch = [&](int f0) {
#pragma unroll
      for (int i = 0; i < B_PT; i++) {
        const int ch = tid + 256 * i;
        if (ch < B_CH) rb[i] = *(const u32x4*)(Bg + (long)(f0 + ch / (DV / 8)) * DV + (ch % (DV / 8)) * 8);
      }
      if (sBg && tid < NN_KF) rs = sBg[f0 + tid];
    };
    auto stash = [&](int stage) {
      T* b = bt + stage * NN_KF * LDB;
#pragma unroll
      for (int i = 0; i < B_PT; i++) {
        const int ch = tid + 256 * i;
        if (ch < B_CH) *(u32x4*)(b + (ch / (DV / 8)) * LDB + (ch % (DV / 8)) * 8) = rb[i];
      }
      if (sBg && tid < NN_KF) {
        const float v = rs * ScaleS<T>::down;
        const T hi = (T)v;
        b[tid * LDB + DV] = hi;
        b[tid * LDB + DV + 1] = (T)(v - (float)hi);
      }
    };

    FeatIter<MULT> cur, nxt;
    cur.init(TT);
    nxt.init(TT);
    fetch(nxt.f0());
    nxt.next();
    PhiRow<T> prow[MT];
    int y_loaded = -1, stage = 0;
    __syncthreads();  // X rows staged, B tiles cleared
    while (!cur.done()) {
      stash(stage);
      __syncthreads();
      if (!nxt.done()) fetch(nxt.f0());
      nxt.next();
      const T* b = bt + stage * NN_KF * LDB;
      if (cur.y != y_loaded) {
        y_loaded = cur.y;
#pragma unroll
        for (int mi = 0; mi < MT; mi++)
          prow[mi].load(xt + (wave * 16 * MT + 16 * mi + (l & 15)) * LDX + 16 * cur.y + 8 * (g & 1));
      }
      v8 vf[NT + 1];
#pragma unroll
      for (int nt = 0; nt <= NT; nt++) vf[nt] = lds_frag_tr<T>(b, LDB, 0, 16 * nt);
#pragma unroll
      for (int mi = 0; mi < MT; mi++) {
        const T xs = xt[(wave * 16 * MT + 16 * mi + (l & 15)) * LDX + cur.X0 + (g >> 1)];
        const v8 af = prow[mi].make(xs);
#pragma unroll
        for (int nt = 0; nt <= NT; nt++) acc[mi][nt] = mfma16(af, vf[nt], acc[mi][nt]);
      }
      if (cur.next()) {
#pragma unroll
        for (int mi = 0; mi < MT; mi++)
#pragma unroll
          for (int nt = 0; nt <= NT; nt++) acc[mi][nt] *= 2.f;
      }
      stage ^= 1;
    }
  }

  // epilogue: accumulator element v of lane l is row 4*(l/16)+v, column 16*nt + l%16
  T* out = (T*)a.out + (long)bn * a.c * hA * DV;
  const float log_gamma = 0.5f * __logf((float)D);
#pragma unroll
  for (int mi = 0; mi < MT; mi++) {
#pragma unroll
    for (int v = 0; v < 4; v++) {
      const int row = row0 + wave * 16 * MT + 16 * mi + 4 * g + v;
      if (row >= rows) continue;
      const long ro = row_off(row);
      if (EPI == NN_EPI_PLAIN) {
#pragma unroll
        for (int nt = 0; nt < NT; nt++) out[ro * DV + 16 * nt + (l & 15)] = (T)acc[mi][nt][v];
      } else {
        const float lqs = (row_bcast<0>(acc[mi][NT][v]) + row_bcast<1>(acc[mi][NT][v])) * ScaleS<T>::up;
        float wa = 0.f, wq = 1.f, la = 0.f;
        const T* ya = nullptr;
        if (a.Y_attn) {
          const long go = (long)bn * a.c * hA + ro;
          const float m = a.rowmax[go];
          la = a.l_attn[go];
          const float beta = fmaxf(m, log_gamma);
          wa = __expf(m - beta);
          wq = a.scale_p * __expf(-beta);
          ya = (const T*)a.Y_attn + (long)bn * a.c * hA * DV + ro * DV;
        }
        const float den = la * wa + lqs * wq;
        const float inv = 1.f / den;
#pragma unroll
        for (int nt = 0; nt < NT; nt++) {
          const int e = 16 * nt + (l & 15);
          float num = acc[mi][nt][v] * wq;
          if (ya) num += (float)ya[e] * wa;
          out[ro * DV + e] = (T)(num * inv);
        }
        if ((l & 15) == 0) a.den[(long)bn * a.c * hA + ro] = den;
      }
    }
  }
}

template <typename T, int DK, int DV, bool MULT, int EPI> static int nn_launch(const NNArgs& a, int BN, hipStream_t st) {
  const int rows = a.c * a.r;
  auto go = [&](auto mt) {
    constexpr int MT = decltype(mt)::value;
    constexpr size_t smem = (64 * MT * (DK + 8) + 2 * NN_KF * (DV + 24)) * sizeof(T);
    dim3 grid((rows + 64 * MT - 1) / (64 * MT), (unsigned)(BN * a.h));
    hipLaunchKernelGGL((sympow_nn_kernel<T, DK, DV, MT, MULT, EPI>), grid, dim3(256), smem, st, a);
  };
  if (DK <= 64 && rows >= 256) go(IC<4>{});
  else if (rows >= 128) go(IC<2>{});
  else go(IC<1>{});
  return (int)hipGetLastError();
}

int sympow_nn(const NNArgs& a, int BN, int d, int mult, int epi, int dtype, hipStream_t st) {
#define PR_NN_D(T, DD)                                                                                                 \
  case DD:                                                                                                             \
    if (epi == NN_EPI_MERGE) return nn_launch<T, DD, DD, false, NN_EPI_MERGE>(a, BN, st);                             \
    return mult ? nn_launch<T, DD, DD, true, NN_EPI_PLAIN>(a, BN, st) : nn_launch<T, DD, DD, false, NN_EPI_PLAIN>(a, BN, st);
#define PR_NN_T(T)                                                                                                     \
  switch (d) { PR_NN_D(T, 32) PR_NN_D(T, 64) PR_NN_D(T, 128) default: return -2; }
  if (dtype == DT_BF16) { PR_NN_T(bf16_t) }
  if (dtype == DT_F16) { PR_NN_T(f16_t) }
#undef PR_NN_T
#undef PR_NN_D
  return -1;
}

}  // namespace pr
