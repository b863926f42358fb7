// Chunk-state contraction  S[f, e] = m_f * sum_rows phi(A_row)[f] * B[row, e],
//                          s[f]    = m_f * sum_rows phi(A_row)[f] * w[row]      (w = 1 when absent)
// with phi(a)[f] = a[x_f] * a[w_f] the degree-2 symmetric power features in the tiled state layout
// and m_f = 2 for tiles strictly below the block diagonal when use_mult is set.
//
// Two callers:
//   * update_state forward: A = K, B = V                       (ref: retention/_update_state/reference.py:33-52)
//   * query_state backward, dS/ds: A = Q, B = scaled dO, w = -scaled delta, m = 1
//                                                              (ref: retention/_query_state/triton.py:546-553)
//
// One workgroup = 4 waves; a wave owns XPW of the 16 "x" columns of one 16x16 feature block
// (y, xb) and all DV value columns, and contracts over the rows in steps of 32.  The phi tile is
// never stored: the A-operand of each matrix-core op is produced in registers as the product of a
// row-broadcast (DPP) of column x with the 16 columns 16*y..16*y+15, both read transposed from one
// row-major LDS tile.  s uses the identity s[(x, j)] = (A^T diag(w) A)[x, j], one extra matrix-core op
// per step.
#include "common.h"
#include "kernels.h"

namespace pr {

constexpr int TN_KT = 32;  // rows contracted per step

template <typename T, int X> struct PhiTile;
template <int X> struct PhiTile<bf16_t, X> {
  static __device__ __forceinline__ bf16x8 make(const bf16x8&, const bf16x8&, const float* rowf, const float* srcf) {
    float p[8];
#pragma unroll
    for (int r = 0; r < 8; r++) p[r] = row_bcast<X>(srcf[r]) * rowf[r];
    return pack8<bf16_t>(p);
  }
};
template <int X> struct PhiTile<f16_t, X> {
  static __device__ __forceinline__ f16x8 make(const f16x8& rows, const f16x8& src, const float*, const float*) {
    u32x4 u = __builtin_bit_cast(u32x4, src), b;
#pragma unroll
    for (int i = 0; i < 4; i++) b[i] = row_bcast_u32<X>(u[i]);
    return rows * __builtin_bit_cast(f16x8, b);
  }
};

template <typename T, int DK, int DV, int XPW, int PART, bool HAS_W>
__device__ __forceinline__ void tn_body(const T* __restrict__ A, const T* __restrict__ Bm, const float* __restrict__ w,
                                        T* __restrict__ S, float* __restrict__ s, int c, int hA, int r, int hh,
                                        int bn, int h, int y, int xb, bool active, bool use_mult, char* smem) {
  typedef typename VecOf<T>::v8 v8;
  constexpr int LDA = DK + 8, LDB = DV + 8, NT = DV / 16;
  constexpr int A_CH = TN_KT * DK / 8, B_CH = TN_KT * DV / 8;  // 16-byte chunks per tile
  constexpr int A_PT = (A_CH + 255) / 256, B_PT = (B_CH + 255) / 256;
  T* At = (T*)smem;                                   // [2][KT][LDA]
  T* Bt = At + 2 * TN_KT * LDA;                       // [2][KT][LDB]
  float* wt = (float*)(Bt + 2 * TN_KT * LDB);         // [2][KT]
  const int tid = threadIdx.x, l = tid & 63, g = l >> 4;
  const int rows = c * r;
  const long a_base = (long)bn * c * hA * DK, b_base = (long)bn * c * hA * DV, w_base = (long)bn * c * hA;

  u32x4 ra[A_PT], rb[B_PT];
  float rw = 0.f;
  auto fetch = [&](int step) {
#pragma unroll
    for (int i = 0; i < A_PT; i++) {
      const int ch = tid + 256 * i;
      const int row = step * TN_KT + ch / (DK / 8), col = (ch % (DK / 8)) * 8;
      ra[i] = (u32x4){0, 0, 0, 0};
      if (ch < A_CH && row < rows) {
        const int t = row / r, rr = row - t * r;
        ra[i] = *(const u32x4*)(A + a_base + ((long)t * hA + hh * r + rr) * DK + col);
      }
    }
#pragma unroll
    for (int i = 0; i < B_PT; i++) {
      const int ch = tid + 256 * i;
      const int row = step * TN_KT + ch / (DV / 8), col = (ch % (DV / 8)) * 8;
      rb[i] = (u32x4){0, 0, 0, 0};
      if (ch < B_CH && row < rows) {
        const int t = row / r, rr = row - t * r;
        rb[i] = *(const u32x4*)(Bm + b_base + ((long)t * hA + hh * r + rr) * DV + col);
      }
    }
    if (HAS_W && tid < TN_KT) {
      const int row = step * TN_KT + tid;
      rw = 0.f;
      if (row < rows) {
        const int t = row / r, rr = row - t * r;
        rw = w[w_base + (long)t * hA + hh * r + rr];
      }
    }
  };
  auto stash = [&](int stage) {
#pragma unroll
    for (int i = 0; i < A_PT; i++) {
      const int ch = tid + 256 * i;
      if (ch < A_CH) *(u32x4*)(At + stage * TN_KT * LDA + (ch / (DK / 8)) * LDA + (ch % (DK / 8)) * 8) = ra[i];
    }
#pragma unroll
    for (int i = 0; i < B_PT; i++) {
      const int ch = tid + 256 * i;
      if (ch < B_CH) *(u32x4*)(Bt + stage * TN_KT * LDB + (ch / (DV / 8)) * LDB + (ch % (DV / 8)) * 8) = rb[i];
    }
    if (HAS_W && tid < TN_KT) wt[stage * TN_KT + tid] = rw;
  };

  f32x4 acc[XPW][NT];
#pragma unroll
  for (int i = 0; i < XPW; i++)
#pragma unroll
    for (int j = 0; j < NT; j++) acc[i][j] = (f32x4){0, 0, 0, 0};
  f32x4 sacc = {0, 0, 0, 0};

  const int steps = (rows + TN_KT - 1) / TN_KT;
  fetch(0);
  for (int step = 0; step < steps; step++) {
    const int stage = step & 1;
    stash(stage);
    __syncthreads();
    if (step + 1 < steps) fetch(step + 1);
    if (active) {
      const T* at = At + stage * TN_KT * LDA;
      const T* bt = Bt + stage * TN_KT * LDB;
      v8 kfy = lds_frag_tr<T>(at, LDA, 0, 16 * y);
      v8 kfx = (xb == y) ? kfy : lds_frag_tr<T>(at, LDA, 0, 16 * xb);
      v8 vf[NT];
#pragma unroll
      for (int nt = 0; nt < NT; nt++) vf[nt] = lds_frag_tr<T>(bt, LDB, 0, 16 * nt);
      float rowf[8], srcf[8];
      unpack8(kfy, rowf);
      unpack8(kfx, srcf);
      if (HAS_W) {
        float sc[8];
        const float* wp = wt + stage * TN_KT + 8 * g;
#pragma unroll
        for (int q = 0; q < 8; q++) sc[q] = srcf[q] * wp[q];
        sacc = mfma16(kfy, pack8<T>(sc), sacc);
      } else {
        sacc = mfma16(kfy, kfx, sacc);
      }
      static_for<XPW>([&](auto xi) {
        v8 a = PhiTile<T, PART * XPW + xi.value>::make(kfy, kfx, rowf, srcf);
#pragma unroll
        for (int nt = 0; nt < NT; nt++) acc[xi.value][nt] = mfma16(a, vf[nt], acc[xi.value][nt]);
      });
    }
  }
  if (!active) return;
  const float mul = (use_mult && xb < y) ? 2.f : 1.f;
  constexpr int D = 128 * (DK / 16) * (DK / 16 + 1);
  const int fbase = 128 * y * (y + 1) + 256 * xb;
  const long so = ((long)bn * h + hh) * D;
#pragma unroll
  for (int xi = 0; xi < XPW; xi++) {
    const int X = PART * XPW + xi;
#pragma unroll
    for (int nt = 0; nt < NT; nt++)
#pragma unroll
      for (int v = 0; v < 4; v++)
        S[(so + fbase + 16 * X + 4 * g + v) * DV + 16 * nt + (l & 15)] = (T)(acc[xi][nt][v] * mul);
  }
  const int Xc = l & 15;
  if (Xc >= PART * XPW && Xc < (PART + 1) * XPW) {
#pragma unroll
    for (int v = 0; v < 4; v++) s[so + fbase + 16 * Xc + 4 * g + v] = sacc[v] * mul;
  }
}

template <typename T, int DK, int DV, int XPW, bool HAS_W>
__global__ __launch_bounds__(256, 2) void sympow_tn_kernel(const T* __restrict__ A, const T* __restrict__ Bm,
                                                        const float* __restrict__ w, T* __restrict__ S,
                                                        float* __restrict__ s, int c, int hA, int r, int h,
                                                        int use_mult) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  constexpr int PARTS = 16 / XPW;
  constexpr int NB = (DK / 16) * (DK / 16 + 1) / 2;
  const int task = blockIdx.x * 4 + (threadIdx.x >> 6);
  const bool active = task < NB * PARTS;
  const int t2 = active ? task : 0;
  const int part = t2 % PARTS;
  int y, xb;
  block_to_yx(t2 / PARTS, y, xb);
  const int bn = blockIdx.y / h, hh = blockIdx.y % h;
#define PR_TN_CASE(P)                                                                                                  \
  case P:                                                                                                              \
    if (P < PARTS)                                                                                                     \
      tn_body<T, DK, DV, XPW, (P < PARTS ? P : 0), HAS_W>(A, Bm, w, S, s, c, hA, r, hh, bn, h, y, xb, active,         \
                                                          use_mult != 0, smem);                                        \
    break;
  switch (part) {
    PR_TN_CASE(0)
    PR_TN_CASE(1)
    PR_TN_CASE(2)
    PR_TN_CASE(3)
  }
#undef PR_TN_CASE
}

template <typename T, int DK, int DV>
static int tn_launch(const void* A, const void* Bm, const float* w, void* S, float* s, int BN, int c, int h, int r,
                     int use_mult, hipStream_t st) {
  constexpr int XPW = DV <= 64 ? 8 : 4;
  constexpr int NB = (DK / 16) * (DK / 16 + 1) / 2;
  constexpr int TASKS = NB * (16 / XPW);
  constexpr size_t smem = 2 * TN_KT * ((DK + 8) + (DV + 8)) * sizeof(T) + 2 * TN_KT * sizeof(float);
  dim3 grid((TASKS + 3) / 4, (unsigned)(BN * h));
  if (w)
    hipLaunchKernelGGL((sympow_tn_kernel<T, DK, DV, XPW, true>), grid, dim3(256), smem, st, (const T*)A, (const T*)Bm, w,
                       (T*)S, s, c, h * r, r, h, use_mult);
  else
    hipLaunchKernelGGL((sympow_tn_kernel<T, DK, DV, XPW, false>), grid, dim3(256), smem, st, (const T*)A, (const T*)Bm,
                       w, (T*)S, s, c, h * r, r, h, use_mult);
  return (int)hipGetLastError();
}

// A: [BN, c, h*r, d], Bm: [BN, c, h*r, d], w: [BN, c, h*r] or null -> S: [BN, h, D, d], s: [BN, h, D]
int sympow_tn(const void* A, const void* Bm, const float* w, void* S, float* s, int BN, int c, int h, int r, int d,
              int use_mult, int dtype, hipStream_t st) {
#define PR_TN_DISPATCH(T)                                                                                              \
  switch (d) {                                                                                                         \
    case 32: return tn_launch<T, 32, 32>(A, Bm, w, S, s, BN, c, h, r, use_mult, st);                                   \
    case 64: return tn_launch<T, 64, 64>(A, Bm, w, S, s, BN, c, h, r, use_mult, st);                                   \
    case 128: return tn_launch<T, 128, 128>(A, Bm, w, S, s, BN, c, h, r, use_mult, st);                                \
    default: return -2;                                                                                                \
  }
  if (dtype == DT_BF16) { PR_TN_DISPATCH(bf16_t) }
  if (dtype == DT_F16) { PR_TN_DISPATCH(f16_t) }
#undef PR_TN_DISPATCH
  return -1;
}

}  // namespace pr
