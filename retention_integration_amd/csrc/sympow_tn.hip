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
// (y, xb) and all DV value columns, and contracts over the rows 32 at a time.  The phi tile is
// never stored: the A-operand of each matrix-core op is produced in registers as the product of a
// row-broadcast (DPP) of column x with the 16 columns 16*y..16*y+15, both read transposed from one
// row-major LDS tile.  s uses the identity s[(x, j)] = (A^T diag(w) A)[x, j], one extra matrix-core op
// per step.  Row tiles of A and B arrive through a 3-deep ring of asynchronous global->LDS copies.
#include "common.h"
#include "kernels.h"

namespace pr {

constexpr int TN_KT = 64;   // rows per pipeline stage (two contraction steps of 32)
constexpr int TN_NST = 3;   // stages in the ring

template <typename T, int X> struct PhiTile;
template <int X> struct PhiTile<bf16_t, X> {
  static __device__ __forceinline__ bf16x8 make(const bf16x8&, const bf16x8&, const float* rowf, const float* srcf) {
    float p[8];
#pragma unroll
    for (int r = 0; r < 8; r++) p[r] = mul_row_bcast<X>(srcf[r], rowf[r]);
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
  constexpr int NT = DV / 16, CA = DK / 8, CB = DV / 8;            // 16-byte chunks per row
  constexpr int A_BYTES = TN_KT * DK * 2, B_BYTES = TN_KT * DV * 2, W_BYTES = TN_KT * 4;
  constexpr int STAGE = A_BYTES + B_BYTES + W_BYTES;
  constexpr int LOADS = (TN_KT * CA + TN_KT * CB) / 256;           // copies per thread per stage (w rides on wave 0)
  const int tid = threadIdx.x, l = tid & 63, g = l >> 4;
  const int rows = c * r;
  const char* a_base = (const char*)(A + (long)bn * c * hA * DK);
  const char* b_base = (const char*)(Bm + (long)bn * c * hA * DV);
  const float* w_base = w + (long)bn * c * hA;
  auto row_index = [&](int row) -> long {   // element offset of a (clamped) folded row, per unit of the last dim
    row = min(row, rows - 1);
    const int t = row / r, rr = row - t * r;
    return (long)t * hA + hh * r + rr;
  };
  auto issue = [&](int step) {
    char* st = smem + (step % TN_NST) * STAGE;
    const int r0 = step * TN_KT;
    async_load_tile<CA, TN_KT>(st, [&](int row) { return a_base + row_index(r0 + row) * (DK * 2); });
    async_load_tile<CB, TN_KT>(st + A_BYTES, [&](int row) { return b_base + row_index(r0 + row) * (DV * 2); });
    if (HAS_W && tid < 64) async_copy4(w_base + row_index(r0 + tid), st + A_BYTES + B_BYTES);
  };

  f32x4 acc[XPW][NT];
#pragma unroll
  for (int i = 0; i < XPW; i++)
#pragma unroll
    for (int j = 0; j < NT; j++) acc[i][j] = (f32x4){0, 0, 0, 0};
  f32x4 sacc = {0, 0, 0, 0};

  const int steps = (rows + TN_KT - 1) / TN_KT;
  issue(0);
  if (steps > 1) issue(1);
  for (int step = 0; step < steps; step++) {
    char* st = smem + (step % TN_NST) * STAGE;
    if (step + 1 < steps) wait_vmcnt<LOADS>(); else wait_vmcnt<0>();
    if ((step + 1) * TN_KT > rows) zero_tile_rows<CA, TN_KT>(st, rows - step * TN_KT);
    lds_barrier();
    if (step + 2 < steps) issue(step + 2);
    if (active) {
      const float* wt = (const float*)(st + A_BYTES + B_BYTES);
#pragma unroll 1
      for (int ks = 0; ks < TN_KT / 32; ks++) {
        v8 kfy = sw_frag_tr<T, CA>(st, 32 * ks, 16 * y);
        v8 kfx = (xb == y) ? kfy : sw_frag_tr<T, CA>(st, 32 * ks, 16 * xb);
        v8 vf[NT];
#pragma unroll
        for (int nt = 0; nt < NT; nt++) vf[nt] = sw_frag_tr<T, CB>(st + A_BYTES, 32 * ks, 16 * nt);
        float rowf[8], srcf[8];
        unpack8(kfy, rowf);
        unpack8(kfx, srcf);
        if (HAS_W) {
          float sc[8];
          const float* wp = wt + 32 * ks + 8 * g;
#pragma unroll
          for (int q = 0; q < 8; q++) sc[q] = srcf[q] * wp[q];
          sacc = mfma16(kfy, pack8<T>(sc), sacc);
        } else {
          sacc = mfma16(kfy, kfx, sacc);
        }
        dpp_fence();  // srcf is read through DPP below
        static_for<XPW>([&](auto xi) {
          v8 a = PhiTile<T, PART * XPW + xi.value>::make(kfy, kfx, rowf, srcf);
#pragma unroll
          for (int nt = 0; nt < NT; nt++) acc[xi.value][nt] = mfma16(a, vf[nt], acc[xi.value][nt]);
        });
      }
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
  extern __shared__ __attribute__((aligned(1024))) char smem[];
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
  constexpr size_t smem = TN_NST * (TN_KT * DK * 2 + TN_KT * DV * 2 + TN_KT * 4);
  dim3 grid((TASKS + 3) / 4, (unsigned)(BN * h));
  if (w) {
    auto kern = sympow_tn_kernel<T, DK, DV, XPW, true>;
    allow_big_lds((const void*)kern, smem);
    hipLaunchKernelGGL(kern, grid, dim3(256), smem, st, (const T*)A, (const T*)Bm, w, (T*)S, s, c, h * r, r, h, use_mult);
  } else {
    auto kern = sympow_tn_kernel<T, DK, DV, XPW, false>;
    allow_big_lds((const void*)kern, smem);
    hipLaunchKernelGGL(kern, grid, dim3(256), smem, st, (const T*)A, (const T*)Bm, w, (T*)S, s, c, h * r, r, h, use_mult);
  }
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
