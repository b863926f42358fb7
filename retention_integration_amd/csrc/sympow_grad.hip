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
// dphi is never stored.  A workgroup = 4 waves owns 64*MT rows (16*MT per wave) and sweeps B in memory order,
// 64 feature rows (four x columns of one 16-wide strip y) per pipeline stage, through a 2-deep ring of
// asynchronous global->LDS copies.  For an x column X the wave forms the 16x16 tile dphi^T[i, row] on the matrix
// cores (B rows from LDS as the A operand, G^T from registers as the B operand) and folds it twice:
//   * into dX[row, 16y+i]: multiply by the per-row scalar X[row, X] and accumulate (VALU);
//   * into dX[row, X]: multiply elementwise by X[row, 16y+i], round to 16 bit and sum over i on the matrix
//     cores with a 0/1 selector operand that routes the sum of column X to accumulator row X % 16.
// Both land in the same accumulator layout (coordinate on the accumulator rows, workgroup row on the lanes), so
// the result never leaves registers.  The sB term is linear in X: dX_s = cvec * (X M) with the symmetric d x d
// matrix M[a, b] = sum of m_f sB[f] over the stored features pairing a and b; it is one small product at the end.
// Workgroups that share a state (the row blocks of one (chunk, head)) are placed on the same XCD so that the
// state is fetched from HBM once and re-read from that XCD's L2.
#include "sympow_grad_dev.h"

namespace pr {

template <typename T, int DK, int DV, bool MULT, bool SYM>
static int grad_launch(const GradArgs& a_, int BN, hipStream_t st) {
  GradArgs a = a_;
  if (!g_gate_skip) {   // every row block is swept and the scan's own output is read
    a.live_rows = nullptr;
    a.B_alt = nullptr;
  }
  const int rows = a.c * a.r, npairs = BN * a.h;
  auto go = [&](auto mt, auto alone_c) {
    constexpr int MT = decltype(mt)::value;
    constexpr bool ALONE = decltype(alone_c)::value != 0;
    constexpr size_t ring = GR_NST * GR_FR * DV * 2, mtile = (size_t)DK * (DK + 8) * 2;
    constexpr size_t smem = ((ring > mtile ? ring : mtile) + 1023) / 1024 * 1024 + 64 * MT * DK * 2;
    const int row_blocks = (rows + 64 * MT - 1) / (64 * MT);
    dim3 grid((unsigned)(((npairs + 7) / 8) * 8 * row_blocks));
    auto kern = sympow_grad_kernel<T, DK, DV, MT, MULT, SYM, ALONE>;
    allow_big_lds((const void*)kern, smem);
    PR_LAUNCH("sympow_grad", kern, grid, dim3(256), smem, st, a, row_blocks, npairs);
  };
  // 128 rows per workgroup.  Up to d = 64 that is four workgroups (16 waves) per compute unit, and the vector
  // instructions of the two folds issue at twice the rate of a 256-row tiling at two workgroups (measured 7 %
  // faster at d = 64 although a state tile is reused half as often, equal at d = 32).  At d = 128 a workgroup
  // streams the whole 2.4 MB state from L2, and 128 rows instead of 64 halve that traffic (27 % faster).
  if (rows > 128) go(IC<2>{}, IC<0>{});
  else if (rows > 64) go(IC<2>{}, IC<1>{});
  else go(IC<1>{}, IC<1>{});
  return (int)hipGetLastError();
}

int sympow_grad(const GradArgs& a, int BN, int d, int mult, int dtype, hipStream_t st) {
#define PR_G_D(T, DD)                                                                                                  \
  case DD:                                                                                                             \
    if (a.sym_diag) return mult ? grad_launch<T, DD, DD, true, true>(a, BN, st) : grad_launch<T, DD, DD, false, true>(a, BN, st); \
    return mult ? grad_launch<T, DD, DD, true, false>(a, BN, st) : grad_launch<T, DD, DD, false, false>(a, BN, st);
#define PR_G_T(T)                                                                                                      \
  switch (d) { PR_G_D(T, 32) PR_G_D(T, 64) PR_G_D(T, 128) default: return -2; }
  if (dtype == DT_BF16) { PR_G_T(bf16_t) }
  if (dtype == DT_F16) { PR_G_T(f16_t) }
#undef PR_G_T
#undef PR_G_D
  return -1;
}

}  // namespace pr
