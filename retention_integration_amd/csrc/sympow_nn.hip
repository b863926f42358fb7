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
// A workgroup = 4 waves owns 64*MT rows; each wave 16*MT rows and all DV columns.  B streams through a
// 2-deep ring of asynchronous global->LDS copies in its memory order, 64 features (four x columns of one
// 16-wide y strip) per stage, and is read with the transposing LDS load; the phi operand is built in
// registers from the wave's own rows (one scalar x[X] times eight x[16y+..] values per lane).
// aux is a quadratic form, aux[row] = x_row^T M x_row with M[a, b] = sB[f(a, b)] on the stored pairs, so it
// costs one small d x d product per row tile instead of an extra column in every step.
// Row blocks that share a state are placed on the same XCD (one HBM fetch, L2 re-reads).
#include "sympow_nn_dev.h"

namespace pr {

template <typename T, int DK, int DV, bool MULT, int EPI, bool SYM>
static int nn_launch(const NNArgs& a_, int BN, hipStream_t st) {
  NNArgs a = a_;
  if (!g_gate_skip) {   // every row block is swept and the scan's own output is read
    a.live_rows = nullptr;
    a.B_alt = nullptr;
  }
  const int rows = a.c * a.r, npairs = BN * a.h;
  auto go = [&](auto mt, auto alone_c) {
    constexpr int MT = decltype(mt)::value;
    constexpr bool ALONE = decltype(alone_c)::value != 0;
    constexpr size_t ring = NN_NST * NN_FR * DV * 2, mtile = (size_t)DK * (DK + 8) * 2;
    constexpr size_t smem = ((ring > mtile ? ring : mtile) + 1023) / 1024 * 1024 + 64 * MT * DK * 2;
    const int row_blocks = (rows + 64 * MT - 1) / (64 * MT);
    dim3 grid((unsigned)(((npairs + 7) / 8) * 8 * row_blocks));
    auto kern = sympow_nn_kernel<T, DK, DV, MT, MULT, EPI, SYM, ALONE>;
    allow_big_lds((const void*)kern, smem);
    PR_LAUNCH("sympow_nn", kern, grid, dim3(256), smem, st, a, row_blocks, npairs);
  };
  if constexpr (DK <= 64) {
    if (rows >= 256) { go(IC<4>{}, IC<0>{}); return (int)hipGetLastError(); }
  }
  if (rows > 128) go(IC<2>{}, IC<0>{});
  else if (rows > 64) go(IC<2>{}, IC<1>{});
  else go(IC<1>{}, IC<1>{});
  return (int)hipGetLastError();
}

int sympow_nn(const NNArgs& a, int BN, int d, int mult, int epi, int dtype, hipStream_t st) {
  // two forms exist: the merge epilogue without the multiplier (query_state forward) and the plain epilogue with it
  // (update_state's dV)
  if ((epi == NN_EPI_MERGE) == (mult != 0)) return -1;
#define PR_NN_D(T, DD)                                                                                                 \
  case DD:                                                                                                             \
    if (a.sym_diag) {                                                                                                  \
      if (epi == NN_EPI_MERGE) return nn_launch<T, DD, DD, false, NN_EPI_MERGE, true>(a, BN, st);                     \
      return nn_launch<T, DD, DD, true, NN_EPI_PLAIN, true>(a, BN, st);                                               \
    }                                                                                                                  \
    if (epi == NN_EPI_MERGE) return nn_launch<T, DD, DD, false, NN_EPI_MERGE, false>(a, BN, st);                      \
    return nn_launch<T, DD, DD, true, NN_EPI_PLAIN, false>(a, BN, st);
#define PR_NN_T(T)                                                                                                     \
  switch (d) { PR_NN_D(T, 32) PR_NN_D(T, 64) PR_NN_D(T, 128) default: return -2; }
  if (dtype == DT_BF16) { PR_NN_T(bf16_t) }
  if (dtype == DT_F16) { PR_NN_T(f16_t) }
#undef PR_NN_T
#undef PR_NN_D
  return -1;
}

}  // namespace pr
