// dV and dK of update_state's backward (ref: retention/_update_state/reference.py:55-83) in ONE launch, for chunks of at
// most 128 rows.
//
// With one row block per (chunk, head) the two kernels -- sympow_nn (dV = phi(K) dS) and sympow_grad (dK through the
// feature map) -- each stream the whole gradient state dS of their pair once, and at d = 128 that stream (2.4 MB per
// pair, 19 GB at b=4, t=16384, h=16, chunk 128) is all they wait for: both run at the rate a plain copy reaches.  Here
// the two bodies are dealt to neighbouring workgroups of the same XCD, pair by pair: the two readers of a state start
// together, the one that runs ahead brings the state's lines into the XCD's L2 and the other finds them there, which
// holds it close behind -- the state comes from HBM once instead of twice.  (Side by side on two streams the two kernels
// do not pair up: measured, no gain.)  The bodies are the kernels' own, unchanged (sympow_nn_dev.h, sympow_grad_dev.h):
// every result is bit for bit that of the two launches.
#include "sympow_grad_dev.h"
#include "sympow_nn_dev.h"

namespace pr {

// Workgroups are handed to the 8 XCDs round-robin by linear id (id % 8); ids 8 apart are neighbours on one XCD.  Even
// slots of an XCD run dV, odd slots dK, of the same (chunk, head).
template <typename T, int DK, int MT, bool SYM>
__global__ __launch_bounds__(256, DK <= 64 ? 3 : 2) void sympow_dvdk_kernel(NNArgs na, GradArgs ga, int npairs) {
  const int xcd = blockIdx.x % 8, s = blockIdx.x / 8;
  const int vblock = (s >> 1) * 8 + xcd;   // the block id the body would have in a launch of its own (one row block per pair)
  // (ALONE = false: the state's copies are NOT marked non-temporal here -- the neighbour reads the same lines)
  if (s & 1) sympow_grad_body<T, DK, DK, MT, true, SYM, false>(ga, 1, npairs, vblock);
  else sympow_nn_body<T, DK, DK, MT, true, NN_EPI_PLAIN, SYM, false>(na, 1, npairs, vblock);
}

template <typename T, int DK, bool SYM>
static int dvdk_launch(const NNArgs& na_, const GradArgs& ga_, int BN, hipStream_t st) {
  NNArgs na = na_;
  GradArgs ga = ga_;
  if (!g_gate_skip) {   // every row block is swept and the scan's own output is read
    na.live_rows = nullptr, na.B_alt = nullptr;
    ga.live_rows = nullptr, ga.B_alt = nullptr;
  }
  const int rows = na.c * na.r, npairs = BN * na.h;
  auto go = [&](auto mt) {
    constexpr int MT = decltype(mt)::value;
    constexpr size_t ring_n = NN_NST * NN_FR * DK * 2, ring_g = GR_NST * GR_FR * DK * 2, mtile = (size_t)DK * (DK + 8) * 2;
    constexpr size_t ring = ring_n > ring_g ? ring_n : ring_g;
    constexpr size_t smem = ((ring > mtile ? ring : mtile) + 1023) / 1024 * 1024 + 64 * MT * DK * 2;
    dim3 grid((unsigned)(((npairs + 7) / 8) * 8 * 2));
    auto kern = sympow_dvdk_kernel<T, DK, MT, SYM>;
    allow_big_lds((const void*)kern, smem);
    PR_LAUNCH("sympow_dvdk", kern, grid, dim3(256), smem, st, na, ga, npairs);
  };
  if (rows > 64) go(IC<2>{});
  else go(IC<1>{});
  return (int)hipGetLastError();
}

// 1 where the one-launch form applies: a (chunk, head) is one row block of both kernels
int sympow_dvdk_ok(int c, int r) { return (long)c * r <= 128; }

// na: the arguments of sympow_nn's plain form with the key multiplier (dV), ga: those of sympow_grad with it (dK); both
// describe the same K, dS and chunk geometry.
int sympow_dvdk(const NNArgs& na, const GradArgs& ga, int BN, int d, int dtype, hipStream_t st) {
  if (!sympow_dvdk_ok(na.c, na.r) || na.c != ga.c || na.r != ga.r || na.h != ga.h) return -3;
#define PR_DK_D(T, DD)                                                                                                 \
  case DD:                                                                                                             \
    return (na.sym_diag && ga.sym_diag) ? dvdk_launch<T, DD, true>(na, ga, BN, st) : dvdk_launch<T, DD, false>(na, ga, BN, st);
#define PR_DK_T(T)                                                                                                     \
  switch (d) { PR_DK_D(T, 32) PR_DK_D(T, 64) PR_DK_D(T, 128) default: return -2; }
  if (dtype == DT_BF16) { PR_DK_T(bf16_t) }
  if (dtype == DT_F16) { PR_DK_T(f16_t) }
#undef PR_DK_T
#undef PR_DK_D
  return -1;
}

}  // namespace pr
