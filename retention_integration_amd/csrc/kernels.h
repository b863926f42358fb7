// Host-side entry points of the kernel translation units and their argument blocks.
#pragma once
#include <hip/hip_runtime.h>

namespace pr {

// 1 (default): kernels leave out work whose every term the gates have decayed to an exact zero (pr_set_gate_skipping)
extern int g_gate_skip;

// discumsum.hip
int discumsum_fwd(const void* X, const float* logG, void* Y, int B, int n, int n_out, int H, long F, int dtype,
                  hipStream_t st);
int discumsum_bwd(const void* dY, const void* Y, const float* logG, void* dX, float* dlogG, float* partial, int B,
                  int n, int n_out, int H, long F, int dtype, hipStream_t st);
// the state and its fp32 key sums (same gates) in one launch each way; dlogG is the sum of both contributions.
// ScanCarry (all optional) connects a scan to the calls before and after it:
//   forward:  in / in2 [B, H, F / F2]: the value the scan starts from (Y[0] = in instead of 0);
//             out / out2: receive entry n of the scan when the tensors keep n entries (n_out == n);
//   backward: in / in2: the gradient of that entry n;  out / out2: receive the gradient of the starting value.
struct ScanCarry {
  const void* in = nullptr;
  const float* in2 = nullptr;
  void* out = nullptr;
  float* out2 = nullptr;
};
// consumers_follow_gates != 0 (both directions; only without a ScanCarry and with n_out == n): the caller promises that
// whoever reads entry k of the scan's output reads the scan's input instead wherever the two are equal because the
// carry into it is an exact zero (forward: Y[k] = X[k-1] when exp(logG[k-1]) == 0 or k == 1; backward: dX[k] = dY[k+1]
// when exp(logG[k+1]) == 0).  A (batch, head) whose every factor exp(logG[k]), k >= 1, is zero is then not scanned at
// all: nothing of it is read or written (backward: its gate gradient is written as zero).
int discumsum_pair_fwd(const void* X, const float* X2, const float* logG, void* Y, float* Y2, int B, int n, int n_out,
                       int H, long F, long F2, const ScanCarry& cy, int consumers_follow_gates, int dtype,
                       hipStream_t st);
long discumsum_pair_bwd_workspace_floats(int B, int n, int H, long F, long F2);
int discumsum_pair_bwd(const void* dY, const void* Y, const float* dY2, const float* Y2, const float* logG, void* dX,
                       float* dX2, float* dlogG, float* partial, int B, int n, int n_out, int H, long F, long F2,
                       const ScanCarry& cy, int consumers_follow_gates, int dtype, hipStream_t st);
long discumsum_bwd_workspace_floats(int B, int n, int H, long F, int dtype);
// gate gradient of the pair of scans from the scans Y, Y2 and the already formed input gradients R, R2 ([B,n,H,*])
long scan_gate_grad_workspace_floats(int B, int n, int H, long F, long F2);
int scan_gate_grad(const void* Y, const void* R, const float* Y2, const float* R2, const float* logG, float* dlogG,
                   float* partial, int B, int n, int H, long F, long F2, int dtype, hipStream_t st);

// sympow_tn.hip: A [BN,c,h*r,d], Bm [BN,c,h*r,d], w [BN,c,h*r] or null -> S [BN,h,D,d], s [BN,h,D]
// skip: 0 = every chunk; +n = the last chunk of every n is not computed and its S, s are left unwritten (nobody reads
// them); -n = the first chunk of every n is not computed and its S, s are written as zeros.
// live [BN, h, 2] or null: per (chunk, kv head) {first time step whose A rows are not all zero, end of the time steps
// whose Bm rows are not all zero} (chunk_prep_fwd writes them from the gates); live_side 0 / 1 says which of the two
// holds for this call's operands: the stages of rows outside it are not read.
int sympow_tn(const void* A, const void* Bm, const float* w, void* S, float* s, int BN, int c, int h, int r, int d,
              int use_mult, int skip, const int* live, int live_side, int dtype, hipStream_t st);
// The same contraction chained with the gated scan over the n chunks of a batch element (A, Bm [B,n*c,h*r,d],
// lcs [B,n,h] or null): entry k of S, s [B*n,h,D,*] is the scan's k-th value (forward) or the scan's input gradient
// (reverse).  sympow_tn_chain_ok: 0 = shape not supported, 1 = supported, 2 = and enough independent work to pay.
int sympow_tn_chain_ok(int B, int n, int c, int h, int r, int d);
int sympow_tn_chain(const void* A, const void* Bm, const float* w, const float* lcs, void* S, float* s, int B, int n,
                    int c, int h, int r, int d, int use_mult, int reverse, int dtype, hipStream_t st);

// sympow_nn.hip
enum { NN_EPI_PLAIN = 0, NN_EPI_MERGE = 1 };
struct NNArgs {
  const void* X;        // [BN, c, h*r, d]
  const void* B;        // [BN, h, D, d]
  const float* sB;      // [BN, h, D] or null
  void* out;            // [BN, c, h*r, d]
  float* den;           // [BN, c, h*r]   (merge only)
  const void* Y_attn;   // [BN, c, h*r, d] or null
  const float* l_attn;  // [BN, c, h*r]
  const float* rowmax;  // [BN, c, h*r]
  float scale_p;        // scale^deg
  int c, h, r, n;       // n: chunks per batch entry
  int skip_first;       // chunk 0 of every batch entry has a zero state
  int skip_last;        // chunk n-1 of every batch entry has a zero B: the output there is zero (nothing is read)
  int sym_diag;         // B[(a, b)] == B[(b, a)] in the blocks on the diagonal (the caller's promise): the mirrored
                        // quarter of every such block is not read
  const float* qgate;   // [BN, c, h] or null (merge only): log of a factor on the state part of every row of a kv head
                        // at a position -- out and den are those of X * exp(qgate / 2) without forming that product
  const int* live_rows = nullptr;   // [BN, h, 2] or null (plain only): X rows before time step live_rows[bn, hh, 0] are
                                    // exact zeros (chunk_prep_fwd writes it); their output is zero and is not computed
  // Optional stand-in for B (plain only; all null otherwise).  B is the output of the reverse gated scan over the
  // chunks, whose entry bn equals the scan's INPUT entry bn + 1 exactly when the carry exp(carry[bn + 1, hh]) is zero:
  // the kernel then reads B_alt[bn + 1] (and the scan need not have written B[bn]; see discumsum_pair_bwd).
  const void* B_alt = nullptr;      // [BN, h, D, d]
  const float* carry = nullptr;     // [BN, h] log of the scan's factors
};
int sympow_nn(const NNArgs& a, int BN, int d, int mult, int epi, int dtype, hipStream_t st);

// chunk_fwd.hip: attention inside every chunk, the query of the chunk's starting state and their merge, in one kernel
struct ChunkFwdArgs {
  const void* Q;     // [BN, c, h*r, d]  (ungated)
  const void* K;     // [BN, c, h, d]
  const void* V;     // [BN, c, h, d]
  const float* G;    // [BN, c, h] accumulated log gates inside the chunk, or null
  const void* S;     // [BN, h, D, d]   state at the start of each chunk, symmetric in the diagonal blocks
  const float* s;    // [BN, h, D]
  void* O;           // [BN, c, h*r, d]
  float* rowmax;     // [BN, c, h*r]  log of the largest attention weight of the row
  float* den;        // [BN, c, h*r]  normaliser, in the units sympow_nn's merge writes
  int c, h, r, n;    // n: chunks per batch entry
  float scale;
  int skip_first;    // chunk 0 of every batch entry has a zero state (not read)
  int gate_skip;     // leave out what the gates have decayed to exact zeros (key tiles, the state sweep of a row block)
  // Optional stand-ins for S, s (null otherwise): the per-chunk sums that the forward scan turned into S, s.  Entry bn of
  // the scan equals entry bn - 1 of its input exactly when the carry exp(carry[bn - 1, hh]) is zero (or, with
  // skip_first, bn - 1 is the first chunk of its batch entry): the kernel then reads S_alt[bn - 1], s_alt[bn - 1].
  const void* S_alt = nullptr;
  const float* s_alt = nullptr;
  const float* carry = nullptr;   // [BN, h]
};
int chunk_fwd_supported(int d, int dtype);
int chunk_fwd(const ChunkFwdArgs& a, int BN, int d, int dtype, hipStream_t st);

// chunk_bwd_dq.hip: the query side of the chunked backward in one kernel (attention dQ/dGq + the state path's dQ)
struct ChunkBwdDqArgs {
  const void* Q;          // [BN, c, h*r, d] (ungated)
  const void* K;          // [BN, c, h, d]
  const void* V;          // [BN, c, h, d]
  const float* G;         // [BN, c, h] accumulated log gates inside the chunk, or null
  const float* rowmax;    // [BN, c, h*r]   from the forward
  const float* den;       // [BN, c, h*r]   from the forward
  const void* dO;         // [BN, c, h*r, d]
  const float* dl;        // [BN, c, h*r]   gradient of the attention part's row sum (row-wise preparation)
  const float* dO_scale;  // [BN, c, h*r]   factor on dO for the attention part (row-wise preparation)
  const float* cvec;      // [BN, c, h*r]   factor of the key-sum term of the state part (row-wise preparation)
  const void* S;          // [BN, h, D, d]  states at the start of each chunk, symmetric in the diagonal blocks
  const float* s;         // [BN, h, D]
  void* dQ;               // [BN, c, h*r, d]
  float* dGq;             // [BN, c, h*r] or null
  int c, h, r, n;         // n: chunks per batch entry
  float scale;
  int skip_first;         // chunk 0 of every batch entry has a zero state (not read)
  int gate_skip;          // leave out what the gates have decayed to exact zeros (key tiles, the state sweep of a row block)
  const void* S_alt = nullptr;    // stand-ins for S, s as in ChunkFwdArgs
  const float* s_alt = nullptr;
  const float* carry = nullptr;
};
int chunk_bwd_dq_supported(int d, int dtype);
int chunk_bwd_dq(const ChunkBwdDqArgs& a, int BN, int d, int dtype, hipStream_t st);

// sympow_grad.hip
struct GradArgs {
  const void* X;      // [BN, c, h*r, d]
  const void* G;      // [BN, c, h*r, d]
  const float* cvec;  // [BN, c, h*r] or null (= 1)
  const void* B;      // [BN, h, D, d]
  const float* sB;    // [BN, h, D]
  void* dX;           // [BN, c, h*r, d]
  int c, h, r, n;
  int skip_first;     // bit 0: chunk 0 of every batch entry has a zero state, bit 1: chunk n-1 has a zero B: dX = 0
                      // there and nothing is read
  int sym_diag;       // B[(a, b)] == B[(b, a)] in the blocks on the diagonal (the caller's promise)
  // [BN, h, 2] or null (chunk_prep_fwd writes it): live_side 0 -- X rows before time step live_rows[bn, hh, 0] are exact
  // zeros; live_side 1 -- G rows and cvec from time step live_rows[bn, hh, 1] on are.  dX is zero there, not computed.
  const int* live_rows = nullptr;
  int live_side = 0;
  // Optional stand-ins for B, sB as in NNArgs (alt_shift = +1: B is a reverse scan's output and B_alt its input; -1: B
  // is a forward scan's output, whose entry bn equals the input entry bn - 1 when exp(carry[bn - 1, hh]) is zero or,
  // with bit 0 of skip_first, bn - 1 is the first chunk of its batch entry).
  const void* B_alt = nullptr;
  const float* sB_alt = nullptr;
  const float* carry = nullptr;
  int alt_shift = 0;
};
int sympow_grad(const GradArgs& a, int BN, int d, int mult, int dtype, hipStream_t st);

// sympow_dvdk.hip: sympow_nn's plain form (dV) and sympow_grad (dK), both with the key multiplier, of the same K and dS
// in one launch, for chunks that are one row block of either (sympow_dvdk_ok): their workgroups are dealt pair by pair
// to one XCD, so that the state both stream comes from HBM once.  Results are those of the two launches, bit for bit.
int sympow_dvdk_ok(int c, int r);
int sympow_dvdk(const NNArgs& na, const GradArgs& ga, int BN, int d, int dtype, hipStream_t st);

// attention_fwd.hip / attention_bwd.hip
struct AttnFwdArgs {
  const void* Q;    // [B, tq, h*r, d]
  const void* K;    // [B, tk, h, d]
  const void* V;    // [B, tk, h, d]
  const float* G;   // [B, tk, h] accumulated log gate, or null
  void* O;          // [B, tq, h*r, d]
  float* l;         // [B, tq, h*r]
  float* rowmax;    // [B, tq, h*r]
  int tq, tk, h, r;
  float scale, deg;
  int norm;
  int kv_rows;      // rows per batch entry of the K, V, G buffers (tk for dense tensors, the capacity of a cache)
};
int attention_fwd(const AttnFwdArgs& a, int B, int d, int dtype, hipStream_t st);
struct AttnBwdArgs {
  const void* Q;        // [B, tq, h*r, d]
  const void* K;        // [B, tk, h, d]
  const void* V;        // [B, tk, h, d]
  const float* G;       // [B, tk, h] or null
  const float* rowmax;  // [B, tq, h*r]
  const void* dO;       // [B, tq, h*r, d]
  const float* dl;      // [B, tq, h*r] or null
  const float* dO_scale;  // [B, tq, h*r] or null: dO is used as dO * dO_scale[row] (scaled in fp32)
  void* dQ;             // [B, tq, h*r, d]
  void* dK;             // [B, tk, h, d]
  void* dV;             // [B, tk, h, d]
  float* dGq;           // [B, tq, h*r]   (only when G)
  float* dGk;           // [B, tk, h]     (only when G; already negated)
  int tq, tk, h, r;
  float scale, deg;
  // optional epilogue of the chunked algorithm (all null otherwise): gradients that arrive through the gated
  // copies Q*exp(G/deg) and K*exp((G_last - G)/deg) and the value gradient of the state path
  const void* dQs;      // [B, tq, h*r, d]: dQ = dQ_attn + dQs * exp(G_q/deg);  dGq += (Q.dQs) exp(G_q/deg) / deg
  const void* dKs;      // [B, tk, h, d]:   dK = dK_attn + dKs * w, w = exp((G_last - G_k)/deg); dGk -= (K.dKs) w / deg
  const void* dVs;      // [B, tk, h, d]:   dV = dV_attn + dVs
  float* dotk;          // [B, tk, h]:      (K.dKs) w
  int dQs_plain;        // dQs is already the gradient w.r.t. Q itself: dQ = dQ_attn + dQs, dGq += (Q.dQs) / deg
  // [B, h, 2] or null (chunk_prep_fwd writes it): dKs and dVs are zero at the keys before time step live_rows[b, hh, 0]
  // and need not have been written before the last multiple of 256 below it -- a key block of such keys reads neither
  const int* live_rows = nullptr;
};
int attention_bwd(const AttnBwdArgs& a, int B, int d, int dtype, hipStream_t st);

// elementwise.hip
// qgate [rows / (h*r), h] or null: the forward's log factor on the state part (see NNArgs); rows are (.., position, h*r)
// live_rows [rows / (c*h*r), h, 2] or null (with chunks of c positions; chunk_prep_fwd writes it): the rows of dOs from
// the first multiple of 256 positions at or after live_rows[.., 1] on are left unwritten -- only for a reader that
// stops there (sympow_tn with live_side 1); ignored while gate skipping is switched off
int qs_bwd_prep(const void* O, const void* dO, const float* den, const float* rowmax, const float* qgate, void* dOs,
                float* cvec, void* dY_attn, float* dl_attn, float* dY_scale, long rows, int h, int r, int d, float scale_p,
                const int* live_rows, int c, int dtype, hipStream_t st);

// chunk_glue.hip (return -5: chunk longer than the LDS-resident gate vector allows)
int gate_cumsum(const float* logG, float* A, int B, int t, int h, hipStream_t st);
// (Qg may be null: the gated queries are then not formed)
// live [BN, h, 2] or null: receives, per (chunk, kv head), the first time step whose discounted key is not zeroed by
// its factor exp((A_last - A_t) / deg), and one past the last time step whose factor exp(A_t) on the state part of a
// query is not zero (written with the sums, i.e. when logG is given).  Given WITHOUT logG it is an input: the caller's
// promise that every reader of Kd leaves out the time steps before live[bn, hh, 0] (as sympow_tn, sympow_nn and
// sympow_grad do when handed the same array); those rows of Kd, exact zeros, are then not written
// (up to the block of 256 rows that holds the first live one).
int chunk_prep_fwd(const float* logG, const void* K, const void* Q, float* A, float* lcs, void* Kd, void* Qg, int* live,
                   int BN, int c, int h, int r, int d, int deg, int dtype, hipStream_t st);
int chunk_gate_scan_bwd(float* dA, const float* dGq, const float* dotk, const float* dlcs_a, const float* dlcs_b, int BN,
                        int c, int h, int r, int deg, hipStream_t st);

// cache.hip
int cache_append(void* Kc, void* Vc, float* Ac, const void* k, const void* v, const float* g, float* a_last, int B,
                 int cap, int pos, int t_new, int h, int d, int dtype, hipStream_t st);

// decode.hip (return -3: more than 16 query rows per (batch, kv head))
long decode_workspace_floats(int B, int h, int r, int tq, int d);
int decode_step(const void* Q, const float* gq, const void* S, const float* s, const void* Y_attn, const float* l_attn,
                const float* rowmax, const void* Knew, const void* Vnew, const float* decay, void* Sout, float* sout,
                void* out, float* workspace, int B, int tq, int h, int r, int d, int deg, float scale_p, int dtype,
                int attend_new, hipStream_t st);

// the same step with its partial sums in a per-GPU array of the library (return -6: the step needs more than
// decode_static_floats() floats of partial sums; -7: the stream belongs to another GPU than the current one).
// decode_static_prepare() takes the array's address on the current GPU ahead of the first step (0 or a hipError_t).
long decode_static_floats();
int decode_static_prepare();
int decode_step_static(const void* Q, const float* gq, const void* S, const float* s, const void* Y_attn,
                       const float* l_attn, const float* rowmax, const void* Knew, const void* Vnew,
                       const float* decay, void* Sout, float* sout, void* out, int B, int tq, int h, int r, int d,
                       int deg, float scale_p, int dtype, int attend_new, hipStream_t st);

}  // namespace pr
