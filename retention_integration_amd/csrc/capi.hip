// extern "C" surface of libpower_retention_hip.so: argument checks and dispatch only.
#include "../../include/power_retention_hip.h"

#include <cstdarg>
#include <cstdio>

#include "common.h"
#include "kernels.h"


namespace pr {
launch_hook_t g_launch_hook = nullptr;
void* g_launch_hook_user = nullptr;
int g_gate_skip = 1;
}  // namespace pr

namespace {
thread_local char g_err[256] = "";
int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}
bool bad_ptr(const void* p) { return p == nullptr || (reinterpret_cast<uintptr_t>(p) & 15u) != 0; }
bool bad_opt(const void* p) { return p != nullptr && (reinterpret_cast<uintptr_t>(p) & 15u) != 0; }
int finish(int rc, const char* what) {
  if (rc == 0) return 0;
  if (rc == -1) return fail(PR_ERR_DTYPE, "%s: unsupported dtype", what);
  if (rc == -2) return fail(PR_ERR_HEAD_DIM, "%s: head dim must be 32, 64 or 128", what);
  if (rc == -5) return fail(PR_ERR_ARG, "%s: chunk longer than 8192 is not supported", what);
  return fail(rc, "%s: launch failed: %s", what, hipGetErrorString((hipError_t)rc));
}
int check_common(const char* what, int d, int deg, int dtype, bool state) {
  if (state && deg != 2) return fail(PR_ERR_DEG, "%s: only deg=2 has a state layout (got %d)", what, deg);
  if (!state && (deg <= 0 || deg % 2 != 0)) return fail(PR_ERR_DEG, "%s: deg must be a positive even integer (got %d)", what, deg);
  if (dtype != PR_BF16 && dtype != PR_F16) return fail(PR_ERR_DTYPE, "%s: dtype must be bf16 or fp16", what);
  if (d != 32 && d != 64 && d != 128) return fail(PR_ERR_HEAD_DIM, "%s: head dim must be 32, 64 or 128 (got %d)", what, d);
  return 0;
}
size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }
}  // namespace

extern "C" {

int pr_abi_version(void) { return 9; }

void pr_set_launch_hook(pr_launch_hook_t hook, void* user) {
  pr::g_launch_hook = nullptr;   // (never a new hook with the old user pointer)
  pr::g_launch_hook_user = user;
  pr::g_launch_hook = hook;
}
void pr_set_gate_skipping(int on) { pr::g_gate_skip = on ? 1 : 0; }
int pr_get_gate_skipping(void) { return pr::g_gate_skip; }
const char* pr_last_error(void) { return g_err; }

int pr_expanded_dim(int d, int deg) {
  if (deg != 2 || d <= 0 || d % 16 != 0) return -1;
  return pr::expanded_dim(d);
}

int pr_attention_fwd(const void* Q, const void* K, const void* V, const float* G, void* O, float* l, float* rowmax,
                     int B, int tq, int tk, int h, int r, int d, float scale, int deg, int norm, int dtype,
                     void* stream) {
  if (int rc = check_common("attention_fwd", d, deg, dtype, false)) return rc;
  if (bad_ptr(Q) || bad_ptr(K) || bad_ptr(V) || bad_ptr(O) || bad_opt(G) || bad_opt(l) || bad_opt(rowmax))
    return fail(PR_ERR_ARG, "attention_fwd: null or misaligned pointer");
  if (!norm && (!l || !rowmax)) return fail(PR_ERR_ARG, "attention_fwd: l and rowmax are required when norm == 0");
  if (B <= 0 || tq <= 0 || tk <= 0 || h <= 0 || r <= 0 || tq > tk)
    return fail(PR_ERR_ARG, "attention_fwd: need B,tq,tk,h,r > 0 and tq <= tk (got %d %d %d %d %d)", B, tq, tk, h, r);
  pr::AttnFwdArgs a{Q, K, V, G, O, l, rowmax, tq, tk, h, r, scale, (float)deg, norm, tk};
  return finish(pr::attention_fwd(a, B, d, dtype, (hipStream_t)stream), "attention_fwd");
}

int pr_attention_bwd(const void* Q, const void* K, const void* V, const float* G, const float* rowmax,
                     const void* dO, const float* dl, const float* dO_scale, void* dQ, void* dK, void* dV,
                     float* dGq, float* dGk, int B, int tq, int tk, int h, int r, int d, float scale, int deg,
                     int dtype, void* stream) {
  if (int rc = check_common("attention_bwd", d, deg, dtype, false)) return rc;
  if (bad_ptr(Q) || bad_ptr(K) || bad_ptr(V) || bad_ptr(rowmax) || bad_ptr(dO) || bad_opt(dQ) || bad_opt(dK) ||
      bad_opt(dV) || bad_opt(G) || bad_opt(dl) || bad_opt(dGq) || bad_opt(dGk))
    return fail(PR_ERR_ARG, "attention_bwd: null or misaligned pointer");
  if ((dK == nullptr) != (dV == nullptr) || (!dQ && !dK))
    return fail(PR_ERR_ARG, "attention_bwd: ask for dQ, for dK and dV, or for all three");
  if (G && ((dQ && !dGq) || (dK && !dGk)))
    return fail(PR_ERR_ARG, "attention_bwd: dGq (with dQ) and dGk (with dK, dV) are required when G is given");
  if (B <= 0 || tq <= 0 || tk <= 0 || h <= 0 || r <= 0 || tq > tk)
    return fail(PR_ERR_ARG, "attention_bwd: need B,tq,tk,h,r > 0 and tq <= tk");
  pr::AttnBwdArgs a{Q, K, V, G, rowmax, dO, dl, dO_scale, dQ, dK, dV, G ? dGq : nullptr, G ? dGk : nullptr,
                    tq, tk, h, r, scale, (float)deg, nullptr, nullptr, nullptr, nullptr, 0};
  return finish(pr::attention_bwd(a, B, d, dtype, (hipStream_t)stream), "attention_bwd");
}

int pr_chunk_attention_bwd(const void* Q, const void* K, const void* V, const float* A, const float* rowmax,
                           const void* dO, const float* dl, const float* dO_scale, const void* dQ_state,
                           const void* dK_state, const void* dV_state, const int* live_rows, void* dQ, void* dK, void* dV,
                           float* dGq, float* dGk, float* dotk, int BN, int c, int h, int r, int d, float scale, int deg,
                           int dQ_state_plain, int dtype, void* stream) {
  if (int rc = check_common("chunk_attention_bwd", d, deg, dtype, false)) return rc;
  if (bad_ptr(Q) || bad_ptr(K) || bad_ptr(V) || bad_ptr(rowmax) || bad_ptr(dO) || bad_opt(dQ) || bad_opt(dK) ||
      bad_opt(dV) || bad_opt(dQ_state) || bad_opt(dK_state) || bad_opt(dV_state) || bad_opt(A) || bad_opt(dl) ||
      bad_opt(dO_scale) || bad_opt(dGq) || bad_opt(dGk) || bad_opt(dotk))
    return fail(PR_ERR_ARG, "chunk_attention_bwd: null or misaligned pointer");
  if ((dK == nullptr) != (dV == nullptr) || (!dQ && !dK))
    return fail(PR_ERR_ARG, "chunk_attention_bwd: ask for dQ, for dK and dV, or for all three");
  if ((dQ && !dQ_state) || (dK && (!dK_state || !dV_state)))
    return fail(PR_ERR_ARG, "chunk_attention_bwd: the state-path gradients of the requested outputs are required");
  if (A && ((dQ && !dGq) || (dK && (!dGk || !dotk))))
    return fail(PR_ERR_ARG, "chunk_attention_bwd: dGq (with dQ), dGk and dotk (with dK, dV) are required when A is given");
  if (BN <= 0 || c <= 0 || h <= 0 || r <= 0) return fail(PR_ERR_ARG, "chunk_attention_bwd: need BN,c,h,r > 0");
  pr::AttnBwdArgs a{Q, K, V, A, rowmax, dO, dl, dO_scale, dQ, dK, dV, A ? dGq : nullptr, A ? dGk : nullptr,
                    c, c, h, r, scale, (float)deg, dQ_state, dK_state, dV_state, A ? dotk : nullptr, dQ_state_plain ? 1 : 0};
  if (live_rows && (!A || !dK)) return fail(PR_ERR_ARG, "chunk_attention_bwd: live_rows describes the gates' effect on dK_state and dV_state");
  a.live_rows = live_rows;
  return finish(pr::attention_bwd(a, BN, d, dtype, (hipStream_t)stream), "chunk_attention_bwd");
}

int pr_update_state_fwd(const void* K, const void* V, void* S, float* s, const int* live_rows, int BN, int c, int h,
                        int d, int deg, int skip_last_of, int dtype, void* stream) {
  if (int rc = check_common("update_state_fwd", d, deg, dtype, true)) return rc;
  if (bad_ptr(K) || bad_ptr(V) || bad_ptr(S) || bad_ptr(s)) return fail(PR_ERR_ARG, "update_state_fwd: null or misaligned pointer");
  if (BN <= 0 || c <= 0 || h <= 0) return fail(PR_ERR_ARG, "update_state_fwd: need BN,c,h > 0");
  if (skip_last_of < 0 || (skip_last_of > 0 && BN % skip_last_of != 0))
    return fail(PR_ERR_ARG, "update_state_fwd: skip_last_of must be 0 or a divisor of BN (got %d, BN %d)", skip_last_of, BN);
  return finish(pr::sympow_tn(K, V, nullptr, S, s, BN, c, h, 1, d, 1, skip_last_of, live_rows, 0, dtype, (hipStream_t)stream),
                "update_state_fwd");
}

int pr_update_state_bwd(const void* K, const void* V, const void* dS, const float* ds, const void* dS_scan_in,
                        const float* ds_scan_in, const float* scan_log_G, const int* live_rows, void* dK, void* dV,
                        int BN, int c, int h, int d, int deg, int dS_symmetric, int zero_last_of, int dtype,
                        void* stream) {
  if (int rc = check_common("update_state_bwd", d, deg, dtype, true)) return rc;
  if (bad_ptr(K) || bad_ptr(V) || bad_ptr(dS) || bad_ptr(ds) || bad_opt(dK) || bad_opt(dV) || (!dK && !dV) ||
      bad_opt(dS_scan_in))
    return fail(PR_ERR_ARG, "update_state_bwd: null or misaligned pointer");
  if ((dS_scan_in != nullptr) != (ds_scan_in != nullptr) || (dS_scan_in != nullptr) != (scan_log_G != nullptr))
    return fail(PR_ERR_ARG, "update_state_bwd: dS_scan_in, ds_scan_in and scan_log_G come together");
  if (dS_scan_in && zero_last_of <= 0)
    return fail(PR_ERR_ARG, "update_state_bwd: dS_scan_in needs zero_last_of (the chunks per scanned sequence)");
  if (BN <= 0 || c <= 0 || h <= 0) return fail(PR_ERR_ARG, "update_state_bwd: need BN,c,h > 0");
  if (zero_last_of < 0 || (zero_last_of > 0 && BN % zero_last_of != 0))
    return fail(PR_ERR_ARG, "update_state_bwd: zero_last_of must be 0 or a divisor of BN (got %d, BN %d)", zero_last_of, BN);
  const int nn_ = zero_last_of > 0 ? zero_last_of : 1, skl = zero_last_of > 0 ? 1 : 0;
  pr::NNArgs nn{K, dS, nullptr, dV, nullptr, nullptr, nullptr, nullptr, 1.f, c, h, 1, nn_, 0, skl, dS_symmetric ? 1 : 0, nullptr};
  nn.live_rows = live_rows;
  nn.B_alt = dS_scan_in;
  nn.carry = scan_log_G;
  pr::GradArgs g{K, V, nullptr, dS, ds, dK, c, h, 1, nn_, skl ? 2 : 0, dS_symmetric ? 1 : 0};
  g.live_rows = live_rows;
  g.live_side = 0;
  g.B_alt = dS_scan_in;
  g.sB_alt = ds_scan_in;
  g.carry = scan_log_G;
  g.alt_shift = 1;
  // short chunks, both gradients: one launch whose two readers of every chunk's dS share it through L2
  if (dV && dK && pr::sympow_dvdk_ok(c, 1))
    return finish(pr::sympow_dvdk(nn, g, BN, d, dtype, (hipStream_t)stream), "update_state_bwd(dV, dK)");
  if (dV)
    if (int rc = finish(pr::sympow_nn(nn, BN, d, 1, 0, dtype, (hipStream_t)stream), "update_state_bwd(dV)")) return rc;
  if (!dK) return 0;
  return finish(pr::sympow_grad(g, BN, d, 1, dtype, (hipStream_t)stream), "update_state_bwd(dK)");
}

int pr_discumsum_fwd(const void* X, const float* log_G, void* Y, int B, int n, int n_out, int H, int64_t F,
                     int dtype, void* stream) {
  if (dtype != PR_BF16 && dtype != PR_F16 && dtype != PR_F32) return fail(PR_ERR_DTYPE, "discumsum_fwd: unsupported dtype");
  if (bad_ptr(X) || bad_ptr(Y) || log_G == nullptr) return fail(PR_ERR_ARG, "discumsum_fwd: null or misaligned pointer");
  const int vec = dtype == PR_F32 ? 4 : 8;
  if (B <= 0 || n <= 0 || H <= 0 || F <= 0 || F % vec != 0 || (n_out != n && n_out != n + 1))
    return fail(PR_ERR_ARG, "discumsum_fwd: need B,n,H > 0, F a multiple of %d, n_out in {n, n+1}", vec);
  return finish(pr::discumsum_fwd(X, log_G, Y, B, n, n_out, H, (long)F, dtype, (hipStream_t)stream), "discumsum_fwd");
}

size_t pr_discumsum_bwd_workspace(int B, int n, int H, int64_t F, int dtype) {
  return (size_t)pr::discumsum_bwd_workspace_floats(B, n, H, (long)F, dtype) * sizeof(float);
}

int pr_discumsum_bwd(const void* dY, const void* Y, const float* log_G, void* dX, float* dlog_G, void* workspace,
                     int B, int n, int n_out, int H, int64_t F, int dtype, void* stream) {
  if (dtype != PR_BF16 && dtype != PR_F16 && dtype != PR_F32) return fail(PR_ERR_DTYPE, "discumsum_bwd: unsupported dtype");
  if (bad_ptr(dY) || bad_ptr(Y) || log_G == nullptr || bad_ptr(dX) || dlog_G == nullptr || bad_ptr(workspace))
    return fail(PR_ERR_ARG, "discumsum_bwd: null or misaligned pointer");
  const int vec = dtype == PR_F32 ? 4 : 8;
  if (B <= 0 || n <= 0 || H <= 0 || F <= 0 || F % vec != 0 || (n_out != n && n_out != n + 1))
    return fail(PR_ERR_ARG, "discumsum_bwd: need B,n,H > 0, F a multiple of %d, n_out in {n, n+1}", vec);
  return finish(pr::discumsum_bwd(dY, Y, log_G, dX, dlog_G, (float*)workspace, B, n, n_out, H, (long)F, dtype,
                                  (hipStream_t)stream), "discumsum_bwd");
}

int pr_state_scan_fwd(const void* S, const float* s, const float* log_G, void* S_out, float* s_out,
                      const void* S_init, const float* s_init, void* S_final, float* s_final, int B, int n,
                      int n_out, int H, int64_t F, int64_t F2, int consumers_follow_gates, int dtype, void* stream) {
  if (dtype != PR_BF16 && dtype != PR_F16) return fail(PR_ERR_DTYPE, "state_scan_fwd: unsupported dtype");
  if (bad_ptr(S) || bad_ptr(s) || log_G == nullptr || bad_ptr(S_out) || bad_ptr(s_out))
    return fail(PR_ERR_ARG, "state_scan_fwd: null or misaligned pointer");
  if (B <= 0 || n <= 0 || H <= 0 || F <= 0 || F2 <= 0 || F % 8 != 0 || (n_out != n && n_out != n + 1))
    return fail(PR_ERR_ARG, "state_scan_fwd: need B,n,H,F2 > 0, F a multiple of 8, n_out in {n, n+1}");
  if ((S_init != nullptr) != (s_init != nullptr) || (S_final != nullptr) != (s_final != nullptr) || bad_opt(S_init) ||
      bad_opt(S_final))
    return fail(PR_ERR_ARG, "state_scan_fwd: S_init / s_init and S_final / s_final come in pairs, 16-byte aligned");
  if (S_final && n_out != n) return fail(PR_ERR_ARG, "state_scan_fwd: S_final is entry n of a scan that keeps n entries");
  pr::ScanCarry cy;
  cy.in = S_init, cy.in2 = s_init, cy.out = S_final, cy.out2 = s_final;
  return finish(pr::discumsum_pair_fwd(S, s, log_G, S_out, s_out, B, n, n_out, H, (long)F, (long)F2, cy,
                                       consumers_follow_gates, dtype, (hipStream_t)stream), "state_scan_fwd");
}

size_t pr_state_scan_bwd_workspace(int B, int n, int H, int64_t F, int64_t F2) {
  return (size_t)pr::discumsum_pair_bwd_workspace_floats(B, n, H, (long)F, (long)F2) * sizeof(float);
}

int pr_state_scan_bwd(const void* dS_out, const void* S_out, const float* ds_out, const float* s_out,
                      const float* log_G, void* dS, float* ds, float* dlog_G, void* workspace, const void* dS_final,
                      const float* ds_final, void* dS_init, float* ds_init, int B, int n, int n_out,
                      int H, int64_t F, int64_t F2, int consumers_follow_gates, int dtype, void* stream) {
  if (dtype != PR_BF16 && dtype != PR_F16) return fail(PR_ERR_DTYPE, "state_scan_bwd: unsupported dtype");
  if (bad_ptr(dS_out) || bad_ptr(S_out) || bad_ptr(ds_out) || bad_ptr(s_out) || log_G == nullptr || bad_ptr(dS) ||
      bad_ptr(ds) || dlog_G == nullptr || bad_ptr(workspace))
    return fail(PR_ERR_ARG, "state_scan_bwd: null or misaligned pointer");
  if (B <= 0 || n <= 0 || H <= 0 || F <= 0 || F2 <= 0 || F % 8 != 0 || (n_out != n && n_out != n + 1))
    return fail(PR_ERR_ARG, "state_scan_bwd: need B,n,H,F2 > 0, F a multiple of 8, n_out in {n, n+1}");
  if ((dS_final != nullptr) != (ds_final != nullptr) || (dS_init != nullptr) != (ds_init != nullptr) ||
      bad_opt(dS_final) || bad_opt(dS_init))
    return fail(PR_ERR_ARG, "state_scan_bwd: dS_final / ds_final and dS_init / ds_init come in pairs, 16-byte aligned");
  if (dS_final && n_out != n) return fail(PR_ERR_ARG, "state_scan_bwd: dS_final belongs to a scan that keeps n entries");
  pr::ScanCarry cy;
  cy.in = dS_final, cy.in2 = ds_final, cy.out = dS_init, cy.out2 = ds_init;
  return finish(pr::discumsum_pair_bwd(dS_out, S_out, ds_out, s_out, log_G, dS, ds, dlog_G, (float*)workspace, B, n,
                                       n_out, H, (long)F, (long)F2, cy, consumers_follow_gates, dtype,
                                       (hipStream_t)stream), "state_scan_bwd");
}

int pr_query_state_fwd(const void* Q, const void* S, const float* s, const void* Y_attn, const float* l_attn,
                       const float* rowmax, const float* q_log_gate, void* O, float* den, int BN, int n, int c, int h,
                       int r, int d, float scale_p, int deg, int zero_initial_state, int S_symmetric, int dtype,
                       void* stream) {
  if (int rc = check_common("query_state_fwd", d, deg, dtype, true)) return rc;
  if (bad_ptr(Q) || bad_ptr(S) || bad_ptr(s) || bad_ptr(O) || bad_ptr(den) || bad_opt(Y_attn) || bad_opt(l_attn) ||
      bad_opt(rowmax))
    return fail(PR_ERR_ARG, "query_state_fwd: null or misaligned pointer");
  if ((Y_attn != nullptr) != (l_attn != nullptr) || (Y_attn != nullptr) != (rowmax != nullptr))
    return fail(PR_ERR_ARG, "query_state_fwd: Y_attn, l_attn and rowmax must be given together");
  if (q_log_gate && !Y_attn) return fail(PR_ERR_ARG, "query_state_fwd: q_log_gate needs the attention part (it enters the merge)");
  if (BN <= 0 || n <= 0 || c <= 0 || h <= 0 || r <= 0 || BN % n != 0)
    return fail(PR_ERR_ARG, "query_state_fwd: need BN,n,c,h,r > 0 and BN a multiple of n");
  pr::NNArgs a{Q, S, s, O, den, Y_attn, l_attn, rowmax, scale_p, c, h, r, n, zero_initial_state ? 1 : 0, 0,
               S_symmetric ? 1 : 0, q_log_gate};
  return finish(pr::sympow_nn(a, BN, d, 0, 1, dtype, (hipStream_t)stream), "query_state_fwd");
}

int pr_chunk_fwd_supported(int d, int deg, int dtype) { return deg == 2 && pr::chunk_fwd_supported(d, dtype); }

int pr_chunk_fwd(const void* Q, const void* K, const void* V, const float* A, const void* S, const float* s,
                 const void* S_scan_in, const float* s_scan_in, const float* scan_log_G, void* O, float* rowmax,
                 float* den, int BN, int n, int c, int h, int r, int d, float scale, int deg, int zero_initial_state,
                 int dtype, void* stream) {
  if (int rc = check_common("chunk_fwd", d, deg, dtype, true)) return rc;
  if (!pr_chunk_fwd_supported(d, deg, dtype))
    return fail(PR_ERR_DTYPE, "chunk_fwd: bf16, head dim 32 or 64, degree 2 (ask pr_chunk_fwd_supported); other cases "
                              "take pr_chunk_attention_fwd and pr_query_state_fwd");
  if (bad_ptr(Q) || bad_ptr(K) || bad_ptr(V) || bad_opt(A) || bad_ptr(S) || bad_ptr(s) || bad_ptr(O) ||
      bad_ptr(rowmax) || bad_ptr(den))
    return fail(PR_ERR_ARG, "chunk_fwd: null or misaligned pointer");
  if (BN <= 0 || n <= 0 || c <= 0 || h <= 0 || r <= 0 || BN % n != 0)
    return fail(PR_ERR_ARG, "chunk_fwd: need BN,n,c,h,r > 0 and BN a multiple of n");
  if ((S_scan_in != nullptr) != (s_scan_in != nullptr) || (S_scan_in != nullptr) != (scan_log_G != nullptr) ||
      bad_opt(S_scan_in))
    return fail(PR_ERR_ARG, "chunk_fwd: S_scan_in, s_scan_in and scan_log_G come together, 16-byte aligned");
  pr::ChunkFwdArgs a{Q, K, V, A, S, s, O, rowmax, den, c, h, r, n, scale, zero_initial_state ? 1 : 0, pr::g_gate_skip};
  if (pr::g_gate_skip) a.S_alt = S_scan_in, a.s_alt = s_scan_in, a.carry = scan_log_G;
  return finish(pr::chunk_fwd(a, BN, d, dtype, (hipStream_t)stream), "chunk_fwd");
}

int pr_chunk_bwd_dq_supported(int d, int deg, int dtype) { return deg == 2 && pr::chunk_bwd_dq_supported(d, dtype); }

int pr_chunk_bwd_dq(const void* Q, const void* K, const void* V, const float* A, const float* rowmax, const float* den,
                    const void* dO, const float* dl_attn, const float* dY_scale, const float* cvec, const void* S,
                    const float* s, const void* S_scan_in, const float* s_scan_in, const float* scan_log_G, void* dQ,
                    float* dGq, int BN, int n, int c, int h, int r, int d, float scale, int deg,
                    int zero_initial_state, int dtype, void* stream) {
  if (int rc = check_common("chunk_bwd_dq", d, deg, dtype, true)) return rc;
  if (!pr_chunk_bwd_dq_supported(d, deg, dtype))
    return fail(PR_ERR_DTYPE, "chunk_bwd_dq: bf16, head dim 32 or 64, degree 2 (ask pr_chunk_bwd_dq_supported); other "
                              "cases take pr_query_state_bwd and pr_chunk_attention_bwd");
  if (bad_ptr(Q) || bad_ptr(K) || bad_ptr(V) || bad_opt(A) || bad_ptr(rowmax) || bad_ptr(den) || bad_ptr(dO) ||
      bad_ptr(dl_attn) || bad_ptr(dY_scale) || bad_ptr(cvec) || bad_ptr(S) || bad_ptr(s) || bad_ptr(dQ) || bad_opt(dGq))
    return fail(PR_ERR_ARG, "chunk_bwd_dq: null or misaligned pointer");
  if (A && !dGq) return fail(PR_ERR_ARG, "chunk_bwd_dq: dGq is required when A is given");
  if (BN <= 0 || n <= 0 || c <= 0 || h <= 0 || r <= 0 || BN % n != 0)
    return fail(PR_ERR_ARG, "chunk_bwd_dq: need BN,n,c,h,r > 0 and BN a multiple of n");
  pr::ChunkBwdDqArgs a{Q, K, V, A, rowmax, den, dO, dl_attn, dY_scale, cvec, S, s, dQ, A ? dGq : nullptr,
                       c, h, r, n, scale, zero_initial_state ? 1 : 0, pr::g_gate_skip};
  if ((S_scan_in != nullptr) != (s_scan_in != nullptr) || (S_scan_in != nullptr) != (scan_log_G != nullptr) ||
      bad_opt(S_scan_in))
    return fail(PR_ERR_ARG, "chunk_bwd_dq: S_scan_in, s_scan_in and scan_log_G come together, 16-byte aligned");
  if (pr::g_gate_skip) a.S_alt = S_scan_in, a.s_alt = s_scan_in, a.carry = scan_log_G;
  return finish(pr::chunk_bwd_dq(a, BN, d, dtype, (hipStream_t)stream), "chunk_bwd_dq");
}

size_t pr_query_state_bwd_workspace(int BN, int c, int h, int r, int d, int dtype) {
  (void)dtype;
  const size_t rows = (size_t)BN * c * h * r;
  return align256(rows * d * 2) + align256(rows * sizeof(float));
}

int pr_query_state_bwd(const void* Q, const void* S, const float* s, const float* rowmax, const float* q_log_gate,
                       const void* O, const float* den, const void* dO, void* dQ, void* dS, float* ds, void* dY_attn,
                       float* dl_attn, float* dY_scale, void* workspace, const int* live_rows, int BN, int n, int c,
                       int h, int r, int d, float scale_p, int deg, int zero_initial_state, int S_symmetric,
                       int prepared, int dtype, void* stream) {
  if (int rc = check_common("query_state_bwd", d, deg, dtype, true)) return rc;
  if (live_rows && !q_log_gate) return fail(PR_ERR_ARG, "query_state_bwd: live_rows describes q_log_gate");
  if (bad_ptr(Q) || bad_ptr(S) || bad_ptr(s) || bad_ptr(O) || bad_ptr(den) || bad_ptr(dO) || bad_opt(dQ) ||
      bad_opt(dS) || bad_ptr(workspace) || bad_opt(rowmax) || bad_opt(dY_attn) || bad_opt(dl_attn))
    return fail(PR_ERR_ARG, "query_state_bwd: null or misaligned pointer");
  if ((dS == nullptr) != (ds == nullptr)) return fail(PR_ERR_ARG, "query_state_bwd: dS and ds come together");
  if (rowmax && ((!dY_attn && !dY_scale) || !dl_attn))
    return fail(PR_ERR_ARG, "query_state_bwd: dl_attn and one of dY_attn, dY_scale are required when rowmax is given");
  if (q_log_gate && !rowmax) return fail(PR_ERR_ARG, "query_state_bwd: q_log_gate needs the attention part");
  if (BN <= 0 || n <= 0 || c <= 0 || h <= 0 || r <= 0 || BN % n != 0)
    return fail(PR_ERR_ARG, "query_state_bwd: need BN,n,c,h,r > 0 and BN a multiple of n");

  const size_t rows = (size_t)BN * c * h * r;
  void* dOs = workspace;
  float* cvec = (float*)((char*)workspace + align256(rows * d * 2));
  hipStream_t st = (hipStream_t)stream;
  if (!prepared)
    if (int rc = finish(pr::qs_bwd_prep(O, dO, den, rowmax, q_log_gate, dOs, cvec, rowmax ? dY_attn : nullptr,
                                        rowmax ? dl_attn : nullptr, rowmax ? dY_scale : nullptr, (long)rows, h, r, d,
                                        scale_p, (dS && !dQ) ? live_rows : nullptr, c, dtype, st),
                        "query_state_bwd(prep)"))
      return rc;
  // (zero_initial_state == 2: the caller does not want the gradient of the first chunk's (zero) state either)
  if (dS)
    if (int rc = finish(pr::sympow_tn(Q, dOs, cvec, dS, ds, BN, c, h, r, d, 0, zero_initial_state == 2 ? -n : 0, live_rows, 1,
                                      dtype, st),
                        "query_state_bwd(dS)"))
      return rc;
  if (!dQ) return 0;
  pr::GradArgs g{Q, dOs, cvec, S, s, dQ, c, h, r, n, zero_initial_state ? 1 : 0, S_symmetric ? 1 : 0};
  g.live_rows = live_rows;
  g.live_side = 1;
  return finish(pr::sympow_grad(g, BN, d, 0, dtype, st), "query_state_bwd(dQ)");
}


int pr_state_chain_supported(int B, int n, int c, int h, int r, int d) {
  return pr::sympow_tn_chain_ok(B, n, c, h, r, d);
}

int pr_update_state_scan_fwd(const void* K, const void* V, const float* log_G, void* S_out, float* s_out, int B, int n,
                             int c, int h, int d, int deg, int dtype, void* stream) {
  if (int rc = check_common("update_state_scan_fwd", d, deg, dtype, true)) return rc;
  if (bad_ptr(K) || bad_ptr(V) || bad_ptr(S_out) || bad_ptr(s_out))
    return fail(PR_ERR_ARG, "update_state_scan_fwd: null or misaligned pointer");
  // (the same predicate as pr_state_chain_supported, so a shape the query accepts is never refused here)
  if (B <= 0 || n <= 0 || c <= 0 || h <= 0 || !pr::sympow_tn_chain_ok(B, n < 2 ? 2 : n, c, h, 1, d))
    return fail(PR_ERR_ARG, "update_state_scan_fwd: need B,n,h > 0 and c a positive multiple of the stage (64 rows, 32 at d = 128)");
  return finish(pr::sympow_tn_chain(K, V, nullptr, log_G, S_out, s_out, B, n, c, h, 1, d, 1, 0, dtype,
                                    (hipStream_t)stream), "update_state_scan_fwd");
}

size_t pr_query_state_scan_bwd_workspace(int B, int n, int c, int h, int r, int d, int dtype) {
  const long D = 128L * (d / 16) * (d / 16 + 1);
  return pr_query_state_bwd_workspace(B * n, c, h, r, d, dtype) +
         align256((size_t)pr::scan_gate_grad_workspace_floats(B, n, h, D * d, D) * sizeof(float));
}

int pr_query_state_scan_bwd(const void* Q, const void* S, const float* s, const float* rowmax, const float* q_log_gate,
                            const void* O, const float* den, const void* dO, const float* log_G, void* dQ, void* dS_in,
                            float* ds_in,
                            void* dY_attn, float* dl_attn, float* dY_scale, float* dlog_G, void* workspace, int B,
                            int n, int c, int h, int r, int d, float scale_p, int deg, int dtype, void* stream) {
  if (int rc = check_common("query_state_scan_bwd", d, deg, dtype, true)) return rc;
  if (bad_ptr(Q) || bad_ptr(S) || bad_ptr(s) || bad_ptr(O) || bad_ptr(den) || bad_ptr(dO) || bad_ptr(dQ) ||
      bad_ptr(dS_in) || bad_ptr(ds_in) || bad_ptr(workspace) || bad_opt(rowmax) || bad_opt(dY_attn) || bad_opt(dl_attn))
    return fail(PR_ERR_ARG, "query_state_scan_bwd: null or misaligned pointer");
  if (rowmax && ((!dY_attn && !dY_scale) || !dl_attn))
    return fail(PR_ERR_ARG, "query_state_scan_bwd: dl_attn and one of dY_attn, dY_scale are required when rowmax is given");
  if ((log_G != nullptr) != (dlog_G != nullptr))
    return fail(PR_ERR_ARG, "query_state_scan_bwd: log_G and dlog_G must be given together");
  if (B <= 0 || n <= 0 || c <= 0 || h <= 0 || r <= 0 || !pr::sympow_tn_chain_ok(B, n < 2 ? 2 : n, c, h, r, d))
    return fail(PR_ERR_ARG, "query_state_scan_bwd: need B,n,c,h > 0, r a divisor of the stage (64 rows, 32 at d = 128) and "
                            "c*r a multiple of it");
  const int BN = B * n;
  const size_t rows = (size_t)BN * c * h * r;
  const long D = 128L * (d / 16) * (d / 16 + 1);
  void* dOs = workspace;
  float* cvec = (float*)((char*)workspace + align256(rows * d * 2));
  float* part = (float*)((char*)workspace + pr_query_state_bwd_workspace(BN, c, h, r, d, dtype));
  hipStream_t st = (hipStream_t)stream;
  if (q_log_gate && !rowmax) return fail(PR_ERR_ARG, "query_state_scan_bwd: q_log_gate needs the attention part");
  if (int rc = finish(pr::qs_bwd_prep(O, dO, den, rowmax, q_log_gate, dOs, cvec, rowmax ? dY_attn : nullptr,
                                      rowmax ? dl_attn : nullptr, rowmax ? dY_scale : nullptr, (long)rows, h, r, d,
                                      scale_p, nullptr, 0, dtype, st),
                      "query_state_scan_bwd(prep)"))
    return rc;
  if (int rc = finish(pr::sympow_tn_chain(Q, dOs, cvec, log_G, dS_in, ds_in, B, n, c, h, r, d, 0, 1, dtype, st),
                      "query_state_scan_bwd(dS)"))
    return rc;
  if (log_G)
    if (int rc = finish(pr::scan_gate_grad(S, dS_in, s, ds_in, log_G, dlog_G, part, B, n, h, D * d, D, dtype, st),
                        "query_state_scan_bwd(dlog_G)"))
      return rc;
  pr::GradArgs g{Q, dOs, cvec, S, s, dQ, c, h, r, n, 1, 0};
  return finish(pr::sympow_grad(g, BN, d, 0, dtype, st), "query_state_scan_bwd(dQ)");
}

int pr_gate_cumsum(const float* log_G, float* A, int B, int t, int h, void* stream) {
  if (!log_G || !A) return fail(PR_ERR_ARG, "gate_cumsum: null pointer");
  if (B <= 0 || t <= 0 || h <= 0) return fail(PR_ERR_ARG, "gate_cumsum: need B,t,h > 0");
  if (t > 8192) return fail(PR_ERR_ARG, "gate_cumsum: at most 8192 positions (got %d)", t);
  return finish(pr::gate_cumsum(log_G, A, B, t, h, (hipStream_t)stream), "gate_cumsum");
}

int pr_chunk_prep_fwd(const float* log_G, const void* K, const void* Q, float* A, float* lcs, void* Kd, void* Qg,
                      int* live_rows, int BN,
                      int c, int h, int r, int d, int deg, int dtype, void* stream) {
  if (int rc = check_common("chunk_prep_fwd", d, deg, dtype, false)) return rc;
  if (bad_ptr(K) || bad_ptr(Q) || A == nullptr || lcs == nullptr || bad_opt(Kd) || bad_opt(Qg) || (!log_G && !Kd))
    return fail(PR_ERR_ARG, "chunk_prep_fwd: null or misaligned pointer");
  if (BN <= 0 || c <= 0 || h <= 0 || r <= 0) return fail(PR_ERR_ARG, "chunk_prep_fwd: need BN,c,h,r > 0");
  return finish(pr::chunk_prep_fwd(log_G, K, Q, A, lcs, Kd, Qg, live_rows, BN, c, h, r, d, deg, dtype, (hipStream_t)stream),
                "chunk_prep_fwd");
}

int pr_chunk_gate_scan_bwd(float* dlog_G, const float* dGq, const float* dotk, const float* dlcs_a, const float* dlcs_b,
                           int BN, int c, int h, int r, int deg, void* stream) {
  if (!dlog_G || !dotk || !dlcs_a) return fail(PR_ERR_ARG, "chunk_gate_scan_bwd: null pointer");
  if (BN <= 0 || c <= 0 || h <= 0 || r <= 0 || deg <= 0)
    return fail(PR_ERR_ARG, "chunk_gate_scan_bwd: need BN,c,h,r,deg > 0");
  return finish(pr::chunk_gate_scan_bwd(dlog_G, dGq, dotk, dlcs_a, dlcs_b, BN, c, h, r, deg, (hipStream_t)stream),
                "chunk_gate_scan_bwd");
}

int pr_cache_append(void* K_cache, void* V_cache, float* A_cache, const void* K_new, const void* V_new,
                    const float* log_G_new, float* A_last, int B, int capacity, int pos, int t_new, int h, int d,
                    int dtype, void* stream) {
  if (dtype != PR_BF16 && dtype != PR_F16) return fail(PR_ERR_DTYPE, "cache_append: dtype must be bf16 or fp16");
  if (d <= 0 || d % 8 != 0) return fail(PR_ERR_HEAD_DIM, "cache_append: head dim must be a positive multiple of 8 (got %d)", d);
  if (bad_ptr(K_cache) || bad_ptr(V_cache) || !A_cache || bad_ptr(K_new) || bad_ptr(V_new))
    return fail(PR_ERR_ARG, "cache_append: null or misaligned pointer");
  if (B <= 0 || h <= 0 || t_new <= 0 || pos < 0 || (long)pos + t_new > capacity)
    return fail(PR_ERR_ARG, "cache_append: need B,h,t_new > 0 and 0 <= pos, pos + t_new <= capacity (got pos %d + %d, "
                            "capacity %d)", pos, t_new, capacity);
  return finish(pr::cache_append(K_cache, V_cache, A_cache, K_new, V_new, log_G_new, A_last, B, capacity, pos, t_new, h, d, dtype,
                                 (hipStream_t)stream), "cache_append");
}

int pr_cache_attention_fwd(const void* Q, const void* K_cache, const void* V_cache, const float* A_cache, void* O, float* l,
                           float* rowmax, int B, int tq, int tk, int capacity, int h, int r, int d, float scale, int deg,
                           int norm, int dtype, void* stream) {
  if (int rc = check_common("cache_attention_fwd", d, deg, dtype, false)) return rc;
  if (bad_ptr(Q) || bad_ptr(K_cache) || bad_ptr(V_cache) || bad_ptr(O) || bad_opt(A_cache) || bad_opt(l) || bad_opt(rowmax))
    return fail(PR_ERR_ARG, "cache_attention_fwd: null or misaligned pointer");
  if (!norm && (!l || !rowmax)) return fail(PR_ERR_ARG, "cache_attention_fwd: l and rowmax are required when norm == 0");
  if (B <= 0 || tq <= 0 || tk <= 0 || h <= 0 || r <= 0 || tq > tk || tk > capacity)
    return fail(PR_ERR_ARG, "cache_attention_fwd: need B,tq,tk,h,r > 0 and tq <= tk <= capacity (got %d %d %d %d)", B, tq, tk,
                capacity);
  pr::AttnFwdArgs a{Q, K_cache, V_cache, A_cache, O, l, rowmax, tq, tk, h, r, scale, (float)deg, norm, capacity};
  return finish(pr::attention_fwd(a, B, d, dtype, (hipStream_t)stream), "cache_attention_fwd");
}

size_t pr_decode_step_workspace(int B, int tq, int h, int r, int d) {
  return align256((size_t)pr::decode_workspace_floats(B, h, r, tq, d) * sizeof(float));
}

namespace {
// argument checks shared by pr_decode_step and pr_decode_step_noalloc
int check_decode(const char* what, const void* Q, const void* S, const float* s, const void* Y_attn, const float* l_attn,
                 const float* rowmax, const void* K_new, const void* V_new, const void* S_out, const float* s_out,
                 const void* out, int B, int tq, int h, int r, int d, int deg, int dtype, int attend_new) {
  if (int rc = check_common(what, d, deg, dtype, true)) return rc;
  if (attend_new && (!K_new || tq != 1 || Y_attn))
    return fail(PR_ERR_ARG, "%s: attend_new needs K_new, V_new, tq == 1 and no separate attention part", what);
  if (bad_ptr(Q) || bad_ptr(S) || bad_ptr(s) || bad_ptr(out) || bad_opt(Y_attn) || bad_opt(K_new) || bad_opt(V_new) ||
      bad_opt(S_out))
    return fail(PR_ERR_ARG, "%s: null or misaligned pointer", what);
  if ((Y_attn != nullptr) != (l_attn != nullptr) || (Y_attn != nullptr) != (rowmax != nullptr))
    return fail(PR_ERR_ARG, "%s: Y_attn, l_attn and rowmax must be given together", what);
  if (K_new && (!V_new || !S_out || !s_out)) return fail(PR_ERR_ARG, "%s: V_new, S_out and s_out are required with K_new", what);
  if (K_new && ((S_out == S) != (s_out == s)))
    return fail(PR_ERR_ARG, "%s: update S and s both in place or both out of place", what);
  if (B <= 0 || tq <= 0 || h <= 0 || r <= 0) return fail(PR_ERR_ARG, "%s: need B,tq,h,r > 0", what);
  if (tq * r > 16) return fail(PR_ERR_ARG, "%s: at most 16 query rows per (batch, kv head) (got %d)", what, tq * r);
  return 0;
}
}  // namespace

int pr_decode_step(const void* Q, const float* gq, const void* S, const float* s, const void* Y_attn,
                   const float* l_attn, const float* rowmax, const void* K_new, const void* V_new,
                   const float* log_decay, void* S_out, float* s_out, void* out, void* workspace, int B, int tq, int h,
                   int r, int d, float scale_p, int deg, int dtype, int attend_new, void* stream) {
  if (int rc = check_decode("decode_step", Q, S, s, Y_attn, l_attn, rowmax, K_new, V_new, S_out, s_out, out, B, tq, h, r,
                            d, deg, dtype, attend_new))
    return rc;
  if (bad_ptr(workspace)) return fail(PR_ERR_ARG, "decode_step: null or misaligned workspace");
  return finish(pr::decode_step(Q, gq, S, s, Y_attn, l_attn, rowmax, K_new, V_new, log_decay, S_out, s_out, out,
                                (float*)workspace, B, tq, h, r, d, deg, scale_p, dtype, attend_new ? 1 : 0,
                                (hipStream_t)stream),
                "decode_step");
}

size_t pr_decode_step_noalloc_max_workspace(void) {
  // also the set-up call: the array's address on the current GPU is taken here, so that a first
  // pr_decode_step_noalloc issued while a stream is being captured has no runtime query left to make
  (void)pr::decode_static_prepare();
  return (size_t)pr::decode_static_floats() * sizeof(float);
}

int pr_decode_step_noalloc(const void* Q, const float* gq, const void* S, const float* s, const void* Y_attn,
                           const float* l_attn, const float* rowmax, const void* K_new, const void* V_new,
                           const float* log_decay, void* S_out, float* s_out, void* out, int B, int tq, int h, int r,
                           int d, float scale_p, int deg, int dtype, int attend_new, void* stream) {
  if (int rc = check_decode("decode_step_noalloc", Q, S, s, Y_attn, l_attn, rowmax, K_new, V_new, S_out, s_out, out, B,
                            tq, h, r, d, deg, dtype, attend_new))
    return rc;
  const size_t need = pr_decode_step_workspace(B, tq, h, r, d);
  if (need > pr_decode_step_noalloc_max_workspace())
    return fail(PR_ERR_ARG, "decode_step_noalloc: this step needs %zu bytes of partial sums, the library's array holds %zu "
                            "(use pr_decode_step with a workspace)", need, pr_decode_step_noalloc_max_workspace());
  const int rc = pr::decode_step_static(Q, gq, S, s, Y_attn, l_attn, rowmax, K_new, V_new, log_decay, S_out, s_out, out,
                                        B, tq, h, r, d, deg, scale_p, dtype, attend_new ? 1 : 0, (hipStream_t)stream);
  if (rc == -6) return fail(PR_ERR_ARG, "decode_step_noalloc: the step needs more partial sums than the library's array holds");
  if (rc == -7) return fail(PR_ERR_ARG, "decode_step_noalloc: the stream belongs to another GPU than the current one");
  return finish(rc, "decode_step_noalloc");
}

}  // extern "C"
