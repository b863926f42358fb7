/*
 * C ABI of libpower_retention_hip.so: the gfx950 (MI355X) kernels behind the four operators of
 * symmetric power retention and their backward passes.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer, 16-byte aligned, to a dense row-major tensor of the stated
 *     shape; nothing is allocated, freed or synchronised inside the library; outputs and workspaces are
 *     provided by the caller; inputs are never written.
 *   - dtype: PR_BF16 / PR_F16 for Q, K, V, states and outputs (PR_F32 additionally for pr_discumsum_*);
 *     gates, row statistics and key sums are always fp32.
 *   - stream: a hipStream_t (NULL = default stream); calls only enqueue work.
 *   - return value: 0 on success, PR_ERR_* (< 0) for arguments the kernels do not support (nothing
 *     is launched), or a positive hipError_t from the launch.  pr_last_error() describes the last
 *     failure on the calling thread.
 *   - head dim d (= value dim) in {32, 64, 128}; deg = 2 for everything that touches the state;
 *     r = query heads per kv head.
 *
 * Each entry point names the reference interface it replaces (paths relative to the reference tree).
 */
#ifndef POWER_RETENTION_HIP_H
#define POWER_RETENTION_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { PR_BF16 = 0, PR_F16 = 1, PR_F32 = 2 };
enum {
  PR_OK = 0,
  PR_ERR_DTYPE = -1,     /* unsupported dtype */
  PR_ERR_HEAD_DIM = -2,  /* unsupported head dim */
  PR_ERR_ARG = -3,       /* null / misaligned pointer, non-positive size, inconsistent sizes */
  PR_ERR_DEG = -4        /* unsupported degree */
};

/* 2: pr_update_state_bwd and pr_query_state_bwd take the symmetric-state promise (dS_symmetric, S_symmetric).
 * 3: pr_decode_step_noalloc.  4: pr_cache_append, pr_cache_attention_fwd; pr_update_state_fwd takes skip_last_of and
 * pr_update_state_bwd zero_last_of; pr_query_state_fwd / _bwd / _scan_bwd take q_log_gate and
 * pr_chunk_attention_bwd dQ_state_plain.  5: pr_query_state_fwd takes S_symmetric.  6: pr_set_launch_hook;
 * pr_decode_step takes up to 16 query rows per (batch, kv head); pr_state_scan_fwd / _bwd connect a scan to the calls
 * before and after it (S_init, S_final and their gradients).  7: pr_chunk_fwd, pr_chunk_bwd_dq and their _supported queries.
 * 8: pr_set_gate_skipping / pr_get_gate_skipping; live_rows of pr_chunk_prep_fwd, pr_update_state_fwd / _bwd and
 * pr_query_state_bwd; consumers_follow_gates of pr_state_scan_fwd / _bwd and the *_scan_in arguments of pr_chunk_fwd,
 * pr_chunk_bwd_dq and pr_update_state_bwd.  9: live_rows of pr_chunk_attention_bwd; with live_rows,
 * pr_update_state_bwd leaves whole blocks of 256 dead rows of dK, dV unwritten. */
int pr_abi_version(void);
const char* pr_last_error(void);

/* Per-kernel hook for benchmarks and profilers (no counterpart in the reference, whose harness times whole operators:
 * perf/_timing.py:77-110).  Once set, the hook is called on the launching host thread right before (phase 0) and right
 * after (phase 1) EVERY kernel launch of the library, with the kernel's short name (a static string such as
 * "sympow_grad" or "attention_bwd_dkv") and the stream it is launched on -- record a pair of events there to time a
 * kernel where it runs, inside a step.  NULL removes it.  Process-wide; set it while no other thread is inside the
 * library.  The hook must not call back into the library. */
typedef void (*pr_launch_hook_t)(const char* kernel, int phase, void* stream, void* user);
void pr_set_launch_hook(pr_launch_hook_t hook, void* user);

/* Gate skipping (no counterpart in the reference, whose kernels visit every tile below the diagonal:
 * retention/_attention/impl_triton.py, retention/_query_state/impl_triton.py).  Accumulated log gates only fall along a
 * chunk, and a weight exp(A_i - A_j) of a query i on a key j that underflows fp32 IS zero in the reference's arithmetic
 * too (so is the factor exp(A_i) on the state part of a row, and the factor exp((A_last - A_j) / deg) on a key's
 * contribution to the next state).  With skipping on (the default) the kernels leave out the key tiles, state sweeps and
 * row blocks whose every term is such an exact zero, instead of multiplying through them; results are the same bit for
 * bit wherever a kernel decides per tile, and gates that do not decay that far (|A| below about 87 inside a chunk)
 * change nothing at all.  Off: every tile is visited, whatever the gates -- the data-independent cost.  Process-wide;
 * set it while no other thread is inside the library. */
void pr_set_gate_skipping(int on);
int pr_get_gate_skipping(void);

/* Size D of the expanded state for head dim d: 256 * T(T+1)/2, T = d/16; -1 if d is not a multiple of 16.
 * Replaces retention/_utils.py:18-19 compute_expanded_dim. */
int pr_expanded_dim(int d, int deg);

/* attention(Q, K, V, log_G_accum, deg, scale, norm) -- retention/_attention/reference.py:10-69,
 * Triton twin retention/_attention/triton.py:606-721 (_attn_fwd).
 *   Q [B,tq,h*r,d], K,V [B,tk,h,d], G [B,tk,h] fp32 accumulated log gate or NULL
 *   -> O [B,tq,h*r,d]; l, rowmax [B,tq,h*r] fp32 (either may be NULL when norm != 0).
 *   norm != 0 writes o/l to O, otherwise the unnormalised o. Queries are aligned to the end of the keys. */
int pr_attention_fwd(const void* Q, const void* K, const void* V, const float* G, void* O, float* l, float* rowmax,
                     int B, int tq, int tk, int h, int r, int d, float scale, int deg, int norm, int dtype,
                     void* stream);

/* Backward of the above w.r.t. (o, l) of the norm == 0 form -- retention/_attention/triton.py:228-603,723-810.
 *   rowmax as returned by the forward; dO [B,tq,h*r,d]; dl [B,tq,h*r] fp32 or NULL (zero);
 *   dO_scale [B,tq,h*r] fp32 or NULL: the gradient of o is dO * dO_scale[row], scaled in fp32 (the norm != 0
 *   form passes dY with dO_scale = 1/l and dl = -sum(dY*Y)/l, which keeps the cancellation of rows that see
 *   a single key exact)
 *   -> dQ [B,tq,h*r,d], dK, dV [B,tk,h,d]; when G != NULL also dGq [B,tq,h*r] (sum_j dz_ij) and
 *   dGk [B,tk,h] (-sum_i dz_ij), whose sum over the aligned positions is d log_G_accum.
 *   The query side (dQ, dGq) and the key side (dK, dV, dGk) are separate kernels: with dQ == NULL, or with dK == dV ==
 *   NULL, only the other side runs (two calls may then be issued on two streams). */
int pr_attention_bwd(const void* Q, const void* K, const void* V, const float* G, const float* rowmax,
                     const void* dO, const float* dl, const float* dO_scale, void* dQ, void* dK, void* dV,
                     float* dGq, float* dGk, int B, int tq, int tk, int h, int r, int d, float scale, int deg,
                     int dtype, void* stream);

/* update_state(K, V, deg) -- retention/_update_state/reference.py:33-52,86-94,
 * Triton twin retention/_update_state/triton.py:61-133,280-320.
 *   K, V [BN,c,h,d] (BN = b*n chunks) -> S [BN,h,D,d], s [BN,h,D] fp32.
 *   skip_last_of = n > 0: the last of every n chunks is not computed and its S, s are left unwritten (the composed
 *   function never reads the last chunk's state, retention/power_retention_maker.py:168-170); 0 computes every chunk.
 *   live_rows (NULL, or the [BN,h,2] int32 array that pr_chunk_prep_fwd wrote for the gates that discounted K): the
 *   time steps before live_rows[bn,h,0] hold keys that the discount turned into exact zeros and are not read. */
int pr_update_state_fwd(const void* K, const void* V, void* S, float* s, const int* live_rows, int BN, int c, int h,
                        int d, int deg, int skip_last_of, int dtype, void* stream);

/* Backward -- retention/_update_state/reference.py:55-83, Triton twin retention/_update_state/triton.py:148-260.
 *   dS [BN,h,D,d], ds [BN,h,D] fp32 -> dK, dV [BN,c,h,d]; one of dK, dV may be NULL (that gradient is skipped).
 *   dS_symmetric != 0 is the caller's promise that dS[(a,b)] == dS[(b,a)] for the pairs the layout stores in both
 *   orders (the 16x16 blocks on the diagonal); true of the dS that pr_query_state_bwd and the scans produce, not of
 *   an arbitrary tensor.  The key gradient then takes a shorter path through those blocks; with 0 every feature is
 *   used as given, as the reference does.
 *   zero_last_of = n > 0 is the promise that dS, ds of the last of every n chunks are zero (that chunk's state feeds
 *   nothing): they are not read and dK, dV are written as zeros there; 0 makes no such promise.
 *   live_rows (NULL, or what pr_chunk_prep_fwd wrote for the gates that discounted K): the time steps before
 *   live_rows[bn,h,0] hold keys that are exact zeros; dK, dV are zero there and not computed -- and up to the last
 *   multiple of 256 steps below live_rows[bn,h,0] they are NOT WRITTEN: hand dK, dV to pr_chunk_attention_bwd with the
 *   same live_rows (which does not read them there), or treat those rows as zeros.
 *   dS_scan_in, ds_scan_in, scan_log_G (all NULL, or all given together with zero_last_of = n): dS, ds are the output of
 *   pr_state_scan_bwd and these its inputs dS_out, ds_out, log_G.  Entry k of that scan equals its input entry k + 1
 *   bit for bit when exp(scan_log_G[k + 1]) == 0; the kernels then read the input entry (see consumers_follow_gates
 *   of pr_state_scan_bwd). */
int pr_update_state_bwd(const void* K, const void* V, const void* dS, const float* ds, const void* dS_scan_in,
                        const float* ds_scan_in, const float* scan_log_G, const int* live_rows, void* dK, void* dV, int BN,
                        int c, int h, int d, int deg, int dS_symmetric, int zero_last_of, int dtype, void* stream);

/* discumsum(X, log_G) -- retention/_discumsum/reference.py:3-15, Triton twin retention/_discumsum/triton.py:34-94.
 *   X [B,n,H,F], log_G [B,n,H] fp32 -> Y [B,n_out,H,F], Y[0]=0, Y[k+1]=Y[k]*exp(log_G[k])+X[k];
 *   n_out = n+1 (the operator) or n (the last entry, which the composed path discards, is not produced).
 *   F must be a multiple of 16 bytes / sizeof(dtype). */
int pr_discumsum_fwd(const void* X, const float* log_G, void* Y, int B, int n, int n_out, int H, int64_t F,
                     int dtype, void* stream);

/* Backward -- autograd of retention/_discumsum/reference.py:3-15 (Triton twin retention/_discumsum/triton.py:111-204).
 *   dY, Y [B,n_out,H,F] -> dX [B,n,H,F], dlog_G [B,n,H] fp32 (deterministic two-pass reduction).
 *   workspace: pr_discumsum_bwd_workspace() bytes of device memory. */
size_t pr_discumsum_bwd_workspace(int B, int n, int H, int64_t F, int dtype);
int pr_discumsum_bwd(const void* dY, const void* Y, const float* log_G, void* dX, float* dlog_G, void* workspace,
                     int B, int n, int n_out, int H, int64_t F, int dtype, void* stream);

/* The two scans of the chunked algorithm -- discumsum(S, lcs) and discumsum(s, lcs),
 * retention/power_retention_maker.py:167-170 -- in one launch each way (the small fp32 scan is bound by latency and
 * costs nothing next to the big one).  S [B,n,H,F] 16-bit, s [B,n,H,F2] fp32, same log_G [B,n,H].
 * Backward: dlog_G [B,n,H] receives the SUM of both scans' gate gradients.
 *   workspace: pr_state_scan_bwd_workspace() bytes.
 * State across calls (retention/power_retention_maker.py:131-140,158-172; here the carried state is the state AFTER the
 * last token, decayed by the gates like every chunk's):
 *   S_init [B,H,F], s_init [B,H,F2] or both NULL: the scans start from them (entry 0 = S_init) instead of zero;
 *   S_final, s_final or both NULL (n_out == n only): receive entry n, exp(log_G[n-1]) * entry n-1 + S[n-1].
 *   Backward: dS_final / ds_final (NULL = zero) is the gradient of that entry n, dS_init / ds_init (NULL = not wanted)
 *   receive the gradient of the starting value.
 * consumers_follow_gates != 0 (honoured only without S_init / S_final resp. dS_final / dS_init, with n_out == n, and
 * while gate skipping is on) is the caller's promise that every reader of the scan's output takes the scan's INPUT
 * wherever the two are equal bit for bit because the carry into the entry is an exact zero -- forward: entry k is input
 * k - 1 when exp(log_G[k-1]) == 0 or k == 1, and entry 0 (zero) is not read; backward: entry k is input k + 1 when
 * exp(log_G[k+1]) == 0, and entry n - 1 (zero) is not read.  pr_chunk_fwd, pr_chunk_bwd_dq (S_scan_in ...) and
 * pr_update_state_bwd (dS_scan_in ...) are such readers.  A (batch, head) whose every factor exp(log_G[k]), k >= 1, is
 * zero is then not scanned: nothing of it is read, its output entries are left unwritten and, backward, its gate
 * gradient is written as zero. */
int pr_state_scan_fwd(const void* S, const float* s, const float* log_G, void* S_out, float* s_out,
                      const void* S_init, const float* s_init, void* S_final, float* s_final, int B, int n,
                      int n_out, int H, int64_t F, int64_t F2, int consumers_follow_gates, int dtype, void* stream);
size_t pr_state_scan_bwd_workspace(int B, int n, int H, int64_t F, int64_t F2);
int pr_state_scan_bwd(const void* dS_out, const void* S_out, const float* ds_out, const float* s_out,
                      const float* log_G, void* dS, float* ds, float* dlog_G, void* workspace, const void* dS_final,
                      const float* ds_final, void* dS_init, float* ds_init, int B, int n, int n_out,
                      int H, int64_t F, int64_t F2, int consumers_follow_gates, int dtype, void* stream);

/* Short chunks: update_state followed by the scan that keeps its first n entries
 * (retention/power_retention_maker.py:156,167-170) as ONE pass that never writes the per-chunk states:
 *   K, V [B,n*c,h,d] (keys already discounted), log_G [B,n,h] fp32 chunk gate sums or NULL (no decay)
 *   -> S_out [B*n,h,D,d], s_out [B*n,h,D] fp32 with S_out[b,0] = 0, S_out[b,k+1] = e^{log_G[b,k]} S_out[b,k] + phi(K_k)^T V_k.
 * A workgroup walks the chunks of a batch element serially, so this pays only when B*h is large and the chunks are
 * short.  pr_state_chain_supported() returns 0 when the shape is not supported (it needs c*r a multiple of the 64-row
 * stage and r a divisor of it -- 32 rows at d = 128 -- and n >= 2), 1 when it is, 2 when it also has enough independent work to be the faster form
 * (r = 1 on the key side, the query-head ratio on the query side). */
int pr_state_chain_supported(int B, int n, int c, int h, int r, int d);
int pr_update_state_scan_fwd(const void* K, const void* V, const float* log_G, void* S_out, float* s_out, int B, int n,
                             int c, int h, int d, int deg, int dtype, void* stream);

/* The backward of query_state (below, with zero_initial_state) chained with the backward of that scan: from dO to
 * dQ, to the gradient of the PER-CHUNK states dS_in [B*n,h,D,d], ds_in [B*n,h,D] (what update_state's backward
 * consumes) and, when log_G is given, to dlog_G [B,n,h]; formulas retention/_query_state/triton.py:546-553 and
 * retention/_discumsum/reference.py:3-15 differentiated.  S, s are the scanned states the forward used.
 *   workspace: pr_query_state_scan_bwd_workspace() bytes. */
size_t pr_query_state_scan_bwd_workspace(int B, int n, int c, int h, int r, int d, int dtype);
int pr_query_state_scan_bwd(const void* Q, const void* S, const float* s, const float* rowmax, const float* q_log_gate,
                            const void* O, const float* den, const void* dO, const float* log_G, void* dQ, void* dS_in,
                            float* ds_in, void* dY_attn, float* dl_attn, float* dY_scale, float* dlog_G, void* workspace,
                            int B, int n, int c, int h, int r, int d, float scale_p, int deg, int dtype, void* stream);

/* query_state(Q, S, s, Y_attn, l_attn, rowmax, deg, scale, zero_initial_state) --
 * retention/_query_state/reference.py:36-96,166-191, Triton twin retention/_query_state/triton.py:54-169,478-544.
 *   Q [BN,c,h*r,d] (already gated), S [BN,h,D,d], s [BN,h,D] fp32,
 *   Y_attn [BN,c,h*r,d] / l_attn, rowmax [BN,c,h*r] fp32, all three NULL when there is no attention part
 *   -> O [BN,c,h*r,d] and den [BN,c,h*r] fp32, the normaliser in the scaled units the backward expects.
 *   scale_p = scale^deg; n = chunks per batch entry; zero_initial_state != 0 declares S, s of chunk 0 of every
 *   batch entry to be zero (they are then not read).
 *   q_log_gate [BN,c,h] fp32 or NULL (needs the attention part): the query gating of
 *   retention/power_retention_maker.py:183-186 without the gated copy -- with it, Q is the UNGATED query and the result
 *   is that of Q * exp(q_log_gate / deg): the state part is homogeneous of degree deg in the query, so the gate is a
 *   factor exp(q_log_gate) on that part of each row and is applied in the merge (exact; the reference rounds the gated
 *   copy to 16 bits first).
 *   S_symmetric != 0: the caller's promise that S[(a,b)] == S[(b,a)] in the blocks on the diagonal (true of every
 *   state made by pr_update_state_fwd and the scans): the mirrored quarter of each such block is then not read
 *   (a tenth of the state less to contract). */
int pr_query_state_fwd(const void* Q, const void* S, const float* s, const void* Y_attn, const float* l_attn,
                       const float* rowmax, const float* q_log_gate, void* O, float* den, int BN, int n, int c, int h,
                       int r, int d, float scale_p, int deg, int zero_initial_state, int S_symmetric, int dtype,
                       void* stream);

/* Backward -- formulas of retention/_query_state/triton.py:546-553 (kernels :184-448).
 *   O, den from the forward; dO [BN,c,h*r,d]
 *   -> dQ [BN,c,h*r,d], dS [BN,h,D,d], ds [BN,h,D] fp32, and, when rowmax != NULL,
 *      dY_attn [BN,c,h*r,d], dl_attn [BN,c,h*r] fp32.  dY_attn is dO times a per-row factor; a consumer that scales
 *      on the fly (the dO_scale argument of the attention backward) can ask for that factor instead:
 *      dY_scale [BN,c,h*r] fp32 (then dY_attn may be NULL).
 *   zero_initial_state: 1 as in the forward; 2 additionally declares that nobody needs the gradient of the first
 *   chunk's (zero) state: dS, ds of the first of every n chunks are then written as zeros instead of computed (the
 *   composed function discards them, retention/power_retention_maker.py:167-170).
 *   workspace: pr_query_state_bwd_workspace() bytes (scaled dO and two fp32 row vectors).
 *   q_log_gate as in the forward: Q is then the ungated query and dQ the gradient w.r.t. it through the state part
 *   (the gate's own gradient is (Q . dQ) / deg per row, which pr_chunk_attention_bwd forms with dQ_state_plain).
 *   S_symmetric != 0: the caller's promise that S[(a,b)] == S[(b,a)] in the blocks on the diagonal (true of every
 *   state made by pr_update_state_fwd and the scans); the query gradient then takes a shorter path through them.
 *   The call is three kernels: the row-wise preparation (fills the workspace, dY_attn / dY_scale, dl_attn), dS / ds, and
 *   dQ.  With dS == ds == NULL or dQ == NULL that kernel is skipped; prepared != 0 says that an earlier call with the
 *   same inputs has filled this workspace and skips the preparation -- so the two contractions, which do not depend
 *   on each other, can be issued as two calls on two streams.
 *   live_rows (NULL, or the [BN,h,2] int32 array that pr_chunk_prep_fwd wrote for the gates in q_log_gate): from time
 *   step live_rows[bn,h,1] on, the factor exp(q_log_gate) has underflowed to zero, the state part of those rows has a
 *   zero gradient, and the dS / ds contraction does not read them.  A call that prepares and forms dS / ds but not dQ
 *   (prepared == 0, dQ == NULL) also leaves the scaled dO of the workspace unwritten from the first multiple of 256
 *   time steps at or after live_rows[bn,h,1] on: a later prepared != 0 call for dQ has to pass the same live_rows (its
 *   kernel then does not read those rows), as pr_chunk_bwd_dq, which takes dO itself, need not. */
size_t pr_query_state_bwd_workspace(int BN, int c, int h, int r, int d, int dtype);
int pr_query_state_bwd(const void* Q, const void* S, const float* s, const float* rowmax, const float* q_log_gate,
                       const void* O, const float* den, const void* dO, void* dQ, void* dS, float* ds, void* dY_attn,
                       float* dl_attn, float* dY_scale, void* workspace, const int* live_rows, int BN, int n, int c,
                       int h, int r, int d, float scale_p, int deg, int zero_initial_state, int S_symmetric,
                       int prepared, int dtype, void* stream);

/* Forward of every chunk in one kernel: the attention inside the chunk (retention/_attention/reference.py:10-69), the
 * query of the state the chunk starts from and the merge of the two (retention/_query_state/reference.py:36-96, with
 * the query gating of retention/power_retention_maker.py:183-186 as a row factor) -- what pr_chunk_attention_fwd
 * followed by pr_query_state_fwd(q_log_gate = A, S_symmetric = 1) compute, without the attention part going to memory
 * and back.  bf16, d in {32, 64}, deg 2: pr_chunk_fwd_supported() says whether the case exists; the others take the
 * two calls.
 *   Q [BN,c,h*r,d] (ungated), K, V [BN,c,h,d], A [BN,c,h] fp32 accumulated log gates of the chunk or NULL,
 *   S [BN,h,D,d] / s [BN,h,D] fp32: the scanned states, symmetric in the diagonal feature blocks
 *   -> O [BN,c,h*r,d], rowmax [BN,c,h*r] (log of the row's largest attention weight) and den [BN,c,h*r], both fp32 and
 *      in the units pr_query_state_bwd and pr_chunk_attention_bwd expect.
 *   scale multiplies q.k before the power; n, zero_initial_state as in pr_query_state_fwd.
 *   S_scan_in, s_scan_in, scan_log_G (all NULL, or all given): S, s are the output of pr_state_scan_fwd and these its
 *   inputs S, s, log_G.  Entry k of that scan equals its input entry k - 1 bit for bit when exp(scan_log_G[k-1]) == 0
 *   (and, with zero_initial_state, for k == 1): the kernel then reads the input entry (see consumers_follow_gates). */
int pr_chunk_fwd_supported(int d, int deg, int dtype);
int pr_chunk_fwd(const void* Q, const void* K, const void* V, const float* A, const void* S, const float* s,
                 const void* S_scan_in, const float* s_scan_in, const float* scan_log_G, void* O, float* rowmax,
                 float* den, int BN, int n, int c, int h, int r, int d, float scale, int deg, int zero_initial_state,
                 int dtype, void* stream);

/* Query side of the chunked backward in one kernel: dQ and dGq of the attention inside every chunk
 * (retention/_attention/triton.py:248-387) plus the query gradient through the chunk's starting state
 * (retention/_query_state/triton.py:546-553) and its share of the gate gradient, (q . dQ_state) / deg -- what
 * pr_query_state_bwd (its dQ kernel, q_log_gate = A, S_symmetric = 1) followed by pr_chunk_attention_bwd
 * (dK == dV == NULL, dQ_state_plain = 1) compute, without the state-path gradient going to memory and back.
 * bf16, d in {32, 64}, deg 2: pr_chunk_bwd_dq_supported() says whether the case exists; the others take the two calls.
 *   Q, K, V, A, S, s as for pr_chunk_fwd; rowmax, den [BN,c,h*r] from it; dO [BN,c,h*r,d];
 *   dl_attn, dY_scale [BN,c,h*r] and cvec [BN,c,h*r] fp32: the row vectors an earlier pr_query_state_bwd call on the
 *   same inputs has written (its dl_attn and dY_scale outputs; cvec is the second part of its workspace, behind the
 *   scaled dO: byte offset rows * d * 2 rounded up to 256, rows = BN*c*h*r) -- call it with dQ == dS == NULL for the
 *   preparation alone
 *   S_scan_in, s_scan_in, scan_log_G: as for pr_chunk_fwd
 *   -> dQ [BN,c,h*r,d] (final), dGq [BN,c,h*r] fp32 (required when A is given). */
int pr_chunk_bwd_dq_supported(int d, int deg, int dtype);
int pr_chunk_bwd_dq(const void* Q, const void* K, const void* V, const float* A, const float* rowmax, const float* den,
                    const void* dO, const float* dl_attn, const float* dY_scale, const float* cvec, const void* S,
                    const float* s, const void* S_scan_in, const float* s_scan_in, const float* scan_log_G, void* dQ,
                    float* dGq, int BN, int n, int c, int h, int r, int d, float scale, int deg,
                    int zero_initial_state, int dtype, void* stream);

/* Accumulated gates of the quadratic / inference paths -- log_G.cumsum(1), retention/power_retention_maker.py:129,
 * 348-349.  log_G, A [B,t,h] fp32, t <= 8192. */
int pr_gate_cumsum(const float* log_G, float* A, int B, int t, int h, void* stream);

/* Gate arithmetic of the chunked algorithm, forward -- retention/power_retention_maker.py:146-153,163-164,183-186.
 *   log_G [BN,c,h] fp32 (BN = b*n chunks of length c <= 8192), K [BN,c,h,d], Q [BN,c,h*r,d]
 *   -> A [BN,c,h] = cumsum over the chunk, lcs [BN,h] = A[c-1],
 *      Kd = K * exp((A[c-1] - A)/deg), Qg = Q * exp(A/deg) (Qg may be NULL: not formed).
 *   Two kernels (the sums, then the row-wise products): with Kd == NULL only A and lcs are written; with
 *   log_G == NULL, A and lcs are inputs and only the products are formed.
 *   live_rows (NULL or [BN,h,2] int32, written with the sums): per (chunk, kv head), [0] the first time step whose
 *   factor exp((A[c-1] - A)/deg) has not underflowed to zero -- the rows of Kd before it are exact zeros -- and [1] one
 *   past the last time step with exp(A) != 0 -- from there on the state part of a query row is an exact zero.  Hand it
 *   to pr_update_state_fwd / _bwd and pr_query_state_bwd, which then leave those rows out (see pr_set_gate_skipping).
 *   In a call with log_G == NULL (products only) live_rows is an INPUT and a promise: every reader of Kd is handed the
 *   same array; the rows of Kd before the block of 256 steps that holds live_rows[bn,h,0] -- exact zeros -- are then
 *   left unwritten. */
int pr_chunk_prep_fwd(const float* log_G, const void* K, const void* Q, float* A, float* lcs, void* Kd, void* Qg,
                      int* live_rows, int BN, int c, int h, int r, int d, int deg, int dtype, void* stream);

/* Backward of the same glue plus the final gradient sums (autograd of retention/power_retention_maker.py:143-193).
 * The row-wise part rides in the attention backward's epilogue (no extra pass over the gradients):
 * pr_chunk_attention_bwd is pr_attention_bwd on the chunks (B = BN, tq = tk = c, G = A) that also adds the gradients
 * arriving through the gated copies (retention/power_retention_maker.py:163-164, 183-186):
 *   dQ = dQ_attn + dQ_state * exp(A/deg),  dK = dK_attn + dK_state * exp((A[c-1] - A)/deg),  dV = dV_attn + dV_state,
 *   dGq [BN,c,h*r] and dGk [BN,c,h]: gradients w.r.t. A, including (Q.dQ_state) exp(A/deg)/deg and
 *   -(K.dK_state) exp((A[c-1]-A)/deg)/deg,  dotk [BN,c,h] = (K.dK_state) exp((A[c-1]-A)/deg).
 *   dQ_state = gradient w.r.t. Qg (query_state backward), dK_state, dV_state = gradients w.r.t. Kd, V
 *   (update_state backward).  With A = NULL the factors are 1 and dGq, dGk, dotk are not written.
 *   dQ_state_plain != 0: dQ_state is already the gradient w.r.t. Q itself (pr_query_state_bwd with q_log_gate):
 *   dQ = dQ_attn + dQ_state and dGq gets (Q.dQ_state)/deg.
 *   live_rows (NULL, or the array that pr_chunk_prep_fwd wrote for A; needs A, dK and dV): the factor
 *   exp((A[c-1] - A)/deg) is an exact zero at the keys before live_rows[bn,h,0]; dK_state and dV_state are not read
 *   there (they are zeros, or were left unwritten by a pr_update_state_bwd that was given the same live_rows).
 * pr_chunk_gate_scan_bwd finishes the gate gradient: dlog_G holds dGk on entry; the r query heads' dGq [BN,c,h*r]
 *   are added (dGq may be NULL), dlog_G[c-1] += (sum_t dotk)/deg + dlcs_a + dlcs_b (dlcs_b may be NULL), then the
 *   reverse cumulative sum over the chunk, in place. */
int pr_chunk_attention_bwd(const void* Q, const void* K, const void* V, const float* A, const float* rowmax,
                           const void* dO, const float* dl, const float* dO_scale, const void* dQ_state,
                           const void* dK_state, const void* dV_state, const int* live_rows, void* dQ, void* dK,
                           void* dV, float* dGq, float* dGk, float* dotk, int BN, int c, int h, int r, int d, float scale,
                           int deg, int dQ_state_plain, int dtype, void* stream);
int pr_chunk_gate_scan_bwd(float* dlog_G, const float* dGq, const float* dotk, const float* dlcs_a, const float* dlcs_b,
                           int BN, int c, int h, int r, int deg, void* stream);

/* Single-token inference step on the state -- query: retention/power_retention_maker.py:358-363 with
 * retention/_query_state/reference.py:36-96 (one query position per sequence); update:
 * retention/power_retention_maker.py:366-382 with retention/_update_state/reference.py:33-52 for ONE new token.
 *   Q [B,tq,h*r,d] with tq*r <= 16, gq [B,h] fp32 or NULL: accumulated log gate at the query position
 *   (Q is used as Q * exp(gq/deg), rounded to dtype), S [B,h,D,d], s [B,h,D] fp32,
 *   Y_attn [B,tq,h*r,d], l_attn, rowmax [B,tq,h*r] fp32 or all NULL (attention over the not yet folded cache)
 *   -> out [B,tq,h*r,d] = the merged, normalised output.
 *   If K_new is not NULL: K_new, V_new [B,h,d], log_decay [B,h] fp32 or NULL (= 0)
 *   -> S_out = exp(log_decay) * S + phi(K_new)^T V_new, s_out = exp(log_decay) * s + phi(K_new), read in the same
 *      pass as the query (which sees the OLD state).  S_out/s_out may be S/s themselves (in-place update: every
 *      element is read and written by the same thread) or separate buffers, both or neither.
 *   attend_new != 0 (needs K_new, tq == 1, Y_attn == NULL): the attention part is that of the new token attending to
 *      itself -- the recurrent loop that folds every token (switch_over_seq_len = 1) in one call: Y_attn = V_new,
 *      l_attn = 1 + 1e-6, rowmax = log((scale q.k)^deg), retention/_attention/reference.py:42-69 with one key.
 *   workspace: pr_decode_step_workspace() bytes. */
size_t pr_decode_step_workspace(int B, int tq, int h, int r, int d);
int pr_decode_step(const void* Q, const float* gq, const void* S, const float* s, const void* Y_attn,
                   const float* l_attn, const float* rowmax, const void* K_new, const void* V_new,
                   const float* log_decay, void* S_out, float* s_out, void* out, void* workspace, int B, int tq, int h,
                   int r, int d, float scale_p, int deg, int dtype, int attend_new, void* stream);

/* Preallocated K / V / gate cache of the decode loop -- replaces the three torch.cat per layer and step of
 * deploy/models/powercoder/kvgs_dynamic_cache.py:131-161 (DynamicLayer.update_kv) and the cumulative sum over the whole
 * cache of retention/power_retention_maker.py:347.
 *   K_cache, V_cache [B,capacity,h,d], A_cache [B,capacity,h] fp32: ACCUMULATED log gates since the start of the cache;
 *   K_new, V_new [B,t_new,h,d], log_G_new [B,t_new,h] fp32 or NULL (no gates: zeros are written)
 *   -> rows pos .. pos+t_new-1 of the three buffers (A_cache[pos+i] = A_cache[pos-1] + log_G_new[0] + ... + log_G_new[i],
 *      A_cache[-1] = 0); A_last [B,h] fp32 or NULL also receives the last of them (dense: the gq argument of
 *      pr_decode_step).  The caller keeps the length; rows beyond it are never read.
 * pr_cache_attention_fwd is pr_attention_fwd over the first tk rows of such buffers (batch stride = capacity rows). */
int pr_cache_append(void* K_cache, void* V_cache, float* A_cache, const void* K_new, const void* V_new,
                    const float* log_G_new, float* A_last, int B, int capacity, int pos, int t_new, int h, int d,
                    int dtype, void* stream);
int pr_cache_attention_fwd(const void* Q, const void* K_cache, const void* V_cache, const float* A_cache, void* O, float* l,
                           float* rowmax, int B, int tq, int tk, int capacity, int h, int r, int d, float scale, int deg,
                           int norm, int dtype, void* stream);

/* pr_decode_step without a workspace argument.  No counterpart in the reference: it is for callers that cannot
 * allocate device memory -- code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.
 * The partial query sums live in an array of pr_decode_step_noalloc_max_workspace() bytes (8 MiB) that the library
 * holds on every GPU it runs on until the process ends; the call allocates and frees nothing.  A step whose
 * pr_decode_step_workspace() exceeds that size is refused with PR_ERR_ARG (use pr_decode_step).  All calls on one
 * GPU share the array: calls that overlap in time on one GPU (two streams) race; calls on one stream do not.
 * The array is that of the GPU the stream belongs to, which must be the current device (PR_ERR_ARG otherwise).
 * Set-up: the array's address is looked up once per GPU (hipGetSymbolAddress, not stream work).
 * pr_decode_step_noalloc_max_workspace() does that for the current device, so call it once per GPU before a first
 * pr_decode_step_noalloc that is issued under stream capture; outside capture the first step does it by itself.
 * Same arguments, results and in-place rules as pr_decode_step. */
size_t pr_decode_step_noalloc_max_workspace(void);
int pr_decode_step_noalloc(const void* Q, const float* gq, const void* S, const float* s, const void* Y_attn,
                           const float* l_attn, const float* rowmax, const void* K_new, const void* V_new,
                           const float* log_decay, void* S_out, float* s_out, void* out, int B, int tq, int h, int r,
                           int d, float scale_p, int deg, int dtype, int attend_new, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* POWER_RETENTION_HIP_H */
