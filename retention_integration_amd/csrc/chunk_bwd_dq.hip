// Query side of the chunked algorithm's backward in ONE kernel per (chunk, kv head, block of 128 folded rows):
//
//   attention part   dQ_attn, dGq of the chunk's own keys        (attention_bwd.hip, its dQ kernel;
//                                                                 ref: retention/_attention/triton.py:248-387)
//   state part       dQ_state = gradient of  kappa_i phi(q_i) . (Sc, sc)  w.r.t. q_i      (sympow_grad.hip;
//                                                                 ref: retention/_query_state/triton.py:546-553)
//   dQ = dQ_attn + dQ_state,   dGq_i = sum_j dz_ij + (q_i . dQ_state_i) / 2
//                                      (the gate of a row multiplies its state part, which is homogeneous of degree 2
//                                       in q: ref retention/power_retention_maker.py:183-186 and its autograd)
//
// Both parts own the same 128 rows per workgroup, 32 per wave, in the same accumulator layout (coordinate on the
// accumulator rows, row on the lanes), so the second is accumulated on top of the first: the state-path gradient is
// not written, read back and rounded to 16 bits in between, the rows are loaded once, and a block has one prologue
// and one store phase.  Order: attention first -- its accumulation carries a row factor that is applied once after the
// tiles in a wave's past, the state sweep adds plain terms.  The block's own rows (for the sweep's per-row values) and
// the first two state stages ride through the attention ring as two more stages behind the last key tile, so they
// arrive under the last tiles' work.
//
// bf16, head dims 32 and 64, degree 2, states symmetric in the diagonal feature blocks; other cases run the two
// kernels.
#include "common.h"
#include "kernels.h"

namespace pr {

constexpr int CB_BN = 64;    // keys per attention stage
constexpr int CB_FR = 64;    // feature rows per state stage
constexpr int CB_NST = 3;    // attention ring
constexpr int CB_LEAD_BLOCKS = 2;   // row blocks of a chunk that are started before the longest ones (see the kernel)
constexpr float CB_LOG_EPS = 1e-7f, CB_EXP_CLAMP = 80.f;
constexpr float CB_LOG2E = 1.4426950408889634f, CB_EXP2_CLAMP = CB_EXP_CLAMP * CB_LOG2E;

typedef __attribute__((address_space(3))) s16x4 cb_lds_s16x4;
typedef __attribute__((address_space(3))) f32x4 cb_lds_f32x4;
typedef __attribute__((address_space(3))) char cb_lds_char;

template <typename T> __device__ __forceinline__ typename VecOf<T>::v8 cb_tr8(uint32_t lo_addr, uint32_t hi_addr) {
  const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((cb_lds_s16x4*)lo_addr);
  const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((cb_lds_s16x4*)hi_addr);
  const s16x8 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  return __builtin_bit_cast(typename VecOf<T>::v8, both);
}

template <typename T, int DH>
__global__ __launch_bounds__(256, 3) void chunk_bwd_dq_kernel(ChunkBwdDqArgs a, int nblocks, int npairs) {
  typedef typename VecOf<T>::v8 v8;
  typedef typename VecOf<T>::v4 v4;
  typedef __attribute__((address_space(3))) v8 lds_v8;
  typedef __attribute__((address_space(3))) uint32_t lds_u32;
  constexpr int MT = 2, KS = DH / 32, NT = DH / 16, TT = DH / 16, KT = CB_BN / 16, ROWS = 64 * MT, CPR = DH / 8, RB = CPR * 16;
  constexpr int TILE = CB_BN * RB;
  constexpr int STAGE = 2 * TILE + 4 * CB_BN * 4;   // K, V, raw gates, two sets of key gate factors
  constexpr int LOADS = 2 * CB_BN * CPR / 256;
  constexpr int D = 128 * TT * (TT + 1), NSTEP = D / CB_FR;
  constexpr int SSTAGE = CB_FR * DH * 2, SLOADS = CB_FR * CPR / 256, LDM = DH + 8;
  static_assert(ROWS * DH * 2 <= 2 * TILE && 2 * SSTAGE <= 2 * TILE, "the rows and two state stages fit a ring stage");
  static_assert(DH * LDM * 2 <= 2 * SSTAGE, "the key-sum matrix fits the state ring");
  extern __shared__ __attribute__((aligned(1024))) char smem[];

  // placement: see attention_bwd.hip (whole (chunk, head) pairs per (XCD, shader engine) group)
  const int grp = blockIdx.x % 32, u = blockIdx.x / 32, ppg = (npairs + 31) / 32;
  int pig, blk;
  deal_causal_blocks(u, nblocks, ppg, pig, blk);
  const int pair = pig * 32 + grp;
  if (pair >= npairs) return;
  const int tid = threadIdx.x, l = tid & 63, g = l >> 4, tcol = l & 15;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int b = __builtin_amdgcn_readfirstlane(pair / a.h), hh = pair - b * a.h;
  const int hq = a.h * a.r, rows = a.c * a.r;
  // Order of a pair's row blocks: the first two of the chunk, then the others from the last (late rows see the most
  // keys) backwards.  Under gates that forget within a hundred steps or so only those first blocks sweep the state and
  // are the long ones of the pair by far (156 for 172 us when they are started first); where every block sweeps it they
  // are the shortest, and two short blocks at the front cost nothing.
  const int lead = nblocks > CB_LEAD_BLOCKS ? CB_LEAD_BLOCKS : 0;
  const int row0 = (blk < lead ? blk : nblocks - 1 - (blk - lead)) * ROWS;
  const T* Qg = (const T*)a.Q + (long)b * a.c * hq * DH;
  const T* dOg = (const T*)a.dO + (long)b * a.c * hq * DH;
  const char* Kg = (const char*)((const T*)a.K + (long)b * a.c * a.h * DH + hh * DH);
  const char* Vg = (const char*)((const T*)a.V + (long)b * a.c * a.h * DH + hh * DH);
  const float* Gg = a.G ? a.G + (long)b * a.c * a.h + hh : nullptr;
  const char* Sg = (const char*)((const T*)a.S + ((long)b * a.h + hh) * D * DH);
  const float* sg = a.s + ((long)b * a.h + hh) * D;
  // (S, s are a gated scan's output: with a zero carry into it -- and, whatever the gate, at the second chunk of a
  // sequence that starts from nothing -- an entry is the scan's input entry before it, bit for bit)
  if (a.S_alt && b % a.n != 0 &&
      ((a.skip_first && (b - 1) % a.n == 0) || __expf(a.carry[(long)(b - 1) * a.h + hh]) == 0.f)) {
    Sg = (const char*)((const T*)a.S_alt + ((long)(b - 1) * a.h + hh) * D * DH);
    sg = a.s_alt + ((long)(b - 1) * a.h + hh) * D;
  }
  const long kstride = (long)a.h * DH * 2;
  const float eps_s = CB_LOG_EPS / a.scale, eps2 = eps_s * eps_s;
  const float scale_p = a.scale * a.scale;
  const float l2sp = __log2f(scale_p);
  bool has_state = !(a.skip_first && (b % a.n == 0));

  const int last_row = min(row0 + ROWS, rows) - 1;
  const int kmax = min(a.c, last_row / a.r + 1);
  const int ntiles = (kmax + CB_BN - 1) / CB_BN;
  const int wslice = (u & 1) ? 3 - wave : wave;   // alternate which wave is nearest the diagonal
  const int wrow0 = row0 + wslice * 16 * MT;
  const int w_first_ti = min(wrow0, rows - 1) / a.r;
  const int w_last_ti = min(wrow0 + 16 * MT - 1, rows - 1) / a.r;
  auto row_off = [&](int row) -> long {   // element offset of a (clamped) folded row, per unit of the last dim
    row = min(row, rows - 1);
    const int t = row / a.r, rr = row - t * a.r;
    return (long)t * hq + hh * a.r + rr;
  };

  uint32_t goff[LOADS / 2];
#pragma unroll
  for (int ii = 0; ii < LOADS / 2; ii++) {
    const int pos = (ii * 4 + wave) * 64 + l, row = pos / CPR;
    goff[ii] = (uint32_t)(row * (int)kstride + 16 * ((pos % CPR) ^ swz<CPR, SWZ_ROW>(row)));
  }
  // What the gates have already forgotten (see chunk_fwd.hip): the oldest key tiles whose factor exp(R - A_last) has
  // underflowed to zero for the largest gate sum among the workgroup's rows contribute exact zeros to every row -- dQ,
  // dGq -- and are neither copied nor visited; a state part whose factor exp(A_row) has underflowed for that largest sum
  // has a zero gradient for every row (its scaled dO and its key-sum factor are zeros), so the sweep is left out.
  int it0 = 0;
  if (Gg && a.gate_skip) {
    // (the largest gate sum among the workgroup's rows: the first row's, unless the caller's log gates are positive)
    float a_first = -INFINITY;
    for (int i = l; i < ROWS; i += 64) a_first = fmaxf(a_first, Gg[(long)(min(row0 + i, rows - 1) / a.r) * a.h]);
#pragma unroll
    for (int m = 32; m > 0; m >>= 1) a_first = fmaxf(a_first, __shfl_xor(a_first, m));
    if (__expf(a_first) == 0.f) has_state = false;
    for (int base = 0; base < ntiles; base += 64) {
      const int tl = min(base + l, ntiles - 1);
      const float a_last = Gg[(long)min(CB_BN * tl + CB_BN - 1, a.c - 1) * a.h];
      const unsigned long long dead = __ballot(__expf(fminf(a_first - a_last, CB_EXP_CLAMP)) == 0.f);
      const int lanes = min(64, ntiles - base);
      const int nd = __builtin_popcountll(lanes == 64 ? dead : (dead & ((1ull << lanes) - 1)));
      it0 += nd;
      if (nd < lanes) break;
    }
    it0 = __builtin_amdgcn_readfirstlane(min(min(it0, ntiles - 1), min(row0 / a.r + 1, a.c) / CB_BN));
  }
  // Stage ntiles of the ring: the block's rows of Q (the sweep's row values; chunk slots rotated per row as the state
  // kernels read them).  Stage ntiles + 1: the first two stages of the state.
  const int ntot = ntiles + (has_state ? 2 : 0);
  auto issue = [&](int it) __attribute__((always_inline)) {
    char* st = smem + (it % CB_NST) * STAGE;
    if (it == ntiles) {
      async_load_tile<CPR, ROWS>(st, [&](int row) { return (const char*)(Qg + row_off(row0 + row) * DH); });
      if (Gg && wave == 0) async_copy4(Gg, st + 2 * TILE);   // keeps the count of copies per stage fixed
      return;
    }
    if (it > ntiles) {
      const uint32_t sa = lds_addr(st) + wave * 1024;
#pragma unroll
      for (int s2 = 0; s2 < 2; s2++)
#pragma unroll
        for (int ii = 0; ii < SLOADS; ii++) {
          const int pos = (ii * 4 + wave) * 64 + l, row = pos / CPR;
          async_copy16_sv(Sg + (long)s2 * SSTAGE, (uint32_t)(row * (DH * 2) + 16 * ((pos % CPR) ^ swz<CPR, SWZ_ROW>(row))),
                          sa + s2 * SSTAGE + ii * 4096);
        }
      return;
    }
    const int j0 = it * CB_BN;
    if (j0 + CB_BN <= a.c) {
      const char* kb_ = Kg + (long)j0 * kstride;
      const char* vb_ = Vg + (long)j0 * kstride;
      const uint32_t sa = lds_addr(st) + wave * 1024;
#pragma unroll
      for (int ii = 0; ii < LOADS / 2; ii++) async_copy16_sv(kb_, goff[ii], sa + ii * 4096);
#pragma unroll
      for (int ii = 0; ii < LOADS / 2; ii++) async_copy16_sv(vb_, goff[ii], sa + TILE + ii * 4096);
    } else {   // last, partial tile: rows past the end repeat the last key (they are masked)
      async_load_tile<CPR, CB_BN, SWZ_ROW>(st, [&](int row) { return Kg + (long)min(j0 + row, a.c - 1) * kstride; });
      async_load_tile<CPR, CB_BN, SWZ_ROW>(st + TILE, [&](int row) { return Vg + (long)min(j0 + row, a.c - 1) * kstride; });
    }
    if (Gg && wave == 0) async_copy4(Gg + (long)min(j0 + l, a.c - 1) * a.h, st + 2 * TILE);
  };
  issue(it0);
  if (ntot > it0 + 1) issue(it0 + 1);

  v8 Qf[MT][KS], dOf[MT][KS];
  int ti[MT];
  bool live[MT];
  float base2[MT], dlr[MT], dgq[MT], osc[MT];   // base2 = log2(scale^2 exp(G_q - m))
  // the state part's factor on dO, one per row: parked in LDS until the sweep (a register pair through the tile loops
  // would be a spilled one)
  float* cq_lds = (float*)(smem + CB_NST * STAGE);
#pragma unroll
  for (int mi = 0; mi < MT; mi++) {
    const int row = wrow0 + 16 * mi + tcol;
    live[mi] = row < rows;
    const int rr = live[mi] ? row : 0;
    const int t = rr / a.r;
    ti[mi] = t;
    const long qoff = (long)t * hq + hh * a.r + (rr - t * a.r);
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      u32x4 z = {0, 0, 0, 0}, z2 = {0, 0, 0, 0};
      if (live[mi]) {
        z = *(const u32x4*)(Qg + qoff * DH + 32 * ks + 8 * g);
        z2 = *(const u32x4*)(dOg + qoff * DH + 32 * ks + 8 * g);
      }
      Qf[mi][ks] = __builtin_bit_cast(v8, z);
      dOf[mi][ks] = __builtin_bit_cast(v8, z2);
    }
    const long so = (long)b * a.c * hq + qoff;
    const float gq = Gg ? Gg[(long)t * a.h] : 0.f, m = a.rowmax[so];
    base2[mi] = __builtin_fmaf(gq - m, CB_LOG2E, l2sp);
    dlr[mi] = a.dl[so];
    osc[mi] = a.dO_scale[so];
    // (the expressions of the row-wise preparation kernel, so that the scaled dO below has its bits)
    const float beta = fmaxf(m, 0.5f * __logf((float)D));
    if (g == 0) cq_lds[wslice * 16 * MT + 16 * mi + tcol] = (scale_p * __expf(gq - beta)) * (1.f / a.den[so]);
    dgq[mi] = 0.f;
  }
  const float Rw = Gg ? Gg[(long)w_first_ti * a.h] : 0.f;   // gate at the wave's first row
  f32x4 acc[MT][NT];
#pragma unroll
  for (int mi = 0; mi < MT; mi++)
#pragma unroll
    for (int nt = 0; nt < NT; nt++) acc[mi][nt] = (f32x4){0, 0, 0, 0};

  int koff[KS], toff[NT];
#pragma unroll
  for (int ks = 0; ks < KS; ks++) koff[ks] = tcol * RB + (((4 * ks + g) ^ swz<CPR, SWZ_ROW>(tcol)) * 16);
  {
    const int vr = 4 * g + (tcol >> 2);
#pragma unroll
    for (int nt = 0; nt < NT; nt++) {
      const int col = 16 * nt + 4 * (tcol & 3);
      toff[nt] = vr * RB + (((col / 8) ^ swz<CPR, SWZ_ROW>(vr)) * 16) + (col % 8) * 2;
    }
  }

  const int n_past = min(ntiles, min(w_first_ti + 1, a.c) / CB_BN);   // tiles with every pair visible
  const int n_seen = min(ntiles, w_last_ti / CB_BN + 1);              // tiles with at least one visible pair

  auto gate_factors = [&](int it) __attribute__((always_inline)) {
    float* graw = (float*)(smem + (it % CB_NST) * STAGE + 2 * TILE);
    const int rpos = min(CB_BN - 1, a.c - 1 - it * CB_BN);
    const float gv = Gg ? graw[l] : 0.f;
    const float R_ = Gg ? graw[rpos] : 0.f;
    graw[CB_BN + l] = __expf(fminf(R_ - gv, CB_EXP_CLAMP));
    graw[2 * CB_BN + l] = gv * CB_LOG2E;   // the gate itself, in powers of two, for the diagonal tiles
    if (!Gg) graw[l] = 0.f;
  };
  if (wave == 0) {
    wait_vmcnt<0>();
    gate_factors(it0);
  }
  auto sync_step = [&](int it) __attribute__((always_inline)) -> char* {
    char* st = smem + (it % CB_NST) * STAGE;
    if (it + 1 < ntot) wait_vmcnt<LOADS>(); else wait_vmcnt<0>();
    lds_barrier();
    if (it + 2 < ntot) issue(it + 2);
    if (wave == 0 && it + 1 < ntiles) {
      if (it + 2 < ntot) wait_vmcnt<LOADS + 1>(); else wait_vmcnt<0>();   // all but the stage just issued
      gate_factors(it + 1);
    }
    return st;
  };

  // One 64-key tile (attention_bwd.hip, the dQ kernel's)
  auto tile = [&](int it, const char* st, auto diag_c) __attribute__((always_inline)) {
    constexpr bool DIAG = decltype(diag_c)::value != 0;
    const int j0 = it * CB_BN;
    const float* graw = (const float*)(st + 2 * TILE);
    uint32_t kb[KS], tb[NT], eb;
    {
      uint32_t sa = (uint32_t)(uintptr_t)(cb_lds_char*)st;
      asm volatile("" : "+s"(sa));
#pragma unroll
      for (int ks = 0; ks < KS; ks++) {
        kb[ks] = sa + koff[ks];
        asm volatile("" : "+v"(kb[ks]));
      }
#pragma unroll
      for (int nt = 0; nt < NT; nt++) { tb[nt] = sa + toff[nt]; asm volatile("" : "+v"(tb[nt])); }
      eb = sa + 2 * TILE + (DIAG ? 2 * CB_BN : CB_BN) * 4 + 16 * g;
      asm volatile("" : "+v"(eb));
    }
    int lim[MT];
#pragma unroll
    for (int mi = 0; mi < MT; mi++) lim[mi] = DIAG ? min(ti[mi], a.c - 1) - j0 - 4 * g : 0;
    const float cw = DIAG ? 1.f : __expf(fminf(Rw - graw[CB_BN - 1], CB_EXP_CLAMP));
    // (forgotten by this wave's rows, though not by the workgroup's first: every term of the tile is an exact zero)
    if (!DIAG && a.gate_skip && __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, cw)) == 0) return;
#pragma unroll
    for (int kp = 0; kp < KT / 2; kp++) {
      if (DIAG && j0 + 32 * kp > w_last_ti) continue;   // these 32 keys come after every row of the wave
      v4 h4[2][MT];
#pragma unroll
      for (int half = 0; half < 2; half++) {
        v8 kf[KS], vf[KS];
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
          kf[ks] = *(const lds_v8*)(kb[ks] + (2 * kp + half) * 16 * RB);
          vf[ks] = *(const lds_v8*)(kb[ks] + TILE + (2 * kp + half) * 16 * RB);
        }
        f32x4 ev = *(const cb_lds_f32x4*)(eb + 64 * (2 * kp + half));
        if (!DIAG) ev *= cw;
        f32x4 sc[MT], dp[MT];
#pragma unroll
        for (int mi = 0; mi < MT; mi++) {
          sc[mi] = (f32x4){0, 0, 0, 0};
          dp[mi] = (f32x4){0, 0, 0, 0};
        }
#pragma unroll
        for (int ks = 0; ks < KS; ks++)
#pragma unroll
          for (int mi = 0; mi < MT; mi++) {
            sc[mi] = mfma16(kf[ks], Qf[mi][ks], sc[mi]);
            dp[mi] = mfma16(vf[ks], dOf[mi][ks], dp[mi]);
          }
#pragma unroll
        for (int mi = 0; mi < MT; mi++) {
          float d4[4];
#pragma unroll
          for (int v = 0; v < 4; v++) {
            const float s = sc[mi][v];
            const float dpl = __builtin_fmaf(dp[mi][v], osc[mi], dlr[mi]);
            float q;                                     // E * dP (past tiles: without the row factor)
            if (DIAG) {
              q = __builtin_amdgcn_exp2f(fminf(base2[mi] - ev[v], CB_EXP2_CLAMP)) * dpl;
              q = (32 * kp + 16 * half + v <= lim[mi]) ? q : 0.f;
            } else {
              q = ev[v] * dpl;
            }
            dgq[mi] = __builtin_fmaf(__builtin_fmaf(s, s, eps2), q, dgq[mi]);
            d4[v] = s * q;
          }
          h4[half][mi] = pack4<T>(d4);
          asm volatile("" : "+v"(h4[half][mi]));
        }
      }
      v8 kT[NT];
#pragma unroll
      for (int nt = 0; nt < NT; nt++) kT[nt] = cb_tr8<T>(tb[nt] + kp * 32 * RB, tb[nt] + kp * 32 * RB + 16 * RB);
      v8 dsf[MT];
#pragma unroll
      for (int mi = 0; mi < MT; mi++) dsf[mi] = __builtin_shufflevector(h4[0][mi], h4[1][mi], 0, 1, 2, 3, 4, 5, 6, 7);
#pragma unroll
      for (int nt = 0; nt < NT; nt++)
#pragma unroll
        for (int mi = 0; mi < MT; mi++) acc[mi][nt] = mfma16(kT[nt], dsf[mi], acc[mi][nt]);
    }
  };

  int it = it0;
  for (; it < n_past; it++) tile(it, sync_step(it), IC<0>{});
  // the past tiles were accumulated without the row factor scale^2 * exp(G_q - m - Rw); apply it once
#pragma unroll
  for (int mi = 0; mi < MT; mi++) {
    const float f = __builtin_amdgcn_exp2f(fminf(base2[mi] - Rw * CB_LOG2E, CB_EXP2_CLAMP));
#pragma unroll
    for (int nt = 0; nt < NT; nt++) acc[mi][nt] *= f;
    dgq[mi] *= f;
  }
  for (; it < n_seen; it++) tile(it, sync_step(it), IC<1>{});
  for (; it < ntiles; it++) sync_step(it);

  // ---- hand over: d(q.k) -> dQ takes the degree; the scaled dO of the state part replaces dO ---------------------
  float tot[MT];
#pragma unroll
  for (int mi = 0; mi < MT; mi++) {
    tot[mi] = sum_over_rows(dgq[mi]);
#pragma unroll
    for (int nt = 0; nt < NT; nt++) acc[mi][nt] *= 2.f;
  }
  T* dQg = (T*)a.dQ + (long)b * a.c * hq * DH;
  // Lane indices for the rest of the kernel, re-derived from a copy of the lane id that the compiler cannot match with
  // the one used so far: nothing that is only needed from here on should stay in registers through the tile loops.
  int lB = threadIdx.x & 63;
  asm volatile("" : "+v"(lB));
  const int g2 = lB >> 4, tc2 = lB & 15;
  int lrow[MT];
#pragma unroll
  for (int mi = 0; mi < MT; mi++) lrow[mi] = wslice * 16 * MT + 16 * mi + tc2;

  if (has_state) {
    v8 Gf[MT][KS];
#pragma unroll
    for (int mi = 0; mi < MT; mi++) {
      const float cq = cq_lds[lrow[mi]];
#pragma unroll
      for (int ks = 0; ks < KS; ks++) {
        float g8[8];
        unpack8(dOf[mi][ks], g8);
#pragma unroll
        for (int i = 0; i < 8; i++) g8[i] *= cq;
        Gf[mi][ks] = pack8<T>(g8);
      }
    }
    wait_vmcnt<0>();
    lds_barrier();   // the rows and the first two state stages are in place
    char* xt = smem + (ntiles % CB_NST) * STAGE;
    char* ring = smem + ((ntiles + 1) % CB_NST) * STAGE;
    auto x_ptr = [&](int mi, int col) -> const char* {   // address of X[lrow[mi], col] in the swizzled tile
      return xt + lrow[mi] * (DH * 2) + (((col / 8) ^ swz<CPR>(lrow[mi])) * 16) + (col % 8) * 2;
    };
    // (q . dQ) so far: the state part's share of the gate gradient is the difference to the same sum afterwards
    float dot0[MT];
#pragma unroll
    for (int mi = 0; mi < MT; mi++) {
      float dsum = 0.f;
#pragma unroll
      for (int nt = 0; nt < NT; nt++) {
        const v4 q4 = *(const v4*)x_ptr(mi, 16 * nt + 4 * g2);
#pragma unroll
        for (int v = 0; v < 4; v++) dsum = __builtin_fmaf((float)q4[v], acc[mi][nt][v], dsum);
      }
      dot0[mi] = dsum;
    }

    uint32_t boffs[SLOADS];
#pragma unroll
    for (int ii = 0; ii < SLOADS; ii++) {
      const int pos = (ii * 4 + wave) * 64 + lB, row = pos / CPR;
      boffs[ii] = (uint32_t)(row * (DH * 2) + 16 * ((pos % CPR) ^ swz<CPR, SWZ_ROW>(row)));
    }
    const uint32_t ring_lds = lds_addr(ring) + wave * 1024;
    auto issue_s = [&](int step) {
      const char* src = Sg + (long)step * SSTAGE;
#pragma unroll
      for (int ii = 0; ii < SLOADS; ii++) async_copy16_sv(src, boffs[ii], ring_lds + (step % 2) * SSTAGE + ii * 4096);
    };
    const uint32_t ring_a = (uint32_t)(uintptr_t)(cb_lds_char*)ring, xt_a = (uint32_t)(uintptr_t)(cb_lds_char*)xt;
    uint32_t aoffa[KS];            // state rows as the first operand: row tcol of a 16-row group, chunk 4*ks + g
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      aoffa[ks] = ring_a + tc2 * (CPR * 16) + (((4 * ks + g2) ^ swz<CPR, SWZ_ROW>(tc2)) * 16);
      asm volatile("" : "+v"(aoffa[ks]));
    }
    uint32_t xrow_a[MT], xsw[MT];
#pragma unroll
    for (int mi = 0; mi < MT; mi++) {
      xrow_a[mi] = xt_a + lrow[mi] * (DH * 2);
      xsw[mi] = swz<CPR>(lrow[mi]);
    }

    // the sweep of sympow_grad.hip (symmetric state, no key-side multiplier): blocks (y, xb) in memory order
    int step = 0;
    static_for<TT>([&](auto yc) {
      constexpr int y = decltype(yc)::value;
      float xr[MT][4];              // X[row, 16y + 4g + v]
      static_for<y + 1>([&](auto xc) {
        constexpr int xb = decltype(xc)::value;
        constexpr bool diag = xb == y;
        auto stage = [&](int sb, auto sl_c) __attribute__((always_inline)) {
          constexpr int SL = decltype(sl_c)::value;
          if (step > 0) {   // (stages 0 and 1 came with the attention ring)
            wait_vmcnt<0>();
            lds_barrier();
            if (step > 0 && step + 1 < NSTEP) issue_s(step + 1);
          }
          if (sb == 0 && xb == 0) {
#pragma unroll
            for (int mi = 0; mi < MT; mi++) {
              const v4 h4 = *(const v4*)x_ptr(mi, 16 * y + 4 * g2);
#pragma unroll
              for (int v = 0; v < 4; v++) xr[mi][v] = (float)h4[v];
            }
          }
          uint32_t xa[MT];
          {
            const int X0 = 16 * xb + (CB_FR / 16) * sb, xc2 = X0 >> 3, xo = (X0 & 7) * 2;
#pragma unroll
            for (int mi = 0; mi < MT; mi++) { xa[mi] = xrow_a[mi] + ((xc2 ^ xsw[mi]) << 4) + xo; asm volatile("" : "+v"(xa[mi])); }
          }
#pragma unroll
          for (int pr2 = 0; pr2 < CB_FR / 32; pr2++) {
            const int m0 = ((CB_FR / 16) * sb + 2 * pr2) % 16;
            v8 af0[KS], af1[KS];
#pragma unroll
            for (int ks = 0; ks < KS; ks++) {
              af0[ks] = *(const lds_v8*)(aoffa[ks] + SL * SSTAGE + (32 * pr2) * (CPR * 16));
              af1[ks] = *(const lds_v8*)(aoffa[ks] + SL * SSTAGE + (32 * pr2 + 16) * (CPR * 16));
            }
            const uint32_t s_lo = (tc2 == m0) ? 0x3F803F80u : 0u, s_hi = (tc2 == m0 + 1) ? 0x3F803F80u : 0u;
            const v8 sel = __builtin_bit_cast(v8, (u32x4){s_lo, s_lo, s_hi, s_hi});
            f32x4 d0[MT], d1[MT];
#pragma unroll
            for (int mi = 0; mi < MT; mi++) {
              d0[mi] = (f32x4){0, 0, 0, 0};
              d1[mi] = (f32x4){0, 0, 0, 0};
            }
#pragma unroll
            for (int ks = 0; ks < KS; ks++)
#pragma unroll
              for (int mi = 0; mi < MT; mi++) {
                d0[mi] = mfma16(af0[ks], Gf[mi][ks], d0[mi]);
                d1[mi] = mfma16(af1[ks], Gf[mi][ks], d1[mi]);
              }
#pragma unroll
            for (int mi = 0; mi < MT; mi++) {
              const uint32_t xx = *(const lds_u32*)(xa[mi] + 4 * pr2);
              float x0 = __builtin_bit_cast(float, xx << 16), x1 = __builtin_bit_cast(float, xx & 0xffff0000u);
              if constexpr (diag) {
                x0 += x0;
                x1 += x1;
              }
              acc[mi][y] = acc[mi][y] + d0[mi] * x0;
              acc[mi][y] = acc[mi][y] + d1[mi] * x1;
              if constexpr (diag) continue;
              float w8[8];
#pragma unroll
              for (int v = 0; v < 4; v++) {
                w8[v] = xr[mi][v] * d0[mi][v];
                w8[4 + v] = xr[mi][v] * d1[mi][v];
              }
              acc[mi][xb] = mfma16(sel, pack8<T>(w8), acc[mi][xb]);   // fold into dX[row, 16*xb + X]
            }
          }
          step++;
        };
#pragma unroll 1
        for (int sb = 0; sb < 256 / CB_FR; sb += 2) {
          stage(sb, IC<0>{});
          stage(sb + 1, IC<1>{});
        }
      });
    });

    // key-sum term: dX_s[row, w] = cvec[row] * sum_a (U[a, w] + U[w, a]) X[row, a], U[a, w] = sc of the stored pair
    T* Mt = (T*)ring;   // [DH (a)][LDM (w)]
    float cv[MT];
#pragma unroll
    for (int mi = 0; mi < MT; mi++) {
      int lr = lrow[mi];
      asm volatile("" : "+v"(lr));
      cv[mi] = row0 + lr < rows ? a.cvec[(long)b * a.c * hq + row_off(row0 + lr)] : 0.f;
    }
    for (int part = 0; part < 2; part++) {
      lds_barrier();
      for (int idx = wave * 64 + lB; idx < DH * TT; idx += 256) {
        const int aa = idx % DH, yb = idx / DH;
        float v16[16];
        if (aa < 16 * (yb + 1)) {
          const f32x4* src = (const f32x4*)(sg + 128 * yb * (yb + 1) + 16 * aa);
#pragma unroll
          for (int q = 0; q < 4; q++) {
            const f32x4 t4 = src[q];
#pragma unroll
            for (int v = 0; v < 4; v++) v16[4 * q + v] = t4[v];
          }
        } else {
#pragma unroll
          for (int q = 0; q < 16; q++) v16[q] = 0.f;
        }
        if (part == 1) {
#pragma unroll
          for (int q = 0; q < 16; q++) v16[q] -= (float)(T)v16[q];
        }
        *(v8*)(Mt + aa * LDM + 16 * yb) = pack8<T>(v16);
        *(v8*)(Mt + aa * LDM + 16 * yb + 8) = pack8<T>(v16 + 8);
      }
      lds_barrier();
#pragma unroll
      for (int mi = 0; mi < MT; mi++) {
        v8 xf[KS];
#pragma unroll
        for (int ks = 0; ks < KS; ks++) xf[ks] = *(const v8*)x_ptr(mi, 32 * ks + 8 * g2);
#pragma unroll
        for (int wt = 0; wt < TT; wt++) {
          f32x4 t = {0, 0, 0, 0};
#pragma unroll
          for (int ks = 0; ks < KS; ks++) {
            // (the operand fetches of lds_frag_tr / lds_frag, on this part's own copy of the lane indices)
            const T* pt = Mt + (32 * ks + 8 * g2 + (tc2 >> 2)) * LDM + 16 * wt + 4 * (tc2 & 3);
            const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((cb_lds_s16x4*)pt);
            const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((cb_lds_s16x4*)(pt + 4 * LDM));
            const v8 ut = __builtin_bit_cast(v8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
            t = mfma16(ut, xf[ks], t);                                                            // sum_a U[a, w] x[a]
            t = mfma16(*(const v8*)(Mt + (16 * wt + tc2) * LDM + 32 * ks + 8 * g2), xf[ks], t);   // sum_a U[w, a] x[a]
          }
          acc[mi][wt] += t * cv[mi];
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    // the gate's share through the state part: (q . dQ_state) / 2  (the rows are read again, from an address the
    // compiler cannot match with the first read: their values should not stay in registers through the sweep)
    uint32_t xt_b = xt_a;
    int lC = threadIdx.x & 63;
    asm volatile("" : "+v"(xt_b), "+v"(lC));
    const int g3 = lC >> 4;
#pragma unroll
    for (int mi = 0; mi < MT; mi++) {
      const int lr3 = wslice * 16 * MT + 16 * mi + (lC & 15);
      float dsum = 0.f;
#pragma unroll
      for (int nt = 0; nt < NT; nt++) {
        const int col = 16 * nt + 4 * g3;
        const v4 q4 = *(const __attribute__((address_space(3))) v4*)(xt_b + lr3 * (DH * 2) + (((col / 8) ^ swz<CPR>(lr3)) * 16) + (col % 8) * 2);
#pragma unroll
        for (int v = 0; v < 4; v++) dsum = __builtin_fmaf((float)q4[v], acc[mi][nt][v], dsum);
      }
      tot[mi] += sum_over_rows(dsum - dot0[mi]) * 0.5f;
    }
  }

#pragma unroll
  for (int mi = 0; mi < MT; mi++) {
    int lr = lrow[mi];
    asm volatile("" : "+v"(lr));
    if (row0 + lr >= rows) continue;
    const long ro = row_off(row0 + lr);
#pragma unroll
    for (int nt = 0; nt < NT; nt++) {
      float o4[4];
#pragma unroll
      for (int v = 0; v < 4; v++) o4[v] = acc[mi][nt][v];
      *(v4*)(dQg + ro * DH + 16 * nt + 4 * g2) = pack4<T>(o4);
    }
    if (g2 == 0 && a.dGq) a.dGq[(long)b * a.c * hq + ro] = tot[mi];
  }
}

template <typename T, int DH> static int chunk_bwd_dq_launch(const ChunkBwdDqArgs& a, int BN, hipStream_t st) {
  constexpr size_t smem = CB_NST * (2 * CB_BN * DH * 2 + 4 * CB_BN * 4) + 128 * sizeof(float);
  const int rows = a.c * a.r, nblocks = (rows + 127) / 128, npairs = BN * a.h;
  dim3 grid((unsigned)((npairs + 31) / 32 * 32 * nblocks));
  auto kern = chunk_bwd_dq_kernel<T, DH>;
  allow_big_lds((const void*)kern, smem);
  PR_LAUNCH("chunk_bwd_dq", kern, grid, dim3(256), smem, st, a, nblocks, npairs);
  return (int)hipGetLastError();
}

// 1 where the one-kernel query side exists: bf16, head dim 32 or 64 (and a chunk of at least 64 keys' worth of ring)
int chunk_bwd_dq_supported(int d, int dtype) { return dtype == DT_BF16 && (d == 32 || d == 64); }

int chunk_bwd_dq(const ChunkBwdDqArgs& a, int BN, int d, int dtype, hipStream_t st) {
  if (dtype != DT_BF16) return -1;
  switch (d) {
    case 32: return chunk_bwd_dq_launch<bf16_t, 32>(a, BN, st);
    case 64: return chunk_bwd_dq_launch<bf16_t, 64>(a, BN, st);
    default: return -2;
  }
}

}  // namespace pr
