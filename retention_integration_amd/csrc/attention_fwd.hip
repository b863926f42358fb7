// Causal power attention, forward (ref: retention/_attention/reference.py:10-69).
//
//   s = scale * q.k,  z = deg*log(|s| + 1e-7) + G_q - G_k  (masked to keys j <= i + tk - tq),
//   m = max_j z,  P = exp(z - m),  l = sum_j P + 1e-6,  o = P V
//   norm: returns o / l;  otherwise (o, l, m).
//
// Query rows of the r query heads that share a kv head are folded into one row axis of length tq*r.
// A workgroup = 4 waves owns 64*MT folded rows of one (batch, kv head); keys stream 64 at a time through a
// 3-deep ring of asynchronous global->LDS copies.  All products are formed transposed (S^T = K Q^T,
// O^T = V^T P^T) so that the accumulator layout of S^T is directly the operand layout of the second
// contraction and no data moves between lanes; row statistics live one row per lane column.
//
// The weights are evaluated without logarithms: w = exp(z) = (|s| + 1e-7)^deg * exp(G_q - G_k) is accumulated
// unnormalised (w <= (|s|+eps)^deg because gates only decay), its running maximum is tracked, and the row is
// divided by max_j w at the end, which gives exactly the exp(z - m) sums.  For key tiles entirely in a wave's
// past the gate factor is split as exp(G_q - R) * exp(R - G_k) with R the gate at the tile's last key, so the
// exponentials are per row and per key, not per pair; only the tile on the wave's diagonal evaluates
// exp(G_q - G_k) per pair, and tiles entirely in the wave's future are skipped.  The row sums come from the
// matrix cores as well (an all-ones operand against the rounded weights), so o / l is an exact average
// (ref rounds p before summing: retention/_attention/reference.py:52-55).
#include "common.h"
#include "kernels.h"

namespace pr {

constexpr int AT_BN = 64;
// stages in the ring: three up to d = 64; two at d = 128, where three would leave room for one workgroup per CU
constexpr int at_stages(int d) { return d <= 64 ? 3 : 2; }
constexpr float AT_LOG_EPS = 1e-7f, AT_SUM_EPS = 1e-6f, AT_EXP_CLAMP = 80.f;
constexpr float AT_LOG2E = 1.4426950408889634f, AT_EXP2_CLAMP = AT_EXP_CLAMP * AT_LOG2E;

template <typename T> struct OnesBits;
template <> struct OnesBits<bf16_t> { static constexpr uint32_t v = 0x3F803F80u; };
template <> struct OnesBits<f16_t> { static constexpr uint32_t v = 0x3C003C00u; };

// (s^2 + eps^2)^half_deg, which stands in for (|s| + eps)^(2*half_deg): equal at s = 0 and within a relative
// 2*eps/|s| elsewhere, and it needs neither the absolute value nor a separate addition.
template <bool DEG2> __device__ __forceinline__ float pow_even(float sv, float eps2, int half_deg) {
  const float a2 = __builtin_fmaf(sv, sv, eps2);
  float p = a2;
  if (!DEG2)
    for (int k = 1; k < half_deg; k++) p *= a2;
  return p;
}

template <typename T, int DH, int MT, bool DEG2, int OCC>
__global__ __launch_bounds__(256, OCC) void attention_fwd_kernel(AttnFwdArgs a, int row_blocks, int npairs, int gate_skip) {
  typedef typename VecOf<T>::v8 v8;
  typedef typename VecOf<T>::v4 v4;
  typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
  typedef __attribute__((address_space(3))) v8 lds_v8;
  typedef __attribute__((address_space(3))) f32x4 lds_f32x4;
  typedef __attribute__((address_space(3))) char lds_char;
  constexpr int KS = DH / 32, NT = DH / 16, KT = AT_BN / 16, ROWS = 64 * MT, CPR = DH / 8, RB = CPR * 16;
  constexpr int TILE = AT_BN * RB;                  // bytes of one K or V tile
  constexpr int STAGE = 2 * TILE + 4 * AT_BN * 4;   // K, V, raw gates, two sets of key gate factors
  constexpr int LOADS = 2 * AT_BN * CPR / 256;      // tile copies per thread per stage
  constexpr int NST = at_stages(DH);
  extern __shared__ __attribute__((aligned(1024))) char smem[];

  const int tid = threadIdx.x, l = tid & 63, g = l >> 4, tcol = l & 15;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // wave-uniform, so branches on it are scalar
  // Workgroups are dealt round-robin by their linear index: to the 8 XCDs first, then inside an XCD to its 4
  // shader engines (index / 8 % 4); only the CU inside a shader engine is chosen by load.  Row blocks differ in
  // length (causal), so each of the 32 (XCD, shader engine) groups is given whole (batch, kv head) pairs: every
  // group then gets the same mix of long and short row blocks and the K/V of a pair stay in one L2.  Inside a
  // group the pairs follow one another, longest row block first, so that the row blocks of a pair run together.
  const int grp = blockIdx.x % 32, u = blockIdx.x / 32, ppg = (npairs + 31) / 32;
  // (the last few pairs of a group are interleaved, see deal_causal_blocks)
  int pig, blk;
  deal_causal_blocks(u, row_blocks, ppg, pig, blk);
  const int pair = pig * 32 + grp;
  const int rblk = row_blocks - 1 - blk;
  if (pair >= npairs) return;
  const int b = __builtin_amdgcn_readfirstlane(pair / a.h), hh = pair - b * a.h;
  const int hq = a.h * a.r, rows = a.tq * a.r, shift = a.tk - a.tq;
  // every other workgroup hands its 16*MT-row slices to the waves in reverse order: the wave nearest the
  // diagonal has the most tiles, and co-resident workgroups then load the four SIMDs evenly
  const int row0 = rblk * ROWS;
  const T* Qg = (const T*)a.Q + (long)b * a.tq * hq * DH;
  const char* Kg = (const char*)((const T*)a.K + (long)b * a.kv_rows * a.h * DH + hh * DH);
  const char* Vg = (const char*)((const T*)a.V + (long)b * a.kv_rows * a.h * DH + hh * DH);
  const float* Gg = a.G ? a.G + (long)b * a.kv_rows * a.h + hh : nullptr;
  const long kstride = (long)a.h * DH * 2;
  const int half_deg = (int)a.deg / 2;
  const float eps_s = AT_LOG_EPS / a.scale;          // |scale*x| + eps = scale * (|x| + eps/scale)
  const float l2sp = a.deg * __log2f(a.scale);

  const int last_row = min(row0 + ROWS, rows) - 1;
  const int kmax = min(a.tk, last_row / a.r + shift + 1);   // keys any row of the workgroup can see
  const int ntiles = (kmax + AT_BN - 1) / AT_BN;
  const int wslice = (u & 1) ? 3 - wave : wave;
  const int wrow0 = row0 + wslice * 16 * MT;
  const int w_first_ti = min(wrow0, rows - 1) / a.r + shift;               // smallest time index in the wave
  const int w_last_ti = min(wrow0 + 16 * MT - 1, rows - 1) / a.r + shift;  // largest

  // Copies of one stage: every thread owns LOADS/2 16-byte chunks of the K tile and the same chunks of the V tile.
  // Its byte offsets inside a tile are fixed, so a full tile costs no address arithmetic beyond a scalar base.
  uint32_t goff[LOADS / 2];
#pragma unroll
  for (int ii = 0; ii < LOADS / 2; ii++) {
    const int pos = (ii * 4 + wave) * 64 + l, row = pos / CPR;
    goff[ii] = (uint32_t)(row * (int)kstride + 16 * ((pos % CPR) ^ swz<CPR, SWZ_ROW>(row)));
  }
  auto issue = [&](int it) __attribute__((always_inline)) {
    char* st = smem + (it % NST) * STAGE;
    const int j0 = it * AT_BN;
    if (j0 + AT_BN <= a.tk) {
      const char* kb_ = Kg + (long)j0 * kstride;
      const char* vb_ = Vg + (long)j0 * kstride;
      const uint32_t sa = lds_addr(st) + wave * 1024;
#pragma unroll
      for (int ii = 0; ii < LOADS / 2; ii++) async_copy16_sv(kb_, goff[ii], sa + ii * 4096);
#pragma unroll
      for (int ii = 0; ii < LOADS / 2; ii++) async_copy16_sv(vb_, goff[ii], sa + TILE + ii * 4096);
    } else {   // last, partial tile: rows past the end repeat the last key (they are masked)
      async_load_tile<CPR, AT_BN, SWZ_ROW>(st, [&](int row) { return Kg + (long)min(j0 + row, a.tk - 1) * kstride; });
      async_load_tile<CPR, AT_BN, SWZ_ROW>(st + TILE, [&](int row) { return Vg + (long)min(j0 + row, a.tk - 1) * kstride; });
    }
    if (Gg && wave == 0) async_copy4(Gg + (long)min(j0 + l, a.tk - 1) * a.h, st + 2 * TILE);
  };
  // What the gates have already forgotten.  A key tile entirely in a wave's past enters with the wave-uniform factor
  // exp(R - A_last) (R: gate sum at the wave's first row, A_last: at the tile's last key; see the tile code).  Once that
  // factor has underflowed to zero for the LARGEST gate sum among the workgroup's rows (its first row's: gate sums only
  // fall along a sequence, unless the caller's log gates are positive) it is zero for every wave: the oldest tiles for
  // which it has, as far as they lie before the workgroup's first row, contribute exact zeros and are neither copied nor
  // visited (it0 = the first tile that is); a wave also returns from a past tile whose factor is zero for its own rows.
  int it0 = 0;
  if (Gg && gate_skip) {
    float a_max = -INFINITY;
    for (int i = l; i < ROWS; i += 64) a_max = fmaxf(a_max, Gg[(long)(min(row0 + i, rows - 1) / a.r + shift) * a.h]);
    const float a_last0 = Gg[(long)min(AT_BN * min(l, ntiles - 1) + AT_BN - 1, a.tk - 1) * a.h];
#pragma unroll
    for (int m = 32; m > 0; m >>= 1) a_max = fmaxf(a_max, __shfl_xor(a_max, m));
    for (int base = 0; base < ntiles; base += 64) {
      const int tl = min(base + l, ntiles - 1);
      const float a_last = base == 0 ? a_last0 : Gg[(long)min(AT_BN * tl + AT_BN - 1, a.tk - 1) * a.h];
      const unsigned long long dead = __ballot(__expf(fminf(a_max - a_last, AT_EXP_CLAMP)) == 0.f);
      const int lanes = min(64, ntiles - base);
      const int nd = __builtin_popcountll(lanes == 64 ? dead : (dead & ((1ull << lanes) - 1)));
      it0 += nd;
      if (nd < lanes) break;
    }
    it0 = __builtin_amdgcn_readfirstlane(min(min(it0, ntiles - 1), min(row0 / a.r + shift + 1, a.tk) / AT_BN));
  }
  issue(it0);
  if (NST == 3 && ntiles > it0 + 1) issue(it0 + 1);

  v8 Qf[MT][KS];
  int ti[MT];
  long qoff[MT];
  bool live[MT];
  float Gq2[MT], mx[MT];   // Gq2 = log2(scale^deg exp(G_q))
  constexpr bool TWO_PASS = sizeof(T) == 2 && !__is_same(T, bf16_t);   // fp16
  float pn[MT], prow[MT];   // (second pass) 1 / row maximum, and that times the past tiles' row factor
#pragma unroll
  for (int mi = 0; mi < MT; mi++) {
    const int row = wrow0 + 16 * mi + tcol;
    live[mi] = row < rows;
    const int rr = live[mi] ? row : 0;
    const int t = rr / a.r;
    ti[mi] = t + shift;
    qoff[mi] = (long)t * hq + hh * a.r + (rr - t * a.r);
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      u32x4 z = {0, 0, 0, 0};
      if (live[mi]) z = *(const u32x4*)(Qg + qoff[mi] * DH + 32 * ks + 8 * g);
      Qf[mi][ks] = __builtin_bit_cast(v8, z);
    }
    Gq2[mi] = __builtin_fmaf(Gg ? Gg[(long)ti[mi] * a.h] : 0.f, AT_LOG2E, l2sp);
    mx[mi] = 0.f;
  }
  f32x4 acc[MT][NT], accl[MT];
#pragma unroll
  for (int mi = 0; mi < MT; mi++) {
#pragma unroll
    for (int nt = 0; nt < NT; nt++) acc[mi][nt] = (f32x4){0, 0, 0, 0};
    accl[mi] = (f32x4){0, 0, 0, 0};
  }
  const float eps2 = eps_s * eps_s;
  const float Rw = Gg ? Gg[(long)w_first_ti * a.h] : 0.f;   // gate at the wave's first row
  const uint32_t one2 = OnesBits<T>::v;
  v8 ones = __builtin_bit_cast(v8, (u32x4){one2, one2, one2, one2});
  asm volatile("" : "+v"(ones));   // keep the four registers instead of rebuilding them at every use

  // Per-lane LDS byte offsets; the swizzle depends only on the lane's row inside a 16-row group.
  int koff[KS], voff[NT];
#pragma unroll
  for (int ks = 0; ks < KS; ks++) koff[ks] = tcol * RB + (((4 * ks + g) ^ swz<CPR, SWZ_ROW>(tcol)) * 16);
  {
    const int vr = 4 * g + (tcol >> 2);   // V^T operand: row 4g + (s>>2) of a 16-key group, columns 16*nt + 4*(s&3) ..
#pragma unroll
    for (int nt = 0; nt < NT; nt++) {
      const int col = 16 * nt + 4 * (tcol & 3);
      voff[nt] = vr * RB + (((col / 8) ^ swz<CPR, SWZ_ROW>(vr)) * 16) + (col % 8) * 2;
    }
  }

  // Every wave runs ntiles steps with one barrier each, split by what the tile is to THIS wave: tiles entirely in
  // its past (no masking code at all), tiles that cross its diagonal, and tiles entirely in its future, for
  // which it only takes part in the copies and the barrier.  Three loops instead of one loop with branches keep
  // the accumulators in place (no copies between control-flow paths).
  const int n_past = min(ntiles, min(w_first_ti + 1, a.tk) / AT_BN);   // tiles with every pair visible
  const int n_seen = min(ntiles, w_last_ti / AT_BN + 1);               // tiles with at least one visible pair

  // Gate factors of tile `it`, written by wave 0 (it issued the gate copy, so it alone can wait for it):
  // exp(R - gate) relative to the tile's last key (<= 1) and relative to the first key of each 16-key group (>= 1).
  auto gate_factors = [&](int it) __attribute__((always_inline)) {
    float* graw = (float*)(smem + (it % NST) * STAGE + 2 * TILE);
    const int rpos = min(AT_BN - 1, a.tk - 1 - it * AT_BN);
    const float gv = Gg ? graw[l] : 0.f;
    const float R_ = Gg ? graw[rpos] : 0.f;
    graw[AT_BN + l] = __expf(fminf(R_ - gv, AT_EXP_CLAMP));
    graw[2 * AT_BN + l] = gv * AT_LOG2E;   // the gate itself, in powers of two, for the diagonal tiles
    if (!Gg) graw[l] = 0.f;
  };
  if (wave == 0) {
    wait_vmcnt<0>();
    gate_factors(it0);
  }
  // Make tile `it` visible to the workgroup, start the copy of tile it+2, and (wave 0) prepare the gate factors of
  // tile it+1 while the others already compute.
  auto sync_step = [&](int it) __attribute__((always_inline)) -> char* {
    char* st = smem + (it % NST) * STAGE;
    if constexpr (NST == 3) {
      if (it + 1 < ntiles) wait_vmcnt<LOADS>(); else wait_vmcnt<0>();
      lds_barrier();
      if (it + 2 < ntiles) issue(it + 2);
      if (wave == 0 && it + 1 < ntiles) {
        if (it + 2 < ntiles) wait_vmcnt<LOADS + 1>(); else wait_vmcnt<0>();   // all but the stage just issued
        gate_factors(it + 1);
      }
    } else {
      wait_vmcnt<0>();   // one stage in flight
      lds_barrier();
      if (it + 1 < ntiles) issue(it + 1);
    }
    return st;
  };
  // two-stage ring: wave 0 prepares the next tile's factors after its own work on this one
  auto after_step = [&](int it) __attribute__((always_inline)) {
    if constexpr (NST == 2) {
      if (wave == 0 && it + 1 < ntiles) {
        wait_vmcnt<0>();
        gate_factors(it + 1);
      }
    }
  };

  // One 64-key tile.  Past tiles use one reference gate (the tile's last key), so both gate factors are <= 1.
  // Diagonal tiles use the first key of every 16-key group instead: for every visible pair the row factor is
  // then <= 1 and the key factor spans only 16 steps of decay, so neither leaves the fp32 range.
  // MODE 0: weights in absolute terms, the row maximum divides the result at the end (bf16: its exponent range
  // covers any row).  fp16 needs the reference's normalisation -- weights relative to the row maximum, <= 1 -- or
  // a row whose largest weight is below 6e-8 would lose all of them: it runs the tiles twice, MODE 1 only for the
  // row maxima (no V, no packing, no accumulation), then MODE 2 with every weight divided by its row's maximum.
  auto tile = [&](int it, const char* st, auto diag_c, auto mode_c) __attribute__((always_inline)) {
    constexpr bool DIAG = decltype(diag_c)::value != 0;
    constexpr int MODE = decltype(mode_c)::value;
    const int j0 = it * AT_BN;
    const float* graw = (const float*)(st + 2 * TILE);
    // LDS byte addresses of this lane's operands; opaque, so that the per-group and per-column-tile displacements
    // stay immediate offsets of the loads instead of one address register each
    uint32_t kb[KS], vb[NT], eb;
    {
      const uint32_t sa = (uint32_t)(uintptr_t)(lds_char*)st;
#pragma unroll
      for (int ks = 0; ks < KS; ks++) { kb[ks] = sa + koff[ks]; asm volatile("" : "+v"(kb[ks])); }
#pragma unroll
      for (int nt = 0; nt < NT; nt++) { vb[nt] = sa + TILE + voff[nt]; asm volatile("" : "+v"(vb[nt])); }
      eb = sa + 2 * TILE + (DIAG ? 2 * AT_BN : AT_BN) * 4 + 16 * g;
      asm volatile("" : "+v"(eb));
    }
    float eu[MT];
    int lim[MT];
#pragma unroll
    for (int mi = 0; mi < MT; mi++) {
      if (DIAG) lim[mi] = min(ti[mi], a.tk - 1) - j0 - 4 * g;   // pair (row, key 16*kt + 4g + v) visible iff 16*kt + v <= lim
      else eu[mi] = MODE == 2 ? prow[mi] : 1.f;
    }
    // past tiles: key factors relative to the gate at the wave's first row (<= 1 for every past key)
    const float cw = DIAG ? 1.f : __expf(fminf(Rw - graw[AT_BN - 1], AT_EXP_CLAMP));
    // (forgotten by this wave's rows, though not by the workgroup's first: every weight of the tile is an exact zero)
    if (!DIAG && gate_skip && __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, cw)) == 0) return;
#pragma unroll
    for (int kp = 0; kp < KT / 2; kp++) {
      if (DIAG && j0 + 32 * kp > w_last_ti) continue;   // these 32 keys come after every row of the wave
      // S^T for 32 keys: operands first, then every product, so the matrix pipe runs back to back
      v8 kf[2][KS];
      f32x4 ev[2];
#pragma unroll
      for (int half = 0; half < 2; half++) {
#pragma unroll
        for (int ks = 0; ks < KS; ks++) kf[half][ks] = *(const lds_v8*)(kb[ks] + (2 * kp + half) * 16 * RB);
        ev[half] = *(const lds_f32x4*)(eb + 64 * (2 * kp + half));
        if (!DIAG) ev[half] *= cw;
      }
      f32x4 sc[2][MT];
#pragma unroll
      for (int half = 0; half < 2; half++)
#pragma unroll
        for (int mi = 0; mi < MT; mi++) sc[half][mi] = (f32x4){0, 0, 0, 0};
#pragma unroll
      for (int ks = 0; ks < KS; ks++)
#pragma unroll
        for (int half = 0; half < 2; half++)
#pragma unroll
          for (int mi = 0; mi < MT; mi++) sc[half][mi] = mfma16(kf[half][ks], Qf[mi][ks], sc[half][mi]);
      // V^T operands for the same 32 keys, in flight while the weights are formed
      v8 vf[NT];
#pragma unroll
      for (int nt = 0; MODE != 1 && nt < NT; nt++) {
        const uint32_t vp = vb[nt] + kp * 32 * RB;
        const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)vp);
        const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(vp + 16 * RB));
        const s16x8 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        vf[nt] = __builtin_bit_cast(v8, both);
      }
      v8 pf[MT];
#pragma unroll
      for (int mi = 0; mi < MT; mi++) {
        float p[8];
#pragma unroll
        for (int half = 0; half < 2; half++) {
#pragma unroll
          for (int v = 0; v < 4; v++) {
            float w = pow_even<DEG2>(sc[half][mi][v], eps2, half_deg);
            if (DIAG) {
              // the pair's own exponent: no reference gate shared by a group of keys, whose two factors could leave
              // the fp32 range against each other where the gates fall steeply
              w *= __builtin_amdgcn_exp2f(fminf(Gq2[mi] - ev[half][v], AT_EXP2_CLAMP));
              if (MODE == 2) w *= pn[mi];
              w = (32 * kp + 16 * half + v <= lim[mi]) ? w : 0.f;
            } else {
              w *= ev[half][v];
              if (MODE == 2) w *= eu[mi];
            }
            p[4 * half + v] = w;
          }
        }
        if (MODE != 2) {
#pragma unroll
          for (int e = 0; e < 8; e++) mx[mi] = fmaxf(mx[mi], p[e]);
        }
        if (MODE != 1) pf[mi] = pack8<T>(p);
      }
      if constexpr (MODE != 1) {
        // O^T += V^T P^T over these 32 keys (elements 0-3 are keys 4g.. of the first 16, 4-7 of the second 16);
        // the all-ones operand adds the row sums of the rounded weights
#pragma unroll
        for (int mi = 0; mi < MT; mi++) accl[mi] = mfma16(ones, pf[mi], accl[mi]);
#pragma unroll
        for (int nt = 0; nt < NT; nt++)
#pragma unroll
          for (int mi = 0; mi < MT; mi++) {
            acc[mi][nt] = mfma16(vf[nt], pf[mi], acc[mi][nt]);
          }
      }
    }
  };

  auto run_pass = [&](auto mode_c) __attribute__((always_inline)) {
    constexpr int MODE = decltype(mode_c)::value;
    int it = it0;
    for (; it < n_past; it++) {
      tile(it, sync_step(it), IC<0>{}, mode_c);
      after_step(it);
    }
    // the past tiles were accumulated without the row factor exp(G_q - Rw) * scale^deg; apply it once
    if constexpr (MODE != 2) {
#pragma unroll
      for (int mi = 0; mi < MT; mi++) {
        const float f = __builtin_amdgcn_exp2f(fminf(Gq2[mi] - Rw * AT_LOG2E, AT_EXP2_CLAMP));
        if (MODE == 0) {
#pragma unroll
          for (int nt = 0; nt < NT; nt++) acc[mi][nt] *= f;
          accl[mi] *= f;
        }
        mx[mi] *= f;
      }
    }
    for (; it < n_seen; it++) {
      tile(it, sync_step(it), IC<1>{}, mode_c);
      after_step(it);
    }
    for (; it < ntiles; it++) {
      sync_step(it);
      after_step(it);
    }
  };
  if constexpr (TWO_PASS) {
    run_pass(IC<1>{});
#pragma unroll
    for (int mi = 0; mi < MT; mi++) {
      mx[mi] = max_over_rows(mx[mi]);
      pn[mi] = mx[mi] > 0.f ? 1.f / mx[mi] : 0.f;
      prow[mi] = __builtin_amdgcn_exp2f(fminf(Gq2[mi] - Rw * AT_LOG2E, AT_EXP2_CLAMP)) * pn[mi];
    }
    lds_barrier();   // every wave is done with the ring: start the copies over
    issue(it0);
    if (NST == 3 && ntiles > it0 + 1) issue(it0 + 1);
    if (wave == 0) {
      wait_vmcnt<0>();
      gate_factors(it0);
    }
    run_pass(IC<2>{});
  } else {
    run_pass(IC<0>{});
  }

  T* Og = (T*)a.O + (long)b * a.tq * hq * DH;
#pragma unroll
  for (int mi = 0; mi < MT; mi++) {
    const float wmax = TWO_PASS ? mx[mi] : max_over_rows(mx[mi]);   // = exp(rowmax)
    if (!live[mi]) continue;
    const float wsum = accl[mi][0];             // every accumulator row of the all-ones product holds the row sum
    const float inv = TWO_PASS ? 1.f : 1.f / wmax;
    const float lrow = wsum * inv + AT_SUM_EPS;
    const float f = a.norm ? inv / lrow : inv;
#pragma unroll
    for (int nt = 0; nt < NT; nt++) {
      float o4[4];
#pragma unroll
      for (int v = 0; v < 4; v++) o4[v] = acc[mi][nt][v] * f;
      *(v4*)(Og + qoff[mi] * DH + 16 * nt + 4 * g) = pack4<T>(o4);
    }
    if (g == 0) {
      const long o = (long)b * a.tq * hq + qoff[mi];
      if (a.l) a.l[o] = lrow;
      if (a.rowmax) a.rowmax[o] = __logf(wmax);
    }
  }
}

template <typename T, int DH, bool DEG2> static int attn_fwd_launch(const AttnFwdArgs& a, int B, hipStream_t st) {
  const int rows = a.tq * a.r;
  auto go = [&](auto mt, auto occ) {
    constexpr int MT = decltype(mt)::value, OCC = decltype(occ)::value;
    constexpr size_t smem = at_stages(DH) * (2 * AT_BN * DH * 2 + 4 * AT_BN * 4);
    const int row_blocks = (rows + 64 * MT - 1) / (64 * MT), npairs = B * a.h;
    dim3 grid((unsigned)(((npairs + 31) / 32) * 32 * row_blocks));
    auto kern = attention_fwd_kernel<T, DH, MT, DEG2, OCC>;
    allow_big_lds((const void*)kern, smem);
    PR_LAUNCH("attention_fwd", kern, grid, dim3(256), smem, st, a, row_blocks, npairs, g_gate_skip);
  };
  // 128 rows per workgroup: 123 registers at d = 32 (four workgroups per CU), 166 at d = 64 (three); measured 9 % and
  // 6 % faster than 256 rows at two workgroups -- the kernel is mostly vector work, which issues faster with more
  // waves resident, and that outweighs streaming K and V twice as often
  if (rows > 64) go(IC<2>{}, IC<2>{});
  else go(IC<1>{}, IC<2>{});
  return (int)hipGetLastError();
}

int attention_fwd(const AttnFwdArgs& a, int B, int d, int dtype, hipStream_t st) {
  const bool deg2 = a.deg == 2.f;
#define PR_AF(T)                                                                                                       \
  switch (d) {                                                                                                         \
    case 32: return deg2 ? attn_fwd_launch<T, 32, true>(a, B, st) : attn_fwd_launch<T, 32, false>(a, B, st);           \
    case 64: return deg2 ? attn_fwd_launch<T, 64, true>(a, B, st) : attn_fwd_launch<T, 64, false>(a, B, st);           \
    case 128: return deg2 ? attn_fwd_launch<T, 128, true>(a, B, st) : attn_fwd_launch<T, 128, false>(a, B, st);        \
    default: return -2;                                                                                                \
  }
  if (dtype == DT_BF16) { PR_AF(bf16_t) }
  if (dtype == DT_F16) { PR_AF(f16_t) }
#undef PR_AF
  return -1;
}

}  // namespace pr
