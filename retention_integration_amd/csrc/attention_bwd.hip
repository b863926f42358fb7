// Causal power attention, backward (formulas: autograd of retention/_attention/reference.py:42-69;
// cross-check retention/_attention/triton.py:248-387).  Inputs are the forward's operands, its row
// maximum m, and the gradients dO (of the unnormalised o) and dl (of the row sum l):
//
//   P = exp(z - m),  dP = dO V^T + dl,  dz = P * dP,  dV = P^T dO,
//   dGq_i = sum_j dz_ij,  dGk_j = -sum_i dz_ij,
//   d(q.k) = dz * deg * sign(s) / (|q.k| + 1e-7/scale),  dQ = d(q.k) K,  dK = d(q.k)^T Q.
//
// Two kernels, each recomputing P: one owns query rows and walks the keys (dQ, dGq), the other owns keys and walks
// the query rows (dK, dV, dGk).  Products are oriented so that every accumulator layout is already the operand
// layout of the next contraction (see attention_fwd.hip), and the streamed operand goes through a 3-deep ring of
// asynchronous global->LDS copies.
//
// No logarithm or division per pair.  As in the forward, a2 = (q.k)^2 + (eps/scale)^2 stands in for
// (|q.k| + eps/scale)^2, so P = a2^(deg/2) * E with E = scale^deg * exp(G_q - m - G_k), and
//   d(q.k)/deg = (q.k) * a2^(deg/2 - 1) * E * dP,      dz = a2^(deg/2) * E * dP.
// E is split into a per-row and a per-key exponential around a reference gate chosen so that both stay in range:
// pairs well off the diagonal share one reference per wave or workgroup and the factor that is constant along the
// accumulation (per row for dQ, per key for dK/dV) is applied once to the accumulators; pairs near the diagonal
// use a reference per group of 16 keys and are masked per pair.
#include "common.h"
#include "kernels.h"

namespace pr {

constexpr int AB_BN = 64;    // keys per stage in the dQ kernel
constexpr int AB_BM = 64;    // query rows per stage in the dK/dV kernel
// stages in the ring: three up to d = 64; two at d = 128, where three would leave room for one workgroup per CU
constexpr int ab_stages(int d) { return d <= 64 ? 3 : 2; }
constexpr float AB_LOG_EPS = 1e-7f, AB_EXP_CLAMP = 80.f;
constexpr float AB_LOG2E = 1.4426950408889634f, AB_EXP2_CLAMP = AB_EXP_CLAMP * AB_LOG2E;

// a2^(half_deg - 1)
template <bool DEG2> __device__ __forceinline__ float pow_hm1(float a2, int half_deg) {
  if (DEG2) return 1.f;
  float p = 1.f;
  for (int k = 1; k < half_deg; k++) p *= a2;
  return p;
}

typedef __attribute__((address_space(3))) s16x4 ab_lds_s16x4;
typedef __attribute__((address_space(3))) f32x4 ab_lds_f32x4;
typedef __attribute__((address_space(3))) char ab_lds_char;

template <typename T> __device__ __forceinline__ typename VecOf<T>::v8 ab_tr8(uint32_t lo_addr, uint32_t hi_addr) {
  const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((ab_lds_s16x4*)lo_addr);
  const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((ab_lds_s16x4*)hi_addr);
  const s16x8 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  return __builtin_bit_cast(typename VecOf<T>::v8, both);
}

// ------------------------------------------------------------------ dQ, dGq
template <typename T, int DH, int MT, bool DEG2, int OCC>
__global__ __launch_bounds__(256, OCC) void attention_bwd_dq_kernel(AttnBwdArgs a, int nblocks, int npairs, int gate_skip) {
  typedef typename VecOf<T>::v8 v8;
  typedef typename VecOf<T>::v4 v4;
  typedef __attribute__((address_space(3))) v8 lds_v8;
  typedef __attribute__((address_space(3))) v4 lds_v4;
  constexpr int KS = DH / 32, NT = DH / 16, KT = AB_BN / 16, ROWS = 64 * MT, CPR = DH / 8, RB = CPR * 16;
  constexpr int TILE = AB_BN * RB;
  constexpr int STAGE = 2 * TILE + 4 * AB_BN * 4;   // K, V, raw gates, two sets of key gate factors
  constexpr int NST = ab_stages(DH);
  constexpr int LOADS = 2 * AB_BN * CPR / 256;
  extern __shared__ __attribute__((aligned(1024))) char smem[];

  // Workgroups are dealt round-robin by their linear index to the 8 XCDs and then to the 4 shader engines of an
  // XCD; only the CU inside a shader engine is chosen by load.  Blocks differ in length (causal), so each of the 32
  // (XCD, shader engine) groups gets whole (batch, kv head) pairs, pair after pair with the longest block of a pair
  // first: the blocks of a pair run at the same time and share its rows in the XCD's L2 (dealing the longest blocks
  // of ALL pairs first instead fetches 2.5x the bytes from HBM); only the last few pairs of a group are interleaved,
  // see deal_causal_blocks.
  const int grp = blockIdx.x % 32, u = blockIdx.x / 32, ppg = (npairs + 31) / 32;
  int pig, blk;
  deal_causal_blocks(u, nblocks, ppg, pig, blk);
  const int pair = pig * 32 + grp;
  if (pair >= npairs) return;
  const int tid = threadIdx.x, l = tid & 63, g = l >> 4, tcol = l & 15;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int b = __builtin_amdgcn_readfirstlane(pair / a.h), hh = pair - b * a.h;
  const int hq = a.h * a.r, rows = a.tq * a.r, shift = a.tk - a.tq;
  const int row0 = (nblocks - 1 - blk) * ROWS;   // late rows see the most keys
  const T* Qg = (const T*)a.Q + (long)b * a.tq * hq * DH;
  const T* dOg = (const T*)a.dO + (long)b * a.tq * hq * DH;
  const char* Kg = (const char*)((const T*)a.K + (long)b * a.tk * a.h * DH + hh * DH);
  const char* Vg = (const char*)((const T*)a.V + (long)b * a.tk * a.h * DH + hh * DH);
  const float* Gg = a.G ? a.G + (long)b * a.tk * a.h + hh : nullptr;
  const long kstride = (long)a.h * DH * 2;
  const int half_deg = (int)a.deg / 2;
  const float eps_s = AB_LOG_EPS / a.scale, eps2 = eps_s * eps_s;
  const float l2sp = a.deg * __log2f(a.scale);

  const int last_row = min(row0 + ROWS, rows) - 1;
  const int kmax = min(a.tk, last_row / a.r + shift + 1);
  const int ntiles = (kmax + AB_BN - 1) / AB_BN;
  const int wslice = (u & 1) ? 3 - wave : wave;   // alternate which wave is nearest the diagonal
  const int wrow0 = row0 + wslice * 16 * MT;
  const int w_first_ti = min(wrow0, rows - 1) / a.r + shift;
  const int w_last_ti = min(wrow0 + 16 * MT - 1, rows - 1) / a.r + shift;

  uint32_t goff[LOADS / 2];
#pragma unroll
  for (int ii = 0; ii < LOADS / 2; ii++) {
    const int pos = (ii * 4 + wave) * 64 + l, row = pos / CPR;
    goff[ii] = (uint32_t)(row * (int)kstride + 16 * ((pos % CPR) ^ swz<CPR, SWZ_ROW>(row)));
  }
  // With the chunked epilogue the workgroup's rows of dQs ride through the ring as one more stage after the last
  // key tile (rows 0..63 in the K area, 64..127 in the V area), so that they arrive under the last tiles' work.
  const T* dQsg = a.dQs ? (const T*)a.dQs + (long)b * a.tq * hq * DH : nullptr;
  const int ntot = ntiles + (dQsg ? 1 : 0);
  auto issue = [&](int it) __attribute__((always_inline)) {
    char* st = smem + (it % NST) * STAGE;
    if (it >= ntiles) {
#pragma unroll
      for (int ii = 0; ii < LOADS; ii++) {
        const int pos = ((ii % (LOADS / 2)) * 4 + wave) * 64 + l, row = pos / CPR;
        const int fr = min(row0 + (ii / (LOADS / 2)) * AB_BN + row, rows - 1), t = fr / a.r;
        const long eo = ((long)t * hq + hh * a.r + (fr - t * a.r)) * DH;
        async_copy16((const char*)(dQsg + eo) + 16 * ((pos % CPR) ^ swz<CPR, SWZ_ROW>(row)),
                     st + (ii / (LOADS / 2)) * TILE + ((ii % (LOADS / 2)) * 4 + wave) * 1024);
      }
      if (Gg && wave == 0) async_copy4(Gg, st + 2 * TILE);   // keeps the count of copies per stage fixed
      return;
    }
    const int j0 = it * AB_BN;
    if (j0 + AB_BN <= a.tk) {
      const char* kb_ = Kg + (long)j0 * kstride;
      const char* vb_ = Vg + (long)j0 * kstride;
      const uint32_t sa = lds_addr(st) + wave * 1024;
#pragma unroll
      for (int ii = 0; ii < LOADS / 2; ii++) async_copy16_sv(kb_, goff[ii], sa + ii * 4096);
#pragma unroll
      for (int ii = 0; ii < LOADS / 2; ii++) async_copy16_sv(vb_, goff[ii], sa + TILE + ii * 4096);
    } else {   // last, partial tile: rows past the end repeat the last key (they are masked)
      async_load_tile<CPR, AB_BN, SWZ_ROW>(st, [&](int row) { return Kg + (long)min(j0 + row, a.tk - 1) * kstride; });
      async_load_tile<CPR, AB_BN, SWZ_ROW>(st + TILE, [&](int row) { return Vg + (long)min(j0 + row, a.tk - 1) * kstride; });
    }
    if (Gg && wave == 0) async_copy4(Gg + (long)min(j0 + l, a.tk - 1) * a.h, st + 2 * TILE);
  };
  // What the gates have already forgotten (as in attention_fwd.hip): the oldest key tiles whose factor exp(R - A_last)
  // has underflowed to zero for the largest gate sum among the workgroup's rows, as far as they lie before its first row,
  // contribute exact zeros to dQ and dGq and are neither copied nor visited; a wave also returns from a past tile whose
  // factor is zero for its own rows.
  int it0 = 0;
  if (Gg && gate_skip) {
    float a_max = -INFINITY;
    for (int i = l; i < ROWS; i += 64) a_max = fmaxf(a_max, Gg[(long)(min(row0 + i, rows - 1) / a.r + shift) * a.h]);
    const float a_last0 = Gg[(long)min(AB_BN * min(l, ntiles - 1) + AB_BN - 1, a.tk - 1) * a.h];
#pragma unroll
    for (int m = 32; m > 0; m >>= 1) a_max = fmaxf(a_max, __shfl_xor(a_max, m));
    for (int base_t = 0; base_t < ntiles; base_t += 64) {
      const int tl = min(base_t + l, ntiles - 1);
      const float a_last = base_t == 0 ? a_last0 : Gg[(long)min(AB_BN * tl + AB_BN - 1, a.tk - 1) * a.h];
      const unsigned long long dead = __ballot(__expf(fminf(a_max - a_last, AB_EXP_CLAMP)) == 0.f);
      const int lanes = min(64, ntiles - base_t);
      const int nd = __builtin_popcountll(lanes == 64 ? dead : (dead & ((1ull << lanes) - 1)));
      it0 += nd;
      if (nd < lanes) break;
    }
    it0 = __builtin_amdgcn_readfirstlane(min(min(it0, ntiles - 1), min(row0 / a.r + shift + 1, a.tk) / AB_BN));
  }
  issue(it0);
  if (NST == 3 && ntot > it0 + 1) issue(it0 + 1);

  v8 Qf[MT][KS], dOf[MT][KS];
  int ti[MT];
  long qoff[MT];
  bool live[MT];
  float base2[MT], dlr[MT], dgq[MT], osc[MT];   // base2 = log2(scale^deg exp(G_q - m))
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
      u32x4 z = {0, 0, 0, 0}, z2 = {0, 0, 0, 0};
      if (live[mi]) {
        z = *(const u32x4*)(Qg + qoff[mi] * DH + 32 * ks + 8 * g);
        z2 = *(const u32x4*)(dOg + qoff[mi] * DH + 32 * ks + 8 * g);
      }
      Qf[mi][ks] = __builtin_bit_cast(v8, z);
      dOf[mi][ks] = __builtin_bit_cast(v8, z2);
    }
    const long so = (long)b * a.tq * hq + qoff[mi];
    base2[mi] = __builtin_fmaf((Gg ? Gg[(long)ti[mi] * a.h] : 0.f) - a.rowmax[so], AB_LOG2E, l2sp);
    dlr[mi] = a.dl ? a.dl[so] : 0.f;
    osc[mi] = a.dO_scale ? a.dO_scale[so] : 1.f;
    dgq[mi] = 0.f;
  }
  const float Rw = Gg ? Gg[(long)w_first_ti * a.h] : 0.f;   // gate at the wave's first row
  f32x4 acc[MT][NT];
#pragma unroll
  for (int mi = 0; mi < MT; mi++)
#pragma unroll
    for (int nt = 0; nt < NT; nt++) acc[mi][nt] = (f32x4){0, 0, 0, 0};

  // per-lane LDS byte offsets inside a tile (the swizzle depends only on the row inside a 16-row group)
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

  const int n_past = min(ntiles, min(w_first_ti + 1, a.tk) / AB_BN);   // tiles with every pair visible
  const int n_seen = min(ntiles, w_last_ti / AB_BN + 1);               // tiles with at least one visible pair

  // exp(R - gate) relative to the tile's last key (<= 1) and to the first key of each 16-key group (>= 1);
  // written by wave 0, which issued the gate copy and so is the one that can wait for it
  auto gate_factors = [&](int it) __attribute__((always_inline)) {
    float* graw = (float*)(smem + (it % NST) * STAGE + 2 * TILE);
    const int rpos = min(AB_BN - 1, a.tk - 1 - it * AB_BN);
    const float gv = Gg ? graw[l] : 0.f;
    const float R_ = Gg ? graw[rpos] : 0.f;
    graw[AB_BN + l] = __expf(fminf(R_ - gv, AB_EXP_CLAMP));
    graw[2 * AB_BN + l] = gv * AB_LOG2E;   // the gate itself, in powers of two, for the diagonal tiles
    if (!Gg) graw[l] = 0.f;
  };
  if (wave == 0) {
    wait_vmcnt<0>();
    gate_factors(it0);
  }
  auto sync_step = [&](int it) __attribute__((always_inline)) -> char* {
    char* st = smem + (it % NST) * STAGE;
    if constexpr (NST == 3) {
      if (it + 1 < ntot) wait_vmcnt<LOADS>(); else wait_vmcnt<0>();
      lds_barrier();
      if (it + 2 < ntot) issue(it + 2);
      if (wave == 0 && it + 1 < ntiles) {
        if (it + 2 < ntot) wait_vmcnt<LOADS + 1>(); else wait_vmcnt<0>();   // all but the stage just issued
        gate_factors(it + 1);
      }
    } else {
      wait_vmcnt<0>();   // one stage in flight
      lds_barrier();
      if (it + 1 < ntot) issue(it + 1);
    }
    return st;
  };
  // two-stage ring: wave 0 prepares the next tile's factors after its own work on this one, when the copy issued at
  // the start of the step has had a tile's time to arrive
  auto after_step = [&](int it) __attribute__((always_inline)) {
    if constexpr (NST == 2) {
      if (wave == 0 && it + 1 < ntiles) {
        wait_vmcnt<0>();
        gate_factors(it + 1);
      }
    }
  };

  // One 64-key tile.  Past tiles: key factors relative to the gate at the wave's first row (<= 1), the row factor
  // is applied to the accumulators after the past tiles.  Diagonal tiles: per-pair exponent, per-pair mask.
  auto tile = [&](int it, const char* st, auto diag_c) __attribute__((always_inline)) {
    constexpr bool DIAG = decltype(diag_c)::value != 0;
    const int j0 = it * AB_BN;
    const float* graw = (const float*)(st + 2 * TILE);
    uint32_t kb[KS], tb[NT], eb;
    {
      uint32_t sa = (uint32_t)(uintptr_t)(ab_lds_char*)st;
      asm volatile("" : "+s"(sa));   // one scalar: or the slot arithmetic is redone inside every address below
#pragma unroll
      for (int ks = 0; ks < KS; ks++) {
        kb[ks] = sa + koff[ks];
        asm volatile("" : "+v"(kb[ks]));
      }
#pragma unroll
      for (int nt = 0; nt < NT; nt++) { tb[nt] = sa + toff[nt]; asm volatile("" : "+v"(tb[nt])); }
      eb = sa + 2 * TILE + (DIAG ? 2 * AB_BN : AB_BN) * 4 + 16 * g;
      asm volatile("" : "+v"(eb));
    }
    int lim[MT];
#pragma unroll
    for (int mi = 0; mi < MT; mi++) lim[mi] = DIAG ? min(ti[mi], a.tk - 1) - j0 - 4 * g : 0;
    const float cw = DIAG ? 1.f : __expf(fminf(Rw - graw[AB_BN - 1], AB_EXP_CLAMP));
    // (forgotten by this wave's rows, though not by the workgroup's first: every term of the tile is an exact zero)
    if (!DIAG && gate_skip && __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, cw)) == 0) return;
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
        f32x4 ev = *(const ab_lds_f32x4*)(eb + 64 * (2 * kp + half));
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
              // the pair's own exponent: no reference gate shared by a group of keys, whose two factors could leave
              // the fp32 range against each other where the gates fall steeply
              q = __builtin_amdgcn_exp2f(fminf(base2[mi] - ev[v], AB_EXP2_CLAMP)) * dpl;
              q = (32 * kp + 16 * half + v <= lim[mi]) ? q : 0.f;
            } else {
              q = ev[v] * dpl;
            }
            if (!DEG2) q *= pow_hm1<DEG2>(__builtin_fmaf(s, s, eps2), half_deg);
            // dz = (s^2 + eps^2) q: the eps^2 part is all there is for a key with q.k = 0 (an all-zero key)
            dgq[mi] = __builtin_fmaf(__builtin_fmaf(s, s, eps2), q, dgq[mi]);
            d4[v] = s * q;
          }
          h4[half][mi] = pack4<T>(d4);
          asm volatile("" : "+v"(h4[half][mi]));
        }
      }
      // K^T operands for the same 32 keys
      v8 kT[NT];
#pragma unroll
      for (int nt = 0; nt < NT; nt++) kT[nt] = ab_tr8<T>(tb[nt] + kp * 32 * RB, tb[nt] + kp * 32 * RB + 16 * RB);
      v8 dsf[MT];
#pragma unroll
      for (int mi = 0; mi < MT; mi++) dsf[mi] = __builtin_shufflevector(h4[0][mi], h4[1][mi], 0, 1, 2, 3, 4, 5, 6, 7);
      // dQ^T[d, row] += K^T[d, key] dsr^T[key, row]
#pragma unroll
      for (int nt = 0; nt < NT; nt++)
#pragma unroll
        for (int mi = 0; mi < MT; mi++) acc[mi][nt] = mfma16(kT[nt], dsf[mi], acc[mi][nt]);
    }
  };

  int it = it0;
  for (; it < n_past; it++) {
    tile(it, sync_step(it), IC<0>{});
    after_step(it);
  }
  // the past tiles were accumulated without the row factor scale^deg * exp(G_q - m - Rw); apply it once
#pragma unroll
  for (int mi = 0; mi < MT; mi++) {
    const float f = __builtin_amdgcn_exp2f(fminf(base2[mi] - Rw * AB_LOG2E, AB_EXP2_CLAMP));
#pragma unroll
    for (int nt = 0; nt < NT; nt++) acc[mi][nt] *= f;
    dgq[mi] *= f;
  }
  for (; it < n_seen; it++) {
    tile(it, sync_step(it), IC<1>{});
    after_step(it);
  }
  for (; it < ntiles; it++) {
    sync_step(it);
    after_step(it);
  }

  T* dQg = (T*)a.dQ + (long)b * a.tq * hq * DH;
  // Indices of this lane for the epilogue, re-derived from a copy of the lane id that the compiler cannot match with
  // the one used before the sweep: nothing that is only needed here should stay in registers through it.
  int le = threadIdx.x & 63;
  asm volatile("" : "+v"(le));
  const int ge = le >> 4, tce = le & 15;
  uint32_t ep = 0;
  if (dQsg) {
    wait_vmcnt<0>();
    lds_barrier();
    ep = (uint32_t)(uintptr_t)(ab_lds_char*)(smem + (ntiles % NST) * STAGE);
  }
#pragma unroll
  for (int mi = 0; mi < MT; mi++) {
    const int row_e = wrow0 + 16 * mi + tce;
    const bool live_e = row_e < rows;
    const int rr_e = live_e ? row_e : 0, t_e = rr_e / a.r;
    const long qoff_e = (long)t_e * hq + hh * a.r + (rr_e - t_e * a.r);
    float tot = sum_over_rows(dgq[mi]);
    float u = 1.f;
    v4 add4[NT];
    if (dQsg) {   // gradient through the gated copy of Q: dQs * u, and (Q . dQs) u / deg for the gate
      const int lr = wslice * 16 * MT + 16 * mi;
      const uint32_t rb = ep + (lr / AB_BN) * TILE + (lr % AB_BN) * RB;
      u = (Gg && !a.dQs_plain) ? __expf(Gg[(long)(t_e + shift) * a.h] / a.deg) : 1.f;
      float dotq = 0.f;
#pragma unroll
      for (int ks = 0; ks < KS; ks++) {
        float q8[8], d8[8];
        unpack8(Qf[mi][ks], q8);
        unpack8((v8)(*(const lds_v8*)(rb + tce * RB + (((4 * ks + ge) ^ swz<CPR, SWZ_ROW>(tce)) * 16))), d8);
#pragma unroll
        for (int i = 0; i < 8; i++) dotq = __builtin_fmaf(q8[i], d8[i], dotq);
      }
#pragma unroll
      for (int nt = 0; nt < NT; nt++)
        add4[nt] = *(const lds_v4*)(rb + tce * RB + (((2 * nt + (ge >> 1)) ^ swz<CPR, SWZ_ROW>(tce)) * 16) + (ge & 1) * 8);
      tot += sum_over_rows(dotq) * u / a.deg;
    }
    if (!live_e) continue;
#pragma unroll
    for (int nt = 0; nt < NT; nt++) {
      float o4[4];
#pragma unroll
      for (int v = 0; v < 4; v++) {
        o4[v] = acc[mi][nt][v] * a.deg;
        if (dQsg) o4[v] = __builtin_fmaf((float)add4[nt][v], u, o4[v]);
      }
      *(v4*)(dQg + qoff_e * DH + 16 * nt + 4 * ge) = pack4<T>(o4);
    }
    if (ge == 0 && a.dGq) a.dGq[(long)b * a.tq * hq + qoff_e] = tot;
  }
}

// ------------------------------------------------------------------ dK, dV, dGk
// A workgroup owns 64*MK keys (16*MK per wave, keys on the lanes) and walks the query-row tiles that can see them
// from the LAST row tile down to the tiles on its diagonal.  Far tiles (every row after every key of the workgroup)
// use one reference gate R for the workgroup: the row factors scale^deg exp(G_q - m - R) (times the dO scale and
// times dl) are prepared once per tile in LDS, and the key factor exp(R - G_k) <= 1 is applied to the accumulators
// once after the far tiles; the tiles near the diagonal then add absolute terms (reference: last key of each 16).
template <typename T, int DH, int MK, bool DEG2>
__global__ __launch_bounds__(256, 2) void attention_bwd_dkv_kernel(AttnBwdArgs a, int nblocks, int npairs, int gate_skip) {
  typedef typename VecOf<T>::v8 v8;
  typedef typename VecOf<T>::v4 v4;
  typedef __attribute__((address_space(3))) v8 lds_v8;
  typedef __attribute__((address_space(3))) v4 lds_v4;
  constexpr int KS = DH / 32, NT = DH / 16, QT = AB_BM / 16, KEYS = 64 * MK, CPR = DH / 8, RB = CPR * 16;
  constexpr int TILE = AB_BM * RB;
  // row vectors of a stage, AB_BM floats each: [0] G_q (raw) -> G_q - m, [1] m (raw) -> time index (as a float),
  // [2] dl, [3] dO scale, [4] far-tile factor * dO scale, [5] far-tile factor * dl
  constexpr int NV = 6;
  constexpr int STAGE = 2 * TILE + NV * AB_BM * 4;
  constexpr int NST = ab_stages(DH);
  constexpr bool EARLY_T = DEG2 && DH <= 64;   // the other instances have no registers left for it
  constexpr int LOADS = 2 * AB_BM * CPR / 256;
  extern __shared__ __attribute__((aligned(1024))) char smem[];

  const int grp = blockIdx.x % 32, u = blockIdx.x / 32, ppg = (npairs + 31) / 32;
  int pig, blk;
  deal_causal_blocks(u, nblocks, ppg, pig, blk);
  const int pair = pig * 32 + grp;
  if (pair >= npairs) return;
  const int tid = threadIdx.x, l = tid & 63, g = l >> 4, kcol = l & 15;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int b = __builtin_amdgcn_readfirstlane(pair / a.h), hh = pair - b * a.h;
  const int hq = a.h * a.r, rows = a.tq * a.r, shift = a.tk - a.tq;
  const int key0 = blk * KEYS;   // early keys are seen by the most rows
  const char* Qg = (const char*)((const T*)a.Q + (long)b * a.tq * hq * DH);
  const char* dOg = (const char*)((const T*)a.dO + (long)b * a.tq * hq * DH);
  const T* Kg = (const T*)a.K + (long)b * a.tk * a.h * DH + hh * DH;
  const T* Vg = (const T*)a.V + (long)b * a.tk * a.h * DH + hh * DH;
  const float* Gg = a.G ? a.G + (long)b * a.tk * a.h + hh : nullptr;
  const float* rmg = a.rowmax + (long)b * a.tq * hq;
  const float* dlg = a.dl ? a.dl + (long)b * a.tq * hq : nullptr;
  const float* osg = a.dO_scale ? a.dO_scale + (long)b * a.tq * hq : nullptr;
  const long kstride = (long)a.h * DH;
  const int half_deg = (int)a.deg / 2;
  const float eps_s = AB_LOG_EPS / a.scale, eps2 = eps_s * eps_s;
  const float scale_p = __expf(a.deg * __logf(a.scale));
  const int last_key = min(key0 + KEYS, a.tk) - 1;
  const float Rblk = Gg ? Gg[(long)last_key * a.h] : 0.f;   // reference gate of the workgroup's far tiles
  const float Glast = Gg ? Gg[(long)(a.tk - 1) * a.h] : 0.f;  // (for the epilogue; fetched here, where its latency hides)

  const int wslice = (u & 1) ? 3 - wave : wave;
  const int wkey0 = key0 + wslice * 16 * MK;

  // row tiles, walked downwards from the last one
  const int ntile_total = (rows + AB_BM - 1) / AB_BM;
  const int tile_lo = max(0, (key0 - shift) * a.r) / AB_BM;               // first tile that sees any key of the block
  const int nsteps = max(0, ntile_total - tile_lo);
  // far tiles: every row's time index >= last_key  <=>  tile >= ceil((last_key - shift) * r / BM)
  // (per workgroup, not per wave: the row factors in LDS are relative to the gate at the workgroup's last key and
  // stay <= 1 only for rows after it)
  const int tile_far = max(tile_lo, (max(0, (last_key - shift) * a.r) + AB_BM - 1) / AB_BM);
  const int n_far = max(0, ntile_total - tile_far);
  const int row_vis = (wkey0 - shift) * a.r;   // folded rows before this one see none of the wave's keys
  // tiles with at least one row that sees the wave's first key
  const int tile_w = max(tile_lo, max(0, (wkey0 - shift) * a.r) / AB_BM);
  const int n_seen = max(n_far, ntile_total - tile_w);

  // copies of one stage: row inside the tile and byte offset of the 16-byte chunk in its row for this thread's
  // copy number ii (recomputed where needed: only the irregular paths use them)
  auto grow = [&](int ii) __attribute__((always_inline)) -> int { return ((ii * 4 + wave) * 64 + l) / CPR; };
  auto gchk = [&](int ii) __attribute__((always_inline)) -> uint32_t {
    const int pos = (ii * 4 + wave) * 64 + l;
    return 16 * ((pos % CPR) ^ swz<CPR, SWZ_ROW>(pos / CPR));
  };
  auto row_elem = [&](int row) __attribute__((always_inline)) -> long {   // element offset of a (clamped) folded row in a [tq, hq] array
    row = min(row, rows - 1);
    const int t = row / a.r;
    return (long)t * hq + hh * a.r + (row - t * a.r);
  };
  // With the chunked epilogue the workgroup's rows of dKs and dVs ride through the ring as two more stages after
  // the last row tile (keys 0..63 in the Q area, 64..127 in the dO area): they arrive under the last tiles' work.
  // (not for a block of keys whose discount is an exact zero: their rows of dKs and dVs are zeros, or not written at all)
  const bool dead_keys = gate_skip && a.live_rows && a.dKs && key0 + KEYS <= a.live_rows[((long)b * a.h + hh) * 2];
  const T* dKsg = a.dKs && !dead_keys ? (const T*)a.dKs + (long)b * a.tk * a.h * DH + hh * DH : nullptr;
  const T* dVsg = a.dVs && !dead_keys ? (const T*)a.dVs + (long)b * a.tk * a.h * DH + hh * DH : nullptr;
  const int ntot = nsteps + (dKsg ? 2 : 0);
  // lane offsets of the copies of a regular tile (r a power of two): folded row j of a tile is time step j / r, head
  // hh * r + j % r, whatever the tile
  const bool regular = (a.r & (a.r - 1)) == 0 && a.r <= AB_BM;
  const int rsh = 31 - __builtin_clz(a.r);
  const uint32_t smem_a = lds_addr(smem);
  uint32_t voff[LOADS / 2];
#pragma unroll
  for (int ii = 0; ii < LOADS / 2; ii++)
    voff[ii] = (uint32_t)((((grow(ii) >> rsh) * hq + hh * a.r + (grow(ii) & (a.r - 1))) * (DH * 2))) + gchk(ii);
  auto issue = [&](int step) __attribute__((always_inline)) {
    char* st = smem + (step % NST) * STAGE;
    if (step >= nsteps) {
      const T* src = step == nsteps ? dKsg : dVsg;
#pragma unroll
      for (int ii = 0; ii < LOADS; ii++) {
        const int half = ii / (LOADS / 2), i2 = ii % (LOADS / 2);
        const long eo = (long)min(key0 + half * AB_BM + grow(i2), a.tk - 1) * kstride;
        async_copy16((const char*)(src + eo) + gchk(i2), st + half * TILE + (i2 * 4 + wave) * 1024);
      }
      if (wave == 0) {   // keeps the count of copies per stage fixed
        float* rv = (float*)(st + 2 * TILE);
#pragma unroll
        for (int i = 0; i < 4; i++) async_copy4(rmg, rv + i * AB_BM);
      }
      return;
    }
    const int rbase = (ntile_total - 1 - step) * AB_BM;
    if (regular && rbase + AB_BM <= rows) {
      // a whole tile of whole time steps: lane offsets are fixed, the tile's base moves in scalar registers
      const long tb = (long)(rbase >> rsh) * hq;   // first [t, hq] row of the tile
      const uint32_t sa = __builtin_amdgcn_readfirstlane(smem_a + (step % NST) * STAGE + wave * 1024);
      const void* qb_ = uniform_ptr(Qg + tb * (DH * 2));
      const void* ob_ = uniform_ptr(dOg + tb * (DH * 2));
#pragma unroll
      for (int ii = 0; ii < LOADS / 2; ii++) {
        async_copy16_sv(qb_, voff[ii], sa + ii * 4096);
        async_copy16_sv(ob_, voff[ii], sa + TILE + ii * 4096);
      }
      if (wave == 0) {   // always four copies so that the count per stage is fixed
        const uint32_t rv = sa + 2 * TILE;
        const uint32_t voffR = (uint32_t)((((l >> rsh) * hq + hh * a.r + (l & (a.r - 1)))) * 4);
        const uint32_t voffG = (uint32_t)((l >> rsh) * a.h * 4);
        const void* rb_ = uniform_ptr(rmg + tb);
        if (Gg) async_copy4_sv(uniform_ptr(Gg + (long)((rbase >> rsh) + shift) * a.h), voffG, rv);
        else async_copy4_sv(rb_, voffR, rv);
        async_copy4_sv(rb_, voffR, rv + AB_BM * 4);
        async_copy4_sv(uniform_ptr((dlg ? dlg : rmg) + tb), voffR, rv + 2 * AB_BM * 4);
        async_copy4_sv(uniform_ptr((osg ? osg : rmg) + tb), voffR, rv + 3 * AB_BM * 4);
      }
      return;
    }
#pragma unroll
    for (int ii = 0; ii < LOADS / 2; ii++) {
      const long ro = row_elem(rbase + grow(ii)) * (DH * 2) + gchk(ii);
      async_copy16(Qg + ro, st + (ii * 4 + wave) * 1024);
      async_copy16(dOg + ro, st + TILE + (ii * 4 + wave) * 1024);
    }
    if (wave == 0) {   // always four copies so that the count per stage is fixed
      const int row = min(rbase + l, rows - 1);
      const long ro = row_elem(row);
      const int t = row / a.r + shift;
      float* rv = (float*)(st + 2 * TILE);
      async_copy4(Gg ? Gg + (long)t * a.h : rmg + ro, rv);
      async_copy4(rmg + ro, rv + AB_BM);
      async_copy4(dlg ? dlg + ro : rmg + ro, rv + 2 * AB_BM);
      async_copy4(osg ? osg + ro : rmg + ro, rv + 3 * AB_BM);
    }
  };
  // (the keys and values of the workgroup first: their loads are in flight while the far tiles are tested)
  v8 Kf[MK][KS], Vf[MK][KS];
  int key[MK];
  bool live[MK];
  float Gk[MK], Rk[MK], dk[MK], dgk[MK], keyf[MK];
#pragma unroll
  for (int kj = 0; kj < MK; kj++) {
    key[kj] = wkey0 + 16 * kj + kcol;
    live[kj] = key[kj] < a.tk;
    keyf[kj] = (float)key[kj];
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      u32x4 z = {0, 0, 0, 0}, z2 = {0, 0, 0, 0};
      if (live[kj]) {
        z = *(const u32x4*)(Kg + key[kj] * kstride + 32 * ks + 8 * g);
        z2 = *(const u32x4*)(Vg + key[kj] * kstride + 32 * ks + 8 * g);
      }
      Kf[kj][ks] = __builtin_bit_cast(v8, z);
      Vf[kj][ks] = __builtin_bit_cast(v8, z2);
    }
    Gk[kj] = Gg ? Gg[(long)min(key[kj], a.tk - 1) * a.h] : 0.f;
    // Near the diagonal the exponent of a pair is G_q - m - G_k itself: a key factor and a row factor relative to a
    // shared reference gate leave the fp32 range against each other once the gates of a group of keys differ by more
    // than 87.  It is formed as (G_q - m - Rk) - (G_k - Rk) with Rk the gate at the group's last key, which is the
    // same for the whole wave and stays in a scalar register.
    Rk[kj] = Gg ? Gg[(long)min(wkey0 + 16 * kj + 15, a.tk - 1) * a.h] : 0.f;
    dk[kj] = Gk[kj] - Rk[kj];
    dgk[kj] = 0.f;
  }
  // ---- far tiles that the gates have already forgotten -------------------------------------------------------------
  // Every term of a far tile carries its row's factor scale^deg exp(G_q - m - R) (row_factors below).  The walk starts
  // at the last tile, the one the gates have decayed most: while that factor has underflowed to zero for every row of
  // a tile, the tile adds exact zeros to dK, dV and the gate sums, and is neither copied nor visited (step0 = the first
  // tile that is).  Each wave tests every fourth tile, a row per lane, eight tiles at a time so that the latencies of
  // their loads overlap.
  // (Tested only when the gates fall by more than 40 from the workgroup's keys to the last row: short of that no factor
  // can have underflowed unless a row's largest weight exceeds e^47, and such a tile is merely visited.)
  int step0 = 0;
  if (gate_skip && Gg && n_far > 0 && Gg[(long)((rows - 1) / a.r + shift) * a.h] - Rblk < -40.f) {
    int* first = (int*)smem;
    for (int base = 0; base < n_far; base += 32) {
      float bsv[8];
#pragma unroll
      for (int i = 0; i < 8; i++) {
        const int s = base + 4 * i + wave;
        const int row = (ntile_total - 1 - s) * AB_BM + l;
        const bool real = s < n_far && row < rows;
        const int rc = min(max(row, 0), rows - 1);
        bsv[i] = real ? Gg[(long)(rc / a.r + shift) * a.h] - rmg[row_elem(rc)] : -INFINITY;
      }
      int fa = n_far;   // this wave's first tile of the round with a row that still counts (tiles past the far ones do)
#pragma unroll
      for (int i = 7; i >= 0; i--) {
        const int s = base + 4 * i + wave;
        const bool alive = s >= n_far || __expf(fminf(bsv[i] - Rblk, AB_EXP_CLAMP)) != 0.f;
        if (__ballot(alive) != 0) fa = min(s, n_far);
      }
      __syncthreads();   // (the previous round's values have been read)
      if (l == 0) first[wave] = fa;
      __syncthreads();
      step0 = min(min(first[0], first[1]), min(first[2], first[3]));
      if (step0 < base + 32) break;
    }
    step0 = __builtin_amdgcn_readfirstlane(min(step0, n_far));
    __syncthreads();   // the first stage's copies land where the four values were
  }
  if (ntot > step0) issue(step0);
  if (NST == 3 && ntot > step0 + 1) issue(step0 + 1);

  f32x4 accK[MK][NT], accV[MK][NT];
#pragma unroll
  for (int kj = 0; kj < MK; kj++)
#pragma unroll
    for (int nt = 0; nt < NT; nt++) {
      accK[kj][nt] = (f32x4){0, 0, 0, 0};
      accV[kj][nt] = (f32x4){0, 0, 0, 0};
    }

  int qoff_[KS], toff[NT];
#pragma unroll
  for (int ks = 0; ks < KS; ks++) qoff_[ks] = kcol * RB + (((4 * ks + g) ^ swz<CPR, SWZ_ROW>(kcol)) * 16);
  {
    const int vr = 4 * g + (kcol >> 2);
#pragma unroll
    for (int nt = 0; nt < NT; nt++) {
      const int col = 16 * nt + 4 * (kcol & 3);
      toff[nt] = vr * RB + (((col / 8) ^ swz<CPR, SWZ_ROW>(vr)) * 16) + (col % 8) * 2;
    }
  }

  // Row vectors of a tile (wave 0 issued their copies): G_q - m, time index (-1 for rows past the end), dl, dO
  // scale, and the far-tile factors scale^deg exp(G_q - m - R) * {dO scale, dl} (zero for rows past the end).
  auto row_factors = [&](int step) __attribute__((always_inline)) {
    float* rv = (float*)(smem + (step % NST) * STAGE + 2 * TILE);
    const int row = (ntile_total - 1 - step) * AB_BM + l;
    const bool real = row < rows;
    const float bs = (Gg ? rv[l] : 0.f) - rv[AB_BM + l];
    const float dl_ = (dlg && real) ? rv[2 * AB_BM + l] : 0.f;
    const float os_ = osg ? rv[3 * AB_BM + l] : 1.f;
    const float eu = real ? scale_p * __expf(fminf(bs - Rblk, AB_EXP_CLAMP)) : 0.f;
    rv[l] = bs;
    rv[AB_BM + l] = real ? (float)(min(row, rows - 1) / a.r + shift) : -1.f;
    rv[2 * AB_BM + l] = dl_;
    rv[3 * AB_BM + l] = real ? os_ : 0.f;
    rv[4 * AB_BM + l] = eu * os_;
    rv[5 * AB_BM + l] = eu * dl_;
  };
  if (wave == 0 && nsteps > step0) {
    wait_vmcnt<0>();
    row_factors(step0);
  }
  auto sync_step = [&](int step) __attribute__((always_inline)) -> char* {
    char* st = smem + (step % NST) * STAGE;
    if constexpr (NST == 3) {
      if (step + 1 < ntot) wait_vmcnt<LOADS>(); else wait_vmcnt<0>();
      lds_barrier();
      if (step + 2 < ntot) issue(step + 2);
      if (wave == 0 && step + 1 < nsteps) {
        if (step + 2 < ntot) wait_vmcnt<LOADS + 4>(); else wait_vmcnt<0>();   // all but the stage just issued
        row_factors(step + 1);
      }
    } else {
      wait_vmcnt<0>();   // one stage in flight
      lds_barrier();
      if (step + 1 < ntot) issue(step + 1);
    }
    return st;
  };
  // two-stage ring: wave 0 prepares the next tile's row vectors after its own work on this one
  auto after_step = [&](int step) __attribute__((always_inline)) {
    if constexpr (NST == 2) {
      if (wave == 0 && step + 1 < nsteps) {
        wait_vmcnt<0>();
        row_factors(step + 1);
      }
    }
  };

  auto tile = [&](const char* st, int rbase, auto far_c) __attribute__((always_inline)) {
    constexpr bool FAR = decltype(far_c)::value != 0;
    uint32_t qb[KS], ob[KS], qtb[NT], otb[NT], fb;
    {
      uint32_t sa = (uint32_t)(uintptr_t)(ab_lds_char*)st;
      asm volatile("" : "+s"(sa));   // one scalar: or the slot arithmetic is redone inside every address below
#pragma unroll
      for (int ks = 0; ks < KS; ks++) {
        qb[ks] = sa + qoff_[ks];
        ob[ks] = sa + TILE + qoff_[ks];
        asm volatile("" : "+v"(qb[ks]));
        asm volatile("" : "+v"(ob[ks]));
      }
#pragma unroll
      for (int nt = 0; nt < NT; nt++) {
        qtb[nt] = sa + toff[nt];
        otb[nt] = sa + TILE + toff[nt];
        asm volatile("" : "+v"(qtb[nt]));
        asm volatile("" : "+v"(otb[nt]));
      }
      fb = sa + 2 * TILE + 16 * g;
      asm volatile("" : "+v"(fb));
    }
#pragma unroll
    for (int qp = 0; qp < QT / 2; qp++) {
      if (!FAR && rbase + 32 * qp + 31 < row_vis) continue;   // these 32 rows come before every key of the wave
      v8 qf[2][KS], dof[2][KS];
      f32x4 fa[2], fc[2], fd[2], fe[2];   // FAR: factor*scale, factor*dl;  near: G_q - m, time index, dl, dO scale
#pragma unroll
      for (int half = 0; half < 2; half++) {
        const int qt = 2 * qp + half;
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
          qf[half][ks] = *(const lds_v8*)(qb[ks] + qt * 16 * RB);
          dof[half][ks] = *(const lds_v8*)(ob[ks] + qt * 16 * RB);
        }
        if (FAR) {
          fa[half] = *(const ab_lds_f32x4*)(fb + (4 * AB_BM + 16 * qt) * 4);
          fc[half] = *(const ab_lds_f32x4*)(fb + (5 * AB_BM + 16 * qt) * 4);
        } else {
          fa[half] = *(const ab_lds_f32x4*)(fb + (16 * qt) * 4);
          fc[half] = *(const ab_lds_f32x4*)(fb + (AB_BM + 16 * qt) * 4);
          fd[half] = *(const ab_lds_f32x4*)(fb + (2 * AB_BM + 16 * qt) * 4);
          fe[half] = *(const ab_lds_f32x4*)(fb + (3 * AB_BM + 16 * qt) * 4);
        }
      }
      f32x4 sc[2][MK], dp[2][MK];
#pragma unroll
      for (int half = 0; half < 2; half++)
#pragma unroll
        for (int kj = 0; kj < MK; kj++) {
          sc[half][kj] = (f32x4){0, 0, 0, 0};
          dp[half][kj] = (f32x4){0, 0, 0, 0};
        }
#pragma unroll
      for (int ks = 0; ks < KS; ks++)
#pragma unroll
        for (int half = 0; half < 2; half++)
#pragma unroll
          for (int kj = 0; kj < MK; kj++) {
            sc[half][kj] = mfma16(qf[half][ks], Kf[kj][ks], sc[half][kj]);
            dp[half][kj] = mfma16(dof[half][ks], Vf[kj][ks], dp[half][kj]);
          }
      // dO^T and Q^T operands of the same 32 rows.  Where the registers allow it they are requested here, so that they
      // arrive while the pair terms are formed (they take the registers the plain operands leave); with two waves per
      // SIMD little else covers the LDS latency (6 us of a step).
      v8 doT[NT], qT[NT];
      if constexpr (EARLY_T) {
#pragma unroll
        for (int nt = 0; nt < NT; nt++) {
          doT[nt] = ab_tr8<T>(otb[nt] + qp * 32 * RB, otb[nt] + qp * 32 * RB + 16 * RB);
          qT[nt] = ab_tr8<T>(qtb[nt] + qp * 32 * RB, qtb[nt] + qp * 32 * RB + 16 * RB);
        }
      }
      v8 pf[MK], dsf[MK];
#pragma unroll
      for (int kj = 0; kj < MK; kj++) {
        float p8[8], d8[8];
#pragma unroll
        for (int half = 0; half < 2; half++) {
#pragma unroll
          for (int v = 0; v < 4; v++) {
            const float s = sc[half][kj][v];
            const float a2 = __builtin_fmaf(s, s, eps2);
            float q, pw;   // q = E * dP, pw = P * (dO scale), both without the key factor
            if (FAR) {
              q = __builtin_fmaf(dp[half][kj][v], fa[half][v], fc[half][v]);
              pw = a2 * fa[half][v];
              if (!DEG2) {
                const float h1 = pow_hm1<DEG2>(a2, half_deg);
                q *= h1;
                pw *= h1;
              }
            } else {
              const bool vis = (keyf[kj] <= fc[half][v]) && live[kj];
              float E = scale_p * __expf(fminf((fa[half][v] - Rk[kj]) - dk[kj], AB_EXP_CLAMP)) * pow_hm1<DEG2>(a2, half_deg);
              E = vis ? E : 0.f;
              q = E * __builtin_fmaf(dp[half][kj][v], fe[half][v], fd[half][v]);
              pw = a2 * E * fe[half][v];
            }
            const float dsr = s * q;
            dgk[kj] = __builtin_fmaf(a2, q, dgk[kj]);
            p8[4 * half + v] = pw;
            d8[4 * half + v] = dsr;
          }
        }
        pf[kj] = pack8<T>(p8);
        dsf[kj] = pack8<T>(d8);
      }
      // dV^T[e, key] += dO^T[e, row] P[row, key];  dK^T[d, key] += Q^T[d, row] dsr[row, key]
#pragma unroll
      for (int nt = 0; nt < NT; nt++) {
        if constexpr (!EARLY_T) {
          doT[nt] = ab_tr8<T>(otb[nt] + qp * 32 * RB, otb[nt] + qp * 32 * RB + 16 * RB);
          qT[nt] = ab_tr8<T>(qtb[nt] + qp * 32 * RB, qtb[nt] + qp * 32 * RB + 16 * RB);
        }
#pragma unroll
        for (int kj = 0; kj < MK; kj++) {
          accV[kj][nt] = mfma16(doT[nt], pf[kj], accV[kj][nt]);
          accK[kj][nt] = mfma16(qT[nt], dsf[kj], accK[kj][nt]);
        }
      }
    }
  };

  int step = step0;
  for (; step < n_far; step++) {
    tile(sync_step(step), (ntile_total - 1 - step) * AB_BM, IC<1>{});
    after_step(step);
  }
  // the far tiles were accumulated without the key factor exp(R - G_k) (<= 1); apply it once.  The tiles near
  // the diagonal are accumulated in absolute terms (their packed weights stay <= the true ones).
#pragma unroll
  for (int kj = 0; kj < MK; kj++) {
    const float c = __expf(fminf(Rblk - Gk[kj], AB_EXP_CLAMP));
#pragma unroll
    for (int nt = 0; nt < NT; nt++) {
      accK[kj][nt] *= c;
      accV[kj][nt] *= c;
    }
    dgk[kj] *= c;
  }
  for (; step < n_seen; step++) {
    tile(sync_step(step), (ntile_total - 1 - step) * AB_BM, IC<0>{});
    after_step(step);
  }
  for (; step < nsteps; step++) {
    sync_step(step);
    after_step(step);
  }
  if (NST == 2 && nsteps + 1 < ntot) {   // the second of the two epilogue stages has no step that would copy it
    lds_barrier();
    issue(nsteps + 1);
  }

  T* dKg = (T*)a.dK + (long)b * a.tk * a.h * DH + hh * DH;
  T* dVg = (T*)a.dV + (long)b * a.tk * a.h * DH + hh * DH;
  // Indices of this lane for the epilogue, re-derived from a copy of the lane id that the compiler cannot match with
  // the one used before the sweep: nothing that is only needed here should stay in registers (or in scratch memory,
  // whose reload waits for every copy in flight) through it.
  int le = threadIdx.x & 63;
  asm volatile("" : "+v"(le));
  const int ge = le >> 4, kce = le & 15;
  uint32_t epk = 0, epv = 0;
  if (dKsg) {
    wait_vmcnt<0>();
    lds_barrier();
    epk = (uint32_t)(uintptr_t)(ab_lds_char*)(smem + (nsteps % NST) * STAGE);
    epv = (uint32_t)(uintptr_t)(ab_lds_char*)(smem + ((nsteps + 1) % NST) * STAGE);
  }
#pragma unroll
  for (int kj = 0; kj < MK; kj++) {
    const int key_e = wkey0 + 16 * kj + kce;
    float tot = sum_over_rows(dgk[kj]);
    float w = 1.f, dotk = 0.f;
    v4 addk[NT], addv[NT];
    if (dKsg) {   // gradient through the discounted copy of K: dKs * w, and -(K . dKs) w / deg for the gate
      const int lr = wslice * 16 * MK + 16 * kj;
      const uint32_t ro = (lr / AB_BM) * TILE + (lr % AB_BM) * RB;
      w = Gg ? __expf((Glast - Gk[kj]) / a.deg) : 1.f;
#pragma unroll
      for (int ks = 0; ks < KS; ks++) {
        float k8[8], d8[8];
        unpack8(Kf[kj][ks], k8);
        unpack8((v8)(*(const lds_v8*)(epk + ro + kce * RB + (((4 * ks + ge) ^ swz<CPR, SWZ_ROW>(kce)) * 16))), d8);
#pragma unroll
        for (int i = 0; i < 8; i++) dotk = __builtin_fmaf(k8[i], d8[i], dotk);
      }
#pragma unroll
      for (int nt = 0; nt < NT; nt++) {
        const uint32_t co = ro + kce * RB + (((2 * nt + (ge >> 1)) ^ swz<CPR, SWZ_ROW>(kce)) * 16) + (ge & 1) * 8;
        addk[nt] = *(const lds_v4*)(epk + co);
        addv[nt] = *(const lds_v4*)(epv + co);
      }
      dotk = sum_over_rows(dotk) * w;
      tot += dotk / a.deg;
    }
    if (key_e >= a.tk) continue;
#pragma unroll
    for (int nt = 0; nt < NT; nt++) {
      float k4[4], v4f[4];
#pragma unroll
      for (int v = 0; v < 4; v++) {
        k4[v] = accK[kj][nt][v] * a.deg;
        v4f[v] = accV[kj][nt][v];
        if (dKsg) {
          k4[v] = __builtin_fmaf((float)addk[nt][v], w, k4[v]);
          v4f[v] += (float)addv[nt][v];
        }
      }
      *(v4*)(dKg + key_e * kstride + 16 * nt + 4 * ge) = pack4<T>(k4);
      *(v4*)(dVg + key_e * kstride + 16 * nt + 4 * ge) = pack4<T>(v4f);
    }
    if (ge == 0) {
      const long go = ((long)b * a.tk + key_e) * a.h + hh;
      if (a.dGk) a.dGk[go] = -tot;
      if (a.dotk) a.dotk[go] = dotk;
    }
  }
}

template <typename T, int DH, bool DEG2> static int attn_bwd_launch(const AttnBwdArgs& a, int B, hipStream_t st) {
  const int npairs = B * a.h;
  // dK/dV first: its epilogue reads the state-path gradients that the kernels just before this call wrote (4 us of a
  // training step at the headline shape against the other order).  Either half is skipped when its outputs are null.
  if (a.dK) {
    constexpr int MK = DH <= 64 ? 2 : 1;
    constexpr size_t smem = ab_stages(DH) * (2 * AB_BM * DH * 2 + 6 * AB_BM * 4);
    const int nblocks = (a.tk + 64 * MK - 1) / (64 * MK);
    dim3 grid((unsigned)((npairs + 31) / 32 * 32 * nblocks));
    auto kern = attention_bwd_dkv_kernel<T, DH, MK, DEG2>;
    allow_big_lds((const void*)kern, smem);
    PR_LAUNCH("attention_bwd_dkv", kern, grid, dim3(256), smem, st, a, nblocks, npairs, g_gate_skip);
  }
  if (a.dQ) {
    constexpr int MT = DH <= 64 ? 2 : 1;
    constexpr size_t smem = ab_stages(DH) * (2 * AB_BN * DH * 2 + 4 * AB_BN * 4);
    const int rows = a.tq * a.r;
    const int nblocks = (rows + 64 * MT - 1) / (64 * MT);
    dim3 grid((unsigned)((npairs + 31) / 32 * 32 * nblocks));
    // three workgroups per CU where the registers allow it without spilling (168 at d = 64 and degree 2, the
    // stage-by-stage tile of the kernel is written for that); the ring of d = 128 leaves room for two anyway
    constexpr int OCC = (DH <= 32 || (DH == 64 && DEG2)) ? 3 : 2;
    auto kern = attention_bwd_dq_kernel<T, DH, MT, DEG2, OCC>;
    allow_big_lds((const void*)kern, smem);
    PR_LAUNCH("attention_bwd_dq", kern, grid, dim3(256), smem, st, a, nblocks, npairs, g_gate_skip);
  }
  return (int)hipGetLastError();
}

int attention_bwd(const AttnBwdArgs& a, int B, int d, int dtype, hipStream_t st) {
  const bool deg2 = a.deg == 2.f;
#define PR_AB(T)                                                                                                       \
  switch (d) {                                                                                                         \
    case 32: return deg2 ? attn_bwd_launch<T, 32, true>(a, B, st) : attn_bwd_launch<T, 32, false>(a, B, st);           \
    case 64: return deg2 ? attn_bwd_launch<T, 64, true>(a, B, st) : attn_bwd_launch<T, 64, false>(a, B, st);           \
    case 128: return deg2 ? attn_bwd_launch<T, 128, true>(a, B, st) : attn_bwd_launch<T, 128, false>(a, B, st);        \
    default: return -2;                                                                                                \
  }
  if (dtype == DT_BF16) { PR_AB(bf16_t) }
  if (dtype == DT_F16) { PR_AB(f16_t) }
#undef PR_AB
  return -1;
}

}  // namespace pr
