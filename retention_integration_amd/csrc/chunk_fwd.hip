// Forward of the chunked algorithm for all chunks, in ONE kernel per (chunk, kv head, block of 128 folded rows):
//
//   state part      y_i = sum_f phi(q_i)[f] Sc[f, :],   lq_i = sum_f phi(q_i)[f] sc[f]
//                                      (ref: retention/_query_state/reference.py:36-96, Triton :54-169)
//   attention part  w_ij = (scale q_i.k_j)^2 exp(A_i - A_j)  for the keys j <= i of the same chunk
//                                      (ref: retention/_attention/reference.py:10-69)
//   merge           out_i = (sum_j w_ij v_j + kappa_i y_i) / (sum_j w_ij + 1e-6 max_j w_ij + kappa_i lq_i),
//                   kappa_i = scale^2 exp(A_i)          (ref: retention/_query_state/reference.py:79-87 with the
//                                      query gating of retention/power_retention_maker.py:183-186 as a row factor)
//
// The two parts share one set of accumulators.  Run as two kernels (attention_fwd.hip, then sympow_nn.hip with the
// merge epilogue) the attention result, its row sums and row maxima go to memory and come back, the query rows are
// loaded twice, and each launch has its own start-up and store phase; here the rows are loaded once (into LDS), the
// state sweep runs first and leaves y_i in the accumulators, and the key tiles of the chunk are added on top.
//
// Orientation and scaling are those of attention_fwd.hip: products are formed transposed (O^T = V^T P^T), so an
// accumulator holds out[row = lane % 16, e = 16 nt + 4 (lane / 16) + v]; the state sweep uses the same layout by
// taking the state tile as the first matrix-core operand and phi(q)^T as the second.  Attention weights are
// accumulated in absolute terms; tiles entirely in a wave's past leave out the row factor scale^2 exp(A_i - R)
// (R = the gate at the wave's first row), which is applied once afterwards -- so the state part enters as
// exp(R) y_i and receives the same factor: exp(R) * scale^2 exp(A_i - R) = kappa_i.  No row maximum is needed for
// the result (bf16 holds any row in absolute terms); it is tracked because the backward kernels take it, and the
// normaliser is written in the units they expect: den = exp(-beta) * (denominator above), beta = max(rowmax, log sqrt D).
//
// bf16, head dims 32 and 64, degree 2, a state that is symmetric in the diagonal feature blocks (every state the
// chunked path forms); other cases run the two kernels.
#include "common.h"
#include "kernels.h"

namespace pr {

constexpr int CF_BN = 64;   // keys per attention stage
constexpr int CF_FR = 64;   // feature rows per state stage
constexpr int CF_NST = 3;   // attention ring
constexpr int CF_LEAD_BLOCKS = 2;   // row blocks of a chunk that are started before the longest ones (see the kernel)
constexpr float CF_LOG_EPS = 1e-7f, CF_SUM_EPS = 1e-6f, CF_EXP_CLAMP = 80.f;
constexpr float CF_LOG2E = 1.4426950408889634f, CF_EXP2_CLAMP = CF_EXP_CLAMP * CF_LOG2E;

// Stage order of the state sweep over (strip y, first x column X0): blocks below the diagonal four x columns at a time,
// then the diagonal block as quarters -- x columns 0-3 and 4-7 with the upper eight w counted twice (they stand for
// the mirrored quarter as well), and one "narrow" stage for the quarter of the upper eight x and w.
struct CfFeatIter {
  int y, X0, T;
  __device__ bool narrow() const { return X0 == 16 * y + 8; }
  __device__ bool enters_diag() const { return X0 == 16 * y; }
  __device__ void init(int T_) { T = T_; y = 0; X0 = 0; }
  __device__ bool done() const { return y >= T; }
  __device__ int f0() const { return 128 * y * (y + 1) + 16 * X0; }
  __device__ void next() {
    X0 += narrow() ? 8 : 4;
    if (X0 == 16 * (y + 1)) { y++; X0 = 0; }
  }
};

template <typename T, int DH>
__global__ __launch_bounds__(256, 3) void chunk_fwd_kernel(ChunkFwdArgs a, int row_blocks, int npairs) {
  typedef typename VecOf<T>::v8 v8;
  typedef typename VecOf<T>::v4 v4;
  typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
  typedef __attribute__((address_space(3))) v8 lds_v8;
  typedef __attribute__((address_space(3))) f32x4 lds_f32x4;
  typedef __attribute__((address_space(3))) char lds_char;
  typedef __attribute__((address_space(3))) unsigned short lds_u16;
  constexpr int MT = 2, KS = DH / 32, NT = DH / 16, TT = DH / 16, KT = CF_BN / 16, ROWS = 64 * MT, CPR = DH / 8, RB = CPR * 16;
  constexpr int TILE = CF_BN * RB;                  // bytes of one K or V tile
  constexpr int STAGE = 2 * TILE + 4 * CF_BN * 4;   // K, V, raw gates, two sets of key gate factors
  constexpr int LOADS = 2 * CF_BN * CPR / 256;      // tile copies per thread per attention stage
  constexpr int D = 128 * TT * (TT + 1);
  constexpr int SSTAGE = CF_FR * DH * 2, SLOADS = CF_FR * CPR / 256, LDM = DH + 8;
  // LDS: [attention stage 0 | state ring: two stages, later the key-sum matrix | the workgroup's query rows]; the
  // attention stages 1 and 2 take the memory behind stage 0 once the state sweep is over.
  constexpr int RING_OFF = STAGE, XT_OFF = STAGE + 2 * SSTAGE;
  static_assert(STAGE % 1024 == 0 && SSTAGE % 1024 == 0, "tiles start on 1 KB boundaries");
  static_assert(XT_OFF + ROWS * DH * 2 <= CF_NST * STAGE, "the state phase fits behind attention stage 0");
  static_assert(DH * LDM * 2 <= 2 * SSTAGE, "the key-sum matrix fits the state ring");
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  char* ring = smem + RING_OFF;
  char* xt = smem + XT_OFF;

  const int tid = threadIdx.x, l = tid & 63, g = l >> 4, tcol = l & 15;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // (XCD, shader engine) groups take whole (chunk, head) pairs: see attention_fwd.hip
  const int grp = blockIdx.x % 32, u = blockIdx.x / 32, ppg = (npairs + 31) / 32;
  int pig, blk;
  deal_causal_blocks(u, row_blocks, ppg, pig, blk);
  const int pair = pig * 32 + grp;
  // Order of a pair's row blocks: the first two of the chunk, then the others from the last (which sees the most keys)
  // backwards.  Under gates that forget within a hundred steps or so only those first blocks sweep the state, which
  // then makes them the long ones of the pair by far (123 for 134 us when they are started first); where every block
  // sweeps it they are the shortest, and two short blocks at the front cost nothing.
  const int lead = row_blocks > CF_LEAD_BLOCKS ? CF_LEAD_BLOCKS : 0;
  const int rblk = blk < lead ? blk : row_blocks - 1 - (blk - lead);
  if (pair >= npairs) return;
  const int b = __builtin_amdgcn_readfirstlane(pair / a.h), hh = pair - b * a.h;
  const int hq = a.h * a.r, rows = a.c * a.r;
  const int row0 = rblk * ROWS;
  const T* Qg = (const T*)a.Q + (long)b * a.c * hq * DH;
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
  const float eps_s = CF_LOG_EPS / a.scale, eps2 = eps_s * eps_s;
  const float scale_p = a.scale * a.scale;
  const float l2sp = __log2f(scale_p);
  bool no_state = a.skip_first && (b % a.n == 0);

  const int last_row = min(row0 + ROWS, rows) - 1;
  const int kmax = min(a.c, last_row / a.r + 1);   // keys any row of the workgroup can see
  const int ntiles = (kmax + CF_BN - 1) / CF_BN;
  const int wslice = (u & 1) ? 3 - wave : wave;
  const int wrow0 = row0 + wslice * 16 * MT;
  const int w_first_ti = min(wrow0, rows - 1) / a.r;
  const int w_last_ti = min(wrow0 + 16 * MT - 1, rows - 1) / a.r;

  // ---- attention copies (as attention_fwd.hip) -------------------------------------------------------------------
  uint32_t goff[LOADS / 2];
#pragma unroll
  for (int ii = 0; ii < LOADS / 2; ii++) {
    const int pos = (ii * 4 + wave) * 64 + l, row = pos / CPR;
    goff[ii] = (uint32_t)(row * (int)kstride + 16 * ((pos % CPR) ^ swz<CPR, SWZ_ROW>(row)));
  }
  int it0 = 0;   // first key tile that is visited (set below); ring slots count from it: its slot is the one apart from
                 // the state phase's memory
  auto issue = [&](int it) __attribute__((always_inline)) {
    char* st = smem + ((it - it0) % CF_NST) * STAGE;
    const int j0 = it * CF_BN;
    if (j0 + CF_BN <= a.c) {
      const char* kb_ = Kg + (long)j0 * kstride;
      const char* vb_ = Vg + (long)j0 * kstride;
      const uint32_t sa = lds_addr(st) + wave * 1024;
#pragma unroll
      for (int ii = 0; ii < LOADS / 2; ii++) async_copy16_sv(kb_, goff[ii], sa + ii * 4096);
#pragma unroll
      for (int ii = 0; ii < LOADS / 2; ii++) async_copy16_sv(vb_, goff[ii], sa + TILE + ii * 4096);
    } else {   // last, partial tile: rows past the end repeat the last key (they are masked)
      async_load_tile<CPR, CF_BN, SWZ_ROW>(st, [&](int row) { return Kg + (long)min(j0 + row, a.c - 1) * kstride; });
      async_load_tile<CPR, CF_BN, SWZ_ROW>(st + TILE, [&](int row) { return Vg + (long)min(j0 + row, a.c - 1) * kstride; });
    }
    if (Gg && wave == 0) async_copy4(Gg + (long)min(j0 + l, a.c - 1) * a.h, st + 2 * TILE);
  };
  // ---- the workgroup's query rows, into LDS (operands of both parts) ---------------------------------------------
  auto row_off = [&](int row) -> long {   // element offset of a (clamped) folded row, per unit of the last dim
    row = min(row, rows - 1);
    const int t = row / a.r, rr = row - t * a.r;
    return (long)t * hq + hh * a.r + rr;
  };
  auto x_ptr = [&](int lrow, int col) -> const char* {
    return xt + lrow * (DH * 2) + (((col / 8) ^ swz<CPR>(lrow)) * 16) + (col % 8) * 2;
  };
  async_load_tile<CPR, ROWS>(xt, [&](int row) { return (const char*)(Qg + row_off(row0 + row) * DH); });

  // ---- what the gates have already forgotten -------------------------------------------------------------------
  // A key tile entirely in a wave's past enters with the factor exp(R - A_last), R the gate sum at the wave's first row
  // and A_last the one at the tile's last key.  Once that factor has underflowed to zero for the LARGEST gate sum among
  // the workgroup's rows (its first row's: gate sums only fall along a chunk, unless the caller's log gates are
  // positive) it is zero for every wave: the oldest tiles for which it has, as far as they lie before the workgroup's
  // first row, contribute exact zeros and are neither copied nor visited (it0 = the first tile that is).  Likewise the
  // state part of a wave's rows carries exp(R): with exp of that largest sum underflowed, the sweep over the state adds
  // exact zeros to every row of the workgroup and is left out.  (Nothing changes for gates that do not decay that far.)
  if (Gg && a.gate_skip) {
    // (the largest gate sum among the workgroup's rows: the first row's, unless the caller's log gates are positive)
    float a_first = -INFINITY;
    for (int i = l; i < ROWS; i += 64) a_first = fmaxf(a_first, Gg[(long)(min(row0 + i, rows - 1) / a.r) * a.h]);
#pragma unroll
    for (int m = 32; m > 0; m >>= 1) a_first = fmaxf(a_first, __shfl_xor(a_first, m));
    if (__expf(a_first) == 0.f) no_state = true;
    for (int base = 0; base < ntiles; base += 64) {
      const int tl = min(base + l, ntiles - 1);
      const float a_last = Gg[(long)min(CF_BN * tl + CF_BN - 1, a.c - 1) * a.h];
      const unsigned long long dead = __ballot(__expf(fminf(a_first - a_last, CF_EXP_CLAMP)) == 0.f);
      const int lanes = min(64, ntiles - base);
      const int nd = __builtin_popcountll(lanes == 64 ? dead : (dead & ((1ull << lanes) - 1)));
      it0 += nd;
      if (nd < lanes) break;
    }
    it0 = __builtin_amdgcn_readfirstlane(min(min(it0, ntiles - 1), min(row0 / a.r + 1, a.c) / CF_BN));
  }
  issue(it0);   // older than every copy of the state phase but the rows', so it has landed whenever one of those has

  int ti[MT], lrow[MT];
  long qoff[MT];
  bool live[MT];
  float Gq2[MT], mx[MT], lq[MT];   // Gq2 = log2(scale^2 exp(A_i))
#pragma unroll
  for (int mi = 0; mi < MT; mi++) {
    lrow[mi] = wslice * 16 * MT + 16 * mi + tcol;
    const int row = row0 + lrow[mi];
    live[mi] = row < rows;
    const int rr = live[mi] ? row : 0;
    ti[mi] = rr / a.r;
    qoff[mi] = (long)ti[mi] * hq + hh * a.r + (rr - ti[mi] * a.r);
    Gq2[mi] = __builtin_fmaf(Gg ? Gg[(long)ti[mi] * a.h] : 0.f, CF_LOG2E, l2sp);
    mx[mi] = 0.f;
    lq[mi] = 0.f;
  }
  f32x4 acc[MT][NT], accl[MT];
#pragma unroll
  for (int mi = 0; mi < MT; mi++) {
#pragma unroll
    for (int nt = 0; nt < NT; nt++) acc[mi][nt] = (f32x4){0, 0, 0, 0};
    accl[mi] = (f32x4){0, 0, 0, 0};
  }
  const float Rw = Gg ? Gg[(long)w_first_ti * a.h] : 0.f;   // gate at the wave's first row

  // ---- state part --------------------------------------------------------------------------------------------
  if (no_state) {
    wait_vmcnt<0>();
    lds_barrier();
  } else {
    uint32_t boffs[SLOADS], boffs_n[SLOADS];
#pragma unroll
    for (int ii = 0; ii < SLOADS; ii++) {
      const int pos = (ii * 4 + wave) * 64 + l, row = pos / CPR;
      boffs[ii] = (uint32_t)(row * (DH * 2) + 16 * ((pos % CPR) ^ swz<CPR>(row)));
      // narrow stage: contraction step ks, lane group g take x column 8 + 2 ks + (g & 1) + 4 (g >> 1); stage row
      // 32 ks + 8 g + i is state row 16 * column + 8 + i
      const int gg = (row / 8) % 4, xcol = 2 * (row / 32) + (gg & 1) + 4 * (gg >> 1);
      boffs_n[ii] = (uint32_t)((16 * xcol + 8 + row % 8) * (DH * 2) + 16 * ((pos % CPR) ^ swz<CPR>(row)));
    }
    const uint32_t ring_lds = lds_addr(ring) + wave * 1024;
    auto issue_s = [&](int f0, int ringpos, bool narrow) {
      const char* src = Sg + (long)f0 * DH * 2;
#pragma unroll
      for (int ii = 0; ii < SLOADS; ii++)
        async_copy16_sv(src, narrow ? boffs_n[ii] : boffs[ii], ring_lds + ringpos * SSTAGE + ii * 4096);
    };
    CfFeatIter cur, nxt;
    cur.init(TT);
    nxt.init(TT);
    issue_s(nxt.f0(), 0, nxt.narrow());
    nxt.next();
    int issued = 1, step = 0, y_loaded = -1;
    float prow[MT][8];
    const uint32_t ring_a = (uint32_t)(uintptr_t)(lds_char*)ring, xt_a = (uint32_t)(uintptr_t)(lds_char*)xt;
    uint32_t boff[NT][2];   // state tile, transposed read: rows 8g + (s >> 2) (+4), columns 16 nt + 4 (s & 3) ..
#pragma unroll
    for (int nt = 0; nt < NT; nt++)
#pragma unroll
      for (int hf = 0; hf < 2; hf++) {
        const int row = 8 * g + 4 * hf + (tcol >> 2), col = 16 * nt + 4 * (tcol & 3);
        boff[nt][hf] = ring_a + row * (CPR * 16) + (((col / 8) ^ swz<CPR>(row)) * 16) + (col % 8) * 2;
        asm volatile("" : "+v"(boff[nt][hf]));
      }
    const int xlane = 2 * (g >> 1), xlane_n = 2 * ((g & 1) + 4 * (g >> 1));
    uint32_t xrow_a[MT], xsw[MT];
#pragma unroll
    for (int mi = 0; mi < MT; mi++) {
      xrow_a[mi] = xt_a + lrow[mi] * (DH * 2);
      xsw[mi] = swz<CPR>(lrow[mi]);
    }
    auto stage = [&](auto sl_c) __attribute__((always_inline)) {
      constexpr int SL = decltype(sl_c)::value;
      if (issued > step + 1) wait_vmcnt<SLOADS>(); else wait_vmcnt<0>();
      lds_barrier();
      if (!nxt.done()) {
        issue_s(nxt.f0(), 1 - SL, nxt.narrow());
        nxt.next();
        issued++;
      }
      const bool narrow = cur.narrow();
      if (cur.y != y_loaded || narrow) {
        y_loaded = narrow ? -1 : cur.y;
        const int half = narrow ? 8 : 8 * (g & 1);
#pragma unroll
        for (int mi = 0; mi < MT; mi++) unpack8(*(const v8*)x_ptr(lrow[mi], 16 * cur.y + half), prow[mi]);
      }
      if (cur.enters_diag()) {   // quarter (x < 8, w >= 8) stands for its mirror image as well
        const float f = (g & 1) ? 2.f : 1.f;
#pragma unroll
        for (int mi = 0; mi < MT; mi++)
#pragma unroll
          for (int i = 0; i < 8; i++) prow[mi][i] *= f;
      }
      uint32_t xa[MT];
      {
        const int xc = cur.X0 >> 3, xo = (cur.X0 & 7) * 2 + (narrow ? xlane_n : xlane);
#pragma unroll
        for (int mi = 0; mi < MT; mi++) { xa[mi] = xrow_a[mi] + ((xc ^ xsw[mi]) << 4) + xo; asm volatile("" : "+v"(xa[mi])); }
      }
#pragma unroll
      for (int ks = 0; ks < CF_FR / 32; ks++) {
        v8 vf[NT];
#pragma unroll
        for (int nt = 0; nt < NT; nt++) {
          const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(boff[nt][0] + SL * SSTAGE + ks * 32 * (CPR * 16)));
          const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(boff[nt][1] + SL * SSTAGE + ks * 32 * (CPR * 16)));
          vf[nt] = __builtin_bit_cast(v8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
        }
#pragma unroll
        for (int mi = 0; mi < MT; mi++) {
          const unsigned short xbits = *(const lds_u16*)(xa[mi] + 4 * ks);
          const float xs = (float)__builtin_bit_cast(T, xbits);
          float pr8[8];
#pragma unroll
          for (int i = 0; i < 8; i++) pr8[i] = xs * prow[mi][i];
          const v8 af = pack8<T>(pr8);
          // (state tile first, phi^T second: the accumulator comes out in the attention part's layout)
#pragma unroll
          for (int nt = 0; nt < NT; nt++) acc[mi][nt] = mfma16(vf[nt], af, acc[mi][nt]);
        }
      }
      cur.next();
      step++;
    };
    while (!cur.done()) {
      stage(IC<0>{});
      if (cur.done()) break;
      stage(IC<1>{});
    }

    // lq[row] = x^T M x with M[a, b] = sc of the stored pair (a, b): U^T[b, row] = sum_a M[a, b] x[row, a] on the matrix
    // cores (M in a high and a low 16-bit part), then a dot with x[row, b] down the accumulator rows
    T* Mt = (T*)ring;   // [DH (a)][LDM (b)]
    float aux[MT] = {0.f, 0.f};
    for (int part = 0; part < 2; part++) {
      lds_barrier();
      for (int idx = tid; idx < DH * TT; idx += 256) {
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
        for (int ks = 0; ks < KS; ks++) xf[ks] = *(const v8*)x_ptr(lrow[mi], 32 * ks + 8 * g);
#pragma unroll
        for (int wt = 0; wt < TT; wt++) {
          f32x4 t = {0, 0, 0, 0};
#pragma unroll
          for (int ks = 0; ks < KS; ks++) t = mfma16(lds_frag_tr<T>(Mt, LDM, 32 * ks, 16 * wt), xf[ks], t);
          const v4 xb4 = *(const v4*)x_ptr(lrow[mi], 16 * wt + 4 * g);
#pragma unroll
          for (int v = 0; v < 4; v++) aux[mi] += t[v] * (float)xb4[v];
        }
      }
    }
    // hand over to the attention part: exp(R) times the state part, which the row factor of the past tiles completes
    const float eR = __expf(Rw);   // (may underflow: the state part of these rows is then zero, as its definition has it)
#pragma unroll
    for (int mi = 0; mi < MT; mi++) {
      lq[mi] = sum_over_rows(aux[mi]) * eR;
#pragma unroll
      for (int nt = 0; nt < NT; nt++) acc[mi][nt] *= eR;
    }
  }

  // the wave's query rows as the second operand of S^T = K Q^T, from the LDS copy
  v8 Qf[MT][KS];
#pragma unroll
  for (int mi = 0; mi < MT; mi++)
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      u32x4 z = *(const u32x4*)x_ptr(lrow[mi], 32 * ks + 8 * g);
      if (!live[mi]) z = (u32x4){0, 0, 0, 0};
      Qf[mi][ks] = __builtin_bit_cast(v8, z);
    }
  lds_barrier();   // every wave is done with the state ring and the query rows: attention stages 1, 2 may land there
  if (ntiles > it0 + 1) issue(it0 + 1);

  // ---- attention part (attention_fwd.hip, bf16 path) -----------------------------------------------------------
  const uint32_t one2 = 0x3F803F80u;
  v8 ones = __builtin_bit_cast(v8, (u32x4){one2, one2, one2, one2});
  asm volatile("" : "+v"(ones));
  int koff[KS], voff[NT];
#pragma unroll
  for (int ks = 0; ks < KS; ks++) koff[ks] = tcol * RB + (((4 * ks + g) ^ swz<CPR, SWZ_ROW>(tcol)) * 16);
  {
    const int vr = 4 * g + (tcol >> 2);
#pragma unroll
    for (int nt = 0; nt < NT; nt++) {
      const int col = 16 * nt + 4 * (tcol & 3);
      voff[nt] = vr * RB + (((col / 8) ^ swz<CPR, SWZ_ROW>(vr)) * 16) + (col % 8) * 2;
    }
  }
  const int n_past = min(ntiles, min(w_first_ti + 1, a.c) / CF_BN);   // tiles with every pair visible
  const int n_seen = min(ntiles, w_last_ti / CF_BN + 1);              // tiles with at least one visible pair
  auto gate_factors = [&](int it) __attribute__((always_inline)) {
    float* graw = (float*)(smem + ((it - it0) % CF_NST) * STAGE + 2 * TILE);
    const int rpos = min(CF_BN - 1, a.c - 1 - it * CF_BN);
    const float gv = Gg ? graw[l] : 0.f;
    const float R_ = Gg ? graw[rpos] : 0.f;
    graw[CF_BN + l] = __expf(fminf(R_ - gv, CF_EXP_CLAMP));
    graw[2 * CF_BN + l] = gv * CF_LOG2E;   // the gate itself, in powers of two, for the diagonal tiles
    if (!Gg) graw[l] = 0.f;
  };
  if (wave == 0) {
    if (ntiles > it0 + 1) wait_vmcnt<LOADS + 1>(); else wait_vmcnt<0>();   // all but the stage just issued
    gate_factors(it0);
  }
  auto sync_step = [&](int it) __attribute__((always_inline)) -> char* {
    char* st = smem + ((it - it0) % CF_NST) * STAGE;
    if (it + 1 < ntiles) wait_vmcnt<LOADS>(); else wait_vmcnt<0>();
    lds_barrier();
    if (it + 2 < ntiles) issue(it + 2);
    if (wave == 0 && it + 1 < ntiles) {
      if (it + 2 < ntiles) wait_vmcnt<LOADS + 1>(); else wait_vmcnt<0>();
      gate_factors(it + 1);
    }
    return st;
  };
  auto tile = [&](int it, const char* st, auto diag_c) __attribute__((always_inline)) {
    constexpr bool DIAG = decltype(diag_c)::value != 0;
    const int j0 = it * CF_BN;
    const float* graw = (const float*)(st + 2 * TILE);
    uint32_t kb[KS], vb[NT], eb;
    {
      const uint32_t sa = (uint32_t)(uintptr_t)(lds_char*)st;
#pragma unroll
      for (int ks = 0; ks < KS; ks++) { kb[ks] = sa + koff[ks]; asm volatile("" : "+v"(kb[ks])); }
#pragma unroll
      for (int nt = 0; nt < NT; nt++) { vb[nt] = sa + TILE + voff[nt]; asm volatile("" : "+v"(vb[nt])); }
      eb = sa + 2 * TILE + (DIAG ? 2 * CF_BN : CF_BN) * 4 + 16 * g;
      asm volatile("" : "+v"(eb));
    }
    int lim[MT];
#pragma unroll
    for (int mi = 0; mi < MT; mi++) lim[mi] = min(ti[mi], a.c - 1) - j0 - 4 * g;
    const float cw = DIAG ? 1.f : __expf(fminf(Rw - graw[CF_BN - 1], CF_EXP_CLAMP));
    // (forgotten by this wave's rows, though not by the workgroup's first: every weight of the tile is an exact zero)
    if (!DIAG && a.gate_skip && __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, cw)) == 0) return;
#pragma unroll
    for (int kp = 0; kp < KT / 2; kp++) {
      if (DIAG && j0 + 32 * kp > w_last_ti) continue;   // these 32 keys come after every row of the wave
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
      v8 vf[NT];
#pragma unroll
      for (int nt = 0; nt < NT; nt++) {
        const uint32_t vp = vb[nt] + kp * 32 * RB;
        const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)vp);
        const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(vp + 16 * RB));
        vf[nt] = __builtin_bit_cast(v8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
      }
      v8 pf[MT];
#pragma unroll
      for (int mi = 0; mi < MT; mi++) {
        float p[8];
#pragma unroll
        for (int half = 0; half < 2; half++) {
#pragma unroll
          for (int v = 0; v < 4; v++) {
            float w = __builtin_fmaf(sc[half][mi][v], sc[half][mi][v], eps2);
            if (DIAG) {
              w *= __builtin_amdgcn_exp2f(fminf(Gq2[mi] - ev[half][v], CF_EXP2_CLAMP));
              w = (32 * kp + 16 * half + v <= lim[mi]) ? w : 0.f;
            } else {
              w *= ev[half][v];
            }
            p[4 * half + v] = w;
          }
        }
#pragma unroll
        for (int e = 0; e < 8; e++) mx[mi] = fmaxf(mx[mi], p[e]);
        pf[mi] = pack8<T>(p);
      }
#pragma unroll
      for (int mi = 0; mi < MT; mi++) accl[mi] = mfma16(ones, pf[mi], accl[mi]);
#pragma unroll
      for (int nt = 0; nt < NT; nt++)
#pragma unroll
        for (int mi = 0; mi < MT; mi++) acc[mi][nt] = mfma16(vf[nt], pf[mi], acc[mi][nt]);
    }
  };

  int it = it0;
  for (; it < n_past; it++) tile(it, sync_step(it), IC<0>{});
  // the past tiles and the state part were accumulated without the row factor exp(A_i - R) * scale^2; apply it once
#pragma unroll
  for (int mi = 0; mi < MT; mi++) {
    const float f = __builtin_amdgcn_exp2f(fminf(Gq2[mi] - Rw * CF_LOG2E, CF_EXP2_CLAMP));
#pragma unroll
    for (int nt = 0; nt < NT; nt++) acc[mi][nt] *= f;
    accl[mi] *= f;
    mx[mi] *= f;
    lq[mi] *= f;
  }
  for (; it < n_seen; it++) tile(it, sync_step(it), IC<1>{});
  for (; it < ntiles; it++) sync_step(it);

  // ---- merge and store -------------------------------------------------------------------------------------------
  T* Og = (T*)a.O + (long)b * a.c * hq * DH;
  const float log_gamma = 0.5f * __logf((float)D);
#pragma unroll
  for (int mi = 0; mi < MT; mi++) {
    const float wmax = max_over_rows(mx[mi]);   // = exp(rowmax)
    if (!live[mi]) continue;
    const float den_abs = accl[mi][0] + wmax * CF_SUM_EPS + lq[mi];
    const float inv = 1.f / den_abs;
#pragma unroll
    for (int nt = 0; nt < NT; nt++) {
      float o4[4];
#pragma unroll
      for (int v = 0; v < 4; v++) o4[v] = acc[mi][nt][v] * inv;
      *(v4*)(Og + qoff[mi] * DH + 16 * nt + 4 * g) = pack4<T>(o4);
    }
    if (g == 0) {
      const long o = (long)b * a.c * hq + qoff[mi];
      const float m = __logf(wmax);
      a.rowmax[o] = m;
      a.den[o] = den_abs * __expf(-fmaxf(m, log_gamma));
    }
  }
}

template <typename T, int DH> static int chunk_fwd_launch(const ChunkFwdArgs& a, int BN, hipStream_t st) {
  constexpr int STAGE = 2 * CF_BN * DH * 2 + 4 * CF_BN * 4;
  constexpr size_t smem = CF_NST * STAGE;
  const int rows = a.c * a.r, row_blocks = (rows + 127) / 128, npairs = BN * a.h;
  dim3 grid((unsigned)(((npairs + 31) / 32) * 32 * row_blocks));
  auto kern = chunk_fwd_kernel<T, DH>;
  allow_big_lds((const void*)kern, smem);
  PR_LAUNCH("chunk_fwd", kern, grid, dim3(256), smem, st, a, row_blocks, npairs);
  return (int)hipGetLastError();
}

// 1 where the one-kernel forward exists: bf16, head dim 32 or 64
int chunk_fwd_supported(int d, int dtype) { return dtype == DT_BF16 && (d == 32 || d == 64); }

int chunk_fwd(const ChunkFwdArgs& a, int BN, int d, int dtype, hipStream_t st) {
  if (dtype != DT_BF16) return -1;
  switch (d) {
    case 32: return chunk_fwd_launch<bf16_t, 32>(a, BN, st);
    case 64: return chunk_fwd_launch<bf16_t, 64>(a, BN, st);
    default: return -2;
  }
}

}  // namespace pr
