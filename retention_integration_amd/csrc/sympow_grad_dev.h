// Device side of sympow_grad.hip (constants, helpers and the kernel body), shared with the kernels that run this body next
// to another one in a single launch (sympow_dvdk.hip).
#pragma once
#include "common.h"
#include "kernels.h"

namespace pr {

constexpr int GR_FR = 64;    // feature rows per stage
constexpr int GR_NST = 2;   // ring stages; the stage loop is unrolled over them (see there)

template <typename T> struct OnePair;   // two packed 1.0 values
template <> struct OnePair<bf16_t> { static constexpr uint32_t v = 0x3F803F80u; static constexpr float down = 1.f, up = 1.f; };
template <> struct OnePair<f16_t> { static constexpr uint32_t v = 0x3C003C00u; static constexpr float down = 1.f / 256.f, up = 256.f; };

// the two 16-bit values of one dword as floats
template <typename T> __device__ __forceinline__ void unpack2(uint32_t u, float& lo, float& hi);
template <> __device__ __forceinline__ void unpack2<bf16_t>(uint32_t u, float& lo, float& hi) {
  lo = __builtin_bit_cast(float, u << 16);
  hi = __builtin_bit_cast(float, u & 0xffff0000u);
}
template <> __device__ __forceinline__ void unpack2<f16_t>(uint32_t u, float& lo, float& hi) {
  typedef __attribute__((ext_vector_type(2))) _Float16 h2;
  const h2 p = __builtin_bit_cast(h2, u);
  lo = (float)p[0];
  hi = (float)p[1];
}

// SYM: the caller guarantees B[(a, b)] == B[(b, a)] inside the blocks on the diagonal (true of every state and state
// gradient this library forms: both orders of a pair are the same sum).  dphi is then symmetric there, the two folds
// of a diagonal block are equal, and the block takes twice the first fold instead of both.
template <typename T, int DK, int DV, int MT, bool MULT, bool SYM, bool ALONE>
__device__ __forceinline__ void sympow_grad_body(const GradArgs& a, int row_blocks, int npairs, int vblock) {
  typedef typename VecOf<T>::v8 v8;
  typedef typename VecOf<T>::v4 v4;
  constexpr int TT = DK / 16, KS = DV / 32, KX = DK / 32, ROWS = 64 * MT, CB = DV / 8, CX = DK / 8;
  constexpr int D = 128 * TT * (TT + 1), NSTEP = D / GR_FR;
  constexpr int STAGE = GR_FR * DV * 2;
  constexpr int LOADS = GR_FR * CB / 256;
  constexpr int LDM = DK + 8;
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  char* ring = smem;                                         // [NST][STAGE]; reused for M at the end
  constexpr int RING_BYTES = GR_NST * STAGE > DK * LDM * 2 ? GR_NST * STAGE : DK * LDM * 2;   // the ring later holds M
  char* xt = ring + (RING_BYTES + 1023) / 1024 * 1024;       // [ROWS][DK] T, swizzled

  // XCD-aware placement: consecutive workgroup ids go to different XCDs, so id % 8 picks the XCD
  const int xcd = vblock % 8, slot = vblock / 8;
  const int pair = (slot / row_blocks) * 8 + xcd;
  if (pair >= npairs) return;
  // (the row blocks of a pair stay neighbours in launch order, but which of them comes first rotates from pair to pair:
  // when the blocks of one position finish at once -- zero rows, see below -- the ones that do work would otherwise sit
  // at a fixed stride of the launch order, and with it on a fixed subset of the compute units)
  const int row0 = ((slot + slot / row_blocks) % row_blocks) * ROWS;
  const int bn = pair / a.h, hh = pair % a.h;

  const int tid = threadIdx.x, l = tid & 63, g = l >> 4, tcol = l & 15;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int hA = a.h * a.r, rows = a.c * a.r;
  const T* Xg = (const T*)a.X + (long)bn * a.c * hA * DK;
  const T* Gg = (const T*)a.G + (long)bn * a.c * hA * DV;
  const char* Bg = (const char*)((const T*)a.B + ((long)bn * a.h + hh) * D * DV);
  const float* sBg = a.sB + ((long)bn * a.h + hh) * D;
  // (B, sB are a gated scan's output: with a zero carry into it, an entry is the scan's input entry next to it, bit for
  // bit -- bn + 1 for the reverse scan, bn - 1 for the forward one, whose entry 1 is its input entry 0 whatever the gate)
  if (a.B_alt && (a.alt_shift > 0 ? bn % a.n != a.n - 1 : bn % a.n != 0)) {
    const int nb = bn + a.alt_shift;
    const bool first = a.alt_shift < 0 && (a.skip_first & 1) && nb % a.n == 0;
    if (first || __expf(a.carry[(long)nb * a.h + hh]) == 0.f) {
      Bg = (const char*)((const T*)a.B_alt + ((long)nb * a.h + hh) * D * DV);
      sBg = a.sB_alt + ((long)nb * a.h + hh) * D;
    }
  }
  T* dXg = (T*)a.dX + (long)bn * a.c * hA * DK;
  auto row_off = [&](int row) -> long {
    row = min(row, rows - 1);
    const int t = row / a.r, rr = row - t * a.r;
    return (long)t * hA + hh * a.r + rr;
  };

  // (skip_first: bit 0 = the first, bit 1 = the last chunk of every n contributes nothing and is written as zeros)
  auto write_zeros = [&]() {
    for (int i = tid; i < ROWS * DK / 8; i += 256) {
      const int rl = i / (DK / 8), col = (i % (DK / 8)) * 8;
      if (row0 + rl < rows) *(u32x4*)(dXg + row_off(row0 + rl) * DK + col) = (u32x4){0, 0, 0, 0};
    }
  };
  if (a.skip_first && (((a.skip_first & 1) && bn % a.n == 0) || ((a.skip_first & 2) && bn % a.n == a.n - 1))) {
    write_zeros();
    return;
  }

  // B rows are contiguous: the copies of a stage have fixed lane offsets and a base that moves in scalar registers
  uint32_t boffs[LOADS];
#pragma unroll
  for (int ii = 0; ii < LOADS; ii++) {
    const int pos = (ii * 4 + wave) * 64 + l, row = pos / CB;
    boffs[ii] = (uint32_t)(row * (DV * 2) + 16 * ((pos % CB) ^ swz<CB, SWZ_ROW>(row)));
  }
  const uint32_t ring_lds = lds_addr(ring) + wave * 1024;
  // ALONE: one row block per (chunk, head), so nobody else reads this state and its copies are marked non-temporal
  // (1.5 % of a training step at chunks of 128 rows; with several row blocks the tiles are shared through L2 and the
  // mark costs 10 us of a step at the headline shape).  A template parameter: as a run-time flag it cost the other
  // case 10 us through the registers and the schedule the compiler then chose.
  auto issue = [&](int step) {
    const char* src = Bg + (long)step * GR_FR * DV * 2;
    if constexpr (ALONE) {
#pragma unroll
      for (int ii = 0; ii < LOADS; ii++) async_copy16_sv_nt(src, boffs[ii], ring_lds + (step % GR_NST) * STAGE + ii * 4096);
    } else {
#pragma unroll
      for (int ii = 0; ii < LOADS; ii++) async_copy16_sv(src, boffs[ii], ring_lds + (step % GR_NST) * STAGE + ii * 4096);
    }
  };
  // (live_rows, side 0: up to the last multiple of 256 rows before the first live time step, dX -- a zero -- is not even
  // written: its reader, attention_bwd's epilogue, is given the same live_rows and does not read it)
  if (a.live_rows && a.live_side == 0 && row0 + ROWS <= ((a.live_rows[((long)bn * a.h + hh) * 2] * a.r) & ~255)) return;
  // X rows of this workgroup (waited for together with stage 0), then the first stage(s)
  async_load_tile<CX, ROWS>(xt, [&](int row) { return (const char*)(Xg + row_off(row0 + row) * DK); });
  issue(0);
  if (GR_NST > 2) issue(1);
  // dX is linear in the row's x (every feature is a product of two of its entries) and in the pair (g, cvec) of the
  // row.  live_rows (per (chunk, head): {first time step whose x row -- a discounted key -- is not an exact zero, end of
  // the time steps whose (g, cvec) -- a query row's scaled dO and key-sum factor -- are not}; live_side says which of the
  // two applies to this call) bounds the rows that can have a gradient: a block outside them is written as zeros
  // without the sweep.
  if (a.live_rows) {
    const int v = a.live_rows[((long)bn * a.h + hh) * 2 + a.live_side];
    if (a.live_side == 0 ? row0 + ROWS <= v * a.r : row0 >= v * a.r) {
      wait_vmcnt<0>();
      write_zeros();
      return;
    }
  }

  // per-lane row data (row = this lane's column of the dphi^T tiles)
  v8 Gf[MT][KS];
  int lrow[MT];
  bool live[MT];
#pragma unroll
  for (int mi = 0; mi < MT; mi++) {
    lrow[mi] = wave * 16 * MT + 16 * mi + tcol;
    live[mi] = row0 + lrow[mi] < rows;
    const long ro = row_off(row0 + lrow[mi]);
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      u32x4 z = *(const u32x4*)(Gg + ro * DV + 32 * ks + 8 * g);
      if (!live[mi]) z = (u32x4){0, 0, 0, 0};
      Gf[mi][ks] = __builtin_bit_cast(v8, z);
    }
  }
  auto x_ptr = [&](int mi, int col) -> const char* {   // address of X[lrow[mi], col] in the swizzled tile
    return xt + lrow[mi] * (DK * 2) + (((col / 8) ^ swz<CX>(lrow[mi])) * 16) + (col % 8) * 2;
  };

  f32x4 acc[MT][TT];            // dX^T[16*blk + 4g + v, row]
#pragma unroll
  for (int mi = 0; mi < MT; mi++)
#pragma unroll
    for (int k = 0; k < TT; k++) acc[mi][k] = (f32x4){0, 0, 0, 0};

  // Per-lane LDS byte addresses, hoisted out of the stage loop (the swizzle of a row depends only on its position
  // inside a group of 16 rows, so a stage adds a scalar base and the rest are immediate offsets).
  typedef __attribute__((address_space(3))) char lds_char;
  typedef __attribute__((address_space(3))) v8 lds_v8;
  typedef __attribute__((address_space(3))) uint32_t lds_u32;
  const uint32_t ring_a = (uint32_t)(uintptr_t)(lds_char*)ring, xt_a = (uint32_t)(uintptr_t)(lds_char*)xt;
  uint32_t aoff[KS];            // B rows as the A operand: row tcol of a 16-row group, chunk 4*ks + g
#pragma unroll
  for (int ks = 0; ks < KS; ks++) aoff[ks] = tcol * (CB * 16) + (((4 * ks + g) ^ swz<CB, SWZ_ROW>(tcol)) * 16);
  uint32_t aoffa[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ks++) { aoffa[ks] = ring_a + aoff[ks]; asm volatile("" : "+v"(aoffa[ks])); }
  uint32_t xrow_a[MT], xsw[MT];
#pragma unroll
  for (int mi = 0; mi < MT; mi++) {
    xrow_a[mi] = xt_a + lrow[mi] * (DK * 2);
    xsw[mi] = swz<CX>(lrow[mi]);
  }

  // Blocks (y, xb) in memory order, both compile-time indices so that the two folds accumulate straight into the
  // accumulators of strip y and strip xb; only the four stages of a block are a run-time loop.  With the key-side
  // multiplier (2 below the block diagonal) the strip-y accumulator is doubled once before the diagonal block and
  // the other fold uses doubled X values.
  int step = 0;
  static_for<TT>([&](auto yc) {
    constexpr int y = decltype(yc)::value;
    float xr[MT][4];              // X[row, 16y + 4g + v]
    static_for<y + 1>([&](auto xc) {
      constexpr int xb = decltype(xc)::value;
      constexpr bool diag = xb == y;
      // One stage, held in ring slot SL.  The slot is a compile-time constant (a block has an even number of stages, so
      // its stages alternate between the two slots starting at 0): every operand address is then a lane register plus
      // an immediate, which is worth more than a third stage in the ring (16 us of a training step at the headline
      // shape: the address additions per stage and their pinned registers).
      auto stage = [&](int sb, auto sl_c) __attribute__((always_inline)) {
        constexpr int SL = decltype(sl_c)::value;
        if (GR_NST > 2 && step + 1 < NSTEP) wait_vmcnt<LOADS>(); else wait_vmcnt<0>();
        lds_barrier();
        if (step + GR_NST - 1 < NSTEP) issue(step + GR_NST - 1);
        if (sb == 0 && (xb == 0 || (MULT && diag))) {   // (re)load the strip's X values; X tile is visible after the barrier
          const float m = (MULT && !diag) ? 2.f : 1.f;
#pragma unroll
          for (int mi = 0; mi < MT; mi++) {
            const v4 h4 = *(const v4*)x_ptr(mi, 16 * y + 4 * g);
#pragma unroll
            for (int v = 0; v < 4; v++) xr[mi][v] = (float)h4[v] * m;
            if (MULT && diag) acc[mi][y] *= 2.f;
          }
        }
        uint32_t ab[KS], xa[MT];
        {
#pragma unroll
          for (int ks = 0; ks < KS; ks++) ab[ks] = aoffa[ks];
          // X[row, 16*xb + (GR_FR/16)*sb + 2*pr2 (+1)]: one 32-bit read per pair of columns
          const int X0 = 16 * xb + (GR_FR / 16) * sb, xc = X0 >> 3, xo = (X0 & 7) * 2;
#pragma unroll
          for (int mi = 0; mi < MT; mi++) { xa[mi] = xrow_a[mi] + ((xc ^ xsw[mi]) << 4) + xo; asm volatile("" : "+v"(xa[mi])); }
        }
#pragma unroll
        for (int pr2 = 0; pr2 < GR_FR / 32; pr2++) {
          const int m0 = ((GR_FR / 16) * sb + 2 * pr2) % 16;
          v8 af0[KS], af1[KS];
#pragma unroll
          for (int ks = 0; ks < KS; ks++) {
            af0[ks] = *(const lds_v8*)(ab[ks] + SL * STAGE + (32 * pr2) * (CB * 16));
            af1[ks] = *(const lds_v8*)(ab[ks] + SL * STAGE + (32 * pr2 + 16) * (CB * 16));
          }
          // selector: accumulator row m0 sums the first 16 contraction slots (column X), row m0+1 the last 16
          const uint32_t s_lo = (tcol == m0) ? OnePair<T>::v : 0u, s_hi = (tcol == m0 + 1) ? OnePair<T>::v : 0u;
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
            float x0, x1;
            unpack2<T>(*(const lds_u32*)(xa[mi] + 4 * pr2), x0, x1);
            if constexpr (SYM && diag) {
              x0 += x0;
              x1 += x1;
            }
            acc[mi][y] = acc[mi][y] + d0[mi] * x0;   // each line contracts to one fused multiply-add per element
            acc[mi][y] = acc[mi][y] + d1[mi] * x1;
            if constexpr (SYM && diag) continue;
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
      static_assert(GR_NST == 2 && (256 / GR_FR) % 2 == 0, "stages of a block alternate between the two ring slots");
#pragma unroll 1
      for (int sb = 0; sb < 256 / GR_FR; sb += 2) {
        stage(sb, IC<0>{});
        stage(sb + 1, IC<1>{});
      }
    });
  });

  // sB term: dX_s[row, w] = cvec[row] * sum_a (U[a, w] + U[w, a]) X[row, a] with U[a, w] = m_f sB[f] for the stored
  // pair f = (a, w) and 0 elsewhere.  U is built in the (now idle) ring memory in two 16-bit parts (high, low), one
  // thread per (a, strip of 16 w): 16 consecutive floats of sB, 16 consecutive elements of U; U and U^T are both
  // read from the one tile (plain and transposing operand loads).
  T* Mt = (T*)ring;   // [DK (a)][LDM (w)]
  // Row offsets and cvec are (re)computed here, from a copy of the row index the compiler cannot match with the one
  // used before the sweep: nothing that is only needed now should stay in registers (or scratch) through it.
  float cv[MT];
  long rofs[MT];
#pragma unroll
  for (int mi = 0; mi < MT; mi++) {
    int lr = lrow[mi];
    asm volatile("" : "+v"(lr));
    rofs[mi] = row_off(row0 + lr);
    cv[mi] = live[mi] ? (a.cvec ? a.cvec[(long)bn * a.c * hA + rofs[mi]] : 1.f) : 0.f;
  }
  for (int part = 0; part < 2; part++) {
    lds_barrier();
    for (int idx = tid; idx < DK * TT; idx += 256) {
      const int aa = idx % DK, yb = idx / DK;
      float v16[16];
      if (aa < 16 * (yb + 1)) {
        const float m = ((MULT && aa < 16 * yb) ? 2.f : 1.f) * OnePair<T>::down;
        const f32x4* src = (const f32x4*)(sBg + 128 * yb * (yb + 1) + 16 * aa);
#pragma unroll
        for (int q = 0; q < 4; q++) {
          const f32x4 t4 = src[q];
#pragma unroll
          for (int v = 0; v < 4; v++) v16[4 * q + v] = t4[v] * m;
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
      v8 xf[KX];
#pragma unroll
      for (int ks = 0; ks < KX; ks++) xf[ks] = *(const v8*)x_ptr(mi, 32 * ks + 8 * g);
#pragma unroll
      for (int wt = 0; wt < TT; wt++) {
        f32x4 t = {0, 0, 0, 0};
#pragma unroll
        for (int ks = 0; ks < KX; ks++) {
          t = mfma16(lds_frag_tr<T>(Mt, LDM, 32 * ks, 16 * wt), xf[ks], t);   // sum_a U[a, w] x[a]
          t = mfma16(lds_frag<T>(Mt, LDM, 16 * wt, 32 * ks), xf[ks], t);      // sum_a U[w, a] x[a]
        }
        acc[mi][wt] += t * (cv[mi] * OnePair<T>::up);
      }
      __builtin_amdgcn_sched_barrier(0);   // one row tile at a time: the accumulators leave few registers free
    }
  }

#pragma unroll
  for (int mi = 0; mi < MT; mi++) {
    if (!live[mi]) continue;
    const long ro = rofs[mi];
#pragma unroll
    for (int k = 0; k < TT; k++) {
      float o4[4];
#pragma unroll
      for (int v = 0; v < 4; v++) o4[v] = acc[mi][k][v];
      *(v4*)(dXg + ro * DK + 16 * k + 4 * g) = pack4<T>(o4);
    }
  }
}

template <typename T, int DK, int DV, int MT, bool MULT, bool SYM, bool ALONE>
__global__ __launch_bounds__(256, (MT == 2 && DK <= 64) ? 4 : 2) void sympow_grad_kernel(GradArgs a, int row_blocks, int npairs) {
  sympow_grad_body<T, DK, DV, MT, MULT, SYM, ALONE>(a, row_blocks, npairs, (int)blockIdx.x);
}

}  // namespace pr
