// Device side of sympow_nn.hip (constants, helpers and the kernel body), shared with the kernels that run this body next
// to another one in a single launch (sympow_dvdk.hip).
#pragma once
#include "common.h"
#include "kernels.h"

namespace pr {

constexpr int NN_FR = 64;   // feature rows per stage
constexpr int NN_NST = 2;   // two stages keep three workgroups (12 waves) resident per CU, which hides more than a deeper ring

// Stage order over (strip y, first x column X0, a multiple of 4).  With the key-side multiplier the tiles
// below the block diagonal come first so that the accumulators can be doubled once.
//
// SYM (the caller's promise that B[(a, b)] == B[(b, a)] inside the blocks on the diagonal): a diagonal block is cut
// into its four 8 x 8 quarters (x half, w half).  Quarter (1, 0) is the mirror image of (0, 1) and is never read;
// (0, 1) counts twice instead.  The block then takes three stages instead of four: x columns 0-3 and 4-7 as before
// (with the w half 8..15 weighted 2) and ONE stage for quarter (1, 1), eight x columns times the eight w of the
// upper half ("narrow" stage).
template <bool MULT, bool SYM> struct FeatIter {
  int y, X0, phase, T;
  __device__ bool narrow() const { return SYM && X0 == 16 * y + 8; }
  __device__ bool enters_diag() const { return SYM && X0 == 16 * y; }
  __device__ void init(int T_) {
    T = T_;
    if (MULT && T > 1) { phase = 0; y = 1; X0 = 0; } else { phase = MULT ? 1 : 2; y = 0; X0 = 0; }
  }
  __device__ bool done() const { return y >= T; }
  __device__ int f0() const { return 128 * y * (y + 1) + 16 * X0; }
  // returns true when the stage just consumed was the last one below the diagonal
  __device__ bool next() {
    X0 += narrow() ? 8 : 4;
    if (phase == 0) {
      if (X0 == 16 * y) { y++; X0 = 0; }
      if (y == T) { phase = 1; y = 0; X0 = 0; return true; }
    } else if (phase == 1) {
      if (X0 == 16 * (y + 1)) { y++; X0 = 16 * y; }
    } else {
      if (X0 == 16 * (y + 1)) { y++; X0 = 0; }
    }
    return false;
  }
};

template <typename T> struct ScaleS;  // keeps sB inside the 16-bit range
template <> struct ScaleS<bf16_t> { static constexpr float down = 1.f, up = 1.f; };
template <> struct ScaleS<f16_t> { static constexpr float down = 1.f / 256.f, up = 256.f; };

template <typename T> struct PhiRow;
template <> struct PhiRow<bf16_t> {
  float row[8];
  __device__ __forceinline__ void load(const char* p) { unpack8(*(const bf16x8*)p, row); }
  __device__ __forceinline__ void scale(float f) {
#pragma unroll
    for (int i = 0; i < 8; i++) row[i] *= f;
  }
  __device__ __forceinline__ bf16x8 make(bf16_t x) const {
    const float xs = (float)x;
    float p[8];
#pragma unroll
    for (int i = 0; i < 8; i++) p[i] = xs * row[i];
    return pack8<bf16_t>(p);
  }
};
template <> struct PhiRow<f16_t> {
  f16x8 row;
  __device__ __forceinline__ void load(const char* p) { row = *(const f16x8*)p; }
  __device__ __forceinline__ void scale(float f) { row = row * (f16_t)f; }
  __device__ __forceinline__ f16x8 make(f16_t x) const { return row * x; }
};

template <typename T, int DK, int DV, int MT, bool MULT, int EPI, bool SYM, bool ALONE>
__device__ __forceinline__ void sympow_nn_body(const NNArgs& a, int row_blocks, int npairs, int vblock) {
  typedef typename VecOf<T>::v8 v8;
  typedef typename VecOf<T>::v4 v4;
  constexpr int NT = DV / 16, TT = DK / 16, KX = DK / 32, CB = DV / 8, CX = DK / 8;
  constexpr int D = 128 * TT * (TT + 1);
  constexpr int ROWS = 64 * MT, STAGE = NN_FR * DV * 2, LOADS = NN_FR * CB / 256, LDM = DK + 8;
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  char* ring = smem;                          // [NST][STAGE]; reused for M and the aux exchange at the end
  constexpr int RING_BYTES = NN_NST * STAGE > DK * LDM * 2 ? NN_NST * STAGE : DK * LDM * 2;   // the ring later holds M
  char* xt = ring + (RING_BYTES + 1023) / 1024 * 1024;   // [ROWS][DK] T, swizzled

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
  const char* Bg = (const char*)((const T*)a.B + ((long)bn * a.h + hh) * D * DV);
  // (B is a reverse scan's output: with a zero carry into it, entry bn is the scan's input entry bn + 1, bit for bit)
  if (a.B_alt && bn % a.n != a.n - 1 && __expf(a.carry[(long)(bn + 1) * a.h + hh]) == 0.f)
    Bg = (const char*)((const T*)a.B_alt + ((long)(bn + 1) * a.h + hh) * D * DV);
  const float* sBg = a.sB ? a.sB + ((long)bn * a.h + hh) * D : nullptr;
  auto row_off = [&](int row) -> long {  // element offset of a (clamped) folded row, per unit of the last dim
    row = min(row, rows - 1);
    const int t = row / a.r, rr = row - t * a.r;
    return (long)t * hA + hh * a.r + rr;
  };
  auto x_ptr = [&](int lrow, int col) -> const char* {
    return xt + lrow * (DK * 2) + (((col / 8) ^ swz<CX>(lrow)) * 16) + (col % 8) * 2;
  };
  // B rows are contiguous: the copies of a stage have fixed lane offsets and a base that moves in scalar registers
  uint32_t boffs[LOADS];
#pragma unroll
  for (int ii = 0; ii < LOADS; ii++) {
    const int pos = (ii * 4 + wave) * 64 + l, row = pos / CB;
    boffs[ii] = (uint32_t)(row * (DV * 2) + 16 * ((pos % CB) ^ swz<CB>(row)));
  }
  // the narrow stage of a symmetric diagonal block: eight x columns, the upper eight w of each.  Contraction step
  // ks, lane group g take x column 8 + 2*ks + (g & 1) + 4*(g >> 1), so that, as in every other stage, the x scalar of
  // step ks sits 4*ks bytes past a lane constant; stage row j = 32*ks + 8*g + i is B row 16 * column + 8 + i.
  uint32_t boffs_n[SYM ? LOADS : 1];
  if constexpr (SYM) {
#pragma unroll
    for (int ii = 0; ii < LOADS; ii++) {
      const int pos = (ii * 4 + wave) * 64 + l, row = pos / CB;
      const int gg = (row / 8) % 4, xcol = 2 * (row / 32) + (gg & 1) + 4 * (gg >> 1);
      boffs_n[ii] = (uint32_t)((16 * xcol + 8 + row % 8) * (DV * 2) + 16 * ((pos % CB) ^ swz<CB>(row)));
    }
  }
  const uint32_t ring_lds = lds_addr(ring) + wave * 1024;
  // ALONE: one row block per (chunk, head), so nobody else reads this state and its copies are marked non-temporal
  // (a template parameter: as a run-time flag it changed the registers and the schedule of the other case)
  auto issue = [&](int f0, int ringpos, bool narrow) {
    const char* src = Bg + (long)f0 * DV * 2;
#pragma unroll
    for (int ii = 0; ii < LOADS; ii++) {
      uint32_t bo = boffs[ii];
      if constexpr (SYM) bo = narrow ? boffs_n[ii] : bo;
      if constexpr (ALONE) async_copy16_sv_nt(src, bo, ring_lds + ringpos * STAGE + ii * 4096);
      else async_copy16_sv(src, bo, ring_lds + ringpos * STAGE + ii * 4096);
    }
  };

  const bool skip = ((EPI == NN_EPI_MERGE) && a.skip_first && (bn % a.n == 0)) || (a.skip_last && (bn % a.n == a.n - 1));
  f32x4 acc[MT][NT];
#pragma unroll
  for (int i = 0; i < MT; i++)
#pragma unroll
    for (int j = 0; j < NT; j++) acc[i][j] = (f32x4){0, 0, 0, 0};
  float aux[MT];   // partial aux of the lane's row (row0 + wave*16*MT + 16*mi + tcol), summed over the lane groups at the end
#pragma unroll
  for (int mi = 0; mi < MT; mi++) aux[mi] = 0.f;

  // X rows before time step live_rows[bn, hh, 0] are exact zeros (keys that their discount has turned into zeros), and
  // so are their features and their rows of the output.  Up to the last multiple of 256 rows before that step the
  // output is not even written: its reader (attention_bwd's epilogue, given the same live_rows) does not read it.
  if (EPI == NN_EPI_PLAIN && a.live_rows) {
    const int lv = a.live_rows[((long)bn * a.h + hh) * 2] * a.r;
    if (row0 + ROWS <= (lv & ~255)) return;
  }
  async_load_tile<CX, ROWS>(xt, [&](int row) { return (const char*)(Xg + row_off(row0 + row) * DK); });
  if (skip) {
    wait_vmcnt<0>();
    lds_barrier();
  } else {
    FeatIter<MULT, SYM> cur, nxt;
    cur.init(TT);
    nxt.init(TT);
    int issued = 0;
    for (; issued < NN_NST - 1 && !nxt.done(); issued++) {
      issue(nxt.f0(), issued % NN_NST, nxt.narrow());
      nxt.next();
    }
    // a block of zero rows past that multiple of 256 is written as zeros without the sweep
    bool x_zero = false;
    if (EPI == NN_EPI_PLAIN && a.live_rows) {
      x_zero = row0 + ROWS <= a.live_rows[((long)bn * a.h + hh) * 2] * a.r;
      if (x_zero) {
        wait_vmcnt<0>();
        lds_barrier();
      }
    }
    PhiRow<T> prow[MT];
    int y_loaded = -1, step = 0;
    // Per-lane LDS byte addresses, hoisted out of the stage loop.  The swizzle of a row depends only on the row's
    // position inside its group of 16 (8 for the transposing read), so a stage adds a scalar base and the
    // displacements inside a stage are immediate offsets.
    typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
    typedef __attribute__((address_space(3))) char lds_char;
    typedef __attribute__((address_space(3))) unsigned short lds_u16;
    const uint32_t ring_a = (uint32_t)(uintptr_t)(lds_char*)ring, xt_a = (uint32_t)(uintptr_t)(lds_char*)xt;
    uint32_t boff[NT][2];      // B^T operand (LDS address in slot 0): rows 8g + (s>>2) (+4), columns 16*nt + 4*(s&3) ..
#pragma unroll
    for (int nt = 0; nt < NT; nt++)
#pragma unroll
      for (int hf = 0; hf < 2; hf++) {
        const int row = 8 * g + 4 * hf + (tcol >> 2), col = 16 * nt + 4 * (tcol & 3);
        boff[nt][hf] = ring_a + row * (CB * 16) + (((col / 8) ^ swz<CB>(row)) * 16) + (col % 8) * 2;
        asm volatile("" : "+v"(boff[nt][hf]));   // one register each: the ring slot and the stage's halves are immediates
      }
    const int xlane = 2 * (g >> 1), xlane_n = 2 * ((g & 1) + 4 * (g >> 1));   // byte offsets of the lane's x column
    uint32_t xrow_a[MT], xsw[MT];   // start of this lane's row of the X tile, its swizzle
#pragma unroll
    for (int mi = 0; mi < MT; mi++) {
      const int lrow = wave * 16 * MT + 16 * mi + tcol;
      xrow_a[mi] = xt_a + lrow * (DK * 2);
      xsw[mi] = swz<CX>(lrow);
    }
    static_assert(NN_NST == 2, "the stage loop is unrolled over two ring slots");
    // One stage, held in ring slot SL: a compile-time constant, so that every operand address of the stage is a lane
    // register plus an immediate (with the slot a run-time value the eight address additions per stage cost 7 us of a
    // training step at the headline shape).
    auto stage = [&](auto sl_c) __attribute__((always_inline)) {
      constexpr int SL = decltype(sl_c)::value;
      if (issued > step + 1) wait_vmcnt<LOADS>(); else wait_vmcnt<0>();
      lds_barrier();
      if (!nxt.done()) {
        issue(nxt.f0(), 1 - SL, nxt.narrow());
        nxt.next();
        issued++;
      }
      const bool narrow = cur.narrow();
      if (cur.y != y_loaded || narrow) {
        // (in the narrow stage every lane takes the upper eight w; the strip's values are loaded again afterwards)
        y_loaded = narrow ? -1 : cur.y;
        const int half = narrow ? 8 : 8 * (g & 1);
#pragma unroll
        for (int mi = 0; mi < MT; mi++) prow[mi].load(x_ptr(wave * 16 * MT + 16 * mi + tcol, 16 * cur.y + half));
      }
      if (cur.enters_diag()) {   // quarter (0, 1) stands for (1, 0) as well
        const float f = (g & 1) ? 2.f : 1.f;
#pragma unroll
        for (int mi = 0; mi < MT; mi++) prow[mi].scale(f);
      }
      uint32_t xa[MT];
      {
        // x[row, X0 + 2*ks + g/2] (narrow stage: x[row, X0 + 2*ks + (g & 1) + 4*(g >> 1)]): X0 is a multiple of 4 (8),
        // so the 16-byte chunk is X0/8 and the rest is a lane constant plus an immediate
        const int xc = cur.X0 >> 3, xo = (cur.X0 & 7) * 2 + ((SYM && narrow) ? xlane_n : xlane);
#pragma unroll
        for (int mi = 0; mi < MT; mi++) { xa[mi] = xrow_a[mi] + ((xc ^ xsw[mi]) << 4) + xo; asm volatile("" : "+v"(xa[mi])); }
      }
#pragma unroll
      for (int ks = 0; ks < NN_FR / 32; ks++) {
        v8 vf[NT];
#pragma unroll
        for (int nt = 0; nt < NT; nt++) {
          const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(boff[nt][0] + SL * STAGE + ks * 32 * (CB * 16)));
          const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(boff[nt][1] + SL * STAGE + ks * 32 * (CB * 16)));
          const s16x8 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
          vf[nt] = __builtin_bit_cast(v8, both);
        }
#pragma unroll
        for (int mi = 0; mi < MT; mi++) {
          const unsigned short xbits = *(const lds_u16*)(xa[mi] + 4 * ks);
          const T xs = __builtin_bit_cast(T, xbits);
          const v8 af = prow[mi].make(xs);
#pragma unroll
          for (int nt = 0; nt < NT; nt++) acc[mi][nt] = mfma16(af, vf[nt], acc[mi][nt]);   // phi first: see below
        }
      }
      if (cur.next()) {
#pragma unroll
        for (int mi = 0; mi < MT; mi++)
#pragma unroll
          for (int nt = 0; nt < NT; nt++) acc[mi][nt] *= 2.f;
      }
      step++;
    };
    while (!x_zero && !cur.done()) {
      stage(IC<0>{});
      if (cur.done()) break;
      stage(IC<1>{});
    }

    if (EPI == NN_EPI_MERGE) {
      // aux[row] = sum_{a,b} x[a] M[a,b] x[b]: U^T[b, row] = sum_a M[a,b] x[row,a] on the matrix cores (M in a high
      // and a low 16-bit part), then a dot with x[row, b] down the accumulator rows.
      T* Mt = (T*)ring;   // [DK (a)][LDM (b)]: sB of the stored pair (a, b), read transposed as the A operand
      for (int part = 0; part < 2; part++) {
        lds_barrier();
        // one thread per (a, strip of 16 b): 16 consecutive floats of sB, 16 consecutive elements of M
        for (int idx = tid; idx < DK * TT; idx += 256) {
          const int aa = idx % DK, yb = idx / DK;
          float v16[16];
          if (aa < 16 * (yb + 1)) {
            const f32x4* src = (const f32x4*)(sBg + 128 * yb * (yb + 1) + 16 * aa);
#pragma unroll
            for (int q = 0; q < 4; q++) {
              const f32x4 t4 = src[q];
#pragma unroll
              for (int v = 0; v < 4; v++) v16[4 * q + v] = t4[v] * ScaleS<T>::down;
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
          const int lrow = wave * 16 * MT + 16 * mi + tcol;
          v8 xf[KX];
#pragma unroll
          for (int ks = 0; ks < KX; ks++) xf[ks] = *(const v8*)x_ptr(lrow, 32 * ks + 8 * g);
#pragma unroll
          for (int wt = 0; wt < TT; wt++) {
            f32x4 t = {0, 0, 0, 0};
#pragma unroll
            for (int ks = 0; ks < KX; ks++) t = mfma16(lds_frag_tr<T>(Mt, LDM, 32 * ks, 16 * wt), xf[ks], t);
            const v4 xb4 = *(const v4*)x_ptr(lrow, 16 * wt + 4 * g);
#pragma unroll
            for (int v = 0; v < 4; v++) aux[mi] += t[v] * (float)xb4[v];
          }
        }
      }
    }
  }

  // Epilogue.  The accumulators hold out[row 4*(l/16)+v, column 16*nt + l%16] (the phi operand stays the first
  // matrix-core operand: in the sibling kernel sympow_tn the other order measured ~10 % slower).  Each 16-row tile
  // goes through a private LDS buffer once so that a lane ends up with 4 consecutive columns of ONE row (its own:
  // row0 + wave*16*MT + 16*mi + l%16): per-row scalars are computed once per lane, loads and stores are 8 bytes.
  T* out = (T*)a.out + (long)bn * a.c * hA * DV;
  const float log_gamma = 0.5f * __logf((float)D);
  constexpr int TP = DV + 4;   // pitch of the transposition buffer in floats (conflict-free both ways)
  static_assert(4 * 16 * TP * 4 <= RING_BYTES + 64 * MT * DK * 2, "transposition buffers fit the (idle) LDS");
  float* tbuf = (float*)smem + wave * 16 * TP;
  lds_barrier();   // every wave is done with the ring and the X tile
#pragma unroll
  for (int mi = 0; mi < MT; mi++) {
#pragma unroll
    for (int nt = 0; nt < NT; nt++)
#pragma unroll
      for (int v = 0; v < 4; v++) tbuf[(4 * g + v) * TP + 16 * nt + tcol] = acc[mi][nt][v];
#pragma unroll
    for (int nt = 0; nt < NT; nt++) acc[mi][nt] = *(const f32x4*)(tbuf + tcol * TP + 16 * nt + 4 * g);
  }
#pragma unroll
  for (int mi = 0; mi < MT; mi++) {
    const int row = row0 + wave * 16 * MT + 16 * mi + tcol;
    const bool live = row < rows;
    const long ro = row_off(row);   // clamped
    if (EPI == NN_EPI_MERGE) {
      const float lqs = sum_over_rows(aux[mi]) * ScaleS<T>::up;
      float wa = 0.f, wq = 1.f, la = 0.f;
      v4 ya4[NT];
      if (a.Y_attn) {
        const long go = (long)bn * a.c * hA + ro;
        const float m = a.rowmax[go];
        la = a.l_attn[go];
        const T* ya = (const T*)a.Y_attn + (long)bn * a.c * hA * DV + ro * DV;
#pragma unroll
        for (int nt = 0; nt < NT; nt++) ya4[nt] = *(const v4*)(ya + 16 * nt + 4 * g);
        const float beta = fmaxf(m, log_gamma);
        wa = __expf(m - beta);
        // (gates only decay, so the exponent only shrinks: no range problem; a row whose gate has decayed to nothing
        // keeps its attention part alone, as a gated query rounded to zero would)
        const float qg = a.qgate ? a.qgate[((long)bn * a.c + min(row, rows - 1) / a.r) * a.h + hh] : 0.f;
        wq = a.scale_p * __expf(qg - beta);
      }
      const float den = la * wa + lqs * wq;
      const float inv = 1.f / den;
      if (!live) continue;
#pragma unroll
      for (int nt = 0; nt < NT; nt++) {
        float o4[4];
#pragma unroll
        for (int v = 0; v < 4; v++) {
          float num = acc[mi][nt][v] * wq;
          if (a.Y_attn) num += (float)ya4[nt][v] * wa;
          o4[v] = num * inv;
        }
        *(v4*)(out + ro * DV + 16 * nt + 4 * g) = pack4<T>(o4);
      }
      if (g == 0) a.den[(long)bn * a.c * hA + ro] = den;
    } else {
      if (!live) continue;
#pragma unroll
      for (int nt = 0; nt < NT; nt++) {
        float o4[4];
#pragma unroll
        for (int v = 0; v < 4; v++) o4[v] = acc[mi][nt][v];
        *(v4*)(out + ro * DV + 16 * nt + 4 * g) = pack4<T>(o4);
      }
    }
  }
}

template <typename T, int DK, int DV, int MT, bool MULT, int EPI, bool SYM, bool ALONE>
__global__ __launch_bounds__(256, DK <= 64 ? 3 : 2) void sympow_nn_kernel(NNArgs a, int row_blocks, int npairs) {
  sympow_nn_body<T, DK, DV, MT, MULT, EPI, SYM, ALONE>(a, row_blocks, npairs, (int)blockIdx.x);
}

}  // namespace pr
