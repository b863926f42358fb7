// Chunk-state contraction  S[f, e] = m_f * sum_rows phi(A_row)[f] * B[row, e],
//                          s[f]    = m_f * sum_rows phi(A_row)[f] * w[row]      (w = 1 when absent)
// with phi(a)[f] = a[x_f] * a[w_f] the degree-2 symmetric power features in the tiled state layout
// and m_f = 2 for tiles strictly below the block diagonal when use_mult is set.
//
// Two callers:
//   * update_state forward: A = K, B = V                       (ref: retention/_update_state/reference.py:33-52)
//   * query_state backward, dS/ds: A = Q, B = scaled dO, w = -scaled delta, m = 1
//                                                              (ref: retention/_query_state/triton.py:546-553)
//
// One workgroup = 4 waves; a wave owns XPW of the 16 "x" columns of one 16x16 feature block
// (y, xb) and all DV value columns, and contracts over the rows 32 at a time.  The phi tile is
// never stored: the A-operand of each matrix-core op is produced in registers as the product of a
// row-broadcast (DPP) of column x with the 16 columns 16*y..16*y+15, both read transposed from one
// row-major LDS tile.  Blocks on the diagonal (xb == y) hold every product twice; up to d = 64 one wave computes such
// a block along its nine cyclic diagonals (row rotation instead of row broadcast) and stores each sum at both places.
// s uses the identity s[(x, j)] = (A^T diag(w) A)[x, j], one extra matrix-core op
// per step.  Row tiles of A and B arrive through a 3-deep ring of asynchronous global->LDS copies.
#include "common.h"
#include "kernels.h"

namespace pr {

constexpr int TN_NST = 3;   // stages in the ring
// rows per pipeline stage: two contraction steps of 32 up to d = 64, one at d = 128 (so that the ring of two
// workgroups fits a compute unit's LDS)
constexpr int tn_stage_rows(int d) { return d <= 64 ? 64 : 32; }

template <typename T, int X> struct PhiTile;
template <int X> struct PhiTile<bf16_t, X> {
  static __device__ __forceinline__ bf16x8 make(const bf16x8&, const bf16x8&, const float* rowf, const float* srcf) {
    float p[8];
#pragma unroll
    for (int r = 0; r < 8; r++) p[r] = mul_row_bcast<X>(srcf[r], rowf[r]);
    return pack8<bf16_t>(p);
  }
};
template <int X> struct PhiTile<f16_t, X> {
  static __device__ __forceinline__ f16x8 make(const f16x8& rows, const f16x8& src, const float*, const float*) {
    u32x4 u = __builtin_bit_cast(u32x4, src), b;
#pragma unroll
    for (int i = 0; i < 4; i++) b[i] = row_bcast_u32<X>(u[i]);
    return rows * __builtin_bit_cast(f16x8, b);
  }
};

// Diagonal feature blocks (xb == y) hold every product of the strip's 16 columns twice, (a, b) and (b, a), with equal
// sums.  They are therefore computed along the cyclic diagonals: fragment J holds a[i] * a[(i - J) mod 16] in lane i
// (a row rotation instead of a row broadcast, still one vector op per element); J = 0..8 covers every unordered pair
// (J = 8 covers its eight pairs twice), nine fragments instead of sixteen, and every sum is stored at both places.
template <int J> __device__ __forceinline__ float mul_row_ror(float src, float row) {
  if constexpr (J == 0) return src * row;
  float r;
  asm("v_mul_f32_dpp %0, %1, %2 row_ror:%3 row_mask:0xf bank_mask:0xf" : "=v"(r) : "v"(src), "v"(row), "n"(J));
  return r;
}
template <typename T, int J> struct PhiDiag;
template <int J> struct PhiDiag<bf16_t, J> {
  static __device__ __forceinline__ bf16x8 make(const bf16x8&, const float* rowf) {
    float p[8];
#pragma unroll
    for (int r = 0; r < 8; r++) p[r] = mul_row_ror<J>(rowf[r], rowf[r]);
    return pack8<bf16_t>(p);
  }
};
template <int J> struct PhiDiag<f16_t, J> {
  static __device__ __forceinline__ f16x8 make(const f16x8& rows, const float*) {
    if constexpr (J == 0) return rows * rows;
    u32x4 u = __builtin_bit_cast(u32x4, rows), b;
#pragma unroll
    for (int i = 0; i < 4; i++) b[i] = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)u[i], 0x120 + J, 0xf, 0xf, true);
    return rows * __builtin_bit_cast(f16x8, b);
  }
};
constexpr int TN_NDIAG = 9;   // fragments of a diagonal block

// Writes a wave's 16 x 16 accumulator tile (lane: feature rows 4g+v of value column c0 + lane%16, already rounded:
// pk = {row 4g | row 4g+1 << 16, row 4g+2 | row 4g+3 << 16}) into a row-major LDS buffer of pitch TP bytes.  Neighbouring
// lanes hold neighbouring columns, so a lane pair first trades halves (one DPP move): the even lane then owns rows 4g,
// 4g+1 of both columns and the odd lane rows 4g+2, 4g+3 -- two 4-byte writes per lane instead of four 2-byte ones
// (the 2-byte form cost the chained kernel a quarter of its time in LDS instructions).
// wbase: tb + (4g + 2 (lane & 1)) * TP + 2 (lane%16 & ~1), + 2 * column offset; sel_a / sel_b: byte selectors of the
// lane's parity (tn_pair_selectors).
__device__ __forceinline__ void tn_pair_selectors(uint32_t& sel_a, uint32_t& sel_b) {
  const bool odd = lane_id() & 1;
  sel_a = odd ? 0x01000504u : 0x05040100u;
  sel_b = odd ? 0x03020706u : 0x07060302u;
}
__device__ __forceinline__ void tn_write_pair(u32x2 pk, uint32_t addr, int TP, uint32_t sel_a, uint32_t sel_b) {
  typedef __attribute__((address_space(3))) uint32_t lds_u32;
  const bool odd = lane_id() & 1;
  const uint32_t send = odd ? pk[0] : pk[1], keep = odd ? pk[1] : pk[0];
  const uint32_t recv = (uint32_t)__builtin_amdgcn_mov_dpp((int)send, 0xB1, 0xf, 0xf, true);   // quad_perm [1,0,3,2]
  *(lds_u32*)addr = __builtin_amdgcn_perm(recv, keep, sel_a);
  *(lds_u32*)(addr + TP) = __builtin_amdgcn_perm(recv, keep, sel_b);
}

// The diagonal block's counterpart of tn_store_rows below: fragment J's row i is feature (i, i') with
// i' = (i - J) mod 16, stored at 16 i + i' and at 16 i' + i.  S, s point at the block's first feature.
template <typename T, int DV>
__device__ __forceinline__ void tn_store_diag(const f32x4 (&acc)[TN_NDIAG][DV / 16], const f32x4& sacc, uint32_t tb,
                                              T* __restrict__ S, float* __restrict__ s) {
  typedef __attribute__((address_space(3))) unsigned short lds_u16;
  typedef __attribute__((address_space(3))) u32x4 lds_u32x4;
  constexpr int NT = DV / 16, TP = DV * 2 + 16;
  const int l = lane_id(), g = l >> 4, sl = l & 15;
  const uint32_t tb_w = tb + (4 * g + 2 * (sl & 1)) * TP + (sl & ~1) * 2;
  uint32_t sel_a, sel_b;
  tn_pair_selectors(sel_a, sel_b);
  static_for<TN_NDIAG>([&](auto ji) {
    constexpr int J = decltype(ji)::value;
#pragma unroll
    for (int nt = 0; nt < NT; nt++) {
      float o[4];
#pragma unroll
      for (int v = 0; v < 4; v++) o[v] = acc[J][nt][v];
      tn_write_pair(__builtin_bit_cast(u32x2, pack4<T>(o)), tb_w + 32 * nt, TP, sel_a, sel_b);
    }
    asm volatile("" ::: "memory");   // (LDS operations of one wave execute in order)
#pragma unroll
    for (int j = 0; j < DV / 32; j++) {
      const int q = j * 1024 + l * 16, i = q / (DV * 2), col = q % (DV * 2), i2 = (i - J) & 15;
      const u32x4 v = *(const lds_u32x4*)(tb + i * TP + col);
      __builtin_nontemporal_store(v, (u32x4*)((char*)S + (16 * i + i2) * (DV * 2) + col));
      if (J != 0 && J != 8) __builtin_nontemporal_store(v, (u32x4*)((char*)S + (16 * i2 + i) * (DV * 2) + col));
    }
    asm volatile("" ::: "memory");   // the buffer is rewritten for the next fragment
  });
  *(f32x4*)(s + 16 * sl + 4 * g) = sacc;
}

// Writes a wave's accumulators -- for each of its XPW x values the 16 feature rows (4g+v) x DV value columns
// (16nt + lane%16) of S, times mul -- and its key sums.  Each x goes through a per-wave LDS buffer of 16 padded rows
// (tb, 16 * (2 DV + 16) bytes) so that the tile leaves as whole contiguous kilobytes: the rows of one x are adjacent
// in S.  S, s point at feature fbase of the (chunk, head).
template <typename T, int DV, int XPW, int PART>
__device__ __forceinline__ void tn_store_rows(const f32x4 (&acc)[XPW][DV / 16], const f32x4& sacc, float mul,
                                              uint32_t tb, T* __restrict__ S, float* __restrict__ s) {
  typedef __attribute__((address_space(3))) unsigned short lds_u16;
  typedef __attribute__((address_space(3))) u32x4 lds_u32x4;
  constexpr int NT = DV / 16, TP = DV * 2 + 16;
  const int l = lane_id(), g = l >> 4, sl = l & 15;
  const uint32_t tb_w = tb + (4 * g + 2 * (sl & 1)) * TP + (sl & ~1) * 2;   // + 32*nt (+ TP): see tn_write_pair
  uint32_t sel_a, sel_b;
  tn_pair_selectors(sel_a, sel_b);
  static_for<XPW>([&](auto xi) {
    constexpr int X = PART * XPW + decltype(xi)::value;
#pragma unroll
    for (int nt = 0; nt < NT; nt++) {
      float o[4];
#pragma unroll
      for (int v = 0; v < 4; v++) o[v] = acc[xi.value][nt][v] * mul;
      tn_write_pair(__builtin_bit_cast(u32x2, pack4<T>(o)), tb_w + 32 * nt, TP, sel_a, sel_b);
    }
    asm volatile("" ::: "memory");   // (LDS operations of one wave execute in order)
    char* dst = (char*)(S + 16 * X * DV);
#pragma unroll
    for (int j = 0; j < DV / 32; j++) {   // one kilobyte per store instruction; non-temporal: the scan that reads the
                                          // result streams it once (3 us of a training step at the headline shape)
      const int q = j * 1024 + l * 16;
      __builtin_nontemporal_store(*(const lds_u32x4*)(tb + (q / (DV * 2)) * TP + q % (DV * 2)), (u32x4*)(dst + q));
    }
    asm volatile("" ::: "memory");   // the buffer is rewritten for the next x
  });
  if (sl >= PART * XPW && sl < (PART + 1) * XPW) *(f32x4*)(s + 16 * sl + 4 * g) = sacc * mul;
}

template <typename T, int DK, int DV, int XPW, int PART, bool HAS_W, bool DIAG = false>
__device__ __forceinline__ void tn_body(const T* __restrict__ A, const T* __restrict__ Bm, const float* __restrict__ w,
                                        T* __restrict__ S, float* __restrict__ s, int c, int hA, int r, int hh,
                                        int bn, int h, int y, int xb, bool active, bool use_mult, char* smem,
                                        int k0, int k1) {
  typedef typename VecOf<T>::v8 v8;
  typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
  typedef __attribute__((address_space(3))) f32x4 lds_f32x4;
  constexpr int KT = tn_stage_rows(DV);                            // rows per pipeline stage
  constexpr int NT = DV / 16, CA = DK / 8, CB = DV / 8;            // 16-byte chunks per row
  constexpr int A_BYTES = KT * DK * 2, B_BYTES = KT * DV * 2, W_BYTES = KT * 4;
  constexpr int STAGE = A_BYTES + B_BYTES + W_BYTES;
  constexpr int LA = KT * CA / 256, LB = KT * CB / 256;      // copies per thread per stage (w rides on wave 0)
  constexpr int LOADS = LA + LB;
  static_assert(CA == CB && TN_NST == 3 && (KT == 64 || DV > 64), "the loops below are written for these shapes");
  const int tid = threadIdx.x, l = tid & 63, g = l >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // Stages k0 .. k1-1 of the chunk's rows are walked (the others are known to hold zero rows of A or of Bm): below,
  // rows and stages count from stage k0.
  const int roff = k0 * KT, rows = c * r - roff;
  const char* a_base = (const char*)(A + (long)bn * c * hA * DK);
  const char* b_base = (const char*)(Bm + (long)bn * c * hA * DV);
  const float* w_base = w + (long)bn * c * hA;
  auto row_index = [&](int row) -> long {   // element offset of a (clamped) folded row, per unit of the last dim
    row = min(row, rows - 1) + roff;
    const int t = row / r, rr = row - t * r;
    return (long)t * hA + hh * r + rr;
  };
  // Copies of one stage.  When a stage is a whole number of time steps (KT % r == 0) the folded rows of stage
  // k+1 are those of stage k moved by a fixed distance: lane offsets are computed once, the base moves in scalar
  // registers.  Other shapes and the partial last stage take the general path.
  const bool regular = (KT % r) == 0;
  static_assert(DK == DV, "the A and B tiles share the copy offsets");
  uint32_t voffA[LA], voffW = 0;
#pragma unroll
  for (int ii = 0; ii < LA; ii++) {
    const int pos = (ii * 4 + wave) * 64 + l, row = pos / CA;
    voffA[ii] = (uint32_t)(row_index(row) * (DK * 2) + 16 * ((pos % CA) ^ swz<CA>(row)));
  }
  if (HAS_W) voffW = (uint32_t)(row_index(l) * 4);
  const long stage_rows = (long)(KT / max(r, 1)) * hA;   // rows of the [c, hA] arrays per stage (regular shapes)
  const uint32_t smem_a = lds_addr(smem);
  auto issue = [&](int step) {
    const int slot = step % TN_NST;
    const int r0 = step * KT;
    if (regular && r0 + KT <= rows) {
      const uint32_t sa = smem_a + slot * STAGE + wave * 1024;
      const char* ab = a_base + step * stage_rows * (DK * 2);
      const char* bb = b_base + step * stage_rows * (DV * 2);
#pragma unroll
      for (int ii = 0; ii < LA; ii++) async_copy16_sv(ab, voffA[ii], sa + ii * 4096);
#pragma unroll
      for (int ii = 0; ii < LB; ii++) async_copy16_sv(bb, voffA[ii], sa + A_BYTES + ii * 4096);
      if (HAS_W && wave == 0 && l < KT) async_copy4_sv(w_base + step * stage_rows, voffW, smem_a + slot * STAGE + A_BYTES + B_BYTES);
      return;
    }
    char* st = smem + slot * STAGE;
    async_load_tile<CA, KT>(st, [&](int row) { return a_base + row_index(r0 + row) * (DK * 2); });
    async_load_tile<CB, KT>(st + A_BYTES, [&](int row) { return b_base + row_index(r0 + row) * (DV * 2); });
    if (HAS_W && wave == 0 && l < KT) async_copy4(w_base + row_index(r0 + l), st + A_BYTES + B_BYTES);
  };

  constexpr int NF = DIAG ? TN_NDIAG : XPW;   // operand fragments built per step
  f32x4 acc[NF][NT];
#pragma unroll
  for (int i = 0; i < NF; i++)
#pragma unroll
    for (int j = 0; j < NT; j++) acc[i][j] = (f32x4){0, 0, 0, 0};
  f32x4 sacc = {0, 0, 0, 0};

  // Operand fragments of one contraction step (32 rows).  With PREFETCH they are fetched one step ahead of the
  // matrix-core work that uses them, and a stage's slot is free for the next copy as soon as every wave holds the
  // stage's last fragments in registers.  Every vector instruction in this loop competes with the matrix cores
  // for the SIMD, so the LDS addresses are per-lane registers set up once plus immediates (the stage loop is
  // unrolled over the three slots of the ring).
  struct Frags {
    v8 kfy, kfx, vf[NT];
  };
  constexpr bool PREFETCH = DV <= 64;   // two sets of fragments and their addresses do not fit beyond that
  uint32_t ay[2], ax[2], av[NT][2], aw = smem_a + A_BYTES + B_BYTES + 32 * g;
  if constexpr (PREFETCH) {
    const int sl = l & 15;
#pragma unroll
    for (int hf = 0; hf < 2; hf++) {
      const int row = 8 * g + 4 * hf + (sl >> 2);
      const int cy = 16 * y + 4 * (sl & 3), cx = 16 * xb + 4 * (sl & 3);
      ay[hf] = smem_a + row * (CA * 16) + (((cy / 8) ^ swz<CA>(row)) * 16) + (cy % 8) * 2;
      ax[hf] = smem_a + row * (CA * 16) + (((cx / 8) ^ swz<CA>(row)) * 16) + (cx % 8) * 2;
      asm volatile("" : "+v"(ay[hf]));
      asm volatile("" : "+v"(ax[hf]));
#pragma unroll
      for (int nt = 0; nt < NT; nt++) {
        const int cv = 16 * nt + 4 * (sl & 3);
        av[nt][hf] = smem_a + A_BYTES + row * (CB * 16) + (((cv / 8) ^ swz<CB>(row)) * 16) + (cv % 8) * 2;
        asm volatile("" : "+v"(av[nt][hf]));
      }
    }
    asm volatile("" : "+v"(aw));
  }
  auto tr8 = [&](uint32_t lo, uint32_t hi) -> v8 {
    const s16x4 a = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)lo);
    const s16x4 b = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)hi);
    return __builtin_bit_cast(v8, __builtin_shufflevector(a, b, 0, 1, 2, 3, 4, 5, 6, 7));
  };
  auto load_frags = [&](Frags& F, auto slot_c, auto ks_c) {
    constexpr int OFF = decltype(slot_c)::value * STAGE + decltype(ks_c)::value * 32 * (CA * 16);
    F.kfy = tr8(ay[0] + OFF, ay[1] + OFF);
    if constexpr (!DIAG) F.kfx = tr8(ax[0] + OFF, ax[1] + OFF);
#pragma unroll
    for (int nt = 0; nt < NT; nt++) F.vf[nt] = tr8(av[nt][0] + OFF, av[nt][1] + OFF);
  };
  auto compute = [&](const Frags& F, f32x4 w0, f32x4 w1) {
    float rowf[8], srcf[8];
    unpack8(F.kfy, rowf);
    if constexpr (!DIAG) unpack8(F.kfx, srcf);
    if (HAS_W) {
      float sc[8];
#pragma unroll
      for (int q = 0; q < 4; q++) {
        sc[q] = (DIAG ? rowf[q] : srcf[q]) * w0[q];
        sc[4 + q] = (DIAG ? rowf[4 + q] : srcf[4 + q]) * w1[q];
      }
      sacc = mfma16(F.kfy, pack8<T>(sc), sacc);
    } else {
      sacc = mfma16(F.kfy, DIAG ? F.kfy : F.kfx, sacc);
    }
    dpp_fence();  // srcf / rowf is read through DPP below
    static_for<NF>([&](auto xi) {
      v8 a;
      if constexpr (DIAG) a = PhiDiag<T, xi.value>::make(F.kfy, rowf);
      else a = PhiTile<T, PART * XPW + xi.value>::make(F.kfy, F.kfx, rowf, srcf);
#pragma unroll
      for (int nt = 0; nt < NT; nt++) acc[xi.value][nt] = mfma16(a, F.vf[nt], acc[xi.value][nt]);
    });
  };
  // w of a step is fetched at the end of the previous step's work, when few registers are live
  f32x4 wv0 = {0, 0, 0, 0}, wv1 = {0, 0, 0, 0};
  auto load_w = [&](auto slot_c, auto ks_c) {
    if (HAS_W) {
      constexpr int WOFF = decltype(slot_c)::value * STAGE + decltype(ks_c)::value * 128;
      wv0 = *(const lds_f32x4*)(aw + WOFF);
      wv1 = *(const lds_f32x4*)(aw + WOFF + 16);
    }
  };

  const int steps = k1 - k0;
  if (steps <= 0) {
    // nothing to add up: the zero accumulators are stored
  } else if constexpr (PREFETCH) {
    issue(0);
    if (steps > 1) issue(1);
    if (steps > 2) issue(2);
    if (steps > 2) wait_vmcnt<2 * LOADS>(); else if (steps > 1) wait_vmcnt<LOADS>(); else wait_vmcnt<0>();
    if (KT > rows) zero_tile_rows<CA, KT>(smem, rows);
    lds_barrier();
    Frags F0, F1;
    load_frags(F0, IC<0>{}, IC<0>{});
    load_w(IC<0>{}, IC<0>{});
    // one stage held in slot SL; returns false after the last stage
    auto stage = [&](int step, auto sl_c) -> bool {
      constexpr int SL = decltype(sl_c)::value, NX = (SL + 1) % TN_NST;
      load_frags(F1, IC<SL>{}, IC<1>{});
      if (active) compute(F0, wv0, wv1);
      __builtin_amdgcn_sched_barrier(0);
      load_w(IC<SL>{}, IC<1>{});
      const bool more = step + 1 < steps;
      if (more) {
        if (step + 2 < steps) wait_vmcnt<LOADS>(); else wait_vmcnt<0>();
        if ((step + 2) * KT > rows) zero_tile_rows<CA, KT>(smem + NX * STAGE, rows - (step + 1) * KT);
        lds_barrier();   // every wave holds the last fragments of this stage: its slot can be refilled
        if (step + 3 < steps) issue(step + 3);
        load_frags(F0, IC<NX>{}, IC<0>{});
      }
      if (active) compute(F1, wv0, wv1);
      __builtin_amdgcn_sched_barrier(0);
      if (more) load_w(IC<NX>{}, IC<0>{});
      return more;
    };
    for (int step = 0;; step += 3) {
      if (!stage(step, IC<0>{})) break;
      if (!stage(step + 1, IC<1>{})) break;
      if (!stage(step + 2, IC<2>{})) break;
    }
  } else {
    issue(0);
    if (steps > 1) issue(1);
    Frags F;
    for (int step = 0; step < steps; step++) {
      const char* st = smem + (step % TN_NST) * STAGE;
      if (step + 1 < steps) wait_vmcnt<LOADS>(); else wait_vmcnt<0>();
      if ((step + 1) * KT > rows) zero_tile_rows<CA, KT>(smem + (step % TN_NST) * STAGE, rows - step * KT);
      lds_barrier();
      if (step + 2 < steps) issue(step + 2);
#pragma unroll 1
      for (int ks = 0; ks < KT / 32; ks++) {
        F.kfy = sw_frag_tr<T, CA>(st, 32 * ks, 16 * y);
        F.kfx = (xb == y) ? F.kfy : sw_frag_tr<T, CA>(st, 32 * ks, 16 * xb);
#pragma unroll
        for (int nt = 0; nt < NT; nt++) F.vf[nt] = sw_frag_tr<T, CB>(st + A_BYTES, 32 * ks, 16 * nt);
        f32x4 w0 = {0, 0, 0, 0}, w1 = {0, 0, 0, 0};
        if (HAS_W) {
          const float* wp = (const float*)(st + A_BYTES + B_BYTES) + 32 * ks + 8 * g;
          w0 = *(const f32x4*)wp;
          w1 = *(const f32x4*)(wp + 4);
        }
        if (active) compute(F, w0, w1);
      }
    }
  }
  lds_barrier();   // every wave is done with the ring: its memory stages the stores
  if (!active) return;
  const float mul = (use_mult && xb < y) ? 2.f : 1.f;
  constexpr int D = 128 * (DK / 16) * (DK / 16 + 1);
  const long so = ((long)bn * h + hh) * D + 128 * y * (y + 1) + 256 * xb;
  if constexpr (DIAG) tn_store_diag<T, DV>(acc, sacc, smem_a + wave * (16 * (DV * 2 + 16)), S + so * DV, s + so);
  else tn_store_rows<T, DV, XPW, PART>(acc, sacc, mul, smem_a + wave * (16 * (DV * 2 + 16)), S + so * DV, s + so);
}

// Wave tasks of a (chunk, head).  With eight x columns per wave (XPW == 8) the blocks below the block diagonal give
// two tasks each, numbered first, and every diagonal block is ONE task of nine cyclic fragments; otherwise every
// block, diagonal or not, is cut into 16 / XPW tasks.
template <int DK, int XPW> constexpr int tn_tasks() {
  constexpr int T = DK / 16;
  return XPW == 8 ? T * (T - 1) + T : (T * (T + 1) / 2) * (16 / XPW);
}

template <typename T, int DK, int DV, int XPW, bool HAS_W>
__global__ __launch_bounds__(256, 2) void sympow_tn_kernel(const T* __restrict__ A, const T* __restrict__ Bm,
                                                           const float* __restrict__ w, T* __restrict__ S,
                                                           float* __restrict__ s, int c, int hA, int r, int h,
                                                           int use_mult, int skip, const int* __restrict__ live,
                                                           int live_side) {
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  constexpr int PARTS = 16 / XPW;
  constexpr int NB = (DK / 16) * (DK / 16 + 1) / 2;
  // Workgroups are handed to the 8 XCDs (each with its own L2) round-robin by linear id.  The workgroups of a
  // (chunk, head) read the same rows, so ids are permuted to put them on one XCD: XCD x takes the x-th eighth.
  int bx = blockIdx.x, by = blockIdx.y;
  const int total = gridDim.x * gridDim.y;
  if (total % 8 == 0) {
    const int lin = by * gridDim.x + bx, v = (lin % 8) * (total / 8) + lin / 8;
    by = v / gridDim.x;
    bx = v - by * gridDim.x;
  }
  const int task = bx * 4 + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const bool active = task < tn_tasks<DK, XPW>();
  const int t2 = active ? task : 0;
  int part = t2 % PARTS;
  int y, xb;
  const int bn = by / h, hh = by % h;
  // Chunks whose result nobody reads (skip = +n: the last of every n chunks, left unwritten; skip = -n: the first of
  // every n, whose result is zero by definition and is written as zeros).  Uniform over the workgroup.
  if (skip > 0 && bn % skip == skip - 1) return;
  if (skip < 0 && bn % (-skip) == 0) {
    if (!active) return;
    constexpr int D = 128 * (DK / 16) * (DK / 16 + 1);
    int f0, nf;   // the feature rows this wave owns
    if (XPW == 8 && t2 >= (DK / 16) * (DK / 16 - 1)) {
      y = t2 - (DK / 16) * (DK / 16 - 1);
      f0 = 128 * y * (y + 1) + 256 * y;
      nf = 256;
    } else {
      if (XPW == 8) {
        y = 1;
        while (y * (y + 1) / 2 <= t2 / 2) y++;
        xb = t2 / 2 - y * (y - 1) / 2;
      } else {
        block_to_yx(t2 / PARTS, y, xb);
      }
      f0 = 128 * y * (y + 1) + 256 * xb + 16 * XPW * part;
      nf = 16 * XPW;
    }
    const long so = ((long)bn * h + hh) * D + f0;
    const int l = threadIdx.x & 63;
    for (int q = l * 8; q < nf * DV; q += 512) *(u32x4*)(S + so * DV + q) = (u32x4){0, 0, 0, 0};
    for (int q = l; q < nf; q += 64) s[so + q] = 0.f;
    return;
  }
  // Stages of the chunk's rows that can hold anything but zero rows (live: per (chunk, head) the first time step whose
  // row of A is not zero and the end of the time steps whose rows of Bm are not; live_side picks which one applies).
  constexpr int KT_ = tn_stage_rows(DV);
  int k0 = 0, k1 = (c * r + KT_ - 1) / KT_;
  if (live) {
    const int v = live[((long)bn * h + hh) * 2 + live_side];
    if (live_side == 0) k0 = min(max(v, 0) * r / KT_, k1);
    else k1 = min((max(v, 0) * r + KT_ - 1) / KT_, k1);
  }
  if constexpr (XPW == 8) {
    constexpr int NOFF = (DK / 16) * (DK / 16 - 1);   // tasks below the block diagonal
    if (t2 >= NOFF) {
      y = xb = t2 - NOFF;
      tn_body<T, DK, DV, XPW, 0, HAS_W, true>(A, Bm, w, S, s, c, hA, r, hh, bn, h, y, xb, active, use_mult != 0, smem,
                                              k0, k1);
      return;
    }
    y = 1;
    while (y * (y + 1) / 2 <= t2 / 2) y++;
    xb = t2 / 2 - y * (y - 1) / 2;
  } else {
    block_to_yx(t2 / PARTS, y, xb);
  }
#define PR_TN_CASE(P)                                                                                                  \
  case P:                                                                                                              \
    if (P < PARTS)                                                                                                     \
      tn_body<T, DK, DV, XPW, (P < PARTS ? P : 0), HAS_W>(A, Bm, w, S, s, c, hA, r, hh, bn, h, y, xb, active,         \
                                                          use_mult != 0, smem, k0, k1);                                \
    break;
  switch (part) {
    PR_TN_CASE(0)
    PR_TN_CASE(1)
    PR_TN_CASE(2)
    PR_TN_CASE(3)
  }
#undef PR_TN_CASE
}

// ---------------------------------------------------------------------------------------------------------------
// Chained form (short chunks).  The per-chunk sums S_k of the kernel above are only ever consumed through the gated
// scan over the chunk axis (discumsum.hip).  When a batch element has many short chunks the scan's traffic -- S
// written, read back, and the scanned tensor written -- is what the pair of kernels costs.  Here one workgroup
// walks the chunks of a batch element in order, keeps the running sum in its accumulators and writes only the
// scanned tensor:
//   forward:  Y[0] = 0,    Y[k+1] = e^{g_k} Y[k] + S_k        (the first n entries of the scan)
//   reverse:  R[n-1] = 0,  R[k-1] = e^{g_k} R[k] + S_k        (the scan's backward applied to S_k = per-chunk gradient)
// Rows of all chunks form one stream of stages through the ring; at each chunk boundary the accumulators are
// written (through a small per-wave LDS buffer, so that a wave stores whole contiguous kilobytes) and decayed.
// What bounds it: the scanned tensor is written once, and while a compute unit's burst of stores drains, the copies
// queued behind it wait -- measured, the stores add their drain time to the contraction's instead of hiding under it.
template <typename T, int DK, int DV, int XPW, int NW, int KT, int PART, bool HAS_W, bool REVERSE>
__device__ __forceinline__ void tn_chain_body(const T* __restrict__ A, const T* __restrict__ Bm,
                                              const float* __restrict__ w, const float* __restrict__ lcs,
                                              T* __restrict__ S, float* __restrict__ s, int n, int c, int hA, int r,
                                              int hh, int b, int h, int y, int xb, bool active, bool use_mult,
                                              char* smem) {
  typedef typename VecOf<T>::v8 v8;
  constexpr int NT = DV / 16, CA = DK / 8, CB = DV / 8;
  constexpr int A_BYTES = KT * DK * 2, B_BYTES = KT * DV * 2, W_BYTES = KT * 4;
  constexpr int STAGE = A_BYTES + B_BYTES + W_BYTES;
  constexpr int LA = KT * CA / (64 * NW), LB = KT * CB / (64 * NW);   // copies per thread per stage
  constexpr int LOADS = LA + LB;
  constexpr int NSTORE = XPW * (DV / 32);   // 16-byte stores of a boundary per wave (the key sums add one more)
  static_assert(LOADS + 2 * NSTORE <= 63, "the wait counter has six bits");
  constexpr int D = 128 * (DK / 16) * (DK / 16 + 1);
  static_assert(DK == DV, "the A and B tiles share the copy offsets");
  const int tid = threadIdx.x, l = tid & 63, g = l >> 4, sl = l & 15;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const char* a_base = (const char*)(A + (long)b * n * c * hA * DK);
  const char* b_base = (const char*)(Bm + (long)b * n * c * hA * DV);
  const float* w_base = w + (long)b * n * c * hA;
  // every stage is KT whole folded rows = KT / r time steps (checked by the host)
  auto row_index = [&](int row) -> long {
    const int t = row / r, rr = row - t * r;
    return (long)t * hA + hh * r + rr;
  };
  uint32_t voffA[LA], voffW = 0;
#pragma unroll
  for (int ii = 0; ii < LA; ii++) {
    const int pos = (ii * NW + wave) * 64 + l, row = pos / CA;
    voffA[ii] = (uint32_t)(row_index(row) * (DK * 2) + 16 * ((pos % CA) ^ swz<CA>(row)));
  }
  if (HAS_W) voffW = (uint32_t)(row_index(l % KT) * 4);
  const long stage_rows = (long)(KT / r) * hA;
  const uint32_t smem_a = lds_addr(smem);
  auto issue = [&](int slot, int stage) {
    const uint32_t sa = smem_a + slot * STAGE + wave * 1024;
    const char* ab = a_base + stage * stage_rows * (DK * 2);
    const char* bb = b_base + stage * stage_rows * (DV * 2);
#pragma unroll
    for (int ii = 0; ii < LA; ii++) async_copy16_sv(ab, voffA[ii], sa + ii * (NW * 1024));
#pragma unroll
    for (int ii = 0; ii < LB; ii++) async_copy16_sv(bb, voffA[ii], sa + A_BYTES + ii * (NW * 1024));
    if (HAS_W && wave == 0 && l < KT) async_copy4_sv(w_base + stage * stage_rows, voffW, smem_a + slot * STAGE + A_BYTES + B_BYTES);
  };

  f32x4 acc[XPW][NT];
#pragma unroll
  for (int i = 0; i < XPW; i++)
#pragma unroll
    for (int j = 0; j < NT; j++) acc[i][j] = (f32x4){0, 0, 0, 0};
  f32x4 sacc = {0, 0, 0, 0};

  const float mul = (use_mult && xb < y) ? 2.f : 1.f;
  const int fbase = 128 * y * (y + 1) + 256 * xb;
  // per-wave staging buffer of the boundary's stores, behind the ring
  const uint32_t tb = smem_a + TN_NST * STAGE + wave * (16 * (DV * 2 + 16));
  auto write_out = [&](int k) {
    if (!active) return;
    const long so = ((long)(b * n + k) * h + hh) * D + fbase;
    tn_store_rows<T, DV, XPW, PART>(acc, sacc, mul, tb, S + so * DV, s + so);
  };
  auto decay = [&](int k) {
    if (lcs == nullptr) return;
    const float gk = __expf(lcs[((long)b * n + k) * h + hh]);
#pragma unroll
    for (int i = 0; i < XPW; i++)
#pragma unroll
      for (int j = 0; j < NT; j++) acc[i][j] *= gk;
    sacc *= gk;
  };

  struct Frags {
    v8 kfy, kfx, vf[NT];
  };
  auto compute = [&](const Frags& F, f32x4 w0, f32x4 w1) {
    float rowf[8], srcf[8];
    unpack8(F.kfy, rowf);
    unpack8(F.kfx, srcf);
    if (HAS_W) {
      float sc[8];
#pragma unroll
      for (int q = 0; q < 4; q++) {
        sc[q] = srcf[q] * w0[q];
        sc[4 + q] = srcf[4 + q] * w1[q];
      }
      sacc = mfma16(F.kfy, pack8<T>(sc), sacc);
    } else {
      sacc = mfma16(F.kfy, F.kfx, sacc);
    }
    dpp_fence();
    static_for<XPW>([&](auto xi) {
      v8 a = PhiTile<T, PART * XPW + xi.value>::make(F.kfy, F.kfx, rowf, srcf);
#pragma unroll
      for (int nt = 0; nt < NT; nt++) acc[xi.value][nt] = mfma16(a, F.vf[nt], acc[xi.value][nt]);
    });
  };

  // Step st of the walk: chunk ordinal st / spc (chunk index n-1-ordinal when walking backwards).  The last chunk of
  // the walk contributes to no output and is not read.
  const int spc = (c * r) / KT, steps = (n - 1) * spc;
  int ik = 0, iw = 0;   // chunk ordinal and stage within the chunk of the next stage to copy
  auto issue_next = [&](int st) {
    issue(st % TN_NST, (REVERSE ? n - 1 - ik : ik) * spc + iw);
    if (++iw == spc) {
      iw = 0;
      ik++;
    }
  };
  if (steps > 0) issue_next(0);
  if (steps > 1) issue_next(1);
  int kk = 0, wi = 0;
  int b1 = 0, b2 = 0;   // whether the previous step / the one before wrote a boundary (this wave's stores)
  Frags F;
  for (int step = 0; step < steps; step++) {
    const char* st = smem + (step % TN_NST) * STAGE;
    // Copies and stores of a wave complete in the order issued and share one counter.  Younger than this stage's
    // copies are: the next stage's copies, and the stores of a boundary written in one of the last two steps (at
    // least NSTORE each) -- the boundary's stores are never waited for.
    const int nb = b1 + b2;
    if (step + 1 < steps) {
      if (nb == 0) wait_vmcnt<LOADS>(); else if (nb == 1) wait_vmcnt<LOADS + NSTORE>(); else wait_vmcnt<LOADS + 2 * NSTORE>();
    } else {
      if (nb == 0) wait_vmcnt<0>(); else if (nb == 1) wait_vmcnt<NSTORE>(); else wait_vmcnt<2 * NSTORE>();
    }
    lds_barrier();
    if (step + 2 < steps) issue_next(step + 2);
    b2 = b1;
    b1 = 0;
    if (wi == 0) {
      const int k = REVERSE ? n - 1 - kk : kk;
      write_out(k);
      decay(k);
      b1 = active ? 1 : 0;
    }
#pragma unroll 1
    for (int ks = 0; ks < KT / 32; ks++) {
      F.kfy = sw_frag_tr<T, CA>(st, 32 * ks, 16 * y);
      F.kfx = (xb == y) ? F.kfy : sw_frag_tr<T, CA>(st, 32 * ks, 16 * xb);
#pragma unroll
      for (int nt = 0; nt < NT; nt++) F.vf[nt] = sw_frag_tr<T, CB>(st + A_BYTES, 32 * ks, 16 * nt);
      f32x4 w0 = {0, 0, 0, 0}, w1 = {0, 0, 0, 0};
      if (HAS_W) {
        const float* wp = (const float*)(st + A_BYTES + B_BYTES) + 32 * ks + 8 * g;
        w0 = *(const f32x4*)wp;
        w1 = *(const f32x4*)(wp + 4);
      }
      if (active) compute(F, w0, w1);
    }
    if (++wi == spc) {
      wi = 0;
      kk++;
    }
  }
  write_out(REVERSE ? 0 : n - 1);
}

template <typename T, int DK, int DV, int XPW, int NW, int KT, bool HAS_W, bool REVERSE>
__global__ __launch_bounds__(64 * NW, 2) void sympow_tn_chain_kernel(
    const T* __restrict__ A, const T* __restrict__ Bm, const float* __restrict__ w, const float* __restrict__ lcs,
    T* __restrict__ S, float* __restrict__ s, int n, int c, int hA, int r, int h, int use_mult) {
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  constexpr int PARTS = 16 / XPW;
  constexpr int NB = (DK / 16) * (DK / 16 + 1) / 2;
  // Workgroups are handed to the 8 XCDs (each with its own L2) round-robin by linear id.  All workgroups of a
  // (batch, head) read the same rows, so ids are permuted to put them on one XCD: XCD x takes the x-th eighth.
  int bx = blockIdx.x, by = blockIdx.y;
  const int total = gridDim.x * gridDim.y;
  if (total % 8 == 0) {
    const int lin = by * gridDim.x + bx, v = (lin % 8) * (total / 8) + lin / 8;
    by = v / gridDim.x;
    bx = v - by * gridDim.x;
  }
  const int task = bx * NW + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const bool active = task < NB * PARTS;
  const int t2 = active ? task : 0;
  const int part = t2 % PARTS;
  int y, xb;
  block_to_yx(t2 / PARTS, y, xb);
  const int b = by / h, hh = by % h;
#define PR_TN_CASE(P)                                                                                                  \
  case P:                                                                                                              \
    if (P < PARTS)                                                                                                     \
      tn_chain_body<T, DK, DV, XPW, NW, KT, (P < PARTS ? P : 0), HAS_W, REVERSE>(A, Bm, w, lcs, S, s, n, c, hA, r, hh, \
                                                                                 b, h, y, xb, active, use_mult != 0,   \
                                                                                 smem);                                \
    break;
  switch (part) {
    PR_TN_CASE(0)
    PR_TN_CASE(1)
    PR_TN_CASE(2)
    PR_TN_CASE(3)
  }
#undef PR_TN_CASE
}

template <typename T, int DK, int DV>
static int tn_chain_launch(const void* A, const void* Bm, const float* w, const float* lcs, void* S, float* s, int B,
                           int n, int c, int h, int r, int use_mult, int reverse, hipStream_t st) {
  constexpr int XPW = DV <= 64 ? 8 : 4;
  constexpr int NB = (DK / 16) * (DK / 16 + 1) / 2;
  constexpr int TASKS = NB * (16 / XPW);
  constexpr int NW = 4;                         // waves that share a stage of rows
  constexpr int KT = tn_stage_rows(DV);      // rows per stage: two workgroups per compute unit must fit
  constexpr size_t smem = TN_NST * (KT * DK * 2 + KT * DV * 2 + KT * 4) + NW * 16 * (DV * 2 + 16);
  dim3 grid((TASKS + NW - 1) / NW, (unsigned)(B * h));
#define PR_TN_CHAIN(W, R)                                                                                              \
  {                                                                                                                    \
    auto kern = sympow_tn_chain_kernel<T, DK, DV, XPW, NW, KT, W, R>;                                                          \
    allow_big_lds((const void*)kern, smem);                                                                            \
    PR_LAUNCH("sympow_tn_chain", kern, grid, dim3(64 * NW), smem, st, (const T*)A, (const T*)Bm, w, lcs, (T*)S, s, n, c, h * r, \
                       r, h, use_mult);                                                                                \
  }
  if (w) {
    if (reverse) PR_TN_CHAIN(true, true) else PR_TN_CHAIN(true, false)
  } else {
    if (reverse) PR_TN_CHAIN(false, true) else PR_TN_CHAIN(false, false)
  }
#undef PR_TN_CHAIN
  return (int)hipGetLastError();
}

// 0: the chained form does not apply (it needs whole stages per chunk); 1: it applies; 2: it applies and there are
// enough workgroups to fill the chip although the chunk axis is walked serially.
int sympow_tn_chain_ok(int B, int n, int c, int h, int r, int d) {
  if (d != 32 && d != 64 && d != 128) return 0;
  const int kt = tn_stage_rows(d);
  if (n < 2 || r < 1 || kt % r != 0 || ((long)c * r) % kt != 0) return 0;
  const int xpw = d <= 64 ? 8 : 4;
  const long wgs = (long)B * h * (((d / 16) * (d / 16 + 1) / 2 * (16 / xpw) + 3) / 4);
  return wgs >= 512 ? 2 : 1;
}

// A: [B, n*c, h*r, d], Bm the same, w: [B, n*c, h*r] or null, lcs: [B, n, h] or null (no decay)
// -> S: [B*n, h, D, d], s: [B*n, h, D], entry k of a batch element being the scan value described above
int sympow_tn_chain(const void* A, const void* Bm, const float* w, const float* lcs, void* S, float* s, int B, int n,
                    int c, int h, int r, int d, int use_mult, int reverse, int dtype, hipStream_t st) {
  if (d != 32 && d != 64 && d != 128) return -2;
  if (n < 1 || r < 1 || tn_stage_rows(d) % r != 0 || ((long)c * r) % tn_stage_rows(d) != 0) return -3;
#define PR_TN_DISPATCH(T)                                                                                              \
  switch (d) {                                                                                                         \
    case 32: return tn_chain_launch<T, 32, 32>(A, Bm, w, lcs, S, s, B, n, c, h, r, use_mult, reverse, st);             \
    case 64: return tn_chain_launch<T, 64, 64>(A, Bm, w, lcs, S, s, B, n, c, h, r, use_mult, reverse, st);             \
    case 128: return tn_chain_launch<T, 128, 128>(A, Bm, w, lcs, S, s, B, n, c, h, r, use_mult, reverse, st);          \
    default: return -2;                                                                                                \
  }
  if (dtype == DT_BF16) { PR_TN_DISPATCH(bf16_t) }
  if (dtype == DT_F16) { PR_TN_DISPATCH(f16_t) }
#undef PR_TN_DISPATCH
  return -1;
}

template <typename T, int DK, int DV>
static int tn_launch(const void* A, const void* Bm, const float* w, void* S, float* s, int BN, int c, int h, int r,
                     int use_mult, int skip, const int* live, int live_side, hipStream_t st) {
  constexpr int XPW = DV <= 64 ? 8 : 4;
  constexpr int NB = (DK / 16) * (DK / 16 + 1) / 2;
  constexpr int TASKS = tn_tasks<DK, XPW>();
  constexpr int KT = tn_stage_rows(DV);
  constexpr size_t smem = TN_NST * (KT * DK * 2 + KT * DV * 2 + KT * 4);
  dim3 grid((TASKS + 3) / 4, (unsigned)(BN * h));
  if (w) {
    auto kern = sympow_tn_kernel<T, DK, DV, XPW, true>;
    allow_big_lds((const void*)kern, smem);
    PR_LAUNCH("sympow_tn", kern, grid, dim3(256), smem, st, (const T*)A, (const T*)Bm, w, (T*)S, s, c, h * r, r, h, use_mult, skip,
              live, live_side);
  } else {
    auto kern = sympow_tn_kernel<T, DK, DV, XPW, false>;
    allow_big_lds((const void*)kern, smem);
    PR_LAUNCH("sympow_tn", kern, grid, dim3(256), smem, st, (const T*)A, (const T*)Bm, w, (T*)S, s, c, h * r, r, h, use_mult, skip,
              live, live_side);
  }
  return (int)hipGetLastError();
}

// A: [BN, c, h*r, d], Bm: [BN, c, h*r, d], w: [BN, c, h*r] or null -> S: [BN, h, D, d], s: [BN, h, D]
// skip: 0, or +n / -n to skip the last / first chunk of every n (see the kernel)
// live ([BN, h, 2] or null), live_side: see the kernel; ignored while gate skipping is switched off
int sympow_tn(const void* A, const void* Bm, const float* w, void* S, float* s, int BN, int c, int h, int r, int d,
              int use_mult, int skip, const int* live, int live_side, int dtype, hipStream_t st) {
  if (!g_gate_skip) live = nullptr;
#define PR_TN_DISPATCH(T)                                                                                              \
  switch (d) {                                                                                                         \
    case 32: return tn_launch<T, 32, 32>(A, Bm, w, S, s, BN, c, h, r, use_mult, skip, live, live_side, st);                                   \
    case 64: return tn_launch<T, 64, 64>(A, Bm, w, S, s, BN, c, h, r, use_mult, skip, live, live_side, st);                                   \
    case 128: return tn_launch<T, 128, 128>(A, Bm, w, S, s, BN, c, h, r, use_mult, skip, live, live_side, st);                                \
    default: return -2;                                                                                                \
  }
  if (dtype == DT_BF16) { PR_TN_DISPATCH(bf16_t) }
  if (dtype == DT_F16) { PR_TN_DISPATCH(f16_t) }
#undef PR_TN_DISPATCH
  return -1;
}

}  // namespace pr
