// Shared device helpers for the gfx950 (CDNA4) power-retention kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace pr {

typedef __bf16 bf16_t;
typedef _Float16 f16_t;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(4))) _Float16 f16x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(8))) short s16x8;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

enum { DT_BF16 = 0, DT_F16 = 1, DT_F32 = 2 };

template <typename T> struct VecOf;
template <> struct VecOf<bf16_t> { typedef bf16x8 v8; typedef bf16x4 v4; };
template <> struct VecOf<f16_t> { typedef f16x8 v8; typedef f16x4 v4; };

// One 16x16x32 matrix-core op: D[16x16] += A[16x32] * B[32x16].
// Lane l holds A[row l%16][k = 8*(l/16) .. +7], B[k = 8*(l/16) .. +7][col l%16],
// and D[row 4*(l/16)+v][col l%16] in element v of the accumulator.
__device__ __forceinline__ f32x4 mfma16(bf16x8 a, bf16x8 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ f32x4 mfma16(f16x8 a, f16x8 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
}

// Compile-time loop: f(std::integral_constant<int, I>) for I in [0, N).
template <int I> struct IC { static constexpr int value = I; constexpr operator int() const { return I; } };
template <int I, int N, typename F> __device__ __forceinline__ void static_for_impl(F&& f) {
  if constexpr (I < N) {
    f(IC<I>{});
    static_for_impl<I + 1, N>(f);
  }
}
template <int N, typename F> __device__ __forceinline__ void static_for(F&& f) { static_for_impl<0, N>(f); }

__device__ __forceinline__ int lane_id() { return threadIdx.x & 63; }

// ---- 16-bit <-> fp32 -----------------------------------------------------
__device__ __forceinline__ void unpack8(bf16x8 v, float* f) {
  u32x4 u = __builtin_bit_cast(u32x4, v);
#pragma unroll
  for (int i = 0; i < 4; i++) {
    f[2 * i] = __builtin_bit_cast(float, u[i] << 16);
    f[2 * i + 1] = __builtin_bit_cast(float, u[i] & 0xffff0000u);
  }
}
__device__ __forceinline__ void unpack8(f16x8 v, float* f) {
#pragma unroll
  for (int i = 0; i < 8; i++) f[i] = (float)v[i];
}
template <typename T> __device__ __forceinline__ typename VecOf<T>::v8 pack8(const float* f) {
  typename VecOf<T>::v8 r;
#pragma unroll
  for (int i = 0; i < 8; i++) r[i] = (T)f[i];
  return r;
}
template <typename T> __device__ __forceinline__ typename VecOf<T>::v4 pack4(const float* f) {
  typename VecOf<T>::v4 r;
#pragma unroll
  for (int i = 0; i < 4; i++) r[i] = (T)f[i];
  return r;
}
__device__ __forceinline__ float to_f32(bf16_t x) { return (float)x; }
__device__ __forceinline__ float to_f32(f16_t x) { return (float)x; }
__device__ __forceinline__ float to_f32(float x) { return x; }

// ---- LDS operand loads -----------------------------------------------------
// Row-major LDS tile [k][ld]; returns the MFMA operand whose contraction index runs down the
// rows: element j of lane l is tile[k0 + 8*(l/16) + j][n0 + l%16].  Uses the gfx950 transposing
// LDS read: the 16 lanes of a row each fetch 4 contiguous columns of one of 4 rows, and lane i
// receives column i of those 4 rows.
template <typename T>
__device__ __forceinline__ typename VecOf<T>::v8 lds_frag_tr(const T* tile, int ld, int k0, int n0) {
  const int l = lane_id(), s = l & 15, g = l >> 4;
  const T* p = tile + (k0 + 8 * g + (s >> 2)) * ld + n0 + 4 * (s & 3);
  typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
  s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)p);
  s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(p + 4 * ld));
  s16x8 r = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  return __builtin_bit_cast(typename VecOf<T>::v8, r);
}
// Same, but only 4 rows: element j of lane l is tile[k0 + j][n0 + l%16] with k0 chosen per lane row.
template <typename T>
__device__ __forceinline__ typename VecOf<T>::v4 lds_frag_tr4(const T* tile, int ld, int krow, int n0) {
  const int l = lane_id(), s = l & 15;
  const T* p = tile + (krow + (s >> 2)) * ld + n0 + 4 * (s & 3);
  typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
  s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)p);
  return __builtin_bit_cast(typename VecOf<T>::v4, lo);
}
// Row-major LDS tile [n][ld] whose contraction index runs along the row: element j of lane l is
// tile[n0 + l%16][k0 + 8*(l/16) + j].
template <typename T>
__device__ __forceinline__ typename VecOf<T>::v8 lds_frag(const T* tile, int ld, int n0, int k0) {
  const int l = lane_id();
  return *(const typename VecOf<T>::v8*)(tile + (n0 + (l & 15)) * ld + k0 + 8 * (l >> 4));
}

// ---- swizzled LDS tiles filled by asynchronous global->LDS copies ---------------------------
// A tile is [rows][CPR chunks of 16 bytes] with no padding; chunk c of row r is stored at chunk
// slot c ^ swz(r), which spreads the 16 rows an operand load touches over all banks.  The copy
// instruction (global_load_lds_dwordx4) writes lane i's 16 bytes at wave_base + 16*i, so a wave
// fills 64 consecutive chunk slots and every lane fetches the global chunk that belongs in its slot.
// Completion is tracked by vmcnt only: the consumer waits with wait_vmcnt<N>() and then barriers.
// Which swizzle is free of bank conflicts depends on how the tile is read (measured on gfx950 with every candidate,
// wave-wide reads of a tile with 64-, 128- and 256-byte rows):
//  * SWZ_K8: tiles whose transposing reads take rows 8g + (s >> 2) (contraction index along the rows, eight rows per
//    lane group: the operand tiles of sympow_tn and sympow_nn) -- a bit rotation of the row index;
//  * SWZ_ROW: tiles read row-wise as 16-byte operand chunks (row = lane % 16, chunk 4*ks + g) and/or with transposing
//    reads that take rows 4g + (s >> 2) (the attention tiles, the state tile of sympow_grad) -- the chunk slot advances
//    by one every 128 bytes of rows.
// With the other kind's swizzle these reads take 1.8-1.9 times as long.
enum { SWZ_K8 = 0, SWZ_ROW = 1 };
template <int CPR, int KIND = SWZ_K8> __device__ __forceinline__ int swz(int row) {
  static_assert(CPR == 4 || CPR == 8 || CPR == 16, "rows of 64, 128 or 256 bytes");
  if (KIND == SWZ_ROW) return ((row * CPR) >> 3) & (CPR - 1);
  if (CPR == 8) {
    const int k = (row >> 1) & 7;
    return ((k & 1) << 2) | (k >> 1);
  } else if (CPR == 16) {
    const int k = row & 15;
    return ((k & 3) << 2) | (k >> 2);
  }
  return (row >> 2) & 3;
}

template <int N> __device__ __forceinline__ void wait_vmcnt() {
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
  __builtin_amdgcn_s_waitcnt((N & 0xF) | ((N >> 4) << 14) | (0x7 << 4) | (0xF << 8));
}

// The copies are written as inline assembly on purpose: the compiler tracks copies it knows about and makes every
// later LDS read it cannot prove disjoint wait for ALL of them (vmcnt(0)), which serialises the ring.  Written
// this way they are invisible to that tracking; completion is handled by wait_vmcnt<N>() alone, which counts
// instructions and is therefore safe whatever other vector-memory operations the compiler interleaves.
__device__ __forceinline__ void async_copy16(const void* gsrc, void* lds_wave_base) {
  const uint32_t base = __builtin_amdgcn_readfirstlane(
      (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)lds_wave_base);
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(base), "v"(gsrc) : "memory", "m0");
}
__device__ __forceinline__ void async_copy4(const void* gsrc, void* lds_wave_base) {
  const uint32_t base = __builtin_amdgcn_readfirstlane(
      (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)lds_wave_base);
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, off" ::"s"(base), "v"(gsrc) : "memory", "m0");
}

// The same copies with the global address split into a wave-uniform base (scalar registers) and a per-lane byte
// offset, so that stepping the base through memory costs no vector instruction.  lds_wave_base is the wave-uniform
// LDS byte address (lane i's bytes land at lds_wave_base + 16*i, resp. 4*i).
__device__ __forceinline__ void async_copy16_sv(const void* uniform_base, uint32_t lane_off, uint32_t lds_wave_base) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_wave_base), "v"(lane_off),
               "s"(uniform_base)
               : "memory", "m0");
}
// Non-temporal form, for bytes that no other workgroup reads (a state streamed once).
__device__ __forceinline__ void async_copy16_sv_nt(const void* uniform_base, uint32_t lane_off, uint32_t lds_wave_base) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 nt" ::"s"(lds_wave_base), "v"(lane_off),
               "s"(uniform_base)
               : "memory", "m0");
}
__device__ __forceinline__ void async_copy4_sv(const void* uniform_base, uint32_t lane_off, uint32_t lds_wave_base) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2" ::"s"(lds_wave_base), "v"(lane_off),
               "s"(uniform_base)
               : "memory", "m0");
}
// For values that are uniform but were computed on the vector unit (anything behind an integer division): bring
// them back to scalar registers, as the operands above require.
__device__ __forceinline__ const void* uniform_ptr(const void* p) {
  const uint64_t u = (uint64_t)(uintptr_t)p;
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)u), hi = __builtin_amdgcn_readfirstlane((uint32_t)(u >> 32));
  return (const void*)(uintptr_t)(((uint64_t)hi << 32) | lo);
}
__device__ __forceinline__ uint32_t lds_addr(const void* p) {
  return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const char*)p;
}

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also drains the vector-memory counter, which
// would make every asynchronous global->LDS copy (and every register prefetch) in flight complete at each barrier;
// here only this wave's LDS operations are waited for, and copies are tracked by wait_vmcnt<N>() alone.  The asm
// memory clobber keeps the compiler from moving LDS accesses across it.
__device__ __forceinline__ void lds_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// Issue the copies of a tile of R rows (R*CPR a multiple of 256) by a 256-thread workgroup: every thread
// issues exactly R*CPR/256 copies.  row_ptr(row) returns the global address of the row's first byte and
// must be valid for every row (clamp out-of-range rows; zero them afterwards with zero_tile_rows).
template <int CPR, int R, int KIND = SWZ_K8, typename F> __device__ __forceinline__ void async_load_tile(char* tile, F row_ptr) {
  static_assert((R * CPR) % 256 == 0, "tile must be a whole number of workgroup-wide copies");
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
#pragma unroll
  for (int ii = 0; ii < R * CPR / 256; ii++) {
    const int inst = ii * 4 + wave;
    const int pos = inst * 64 + lane, row = pos / CPR, c = (pos % CPR) ^ swz<CPR, KIND>(row);
    async_copy16(row_ptr(row) + 16 * c, tile + inst * 1024);
  }
}
// Zero rows [first_bad, R) of a tile (same slot ownership as async_load_tile; call after the wait, before the barrier).
template <int CPR, int R> __device__ __forceinline__ void zero_tile_rows(char* tile, int first_bad) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
#pragma unroll
  for (int ii = 0; ii < R * CPR / 256; ii++) {
    const int pos = (ii * 4 + wave) * 64 + lane;
    if (pos / CPR >= first_bad) *(u32x4*)(tile + pos * 16) = (u32x4){0, 0, 0, 0};
  }
}

// Operand loads from a swizzled tile of T (same conventions as lds_frag / lds_frag_tr / lds_frag_tr4).
template <typename T, int CPR>
__device__ __forceinline__ typename VecOf<T>::v8 sw_frag(const char* tile, int n0, int k0) {
  const int l = lane_id(), row = n0 + (l & 15), c = (k0 + 8 * (l >> 4)) / 8;
  return *(const typename VecOf<T>::v8*)(tile + row * (CPR * 16) + ((c ^ swz<CPR>(row)) * 16));
}
template <typename T, int CPR>
__device__ __forceinline__ typename VecOf<T>::v4 sw_frag_tr4(const char* tile, int krow, int n0) {
  const int l = lane_id(), s = l & 15, row = krow + (s >> 2), col = n0 + 4 * (s & 3);
  const char* p = tile + row * (CPR * 16) + (((col / 8) ^ swz<CPR>(row)) * 16) + (col % 8) * 2;
  typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
  s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)p);
  return __builtin_bit_cast(typename VecOf<T>::v4, v);
}
template <typename T, int CPR>
__device__ __forceinline__ typename VecOf<T>::v8 sw_frag_tr(const char* tile, int k0, int n0) {
  const int g = lane_id() >> 4;
  typename VecOf<T>::v4 lo = sw_frag_tr4<T, CPR>(tile, k0 + 8 * g, n0);
  typename VecOf<T>::v4 hi = sw_frag_tr4<T, CPR>(tile, k0 + 8 * g + 4, n0);
  return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
}

// Broadcast lane N of every 16-lane row to the whole row (folds into the consuming VALU op).
template <int N> __device__ __forceinline__ float row_bcast(float x) {
  return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, x), 0x150 + N, 0xf, 0xf, true));
}
template <int N> __device__ __forceinline__ uint32_t row_bcast_u32(uint32_t x) {
  return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x150 + N, 0xf, 0xf, true);
}

// bcast_lane_N_of_row(src) * row in ONE VALU op.  The compiler only folds the row broadcast into the multiply
// for some operand orders, so the instruction is spelled out.  It is opaque to the hazard recogniser: src must
// have been written at least two wait states earlier -- callers put dpp_fence() between producing src and the
// first use.
template <int N> __device__ __forceinline__ float mul_row_bcast(float src, float row) {
  float r;
  asm("v_mul_f32_dpp %0, %1, %2 row_newbcast:%3 row_mask:0xf bank_mask:0xf bound_ctrl:1"
      : "=v"(r)
      : "v"(src), "v"(row), "n"(N));
  return r;
}
__device__ __forceinline__ void dpp_fence() {
  __builtin_amdgcn_sched_barrier(0);
  asm volatile("s_nop 1");
  __builtin_amdgcn_sched_barrier(0);
}

// Sum over the four 16-lane rows of a wave (lanes l, l+16, l+32, l+48); every lane gets the total.
__device__ __forceinline__ float sum_over_rows(float x) {
  x += __shfl_xor(x, 16);
  x += __shfl_xor(x, 32);
  return x;
}
__device__ __forceinline__ float max_over_rows(float x) {
  x = fmaxf(x, __shfl_xor(x, 16));
  x = fmaxf(x, __shfl_xor(x, 32));
  return x;
}
// Sum over the 16 lanes of a row; every lane gets the total.
__device__ __forceinline__ float sum_in_row(float x) {
  x += __shfl_xor(x, 1);
  x += __shfl_xor(x, 2);
  x += __shfl_xor(x, 4);
  x += __shfl_xor(x, 8);
  return x;
}
__device__ __forceinline__ float wave_sum(float x) {
  return sum_over_rows(sum_in_row(x));
}

// Every kernel launch of the library goes through PR_LAUNCH.  A caller may register a hook (pr_set_launch_hook of the
// C ABI) that is called on the host right before and right after each launch with the kernel's name and stream --
// a benchmark records a pair of events there and so times every kernel where it runs.  No hook: one load and a branch.
typedef void (*launch_hook_t)(const char* kernel, int phase, void* stream, void* user);
extern launch_hook_t g_launch_hook;
extern void* g_launch_hook_user;
struct LaunchScope {
  const char* name;
  hipStream_t st;
  launch_hook_t hook;
  LaunchScope(const char* n, hipStream_t s) : name(n), st(s), hook(g_launch_hook) {
    if (hook) hook(name, 0, (void*)st, g_launch_hook_user);
  }
  ~LaunchScope() {
    if (hook) hook(name, 1, (void*)st, g_launch_hook_user);
  }
};
#define PR_LAUNCH(name, kern, grid, block, smem, st, ...)                                                              \
  do {                                                                                                                 \
    ::pr::LaunchScope pr_launch_scope_(name, st);                                                                      \
    hipLaunchKernelGGL(kern, grid, block, smem, st, __VA_ARGS__);                                                      \
  } while (0)

// Kernels that use more than 64 KB of dynamic LDS must opt in once per function.
static inline void allow_big_lds(const void* kernel, size_t bytes) {
  // (a refusal shows up as the launch error that every caller checks right after)
  if (bytes > 48 * 1024) (void)hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
}

// ---- causal blocks of many (batch, head) pairs on one (XCD, shader engine) group ---------------------------------
// The u-th workgroup of a group that owns ppg pairs of nblocks blocks each (block 0 the longest).  Pairs follow one
// another, longest block first, so that the blocks of a pair run together and share its rows in L2 -- except the
// last PR_TAIL_PAIRS pairs, whose blocks are dealt longest first across all of them: with whole pairs to the very end
// the last long blocks start when most slots are already idle (list scheduling of lengths 8..1 on 16 slots ends at
// 39 units for an ideal 36, on 24 slots at 28 for 24; with the last four interleaved at 37 and 25).  Measured at 512
// pairs of 8 blocks: 4 pairs 0.9 % faster for the whole forward + backward step, 8 pairs 0.6 %, all 16 pairs 1.2 % slower.
#ifndef PR_TAIL_PAIRS
#define PR_TAIL_PAIRS 4
#endif
__device__ __forceinline__ void deal_causal_blocks(int u, int nblocks, int ppg, int& pig, int& blk) {
  const int K = ppg < PR_TAIL_PAIRS ? ppg : PR_TAIL_PAIRS, head = (ppg - K) * nblocks;
  int p, b;
  if (u < head) {
    p = u / nblocks;
    b = u - p * nblocks;
  } else {
    const int v = u - head;
    b = v / K;
    p = ppg - K + (v - b * K);
  }
  // (integer division runs on the vector unit: readfirstlane brings the uniform results back to scalar registers)
  pig = __builtin_amdgcn_readfirstlane(p);
  blk = __builtin_amdgcn_readfirstlane(b);
}

// ---- state layout ----------------------------------------------------------
// Features are grouped in blocks of 256 = 16 x 16: block (y, xb), xb <= y, holds the products
// k[16*xb + X] * k[16*y + i] at feature 128*y*(y+1) + 256*xb + 16*X + i.  Blocks are numbered
// in memory order: blk = y*(y+1)/2 + xb.
__host__ __device__ constexpr int expanded_dim(int d) { return 128 * (d / 16) * (d / 16 + 1); }

__device__ __forceinline__ void block_to_yx(int blk, int& y, int& xb) {
  y = 0;
  while ((y + 1) * (y + 2) / 2 <= blk) y++;
  xb = blk - y * (y + 1) / 2;
}

}  // namespace pr
