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

// Broadcast lane N of every 16-lane row to the whole row (folds into the consuming VALU op).
template <int N> __device__ __forceinline__ float row_bcast(float x) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x150 + N, 0xf, 0xf, true));
}
template <int N> __device__ __forceinline__ uint32_t row_bcast_u32(uint32_t x) {
  return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x150 + N, 0xf, 0xf, true);
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

// Kernels that use more than 64 KB of dynamic LDS must opt in once per function.
static inline void allow_big_lds(const void* kernel, size_t bytes) {
  if (bytes > 48 * 1024) hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
}

// ---- state layout ----------------------------------------------------------
// Features are grouped in blocks of 256 = 16 x 16: block (y, xb), xb <= y, holds the products
// k[16*xb + X] * k[16*y + i] at feature 128*y*(y+1) + 256*xb + 16*X + i.  Blocks are numbered
// in memory order: blk = y*(y+1)/2 + xb.
__host__ __device__ __forceinline__ int expanded_dim(int d) { return 128 * (d / 16) * (d / 16 + 1); }
__device__ __forceinline__ void block_to_yx(int blk, int& y, int& xb) {
  y = 0;
  while ((y + 1) * (y + 2) / 2 <= blk) y++;
  xb = blk - y * (y + 1) / 2;
}

}  // namespace pr
