// Preallocated K / V / gate cache of the decode loop: append in place instead of concatenating
// (ref: deploy/models/powercoder/kvgs_dynamic_cache.py:131-161 DynamicLayer.update_kv, which torch.cat's three tensors
// per layer and step).  The gate column holds ACCUMULATED log gates relative to the start of the cache -- what
// attention takes (ref: retention/power_retention_maker.py:347) -- so no cumulative sum over the cache is redone per step.
#include "common.h"
#include "kernels.h"

namespace pr {

// Kc, Vc [B, cap, h, d], Ac [B, cap, h] fp32;  k, v [B, t_new, h, d], g [B, t_new, h] fp32 or null (no gates: zeros).
// Rows pos .. pos + t_new - 1 are written; Ac[pos + i] = Ac[pos - 1] + g[0] + ... + g[i]  (Ac[-1] = 0); the last of
// them also goes to a_last [B, h] (dense: what the state query takes as the gate of the query position) when given.
template <typename T>
__global__ __launch_bounds__(256) void cache_append_kernel(T* __restrict__ Kc, T* __restrict__ Vc, float* __restrict__ Ac,
                                                           const T* __restrict__ k, const T* __restrict__ v,
                                                           const float* __restrict__ g, float* __restrict__ a_last, int B,
                                                           int cap, int pos, int t_new, int h, int d) {
  const long gid = (long)blockIdx.x * 256 + threadIdx.x;
  const int cpr = d / 8;                              // 16-byte pieces per (token, head) row
  const long n_copy = (long)B * t_new * h * cpr;
  if (gid < n_copy) {
    const int piece = (int)(gid % cpr);
    const long row = gid / cpr;                       // (b, i, hh)
    const int hh = (int)(row % h), i = (int)((row / h) % t_new), b = (int)(row / ((long)h * t_new));
    const long src = row * d + 8 * piece, dst = (((long)b * cap + pos + i) * h + hh) * d + 8 * piece;
    *(u32x4*)(Kc + dst) = *(const u32x4*)(k + src);
    *(u32x4*)(Vc + dst) = *(const u32x4*)(v + src);
    return;
  }
  const long j = gid - n_copy;                        // one thread per (b, hh): the running gate sum
  if (j >= (long)B * h) return;
  const int hh = (int)(j % h), b = (int)(j / h);
  float run = pos > 0 ? Ac[((long)b * cap + pos - 1) * h + hh] : 0.f;
  for (int i = 0; i < t_new; i++) {
    if (g) run += g[((long)b * t_new + i) * h + hh];
    Ac[((long)b * cap + pos + i) * h + hh] = run;
  }
  if (a_last) a_last[j] = run;
}

int cache_append(void* Kc, void* Vc, float* Ac, const void* k, const void* v, const float* g, float* a_last, int B,
                 int cap, int pos, int t_new, int h, int d, int dtype, hipStream_t st) {
  const long threads = (long)B * t_new * h * (d / 8) + (long)B * h;
  const dim3 grid((unsigned)((threads + 255) / 256));
  if (dtype == DT_BF16)
    PR_LAUNCH("cache_append", cache_append_kernel<bf16_t>, grid, dim3(256), 0, st, (bf16_t*)Kc, (bf16_t*)Vc, Ac, (const bf16_t*)k,
                       (const bf16_t*)v, g, a_last, B, cap, pos, t_new, h, d);
  else if (dtype == DT_F16)
    PR_LAUNCH("cache_append", cache_append_kernel<f16_t>, grid, dim3(256), 0, st, (f16_t*)Kc, (f16_t*)Vc, Ac, (const f16_t*)k,
                       (const f16_t*)v, g, a_last, B, cap, pos, t_new, h, d);
  else
    return -1;
  return (int)hipGetLastError();
}

}  // namespace pr
