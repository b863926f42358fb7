// Stand-alone timing probe (not part of the library): where a workgroup of the three attention kernels spends its
// time at the chunked headline shape (65536 x 8 rows cut into chunks of c keys, d = 64, bf16, gated, degree 2).
//
// It compiles the kernels' own sources with the PR_STAMP hook points turned into wall-clock stamps (100 MHz counter,
// wave 0 of every workgroup):  0 kernel entry, 1 set-up done (indices, first tile copies issued, own rows and row
// statistics in registers), 2 first tile's gate / row factors ready, 3 tile loop done, 4 results stored; slot 5 holds
// the number of tile steps of the workgroup.  Printed per number of tile steps: how many workgroups, and the mean
// duration of set-up / first factors / tile loop / epilogue in microseconds, plus the launch's span.  (The dK/dV
// kernel, which runs in the same call as the dQ kernel, uses slots 8-13.)
//
// Build and run:  python retention_integration_amd/csrc/build.py --probe && ./retention_integration_amd/probe_attention [c]
#include <hip/hip_runtime.h>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#define PR_STAMP_SLOTS 16
#define PR_STAMP_MAX_WG 16384
__device__ unsigned long long pr_probe_stamps[PR_STAMP_MAX_WG * PR_STAMP_SLOTS];
#define PR_STAMP(i) \
  if (threadIdx.x == 0 && blockIdx.x < PR_STAMP_MAX_WG) pr_probe_stamps[blockIdx.x * PR_STAMP_SLOTS + (i)] = wall_clock64();
#define PR_STAMP_VALUE(i, v) \
  if (threadIdx.x == 0 && blockIdx.x < PR_STAMP_MAX_WG) pr_probe_stamps[blockIdx.x * PR_STAMP_SLOTS + (i)] = (unsigned long long)(v);

#include "attention_fwd.hip"
#include "attention_bwd.hip"

#define CK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__); exit(1); } } while (0)

static unsigned short to_bf16(float f) {
  unsigned u;
  memcpy(&u, &f, 4);
  return (unsigned short)((u + 0x7fff + ((u >> 16) & 1)) >> 16);
}

// one kernel's stamps: rows of the table by number of tile steps
static void report(const char* name, int base) {
  const int first_wg = 0, n_wg = PR_STAMP_MAX_WG;
  std::vector<unsigned long long> st((size_t)PR_STAMP_MAX_WG * PR_STAMP_SLOTS);
  CK(hipMemcpyFromSymbol(st.data(), HIP_SYMBOL(pr_probe_stamps), st.size() * 8));
  static double sum[64][4];
  static int cnt[64];
  memset(sum, 0, sizeof(sum));
  memset(cnt, 0, sizeof(cnt));
  unsigned long long t0 = ~0ull, t1 = 0, gend[32] = {0}, gbusy[32] = {0};
  for (int i = first_wg; i < first_wg + n_wg && i < PR_STAMP_MAX_WG; i++) {
    const unsigned long long* s = &st[(size_t)i * PR_STAMP_SLOTS + base];
    if (s[0] == 0 || s[4] == 0) continue;   // a workgroup without work
    // workgroups go round-robin to the 8 XCDs and, inside an XCD, to its 4 shader engines: group = index % 32
    if (s[4] > gend[i % 32]) gend[i % 32] = s[4];
    gbusy[i % 32] += s[4] - s[0];
    const int nt = (int)s[5];
    if (nt < 0 || nt >= 64) continue;
    if (s[0] < t0) t0 = s[0];
    if (s[4] > t1) t1 = s[4];
    cnt[nt]++;
    for (int k = 0; k < 4; k++) sum[nt][k] += (double)(s[k + 1] - s[k]) * 0.01;
  }
  {
    double lo = 1e30, hi = 0, sum = 0, blo = 1e30, bhi = 0;
    for (int q = 0; q < 32; q++) {
      const double e = (gend[q] - t0) * 0.01, bz = gbusy[q] * 0.01;
      lo = e < lo ? e : lo; hi = e > hi ? e : hi; sum += e;
      blo = bz < blo ? bz : blo; bhi = bz > bhi ? bz : bhi;
    }
    printf("%s: the 32 (XCD, shader engine) groups finish %.1f .. %.1f us after the first workgroup starts (mean %.1f); "
           "workgroup time summed per group %.0f .. %.0f us\n", name, lo, hi, sum / 32, blo, bhi);
  }
  printf("%s: span of the launch %.1f us\n  steps  workgroups  set-up  first factors  tile loop  epilogue   total   (us, mean)\n", name,
         (t1 - t0) * 0.01);
  for (int nt = 0; nt < 64; nt++)
    if (cnt[nt])
      printf("  %5d  %10d  %6.2f  %13.2f  %9.2f  %8.2f  %6.2f\n", nt, cnt[nt], sum[nt][0] / cnt[nt], sum[nt][1] / cnt[nt],
             sum[nt][2] / cnt[nt], sum[nt][3] / cnt[nt], (sum[nt][0] + sum[nt][1] + sum[nt][2] + sum[nt][3]) / cnt[nt]);
}

static void clear_stamps() {
  void* p;
  CK(hipGetSymbolAddress(&p, HIP_SYMBOL(pr_probe_stamps)));
  CK(hipMemset(p, 0, sizeof(unsigned long long) * PR_STAMP_MAX_WG * PR_STAMP_SLOTS));
}

int main(int argc, char** argv) {
  const int c = argc > 1 ? atoi(argv[1]) : 1024, B = 64 * 1024 / c, h = 8, d = 64;
  const size_t n = (size_t)B * c * h * d, nr = (size_t)B * c * h;
  std::vector<unsigned short> hq(n), hk(n), hv(n), hdo(n);
  srand(1);
  auto rnd = [] { float s = 0; for (int i = 0; i < 12; i++) s += rand() / (float)RAND_MAX; return s - 6.f; };   // ~N(0,1)
  for (size_t i = 0; i < n; i++) { hq[i] = to_bf16(rnd()); hk[i] = to_bf16(rnd()); hv[i] = to_bf16(rnd()); hdo[i] = to_bf16(rnd()); }
  std::vector<float> hg(nr);   // accumulated log gates, log-sigmoid of a normal per step
  for (int b = 0; b < B; b++)
    for (int hh = 0; hh < h; hh++) {
      float run = 0;
      for (int t = 0; t < c; t++) { run += -logf(1.f + expf(-rnd())); hg[((size_t)b * c + t) * h + hh] = run; }
    }
  void *Q, *K, *V, *O, *dO, *dQ, *dK, *dV;
  float *G, *l, *m, *dGq, *dGk;
  for (void** p : {&Q, &K, &V, &O, &dO, &dQ, &dK, &dV}) CK(hipMalloc(p, n * 2));
  for (float** p : {&G, &l, &m, &dGq, &dGk}) CK(hipMalloc((void**)p, nr * 4));
  CK(hipMemcpy(Q, hq.data(), n * 2, hipMemcpyHostToDevice));
  CK(hipMemcpy(K, hk.data(), n * 2, hipMemcpyHostToDevice));
  CK(hipMemcpy(V, hv.data(), n * 2, hipMemcpyHostToDevice));
  CK(hipMemcpy(dO, hdo.data(), n * 2, hipMemcpyHostToDevice));
  CK(hipMemcpy(G, hg.data(), nr * 4, hipMemcpyHostToDevice));
  printf("attention kernels, %d chunks of %d keys x %d heads, d = %d, bf16, gated, degree 2\n", B, c, h, d);

  pr::AttnFwdArgs f{Q, K, V, G, O, l, m, c, c, h, 1, 0.125f, 2.f, 0, c};
  for (int i = 0; i < 3; i++) if (int rc = pr::attention_fwd(f, B, d, 0, 0)) { printf("attention_fwd rc=%d\n", rc); return 1; }
  CK(hipDeviceSynchronize());
  clear_stamps();
  pr::attention_fwd(f, B, d, 0, 0);
  CK(hipDeviceSynchronize());
  report("attention_fwd", 0);

  pr::AttnBwdArgs bw{Q, K, V, G, m, dO, nullptr, nullptr, dQ, dK, dV, dGq, dGk, c, c, h, 1, 0.125f, 2.f,
                     nullptr, nullptr, nullptr, nullptr, 0};
  for (int i = 0; i < 3; i++) if (int rc = pr::attention_bwd(bw, B, d, 0, 0)) { printf("attention_bwd rc=%d\n", rc); return 1; }
  CK(hipDeviceSynchronize());
  clear_stamps();
  pr::attention_bwd(bw, B, d, 0, 0);
  CK(hipDeviceSynchronize());
  report("attention_bwd_dq", 0);
  report("attention_bwd_dkv", 8);
  return 0;
}
