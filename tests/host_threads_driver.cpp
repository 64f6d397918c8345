// several host threads ask the library for kernels and sizes at once (no GPU needed): every thread must
// get the answers a single thread gets; the launch entry point is walked up to its (absent) device
#include <cstdio>
#include <cstdint>
#include <thread>
#include <vector>
#include "cascmm.h"
struct Ask { int64_t M, N, K; int fmt, terms; };
static std::vector<Ask> asks() {
  std::vector<Ask> v;
  const int64_t ms[] = {2, 154, 1024, 2048, 4096, 8192}, ns[] = {640, 1280, 1920, 3840, 5120, 10240}, ks[] = {320, 640, 1280, 2048, 2560, 5120};
  const int cas[][2] = {{0, 2}, {0, 3}, {1, 3}, {2, 3}};
  for (int64_t M : ms) for (int64_t N : ns) for (int64_t K : ks) for (auto& c : cas) v.push_back({M, N, K, c[0], c[1]});
  return v;
}
static void answer(const Ask& a, int64_t out[5]) {
  out[0] = cascmm_select_variant(a.M, a.N, a.K, a.K, a.N, a.N, 0, a.fmt, a.terms, 0);
  out[1] = cascmm_select_variant_grouped(3, a.M, a.N, a.K, a.K, a.N, a.N, 0, a.fmt, a.terms, 0);
  out[2] = cascmm_select_variant_prepared(1, a.M, a.N, a.K, a.K, a.N, 0, a.fmt, a.terms, 0);
  out[3] = (int64_t)cascmm_workspace_bytes(a.M, a.N, a.K, 0, a.fmt, a.terms, 0);
  // the launch path as far as it goes on a host without a GPU (the test hides every device from this
  // process): argument checks, selection, the launcher's per-device set-up, which finds no device and
  // must return CASCMM_ERR_LAUNCH before anything is launched; the pointers are never dereferenced
  void* fake = (void*)(uintptr_t)0x100000;
  out[4] = cascmm_gemm(fake, fake, fake, nullptr, a.M, a.N, a.K, a.K, a.N, a.N, 0, a.fmt, a.terms, 0, nullptr, nullptr, 0, nullptr);
}
int main() {
  const std::vector<Ask> q = asks();
  const int T = 8;
  std::vector<std::vector<int64_t>> got(T, std::vector<int64_t>(q.size() * 5));
  std::vector<std::thread> th;
  for (int t = 0; t < T; ++t)
    th.emplace_back([&, t] {
      for (int rep = 0; rep < 3; ++rep)
        for (size_t i = 0; i < q.size(); ++i) { const size_t j = (i + 101 * t) % q.size(); answer(q[j], &got[t][j * 5]); }
    });
  for (auto& x : th) x.join();
  int fails = 0;
  for (size_t i = 0; i < q.size(); ++i) {
    int64_t one[5];
    answer(q[i], one);
    if (one[4] >= 0) { if (fails < 5) printf("FAIL ask %zu: cascmm_gemm returned %lld on a host without a GPU\n", i, (long long)one[4]); ++fails; }
    for (int t = 0; t < T; ++t)
      for (int j = 0; j < 5; ++j)
        if (got[t][i * 5 + j] != one[j]) { if (fails < 5) printf("FAIL ask %zu field %d thread %d: %lld vs %lld\n", i, j, t, (long long)got[t][i * 5 + j], (long long)one[j]); ++fails; }
  }
  printf("%s (%d failures, %zu asks x %d threads)\n", fails ? "FAILED" : "OK", fails, q.size(), T);
  return fails ? 1 : 0;
}
