// host-side exercise of the C ABI's argument checking and selection logic (no GPU needed)
#include <cstdio>
#include <cstdint>
#include <cstring>
#include "cascmm.h"
int main() {
  int fails = 0;
  auto expect = [&](bool ok, const char* what) { if (!ok) { printf("FAIL %s\n", what); ++fails; } };
  expect(cascmm_selftest() == 0, "selftest");
  const int n = cascmm_variant_count();
  expect(n > 50, "variant count");
  for (int i = -2; i < n + 2; ++i) { const char* s = cascmm_variant_name(i); expect((s != nullptr) == (i >= 0 && i < n), "variant name range");
    const char* k = cascmm_variant_kernel(i); expect((k != nullptr) == (i >= 0 && i < n), "variant kernel range"); }
  const int64_t dims[] = {0, 1, 2, 31, 32, 33, 154, 640, 1280, 2048, 5120, 10240, 32768, (1ll << 31) - 1, 1ll << 31, 1ll << 40, -1};
  for (int64_t M : dims) for (int64_t N : dims) for (int64_t K : dims)
    for (int dt = -1; dt < 4; ++dt) for (int fmt = -1; fmt < 4; ++fmt) for (int terms = 0; terms < 5; ++terms) for (int pr = 0; pr < 2; ++pr) {
      if ((M > 40000 || N > 40000 || K > 40000) && (dt != 0 || !((fmt == 0 && terms == 2) || (fmt == 2 && terms == 3) || (fmt == 1 && terms == 3)))) continue;   // keep the run short
      (void)cascmm_select_variant(M, N, K, K, N, N, dt, fmt, terms, pr);
      (void)cascmm_select_variant_grouped(3, M, N, K, K, N, N, dt, fmt, terms, pr);
      (void)cascmm_select_variant_prepared(1, M, N, K, K, N, dt, fmt, terms, pr);
      (void)cascmm_workspace_bytes(M, N, K, dt, fmt, terms, pr);
      (void)cascmm_prepared_bytes(K, N, fmt, terms);
    }
  // the chained feed-forward's size and shape functions over the same range, its launches with refusable arguments
  for (int64_t M : dims) for (int64_t N : dims) for (int64_t K : dims) {
    const size_t sb = cascmm_left_slots_bytes(M, K);
    expect(sb == 0 || sb / 4 / (size_t)M == (size_t)K, "left slots bytes");
    const int ok = cascmm_chained_supported(M, N, K);
    expect(ok == 0 || (K % 16 == 0 && K >= 16 && M > 0 && N > 0), "chained_supported");
    (void)cascmm_select_variant_glu(M, N, K, K, N, N / 2, 0, 0, 2, 0);
  }
  // launches refused before any HIP call: null pointers, bad leading dimensions, misaligned pointers
  char buf[256];
  expect(cascmm_gemm(nullptr, buf, buf, nullptr, 4, 4, 4, 4, 4, 4, 0, 0, 2, 0, nullptr, nullptr, 0, nullptr) != 0, "null A");
  expect(cascmm_gemm(buf, buf, buf, nullptr, 4, 4, 4, 2, 4, 4, 0, 0, 2, 0, nullptr, nullptr, 0, nullptr) != 0, "lda < K");
  expect(cascmm_gemm(buf + 1, buf, buf, nullptr, 4, 4, 4, 4, 4, 4, 0, 0, 2, 0, nullptr, nullptr, 0, nullptr) != 0, "misaligned A");
  expect(cascmm_gemm(buf, buf, buf, nullptr, 4, 4, 4, 4, 4, 4, 7, 0, 2, 0, nullptr, nullptr, 0, nullptr) != 0, "bad dtype");
  expect(cascmm_gemm(buf, buf, buf, nullptr, 0, 4, 4, 4, 4, 4, 0, 0, 2, 0, nullptr, nullptr, 0, nullptr) == 0, "M == 0 is a no-op");
  expect(cascmm_gemm_noalloc(buf, buf, buf, nullptr, 4, 4, 4, 2, 4, 4, 0, 0, 2, 0, nullptr, nullptr) != 0, "noalloc lda < K");
  expect(cascmm_gemm_fp8_autoscale(buf, buf, 0, buf, nullptr, 4, 4, 4, 4, 4, 4, 3, 0, nullptr, nullptr, nullptr, nullptr, 0, nullptr) != 0, "autoscale null exps");
  expect(cascmm_tensor_exp(buf, -1, 4, 4, 0, (int32_t*)buf, nullptr) != 0, "tensor_exp bad rows");
  expect(cascmm_tensor_exps(buf, 4, 4, 2, 0, nullptr, (int32_t*)buf, (int32_t*)buf, nullptr) != 0, "tensor_exps ld < cols");
  expect(cascmm_prepare_weight(buf, 64, 64, 8, 0, 2, 3, nullptr, buf, 16, nullptr) != 0, "prepare ldb < N");
  alignas(16) char slots[256];
  expect(cascmm_prepare_left(slots, 64, 40, 40, slots, sizeof(slots), nullptr) != 0, "prepare_left K % 16");
  expect(cascmm_prepare_left(slots, 64, 64, 64, slots, sizeof(slots), nullptr) != 0, "prepare_left output too small");
  expect(cascmm_prepare_left(slots, 1ll << 40, 64, 64, slots, sizeof(slots), nullptr) != 0, "prepare_left huge M");
  expect(cascmm_prepare_left(nullptr, 0, 64, 64, nullptr, 0, nullptr) == 0, "prepare_left of nothing");
  expect(cascmm_prepare_weight_chained(slots, 64, 64, 32, slots, sizeof(slots), nullptr) != 0, "prepare_weight_chained ldb < N");
  expect(cascmm_prepare_weight_chained(slots, 64, 64, 64, slots, sizeof(slots), nullptr) != 0, "prepare_weight_chained output too small");
  expect(cascmm_gemm_chained(slots, slots, slots, nullptr, 64, 160, 40, 160, nullptr) != 0, "gemm_chained K % 16");
  expect(cascmm_gemm_chained(slots, slots, slots, nullptr, 64, 160, 64, 100, nullptr) != 0, "gemm_chained ldc < N");
  expect(cascmm_gemm_chained(slots + 4, slots, slots, nullptr, 64, 160, 64, 160, nullptr) != 0, "gemm_chained misaligned slots");
  expect(cascmm_gemm_chained(slots, slots, slots, nullptr, 1ll << 31, 160, 64, 160, nullptr) != 0, "gemm_chained huge M");
  expect(cascmm_gemm_chained(slots, slots, slots, nullptr, 0, 160, 64, 160, nullptr) == 0, "gemm_chained of nothing");
  expect(cascmm_gemm_glu_chained(slots, slots, 0, slots, sizeof(slots), nullptr, 256, 330, 64, 64, 330, nullptr) != 0, "glu_chained N % 64");
  expect(cascmm_gemm_glu_chained(slots, slots, 0, slots, sizeof(slots), nullptr, 256, 640, 64, 64, 640, nullptr) != 0, "glu_chained slots too small");
  expect(cascmm_gemm_glu_chained(slots, slots, 1, slots, sizeof(slots), nullptr, 1ll << 33, 640, 64, 64, 640, nullptr) != 0, "glu_chained huge M");
  expect(cascmm_split_terms(buf, (float*)buf, -1, 0, 0, 2, 0, nullptr) != 0, "split n < 0");
  for (int st = -20; st <= 1; ++st) expect(cascmm_strerror(st) != nullptr, "strerror");
  printf("%s (%d failures)\n", fails ? "FAILED" : "OK", fails);
  return fails ? 1 : 0;
}
