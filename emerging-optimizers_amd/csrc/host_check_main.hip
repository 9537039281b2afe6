// Driver of the host-side bounds check (`make host-check`; see host_check.hpp).  Calls the library's C entry points
// with made-up device addresses over a grid of shapes -- every benchmark configuration, the shapes of the GPU tests,
// multiples of 8 on both sides of every tile size, batches, both operand layouts, every option that changes kernel
// choice -- and fails if any lane of any fast-kernel launch would touch a byte outside the buffers of its call, if a
// tile is computed twice or not at all, or if a sanitizer trips in the host code on the way.  No GPU is involved.
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "../../include/mi_ns.h"
#include "host_check.hpp"

using mi::host_check::add_range;
using mi::host_check::clear_ranges;
using mi::host_check::state;

namespace {

// Made-up device memory: addresses that are never dereferenced, 256-byte aligned, a megabyte apart at least, so that
// an access that leaves its buffer lands in no other.
uint64_t g_next = 0x100000000000ull;
void* fake_alloc(size_t bytes, const char* name) {
  void* p = reinterpret_cast<void*>(g_next);
  g_next += (bytes + (1u << 20) + 255) / 256 * 256;
  add_range(p, bytes, name);
  return p;
}
void* fake_alloc_unregistered(size_t bytes) {
  void* p = reinterpret_cast<void*>(g_next);
  g_next += (bytes + (1u << 20) + 255) / 256 * 256;
  return p;
}

long g_calls = 0, g_refused = 0;
std::string g_ctx;
void begin(const std::string& what) {
  clear_ranges();
  g_next = 0x100000000000ull;
  g_ctx = what;
  state().context = g_ctx.c_str();
  ++g_calls;
}
void expect_ok(int rc) {
  if (rc == MI_OK) return;
  if (rc == MI_ERR_UNSUPPORTED_SHAPE) {
    ++g_refused;
    return;
  }
  std::fprintf(stderr, "[host-check] %s: library call failed with %d: %s\n", g_ctx.c_str(), rc, mi_last_error());
  ++state().failures;
}

void syrk_case(int64_t batch, int64_t n, int64_t k, int trans, bool addend, int skip_upper, bool with_workspace) {
  char what[200];
  std::snprintf(what, sizeof what, "syrk batch=%lld n=%lld k=%lld trans=%d addend=%d skip_upper=%d ws=%d", (long long)batch, (long long)n,
                (long long)k, trans, (int)addend, skip_upper, (int)with_workspace);
  begin(what);
  void* a = fake_alloc((size_t)batch * n * k * 2, "A");
  void* c = addend ? fake_alloc((size_t)batch * n * n * 2, "C") : nullptr;
  void* d = fake_alloc((size_t)batch * n * n * 2, "D");
  const int64_t a_ld = trans ? n : k;
  if (with_workspace) {
    const size_t need = skip_upper ? 0 : mi_syrk_workspace_bytes(batch, n, k, trans);
    void* ws = need ? fake_alloc(need, "workspace") : nullptr;
    expect_ok(mi_syrk_bf16_ws(a, batch, n, k, n * k, a_ld, trans, c, n * n, n, 0.5f, addend ? 0.25f : 0.0f, d, n * n, n, skip_upper, ws, need, nullptr));
  } else {
    expect_ok(mi_syrk_bf16(a, batch, n, k, n * k, a_ld, trans, c, n * n, n, 0.5f, addend ? 0.25f : 0.0f, d, n * n, n, skip_upper, nullptr));
  }
}

// `cols`: the product runs on columns [col0, col0 + cols) of matrices that are n columns wide (col0 = 0, cols = n: all)
void gemm_case(int64_t batch, int64_t m, int64_t n, int x_trans, int out_fp32, int64_t col0 = 0, int64_t cols = -1) {
  if (cols < 0) cols = n;
  char what[200];
  std::snprintf(what, sizeof what, "gemm_axpy batch=%lld m=%lld n=%lld x_trans=%d out_fp32=%d columns [%lld, %lld)", (long long)batch,
                (long long)m, (long long)n, x_trans, out_fp32, (long long)col0, (long long)(col0 + cols));
  begin(what);
  char* bm = static_cast<char*>(fake_alloc((size_t)batch * m * m * 2, "Bm"));
  char* x = static_cast<char*>(fake_alloc((size_t)batch * m * n * 2, "X"));
  char* out = static_cast<char*>(fake_alloc((size_t)batch * m * n * (out_fp32 ? 4 : 2), "Xout"));
  const int64_t ld = x_trans ? m : n;
  // a column range of a row-major matrix starts col0 elements in; of a transposed one, col0 rows down
  const int64_t first = x_trans ? col0 * m : col0;
  expect_ok(mi_gemm_axpy_bf16(bm, m * m, m, x + first * 2, m * n, ld, x_trans, out + first * (out_fp32 ? 4 : 2), m * n, ld, batch, m, cols, 0.5f, 0.25f,
                              out_fp32, 2.0f, nullptr));
}

void frob_case(int64_t batch, int64_t numel, int out_bf16, int f64) {
  char what[200];
  std::snprintf(what, sizeof what, "frob_normalize batch=%lld numel=%lld out_bf16=%d f64=%d", (long long)batch, (long long)numel, out_bf16, f64);
  begin(what);
  void* x = fake_alloc((size_t)batch * numel * 4, "x");
  void* out = fake_alloc((size_t)batch * numel * (out_bf16 ? 2 : 4), "out");
  void* partials = fake_alloc(mi_frob_partials_len(batch, numel) * 8, "partials");
  void* norm = fake_alloc((size_t)batch * 4, "norm");
  expect_ok(mi_frob_normalize(static_cast<const float*>(x), batch, numel, 1e-7f, f64, out, out_bf16, static_cast<double*>(partials),
                              static_cast<float*>(norm), nullptr));
}

const float SIMPLE[15] = {3.4445f, -4.7750f, 2.0315f, 3.4445f, -4.7750f, 2.0315f, 3.4445f, -4.7750f, 2.0315f,
                          3.4445f, -4.7750f, 2.0315f, 3.4445f, -4.7750f, 2.0315f};
const float QUINTIC[15] = {4.0848f, -6.8946f, 2.9270f, 3.9505f, -6.3029f, 2.6377f, 3.7418f, -5.5913f, 2.3037f,
                           2.8769f, -3.1427f, 1.2046f, 2.8366f, -3.0525f, 1.2012f};
const float CUBIC[15] = {3.3656576f, -3.3420992f, 0.0f, 2.5744352f, -1.4957376f, 0.0f, 2.5368962f, -1.4312570f, 0.0f,
                         2.4418906f, -1.2764040f, 0.0f, 2.2230472f, -0.9630650f, 0.0f};
const float POLAR8[24] = {8.2051f, -22.9019f, 16.4607f, 4.0664f, -2.8612f, 0.5184f, 3.9096f, -2.8234f, 0.5250f, 3.2856f, -2.4153f, 0.4853f,
                          2.2779f, -1.6198f, 0.3985f, 1.8726f, -1.2307f, 0.3585f, 1.8564f, -1.2132f, 0.3568f, 1.8750f, -1.2500f, 0.3750f};

void ns_case(int64_t batch, int64_t rows, int64_t cols, const float* abc, int steps, const char* kind, bool update) {
  char what[200];
  std::snprintf(what, sizeof what, "%s batch=%lld %lldx%lld %s x %d", update ? "muon_update" : "newton_schulz", (long long)batch, (long long)rows,
                (long long)cols, kind, steps);
  begin(what);
  const size_t elems = (size_t)batch * rows * cols;
  void* x = fake_alloc(elems * 4, "x");
  void* out = fake_alloc(elems * 4, update ? "param" : "out");
  const size_t need = mi_newton_schulz_workspace_bytes(batch, rows, cols);
  void* ws = fake_alloc_unregistered(need);  // (the call registers the segments of its workspace one by one)
  if (update) {
    void* mom = fake_alloc(elems * 4, "momentum");
    expect_ok(mi_muon_update_bf16(static_cast<float*>(out), static_cast<const float*>(x), static_cast<float*>(mom), batch, rows, cols, 0.95f, 1,
                                  0.999f, -0.02f, abc, steps, 1e-15f, 0, ws, need, nullptr));
  } else {
    expect_ok(mi_newton_schulz_bf16(static_cast<const float*>(x), static_cast<float*>(out), batch, rows, cols, abc, steps, 1e-15f, 0, 1.0f, ws, need,
                                    nullptr));
  }
}

void set(const char* name, int value) {
  if (mi_set_option(name, value) != MI_OK) {
    std::fprintf(stderr, "[host-check] mi_set_option(%s, %d) failed\n", name, value);
    ++state().failures;
  }
}

// The refusals of the entry points (what tests/test_c_abi.py checks on the ordinary build), here with the host code
// under the sanitizers: every bad call must come back with its error code and launch nothing.
void validation_cases() {
  begin("argument validation");
  const long launches = state().launches;
  void* p = fake_alloc(1 << 20, "buffer");
  char* odd = static_cast<char*>(p) + 8;  // not 16-byte aligned
  const float abc[3] = {1.0f, 2.0f, 3.0f};
  auto expect = [&](int rc, int want, const char* what) {
    if (rc != want) {
      std::fprintf(stderr, "[host-check] %s returned %d, expected %d (%s)\n", what, rc, want, mi_last_error());
      ++state().failures;
    }
  };
  expect(mi_syrk_bf16(p, 1, 12, 16, 192, 16, 0, nullptr, 0, 12, 1.0f, 0.0f, p, 144, 12, 0, nullptr), MI_ERR_UNSUPPORTED_SHAPE, "syrk, n % 8");
  expect(mi_syrk_bf16(p, 1, 16, 16, 256, 16, 0, nullptr, 0, 16, 1.0f, 0.5f, p, 256, 16, 0, nullptr), MI_ERR_BAD_ARG, "syrk, beta without C");
  expect(mi_syrk_bf16(nullptr, 1, 16, 16, 256, 16, 0, nullptr, 0, 16, 1.0f, 0.0f, p, 256, 16, 0, nullptr), MI_ERR_BAD_ARG, "syrk, null A");
  expect(mi_syrk_bf16(odd, 1, 16, 16, 256, 16, 0, nullptr, 0, 16, 1.0f, 0.0f, p, 256, 16, 0, nullptr), MI_ERR_UNSUPPORTED_SHAPE, "syrk, misaligned A");
  expect(mi_syrk_bf16(p, 1, 16, 16, 256, 8, 0, nullptr, 0, 16, 1.0f, 0.0f, p, 256, 16, 0, nullptr), MI_ERR_BAD_ARG, "syrk, a_ld too small");
  expect(mi_syrk_bf16(p, -1, 16, 16, 256, 16, 0, nullptr, 0, 16, 1.0f, 0.0f, p, 256, 16, 0, nullptr), MI_ERR_BAD_ARG, "syrk, negative batch");
  expect(mi_syrk_bf16_ws(p, 1, 2048, 4096, 2048 * 4096, 2048, 1, nullptr, 0, 2048, 1.0f, 0.0f, nullptr, 2048 * 2048, 2048, 0, p, (size_t)1 << 40, nullptr),
         MI_ERR_BAD_ARG, "syrk with workspace, null D");
  expect(mi_gemm_axpy_bf16(p, 0, 12, p, 0, 16, 0, p, 0, 16, 1, 12, 16, 1.0f, 1.0f, 0, 1.0f, nullptr), MI_ERR_UNSUPPORTED_SHAPE, "gemm, m % 8");
  expect(mi_gemm_axpy_bf16(p, 0, 16, nullptr, 0, 16, 0, p, 0, 16, 1, 16, 16, 1.0f, 1.0f, 0, 1.0f, nullptr), MI_ERR_BAD_ARG, "gemm, null X");
  expect(mi_gemm_axpy_bf16(p, 0, 16, p, 0, 8, 0, p, 0, 16, 1, 16, 16, 1.0f, 1.0f, 0, 1.0f, nullptr), MI_ERR_BAD_ARG, "gemm, x_ld too small");
  expect(mi_newton_schulz_bf16(static_cast<float*>(p), static_cast<float*>(p), 1, 12, 16, abc, 1, 1e-15f, 0, 1.0f, p, 1 << 20, nullptr),
         MI_ERR_UNSUPPORTED_SHAPE, "newton_schulz, rows % 8");
  expect(mi_newton_schulz_bf16(static_cast<float*>(p), static_cast<float*>(p), 1, 16, 16, abc, 1, 1e-15f, 0, 1.0f, p, 8, nullptr), MI_ERR_WORKSPACE,
         "newton_schulz, workspace too small");
  expect(mi_newton_schulz_bf16(static_cast<float*>(p), static_cast<float*>(p), 1, 16, 16, nullptr, 1, 1e-15f, 0, 1.0f, p, 1 << 20, nullptr),
         MI_ERR_BAD_ARG, "newton_schulz, null coefficients");
  expect(mi_newton_schulz_bf16(static_cast<float*>(p), static_cast<float*>(p), 70000, 16, 16, abc, 1, 1e-15f, 0, 1.0f, p, (size_t)1 << 40, nullptr),
         MI_ERR_UNSUPPORTED_SHAPE, "newton_schulz, batch beyond the grid limit");
  expect(mi_muon_update_bf16(static_cast<float*>(p), static_cast<float*>(p), static_cast<float*>(p), 1, 16, 16, 0.9f, 1, 0.0f, 1.0f, abc, 1, 1e-15f, 0, p,
                             1 << 20, nullptr),
         MI_ERR_BAD_ARG, "muon_update, param_decay 0");
  expect(mi_muon_update_bf16(static_cast<float*>(p), static_cast<float*>(p), static_cast<float*>(p), 1, 16, 16, 0.9f, 1, 1.0f, 1.0f, abc, 0, 1e-15f, 0, p,
                             1 << 20, nullptr),
         MI_ERR_BAD_ARG, "muon_update, no steps");
  expect(mi_newton_schulz_bf16_noalloc(static_cast<float*>(p), static_cast<float*>(p), 1, 4096, 14336, abc, 1, 1e-15f, 0, 1.0f, nullptr), MI_ERR_WORKSPACE,
         "noalloc, beyond the built-in buffer");
  expect(mi_set_option("no_such_option", 1), MI_ERR_BAD_ARG, "set_option, unknown name");
  expect(mi_set_option("ns_pairs", 7), MI_ERR_BAD_ARG, "set_option, value out of range");
  int groups[4];
  expect(mi_newton_schulz_schedule(1, 64, 64, nullptr, 5, groups, 4), MI_ERR_BAD_ARG, "schedule, null coefficients");
  expect(mi_syrk_bf16(p, 0, 16, 16, 256, 16, 0, nullptr, 0, 16, 1.0f, 0.0f, p, 256, 16, 0, nullptr), MI_OK, "syrk, empty batch");
  if (state().launches != launches) {
    std::fprintf(stderr, "[host-check] a refused call launched a kernel\n");
    ++state().failures;
  }
}

// The check must notice a buffer that is too small: the same call with the result one row short, the operand one K tile
// short and the addend 16 bytes short, each of which has to be reported.
int selftest() {
  const int64_t n = 1096, k = 192;
  long found[3] = {0, 0, 0};
  for (int which = 0; which < 3; ++which) {
    begin("selftest");
    const size_t a_bytes = (size_t)n * k * 2, c_bytes = (size_t)n * n * 2;
    void* a = fake_alloc(a_bytes - (which == 1 ? 64 * 2 : 0), "A");
    void* c = fake_alloc(c_bytes - (which == 2 ? 16 : 0), "C");
    void* d = fake_alloc(c_bytes - (which == 0 ? (size_t)n * 2 : 0), "D");
    const long before = state().failures;
    std::FILE* quiet = std::freopen("/dev/null", "w", stderr);
    (void)quiet;
    expect_ok(mi_syrk_bf16(a, 1, n, k, n * k, k, 0, c, n * n, n, 0.5f, 0.25f, d, n * n, n, 0, nullptr));
    found[which] = state().failures - before;
  }
  std::printf("host-check selftest: undersized result / operand / addend reported %ld / %ld / %ld times\n", found[0], found[1], found[2]);
  // the self-guarding kernels: a normalisation call whose output, or whose array of partial sums, is too small
  long stated[2] = {0, 0};
  for (int which = 0; which < 2; ++which) {
    begin("selftest");
    const int64_t batch = 3, numel = 256 * 512;
    void* x = fake_alloc((size_t)batch * numel * 4, "x");
    void* out = fake_alloc((size_t)batch * numel * 2 - (which == 0 ? 16 : 0), "out");
    void* partials = fake_alloc(which == 1 ? 8 * (size_t)batch : mi_frob_partials_len(batch, numel) * 8, "partials");  // (one per matrix: too few)
    const long before = state().failures;
    expect_ok(mi_frob_normalize(static_cast<const float*>(x), batch, numel, 1e-7f, 0, out, 1, static_cast<double*>(partials), nullptr, nullptr));
    stated[which] = state().failures - before;
  }
  std::printf("host-check selftest: undersized normalised copy / partial sums reported %ld / %ld times\n", stated[0], stated[1]);
  return (found[0] > 0 && found[1] > 0 && found[2] > 0 && stated[0] > 0 && stated[1] > 0) ? 0 : 1;
}

}  // namespace

int main(int argc, char** argv) {
  if (argc > 1 && std::strcmp(argv[1], "--selftest") == 0) return selftest();
  const bool quick = argc > 1 && std::strcmp(argv[1], "--quick") == 0;
  // --bench: the benchmark's own calls only; --bench-exhaustive: the same calls with no sampling of workgroups or K tiles
  const bool bench_exhaustive = argc > 1 && std::strcmp(argv[1], "--bench-exhaustive") == 0;
  const bool bench_only = bench_exhaustive || (argc > 1 && std::strcmp(argv[1], "--bench") == 0);
  state().exhaustive = bench_exhaustive;
  validation_cases();
  // ---- lower-triangle products
  const int64_t ns_[] = {256, 384, 512, 768, 1024, 1032, 1096, 1152, 1280, 1536, 1792, 1800, 2048, 2304, 3072, 4096, 5120, 8184, 8192};
  const int64_t ks_[] = {64, 128, 192, 448, 1024, 4096, 8192, 14336};
  for (int streamk : {-1, 1}) {
    if (bench_only) break;
    for (int transpose : {-1, 0, 1}) {
      set("streamk", streamk);
      set("syrk_transpose", transpose);
      const bool by_model = streamk == -1 && transpose == -1;
      for (int64_t n : ns_)
        for (int64_t k : ks_) {
          // --quick: the sizes around every tile edge with short K, forced variants on three sizes only
          if (quick && (n > 2304 || k > 1024 || k == 128 || k == 448)) continue;
          if (quick && !by_model && !((n == 1024 || n == 1280 || n == 2048) && k != 64)) continue;
          for (int64_t batch : {1, 3}) {
            if (batch * n * n * k > (int64_t)1 << 38) continue;
            if (quick && batch > 1 && !by_model) continue;
            for (int trans : {0, 1}) {
              if (!trans && transpose != -1) continue;  // (the option only matters for transposed operands)
              syrk_case(batch, n, k, trans, true, 0, true);
              if (by_model) {
                syrk_case(batch, n, k, trans, false, 1, true);
                if (!quick) syrk_case(batch, n, k, trans, true, 0, false);
              }
            }
          }
        }
    }
  }
  set("streamk", -1);
  set("syrk_transpose", -1);
  // the benchmark's SYRK rows: batched call, beta variant, one matrix alone, operand stored transposed
  const int64_t bench_syrk[][3] = {{16, 2048, 8192}, {8, 2048, 2048}, {4, 4096, 4096}, {32, 512, 2048}, {64, 256, 1024}, {1, 4096, 14336},
                                   {2, 1024, 512}, {5, 1024, 448}, {30, 1024, 128}, {26, 1024, 256}, {7, 1024, 64}, {2, 1536, 4096}};
  for (const auto& s : bench_syrk)
    for (int trans : {0, 1})
      for (bool addend : {false, true}) {
        if (quick && s[0] * s[1] * s[2] > (int64_t)1 << 26) continue;
        syrk_case(s[0], s[1], s[2], trans, addend, 0, true);
        syrk_case(1, s[1], s[2], trans, addend, 0, true);
      }
  // ---- GEMM + AXPY
  const int64_t gemm_[][2] = {{1024, 1024}, {1024, 2304}, {2048, 4096}, {4096, 4096}, {4096, 14336}, {1792, 4096}, {1280, 1536}, {128, 512},
                              {384, 768},   {896, 256},   {128, 4096},  {256, 1024},  {1000, 2048},  {1024, 1032}, {1032, 2048}, {64, 64}};
  for (const auto& s : gemm_)
    for (int64_t batch : {1, 2, 8}) {
      if ((quick && batch > 1) || bench_only) continue;
      for (int x_trans : {0, 1})
        for (int out_fp32 : {0, 1}) gemm_case(batch, s[0], s[1], x_trans, out_fp32);
    }
  gemm_case(1, 4096, 14336, 0, 0, 0, 12288);  // a column range of a wider matrix, as the tail split of the library itself
  gemm_case(1, 4096, 14336, 0, 1, 12288, 2048);
  gemm_case(1, 4096, 14336, 1, 1, 12288, 2048);
  // ---- normalisation on its own
  for (int64_t batch : {1, 5})
    for (int64_t numel : {8, 4096, 1 << 20, 4096 * 14336})
      for (int out_bf16 : {0, 1})
        for (int f64 : {0, 1}) frob_case(batch, numel, out_bf16, f64);
  // ---- the single-call driver and the fused optimizer update
  const int64_t nsh[][3] = {{1, 256, 512},   {1, 512, 256},   {1, 64, 64},      {1, 8, 16},      {3, 128, 384},   {2, 384, 128},  {1, 1024, 1280},
                            {4, 128, 1024},  {2, 256, 1536},  {1, 1536, 256},   {1, 1024, 2048}, {2, 1024, 2304}, {1, 200, 456},  {1, 1024, 2560},
                            {1, 4096, 4096}, {1, 4096, 14336}, {1, 14336, 4096}, {8, 1792, 4096}, {8, 4096, 1792}, {32, 128, 4096}, {5, 4096, 128},
                            {1, 3584, 1024}, {2, 2304, 1024},  {1, 2048, 1024},  {6, 128, 1024},  {1, 1024, 4096}, {8, 4096, 4096}, {8, 4096, 14336}};
  struct Kind {
    const float* abc;
    int steps;
    const char* name;
  };
  const Kind kinds[] = {{SIMPLE, 5, "simple"}, {QUINTIC, 5, "quintic"}, {QUINTIC, 4, "quintic"}, {CUBIC, 5, "cubic5"}, {POLAR8, 8, "polar_express"},
                        {SIMPLE, 1, "simple"}, {SIMPLE, 0, "none"}};
  for (int pairs : {-1, 0, 1, 2})
    for (int direct : {1, 0})
      for (int head : {1, 0}) {
        if ((direct == 0 || head == 0) && pairs != -1) continue;
        set("ns_pairs", pairs);
        set("tall_direct", direct);
        set("head_apply", head);
        set("head_front", head);
        if ((quick && (pairs == 1 || direct == 0)) || (bench_only && !(pairs == -1 && direct == 1 && head == 1))) continue;
        for (const auto& s : nsh) {
          if (quick && s[0] * s[1] * s[2] > (int64_t)1 << 22) continue;
          for (const Kind& kd : kinds) {
            if (bench_only && !(kd.steps == 5 && kd.abc != CUBIC)) continue;
            if (pairs != -1 && kd.steps < 4) continue;
            if (quick && (kd.steps == 4 || kd.steps == 1)) continue;
            ns_case(s[0], s[1], s[2], kd.abc, kd.steps, kd.name, false);
            if (kd.steps >= 1 && pairs == -1) ns_case(s[0], s[1], s[2], kd.abc, kd.steps, kd.name, true);
          }
        }
      }
  const mi::host_check::State& st = state();
  std::printf("host-check: %ld library calls (%ld refused as unsupported), %ld fast-kernel launches, %ld workgroups, %ld accesses checked, "
              "%ld other launches with %ld stated blocks, %ld failures\n",
              g_calls, g_refused, st.launches, st.workgroups, st.accesses, st.other_launches, st.footprints, st.failures);
  return st.failures == 0 ? 0 : 1;
}
