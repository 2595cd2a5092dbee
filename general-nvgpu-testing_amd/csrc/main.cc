// beam_host -- C++ host for libbeam_hip.so: a registry of self-checking tests and a small CLI.
//
// It talks to the kernels only through the C ABI (include/beam_hip.h), the same entry points the
// Python package binds.  The checks here need no CPU reference GEMM: they use operands whose
// products are known exactly (identity, all-ones, one-hot), and consistency properties (split-K
// against the plain kernel, run-to-run determinism, LayerNorm invariants).
//
// The reference's counterpart is the pybind11 module initialiser with its three register_*
// functions (cuda/main.cc:31-33,51-60) and the dead timing helper test_pipeline
// (cuda/cublas.cc:12-40); its only test driver is the Python script python/gemm_test.py.
//
//   beam_host --list
//   beam_host --info
//   beam_host --run all | <test name>
//   beam_host --bench [--op gemm|splitk|ln|silu|nn] --m M --n N --k K [--dtype fp16|bf16] [--tile BMxBN]
//             [--wave TMxTN] [--pipeline 0|1] [--group G] [--splitk S] [--iters I] [--warmup W]
//             [--count ELEMENTS]   (silu: GEMM, SiLU alone and GEMM with the SiLU in its K loop)
//             [--data normal|uniform|zeros] (normal: N(0,1)/sqrt(K); uniform: [-1, 1); zeros: all-zero operands,
//                                            for telling schedule limits from power limits)
//             [--ln-mode auto|twopass|fused]   (--op ln)
//             --op probe-empty | probe-empty-pair | probe-splitk-loads: launches that measure what the machine
//             allows (an empty kernel, two of them, the split-K partial kernel with nothing but its loads)
//             --op probe-mfma [--dtype fp16|bf16] [--mfma 16x16x32|32x32x16] [--data normal|zeros] [--passes P]
//             [--seconds S]: a register-only loop of MFMAs on every SIMD (no memory instruction), i.e. what
//             the matrix cores sustain on this data at the clock the power cap allows; S > 0 keeps it running
//             for about S seconds, printing a line per second (for sampling power and clock beside it)
//   beam_host --tune --m M --n N --k K [--dtype fp16|bf16]
//   beam_host --copy MiB      device-to-device copy of known size (calibrates profiler byte counters)
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <map>
#include <string>
#include <vector>

#include "../../include/beam_hip_debug.h"

namespace {

// ---- 16-bit helpers (host) ----------------------------------------------------------------

float half_to_float(uint16_t h) {
  const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  const uint32_t exp = (h >> 10) & 0x1fu;
  const uint32_t man = h & 0x3ffu;
  uint32_t bits;
  if (exp == 0) {
    if (man == 0) {
      bits = sign;
    } else {
      float v = std::ldexp((float)man, -24);
      std::memcpy(&bits, &v, 4);
      bits |= sign;
    }
  } else if (exp == 31) {
    bits = sign | 0x7f800000u | (man << 13);
  } else {
    bits = sign | ((exp + 112u) << 23) | (man << 13);
  }
  float f;
  std::memcpy(&f, &bits, 4);
  return f;
}

float bf16_to_float(uint16_t h) {
  uint32_t bits = (uint32_t)h << 16;
  float f;
  std::memcpy(&f, &bits, 4);
  return f;
}

float to_float(uint16_t v, int dtype) { return dtype == BEAM_BF16 ? bf16_to_float(v) : half_to_float(v); }

// Exact for the small integers and powers of two the tests use.
uint16_t small_to_16(float f, int dtype) {
  uint32_t bits;
  std::memcpy(&bits, &f, 4);
  if (dtype == BEAM_BF16) return (uint16_t)(bits >> 16);
  if ((bits & 0x7fffffffu) == 0) return (uint16_t)(bits >> 16);
  const uint32_t sign = (bits >> 16) & 0x8000u;
  const int exp = (int)((bits >> 23) & 0xff) - 127 + 15;
  return (uint16_t)(sign | ((uint32_t)exp << 10) | ((bits >> 13) & 0x3ffu));
}

// ---- device buffers --------------------------------------------------------------------------

struct Check {
  bool ok = true;
  std::string why;
  void fail(const std::string& s) {
    if (ok) why = s;
    ok = false;
  }
};

#define BEAM_REQUIRE(chk, call)                                                          \
  do {                                                                                   \
    int rc_ = (call);                                                                    \
    if (rc_ != BEAM_OK) {                                                                \
      (chk).fail(std::string(#call) + " -> " + std::to_string(rc_) + ": " + beam_last_error()); \
      return (chk);                                                                      \
    }                                                                                    \
  } while (0)

struct DevBuf {
  void* p = nullptr;
  size_t bytes = 0;
  explicit DevBuf(size_t n) : bytes(n) {
    if (beam_malloc(&p, n) != BEAM_OK) {
      std::fprintf(stderr, "beam_malloc(%zu): %s\n", n, beam_last_error());
      std::exit(2);
    }
  }
  ~DevBuf() { beam_free(p); }
  DevBuf(const DevBuf&) = delete;
  DevBuf& operator=(const DevBuf&) = delete;
  void upload(const std::vector<uint16_t>& h) { beam_memcpy_h2d(p, h.data(), h.size() * 2); }
  std::vector<uint16_t> download16() const {
    std::vector<uint16_t> h(bytes / 2);
    beam_sync(nullptr);
    beam_memcpy_d2h(h.data(), p, bytes);
    return h;
  }
};

std::vector<uint16_t> uniform16(size_t n, int dtype, uint64_t seed, uint64_t id) {
  std::vector<uint16_t> v(n);
  beam_host_fill_uniform(v.data(), n, dtype, seed, id);
  return v;
}

std::vector<uint16_t> normal16(size_t n, int dtype, uint64_t seed, uint64_t id, float mean, float scale) {
  std::vector<uint16_t> v(n);
  beam_host_fill_normal(v.data(), n, dtype, seed, id, mean, scale);
  return v;
}

// ---- tests -------------------------------------------------------------------------------------

typedef std::function<Check()> TestFn;
std::map<std::string, TestFn>& registry() {
  static std::map<std::string, TestFn> r;
  return r;
}
struct Register {
  Register(const char* name, TestFn fn) { registry()[name] = fn; }
};
#define BEAM_TEST(name)                      \
  Check test_##name();                       \
  Register register_##name(#name, test_##name); \
  Check test_##name()

// C = I . B^T must reproduce B^T bit for bit, for every compiled tile and both dtypes.
BEAM_TEST(identity_every_tile) {
  Check c;
  const int n = 256, N = 320;
  for (int dtype = 0; dtype < 2; ++dtype) {
    std::vector<uint16_t> eye((size_t)n * n, 0);
    for (int i = 0; i < n; ++i) eye[(size_t)i * n + i] = small_to_16(1.0f, dtype);
    std::vector<uint16_t> b = uniform16((size_t)N * n, dtype, 1, 1);
    DevBuf da(eye.size() * 2), db(b.size() * 2), dc((size_t)n * N * 2);
    da.upload(eye);
    db.upload(b);
    for (int k = 0; k < beam_num_configs(); ++k) {
      beam_tile_cfg cfg;
      BEAM_REQUIRE(c, beam_get_config(k, &cfg));
      for (int pipe = 0; pipe < 2; ++pipe) {
        cfg.pipeline = pipe;
        beam_memset(dc.p, 0xEE, dc.bytes);
        BEAM_REQUIRE(c, beam_gemmrc(da.p, db.p, dc.p, n, N, n, dtype, &cfg, nullptr));
        std::vector<uint16_t> got = dc.download16();
        for (int m = 0; m < n && c.ok; ++m)
          for (int j = 0; j < N; ++j)
            if (got[(size_t)m * N + j] != b[(size_t)j * n + m]) {
              // +0 and -0 compare equal as numbers
              if (to_float(got[(size_t)m * N + j], dtype) == to_float(b[(size_t)j * n + m], dtype)) continue;
              c.fail("tile " + std::to_string(cfg.block_m) + "x" + std::to_string(cfg.block_n) + " dtype " +
                     std::to_string(dtype) + ": C[" + std::to_string(m) + "][" + std::to_string(j) + "] differs");
              break;
            }
      }
    }
  }
  return c;
}

// All-ones operands: every element equals K (exact in fp16 up to 2048), ragged M and N.
BEAM_TEST(all_ones_ragged) {
  Check c;
  const int M = 300, N = 171 * 4, K = 2048;
  std::vector<uint16_t> a((size_t)M * K, small_to_16(1.0f, BEAM_F16)), b((size_t)N * K, small_to_16(1.0f, BEAM_F16));
  DevBuf da(a.size() * 2), db(b.size() * 2), dc((size_t)M * N * 2);
  da.upload(a);
  db.upload(b);
  beam_memset(dc.p, 0, dc.bytes);
  BEAM_REQUIRE(c, beam_gemmrc(da.p, db.p, dc.p, M, N, K, BEAM_F16, nullptr, nullptr));
  for (uint16_t v : dc.download16())
    if (half_to_float(v) != (float)K) {
      c.fail("expected " + std::to_string(K) + ", got " + std::to_string(half_to_float(v)));
      break;
    }
  return c;
}

// One-hot rows of A select single columns of B, including a short last K tile (K = 3*64 + 40).
BEAM_TEST(one_hot_k_tail) {
  Check c;
  const int M = 200, N = 264, K = 232;
  std::vector<uint16_t> a((size_t)M * K, 0);
  std::vector<int> pick(M);
  for (int m = 0; m < M; ++m) {
    pick[m] = (m * 37 + 5) % K;
    a[(size_t)m * K + pick[m]] = small_to_16(-2.0f, BEAM_F16);
  }
  std::vector<uint16_t> b = uniform16((size_t)N * K, BEAM_F16, 3, 1);
  DevBuf da(a.size() * 2), db(b.size() * 2), dc((size_t)M * N * 2);
  da.upload(a);
  db.upload(b);
  for (int k = 0; k < beam_num_configs(); ++k) {
    beam_tile_cfg cfg;
    BEAM_REQUIRE(c, beam_get_config(k, &cfg));
    beam_memset(dc.p, 0xEE, dc.bytes);
    BEAM_REQUIRE(c, beam_gemmrc(da.p, db.p, dc.p, M, N, K, BEAM_F16, &cfg, nullptr));
    std::vector<uint16_t> got = dc.download16();
    for (int m = 0; m < M && c.ok; ++m)
      for (int n = 0; n < N; ++n)
        if (half_to_float(got[(size_t)m * N + n]) != -2.0f * half_to_float(b[(size_t)n * K + pick[m]])) {
          c.fail("tile " + std::to_string(cfg.block_m) + "x" + std::to_string(cfg.block_n) + ": C[" +
                 std::to_string(m) + "][" + std::to_string(n) + "] wrong");
          break;
        }
  }
  return c;
}

// Split-K: one slice is the plain kernel bit for bit; S slices agree with it to fp32 reorder noise, are
// bit-identical from run to run, and give the same bits in one launch and in two.
BEAM_TEST(splitk_consistency) {
  Check c;
  const int M = 256, N = 256, K = 8192;
  std::vector<uint16_t> a = uniform16((size_t)M * K, BEAM_F16, 5, 0), b = uniform16((size_t)N * K, BEAM_F16, 5, 1);
  DevBuf da(a.size() * 2), db(b.size() * 2), dc((size_t)M * N * 2), dw(beam_splitk_workspace_bytes(M, N, 64));
  da.upload(a);
  db.upload(b);
  beam_tile_cfg cfg = {64, 64, 32, 32, 0, 0};
  BEAM_REQUIRE(c, beam_gemmrc(da.p, db.p, dc.p, M, N, K, BEAM_F16, &cfg, nullptr));
  const std::vector<uint16_t> plain = dc.download16();
  BEAM_REQUIRE(c, beam_gemmrc_splitk(da.p, db.p, dc.p, M, N, K, BEAM_F16, &cfg, 1, dw.p, dw.bytes, nullptr));
  if (dc.download16() != plain) c.fail("split_k = 1 differs from the plain kernel");
  for (int s : {4, 8, 16, 32, 64}) {
    BEAM_REQUIRE(c, beam_gemmrc_splitk(da.p, db.p, dc.p, M, N, K, BEAM_F16, &cfg, s, dw.p, dw.bytes, nullptr));
    const std::vector<uint16_t> first = dc.download16();
    BEAM_REQUIRE(c, beam_gemmrc_splitk(da.p, db.p, dc.p, M, N, K, BEAM_F16, &cfg, s, dw.p, dw.bytes, nullptr));
    if (dc.download16() != first) c.fail("split_k = " + std::to_string(s) + " is not deterministic");
    // both results are rounded to fp16 from fp32 sums that differ only in summation order: they may
    // differ by one unit in the last place (2^-10 relative), never more
    for (size_t i = 0; i < first.size(); ++i) {
      const double r = half_to_float(plain[i]), g = half_to_float(first[i]);
      if (std::fabs(g - r) > std::fmax(std::fabs(r), 1.0) * (1.0 / 1024.0) * 1.001) {
        c.fail("split_k = " + std::to_string(s) + ": element " + std::to_string(i) + " is " + std::to_string(g) +
               ", plain kernel gives " + std::to_string(r));
        break;
      }
    }
    // the same slices as partial kernel + reduce kernel, and on a workspace that holds the partial sums only
    // (no room for the one-launch form's flags): the same bits as the one launch above
    BEAM_REQUIRE(c, beam_set_splitk_two_launches(1));
    const int rc_two = beam_gemmrc_splitk(da.p, db.p, dc.p, M, N, K, BEAM_F16, &cfg, s, dw.p, dw.bytes, nullptr);
    beam_set_splitk_two_launches(0);
    BEAM_REQUIRE(c, rc_two);
    if (dc.download16() != first) c.fail("split_k = " + std::to_string(s) + ": two launches differ from one");
    const int eff = beam_splitk_effective(M, N, K, &cfg, s);
    BEAM_REQUIRE(c, beam_gemmrc_splitk(da.p, db.p, dc.p, M, N, K, BEAM_F16, &cfg, s, dw.p, (size_t)eff * M * N * 4, nullptr));
    if (dc.download16() != first) c.fail("split_k = " + std::to_string(s) + ": a workspace without flags gives other bits");
    int timed_out = 1;
    BEAM_REQUIRE(c, beam_gemmrc_splitk_timed_out(dw.p, dw.bytes, M, N, eff, nullptr, &timed_out));
    if (timed_out) c.fail("split_k = " + std::to_string(s) + ": time-out reported");
  }
  return c;
}

// B stored [K][N]: C = I . B reproduces B, and a random problem matches beam_gemmrc on the transposed
// copy of B bit for bit (the two kernels add the same products in the same order), every tile.
BEAM_TEST(matmul_nn_every_tile) {
  Check c;
  const int M = 200, N = 328, K = 264;
  for (int dtype = 0; dtype < 2; ++dtype) {
    std::vector<uint16_t> a = uniform16((size_t)M * K, dtype, 5, 0), b = uniform16((size_t)K * N, dtype, 5, 1);
    std::vector<uint16_t> bt((size_t)N * K);
    for (int k = 0; k < K; ++k)
      for (int n = 0; n < N; ++n) bt[(size_t)n * K + k] = b[(size_t)k * N + n];
    std::vector<uint16_t> eye((size_t)K * K, 0);
    for (int i = 0; i < K; ++i) eye[(size_t)i * K + i] = small_to_16(1.0f, dtype);
    DevBuf da(a.size() * 2), db(b.size() * 2), dbt(bt.size() * 2), de(eye.size() * 2), dc((size_t)M * N * 2),
        dc2((size_t)M * N * 2), dci((size_t)K * N * 2);
    da.upload(a);
    db.upload(b);
    dbt.upload(bt);
    de.upload(eye);
    for (int k = 0; k < beam_num_configs() && c.ok; ++k) {
      beam_tile_cfg cfg;
      BEAM_REQUIRE(c, beam_get_config(k, &cfg));
      BEAM_REQUIRE(c, beam_matmul_nn(da.p, db.p, dc.p, M, N, K, dtype, &cfg, nullptr));
      BEAM_REQUIRE(c, beam_gemmrc(da.p, dbt.p, dc2.p, M, N, K, dtype, &cfg, nullptr));
      if (dc.download16() != dc2.download16())
        c.fail("tile " + std::to_string(cfg.block_m) + "x" + std::to_string(cfg.block_n) + ": differs from gemmrc on B^T");
      BEAM_REQUIRE(c, beam_matmul_nn(de.p, db.p, dci.p, K, N, K, dtype, &cfg, nullptr));
      std::vector<uint16_t> got = dci.download16();
      for (size_t i = 0; i < got.size() && c.ok; ++i)
        if (got[i] != b[i] && to_float(got[i], dtype) != to_float(b[i], dtype)) c.fail("I . B != B");
    }
  }
  return c;
}

// The same on the kernel of four 128 x 128 wavefronts, which takes K a multiple of 64 from 192 up: several tiles per
// column and row of tiles, edge tiles in M and N.
BEAM_TEST(matmul_nn_four_wavefronts) {
  Check c;
  const int M = 700, N = 520, K = 320;
  beam_tile_cfg cfg = {256, 256, 128, 128, 0, 0};
  for (int dtype = 0; dtype < 2 && c.ok; ++dtype) {
    std::vector<uint16_t> a = uniform16((size_t)M * K, dtype, 6, 0), b = uniform16((size_t)K * N, dtype, 6, 1);
    std::vector<uint16_t> bt((size_t)N * K);
    for (int k = 0; k < K; ++k)
      for (int n = 0; n < N; ++n) bt[(size_t)n * K + k] = b[(size_t)k * N + n];
    DevBuf da(a.size() * 2), db(b.size() * 2), dbt(bt.size() * 2), dc((size_t)M * N * 2), dc2((size_t)M * N * 2);
    da.upload(a);
    db.upload(b);
    dbt.upload(bt);
    BEAM_REQUIRE(c, beam_matmul_nn(da.p, db.p, dc.p, M, N, K, dtype, &cfg, nullptr));
    BEAM_REQUIRE(c, beam_gemmrc(da.p, dbt.p, dc2.p, M, N, K, dtype, &cfg, nullptr));
    if (dc.download16() != dc2.download16()) c.fail(std::string(dtype ? "bf16" : "fp16") + ": differs from gemmrc on B^T");
  }
  return c;
}

// GEMM with the SiLU side job: C equals the plain GEMM bit for bit, Y equals the standalone kernel,
// silu(0) = 0 and silu(x) = x for x >= 20 (fp16), for an array longer than the K loops can carry.
BEAM_TEST(gemm_silu_side_job) {
  Check c;
  const int M = 384, N = 320, K = 200;
  const long long count = 300007;
  std::vector<uint16_t> a = normal16((size_t)M * K, BEAM_F16, 8, 0, 0.0f, 0.1f),
                        b = normal16((size_t)N * K, BEAM_F16, 8, 1, 0.0f, 0.1f),
                        x = normal16((size_t)count, BEAM_F16, 8, 2, 0.0f, 3.0f);
  x[0] = 0;
  x[1] = small_to_16(20.0f, BEAM_F16);
  x[count - 1] = small_to_16(64.0f, BEAM_F16);
  DevBuf da(a.size() * 2), db(b.size() * 2), dc((size_t)M * N * 2), dc2((size_t)M * N * 2), dx(x.size() * 2),
      dy(x.size() * 2), dy2(x.size() * 2);
  da.upload(a);
  db.upload(b);
  dx.upload(x);
  BEAM_REQUIRE(c, beam_parallel_gemmrc_silu(da.p, db.p, dc.p, M, N, K, dx.p, dy.p, count, BEAM_F16, nullptr, nullptr));
  BEAM_REQUIRE(c, beam_gemmrc(da.p, db.p, dc2.p, M, N, K, BEAM_F16, nullptr, nullptr));
  BEAM_REQUIRE(c, beam_silu(dx.p, dy2.p, count, BEAM_F16, nullptr));
  if (dc.download16() != dc2.download16()) c.fail("C differs from the plain GEMM");
  std::vector<uint16_t> y = dy.download16();
  if (y != dy2.download16()) c.fail("Y differs from the standalone SiLU");
  if ((y[0] & 0x7fff) != 0 || y[1] != x[1] || y[count - 1] != x[count - 1]) c.fail("closed forms of silu");
  return c;
}

// LayerNorm invariants: gamma = 1, beta = 0 gives rows of mean 0 and variance 1; x = 0 gives beta.
BEAM_TEST(layernorm_invariants) {
  Check c;
  const int M = 192, N = 2048, K = 256;
  std::vector<uint16_t> a = normal16((size_t)M * K, BEAM_F16, 7, 0, 0.0f, 1.0f / 16),
                        b = normal16((size_t)N * K, BEAM_F16, 7, 1, 0.0f, 1.0f / 16);
  std::vector<uint16_t> ones(N, small_to_16(1.0f, BEAM_F16)), zeros(N, 0);
  std::vector<uint16_t> beta = normal16(N, BEAM_F16, 7, 3, 0.0f, 0.1f);
  DevBuf da(a.size() * 2), db(b.size() * 2), dy((size_t)M * N * 2), dg(N * 2), dbt(N * 2),
      dw(beam_gemmrc_ln_workspace_bytes(M, N, nullptr));
  da.upload(a);
  db.upload(b);
  dg.upload(ones);
  dbt.upload(zeros);
  BEAM_REQUIRE(c, beam_gemmrc_ln(da.p, db.p, dg.p, dbt.p, 1e-5f, dy.p, M, N, K, BEAM_F16, nullptr, dw.p, dw.bytes, nullptr));
  std::vector<uint16_t> y = dy.download16();
  for (int m = 0; m < M; ++m) {
    double s = 0, q = 0;
    for (int n = 0; n < N; ++n) s += half_to_float(y[(size_t)m * N + n]);
    s /= N;
    for (int n = 0; n < N; ++n) q += std::pow(half_to_float(y[(size_t)m * N + n]) - s, 2);
    q /= N;
    if (std::fabs(s) > 2e-3 || std::fabs(q - 1.0) > 5e-3) {
      c.fail("row " + std::to_string(m) + ": mean " + std::to_string(s) + " var " + std::to_string(q));
      break;
    }
  }
  std::vector<uint16_t> za(a.size(), 0);
  da.upload(za);
  dbt.upload(beta);
  BEAM_REQUIRE(c, beam_gemmrc_ln(da.p, db.p, dg.p, dbt.p, 1e-5f, dy.p, M, N, K, BEAM_F16, nullptr, dw.p, dw.bytes, nullptr));
  y = dy.download16();
  for (int m = 0; m < M && c.ok; ++m)
    for (int n = 0; n < N; ++n)
      if (y[(size_t)m * N + n] != beta[n] && half_to_float(y[(size_t)m * N + n]) != half_to_float(beta[n])) {
        c.fail("x = 0 must give y = beta");
        break;
      }
  return c;
}

// Unsupported requests come back as error codes; nothing is written silently.
BEAM_TEST(error_paths) {
  Check c;
  DevBuf da(64 * 64 * 2), db(64 * 64 * 2), dc(64 * 64 * 2);
  beam_tile_cfg bad = {96, 96, 48, 48, 0, 0};
  if (beam_gemmrc(da.p, db.p, dc.p, 64, 64, 64, BEAM_F16, &bad, nullptr) != BEAM_ERR_UNSUPPORTED) c.fail("bad tile accepted");
  if (beam_gemmrc(da.p, db.p, dc.p, 64, 64, 60, BEAM_F16, nullptr, nullptr) != BEAM_OK) c.fail("K % 8 != 0 refused (the plain kernel takes it)");
  if (beam_gemmrc((char*)da.p + 1, db.p, dc.p, 64, 64, 56, BEAM_F16, nullptr, nullptr) != BEAM_ERR_INVALID) c.fail("odd address accepted");
  if (beam_gemmrc(da.p, db.p, dc.p, 64, 64, 64, 9, nullptr, nullptr) != BEAM_ERR_UNSUPPORTED) c.fail("bad dtype accepted");
  if (beam_gemmrc(nullptr, db.p, dc.p, 64, 64, 64, BEAM_F16, nullptr, nullptr) != BEAM_ERR_INVALID) c.fail("null A accepted");
  beam_tile_cfg small = {64, 64, 32, 32, 0, 0};
  DevBuf da2(64 * 512 * 2), db2(64 * 512 * 2);
  if (beam_gemmrc_splitk(da2.p, db2.p, dc.p, 64, 64, 512, BEAM_F16, &small, 4, nullptr, 0, nullptr) != BEAM_ERR_WORKSPACE)
    c.fail("missing workspace accepted");
  return c;
}

// ---- CLI -----------------------------------------------------------------------------------------

struct Args {
  std::map<std::string, std::string> kv;
  bool has(const std::string& k) const { return kv.count(k) != 0; }
  std::string str(const std::string& k, const std::string& d) const { return has(k) ? kv.at(k) : d; }
  int num(const std::string& k, int d) const { return has(k) ? std::atoi(kv.at(k).c_str()) : d; }
};

bool parse_pair(const std::string& s, int* a, int* b) { return std::sscanf(s.c_str(), "%dx%d", a, b) == 2; }

int run_tests(const std::string& which) {
  int failed = 0, ran = 0;
  for (auto& kv : registry()) {
    if (which != "all" && which != kv.first) continue;
    ++ran;
    Check r = kv.second();
    std::printf("[%s] %s%s%s\n", r.ok ? " OK " : "FAIL", kv.first.c_str(), r.ok ? "" : ": ", r.why.c_str());
    std::fflush(stdout);
    failed += r.ok ? 0 : 1;
  }
  if (ran == 0) {
    std::fprintf(stderr, "no test named '%s' (try --list)\n", which.c_str());
    return 2;
  }
  std::printf("%d test(s), %d failed\n", ran, failed);
  return failed ? 1 : 0;
}

struct Problem {
  int M, N, K, dtype;
  DevBuf a, b, c, gamma, beta;
  // zeros: A and B all zero instead of N(0,1)/sqrt(K).  The matrix cores draw far less power on zeros, so the
  // same kernel then runs at the full clock: the pair of timings separates what the schedule costs from
  // what the power cap costs.
  Problem(int m, int n, int k, int d, const std::string& data = "normal")
      : M(m), N(n), K(k), dtype(d), a((size_t)m * k * 2), b((size_t)n * k * 2), c((size_t)m * n * 2), gamma((size_t)n * 2),
        beta((size_t)n * 2) {
    if (data == "uniform") {
      a.upload(uniform16((size_t)m * k, d, 7, 0));
      b.upload(uniform16((size_t)n * k, d, 7, 1));
    } else {
      const float scale = data == "zeros" ? 0.0f : 1.0f / std::sqrt((float)k);
      a.upload(normal16((size_t)m * k, d, 7, 0, 0.0f, scale));
      b.upload(normal16((size_t)n * k, d, 7, 1, 0.0f, scale));
    }
    gamma.upload(normal16(n, d, 7, 2, 1.0f, 0.1f));
    beta.upload(normal16(n, d, 7, 3, 0.0f, 0.1f));
  }
};

int time_op(int op, Problem& p, const beam_tile_cfg* cfg, int split_k, int warmup, int iters, float* ms, int ln_mode = 0) {
  beam_problem q;
  std::memset(&q, 0, sizeof q);
  q.A = p.a.p;
  q.B = p.b.p;
  q.C = p.c.p;
  q.gamma = p.gamma.p;
  q.beta = p.beta.p;
  q.eps = 1e-5f;
  q.M = p.M;
  q.N = p.N;
  q.K = p.K;
  q.dtype = p.dtype;
  q.split_k = split_k;
  q.ln_mode = ln_mode;
  size_t need = 0;
  if (op == BEAM_OP_SPLITK || op == BEAM_OP_PROBE_SPLITK_LOADS) {
    const int s = beam_splitk_effective(p.M, p.N, p.K, cfg, split_k);
    if (s < 0) return BEAM_ERR_UNSUPPORTED;
    need = beam_splitk_workspace_bytes(p.M, p.N, s);
  } else if (op == BEAM_OP_GEMM_LN) {
    need = beam_gemmrc_ln_workspace_bytes_for(p.M, p.N, p.K, cfg, ln_mode);
  }
  DevBuf ws(need ? need : 256);
  q.ws = ws.p;
  q.ws_bytes = ws.bytes;
  return beam_bench(op, &q, cfg, warmup, iters, nullptr, ms);
}

// GEMM alone, SiLU alone and the GEMM carrying the SiLU, interleaved over several rounds.
int cli_bench_silu(const Args& a, Problem& p, const beam_tile_cfg& cfg) {
  const long long count = a.has("count") ? std::atoll(a.str("count", "0").c_str()) : (long long)p.M * p.N;
  DevBuf x((size_t)count * 2 + 16), y((size_t)count * 2 + 16);
  x.upload(normal16((size_t)count, p.dtype, 7, 4, 0.0f, 2.0f));
  beam_problem q;
  std::memset(&q, 0, sizeof q);
  q.A = p.a.p;
  q.B = p.b.p;
  q.C = p.c.p;
  q.M = p.M;
  q.N = p.N;
  q.K = p.K;
  q.dtype = p.dtype;
  q.side_x = x.p;
  q.side_y = y.p;
  q.side_count = count;
  const int warmup = a.num("warmup", 50), iters = a.num("iters", 100);
  float gemm = 0, silu = 0, pair = 0;
  for (int round = 0; round < 3; ++round) {
    if (beam_bench(BEAM_OP_GEMM, &q, &cfg, warmup, iters, nullptr, &gemm) ||
        beam_bench(BEAM_OP_SILU, &q, &cfg, warmup, iters, nullptr, &silu) ||
        beam_bench(BEAM_OP_GEMM_SILU, &q, &cfg, warmup, iters, nullptr, &pair)) {
      std::fprintf(stderr, "bench failed: %s\n", beam_last_error());
      return 1;
    }
  }
  std::printf("silu %dx%dx%d %s tile %dx%d wave %dx%d pipeline %d, %lld elements: gemm %.1f us, silu alone %.1f us "
              "(%.0f GB/s), gemm+silu in one launch %.1f us = %.3f of the two launches, %.1f TFLOP/s\n",
              p.M, p.N, p.K, p.dtype ? "bf16" : "fp16", cfg.block_m, cfg.block_n, cfg.wave_m, cfg.wave_n, cfg.pipeline,
              count, gemm * 1e3, silu * 1e3, 4.0 * count / silu / 1e6, pair * 1e3, pair / (gemm + silu),
              2.0 * p.M * p.N * p.K / pair / 1e9);
  return 0;
}

// The register-only matrix-core loop (beam_probe_mfma): launches of about 0.7 ms, like the 8192^3 kernel.
int cli_probe_mfma(const Args& a) {
  const int dtype = a.str("dtype", "fp16") == "bf16" ? BEAM_BF16 : BEAM_F16;
  const std::string shape = a.str("mfma", "16x16x32"), data = a.str("data", "normal");
  if ((shape != "16x16x32" && shape != "32x32x16") || (data != "normal" && data != "zeros")) {
    std::fprintf(stderr, "--mfma 16x16x32|32x32x16, --data normal|zeros\n");
    return 2;
  }
  const int mfma = shape == "32x32x16" ? BEAM_MFMA_32X32X16 : BEAM_MFMA_16X16X32;
  const int kind = data == "zeros" ? BEAM_PROBE_DATA_ZEROS : BEAM_PROBE_DATA_NORMAL;
  const double seconds = std::atof(a.str("seconds", "0").c_str());
  // (a launch of 1600 passes takes about a millisecond: with --seconds, one line per second or so)
  const int passes = a.num("passes", 1600), iters = a.num("iters", seconds > 0 ? 1000 : 200);
  int warmup = a.num("warmup", 100);
  double spent = 0.0;
  do {
    float ms = 0;
    double flop = 0;
    if (beam_probe_mfma(dtype, mfma, kind, passes, warmup, iters, nullptr, &ms, &flop) != BEAM_OK) {
      std::fprintf(stderr, "probe failed: %s\n", beam_last_error());
      return 1;
    }
    std::printf("probe-mfma %s v_mfma_f32_%s %s operands, %d passes of 1024 matrix-core cycles per wavefront: %.4f ms per launch  "
                "%.1f TFLOP/s = %.3f of 2500\n", dtype ? "bf16" : "fp16", shape.c_str(), data.c_str(), passes, ms, flop / ms / 1e9,
                flop / ms / 1e9 / 2500.0);
    std::fflush(stdout);
    spent += (double)ms * 1e-3 * (warmup + iters);
    warmup = 0;
  } while (spent < seconds);
  return 0;
}

int cli_bench(const Args& a) {
  const int M = a.num("m", 8192), N = a.num("n", 8192), K = a.num("k", 8192);
  const int dtype = a.str("dtype", "fp16") == "bf16" ? BEAM_BF16 : BEAM_F16;
  const std::string opname = a.str("op", "gemm");
  if (opname == "probe-mfma") return cli_probe_mfma(a);
  const int op = opname == "splitk" ? (int)BEAM_OP_SPLITK
                 : opname == "ln"   ? (int)BEAM_OP_GEMM_LN
                 : opname == "nn"   ? (int)BEAM_OP_MATMUL_NN  // B read as [K][N]
                 // what the machine allows: empty launches, and a split-K launch with nothing but its loads
                 : opname == "probe-empty"        ? (int)BEAM_OP_PROBE_EMPTY
                 : opname == "probe-empty-pair"   ? (int)BEAM_OP_PROBE_EMPTY_PAIR
                 : opname == "probe-splitk-loads" ? (int)BEAM_OP_PROBE_SPLITK_LOADS
                                                  : (int)BEAM_OP_GEMM;
  const bool splitk_like = op == BEAM_OP_SPLITK || op == BEAM_OP_PROBE_SPLITK_LOADS;
  beam_tile_cfg cfg;
  int split = 1;
  if (beam_default_config(M, N, K, &cfg, splitk_like ? &split : nullptr) != BEAM_OK) return 2;
  if (a.has("tile") && !parse_pair(a.str("tile", ""), &cfg.block_m, &cfg.block_n)) return 2;
  if (a.has("wave") && !parse_pair(a.str("wave", ""), &cfg.wave_m, &cfg.wave_n)) return 2;
  cfg.pipeline = a.num("pipeline", cfg.pipeline);
  cfg.group_m = a.num("group", cfg.group_m);
  split = a.num("splitk", splitk_like ? 0 : split);
  Problem p(M, N, K, dtype, a.str("data", "normal"));
  if (op == BEAM_OP_MATMUL_NN && cfg.pipeline == 2) cfg.pipeline = 0;
  if (opname == "silu") {
    if (cfg.pipeline == 2) cfg.pipeline = 0;
    return cli_bench_silu(a, p, cfg);
  }
  float ms = 0;
  const std::string lnm = a.str("ln-mode", "auto");  // --op ln: auto | twopass | fused
  const int ln_mode = lnm == "twopass" ? BEAM_LN_TWOPASS : lnm == "fused" ? BEAM_LN_FUSED : BEAM_LN_AUTO;
  // GEMM+LayerNorm without a tile on the command line: the library's own choice for that operator (a cost model
  // of its own, not the plain GEMM's tile); the line below then names what it picked for a device of 256 CUs.
  const bool ln_auto_tile = op == BEAM_OP_GEMM_LN && !a.has("tile") && !a.has("wave") && !a.has("pipeline") && !a.has("group");
  if (ln_auto_tile && ln_mode != BEAM_LN_TWOPASS) {
    beam_tile_cfg picked;
    if (beam_dbg_ln_default_config(M, N, K, 256, &picked) == BEAM_OK) cfg = picked;
  }
  int rc = time_op(op, p, ln_auto_tile ? nullptr : &cfg, split, a.num("warmup", 5), a.num("iters", 20), &ms, ln_mode);
  if (rc != BEAM_OK) {
    std::fprintf(stderr, "bench failed (%d): %s\n", rc, beam_last_error());
    return 1;
  }
  std::printf("%s %dx%dx%d %s tile %dx%d wave %dx%d pipeline %d group %d split %d: %.4f ms  %.1f TFLOP/s\n",
              opname.c_str(), M, N, K, dtype ? "bf16" : "fp16", cfg.block_m, cfg.block_n, cfg.wave_m, cfg.wave_n,
              cfg.pipeline, cfg.group_m, split, ms, 2.0 * M * N * K / ms / 1e9);
  return 0;
}

int cli_tune(const Args& a) {
  const int M = a.num("m", 4096), N = a.num("n", 4096), K = a.num("k", 4096);
  const int dtype = a.str("dtype", "fp16") == "bf16" ? BEAM_BF16 : BEAM_F16;
  Problem p(M, N, K, dtype);
  double best = 1e30;
  std::string best_name;
  for (int i = 0; i < beam_num_configs(); ++i) {
    beam_tile_cfg cfg;
    beam_get_config(i, &cfg);
    for (int split : {1, 4, 8, 16, 32, 64}) {
      if (split > 1 && cfg.block_m * cfg.block_n > 128 * 128) continue;
      float ms = 0;
      int rc = time_op(split > 1 ? BEAM_OP_SPLITK : BEAM_OP_GEMM, p, &cfg, split, 3, 10, &ms);
      if (rc != BEAM_OK) continue;
      char name[128];
      std::snprintf(name, sizeof name, "tile %dx%d wave %dx%d split %d", cfg.block_m, cfg.block_n, cfg.wave_m, cfg.wave_n, split);
      std::printf("  %-40s %9.4f ms %8.1f TFLOP/s\n", name, ms, 2.0 * M * N * K / ms / 1e9);
      if (ms < best) {
        best = ms;
        best_name = name;
      }
    }
  }
  std::printf("best for %dx%dx%d %s: %s (%.4f ms, %.1f TFLOP/s)\n", M, N, K, dtype ? "bf16" : "fp16", best_name.c_str(),
              best, 2.0 * M * N * K / best / 1e9);
  return 0;
}

}  // namespace

int main(int argc, char** argv) {
  Args a;
  for (int i = 1; i < argc; ++i) {
    std::string k = argv[i];
    if (k.rfind("--", 0) != 0) {
      std::fprintf(stderr, "unexpected argument '%s'\n", argv[i]);
      return 2;
    }
    k = k.substr(2);
    if (i + 1 < argc && std::strncmp(argv[i + 1], "--", 2) != 0) a.kv[k] = argv[++i];
    else a.kv[k] = "";
  }
  if (a.has("list")) {
    for (auto& kv : registry()) std::printf("%s\n", kv.first.c_str());
    return 0;
  }
  if (a.kv.empty() || a.has("help")) {
    std::printf("usage: beam_host --list | --info | --run all|<test> | --bench [...] | --tune [...] | --copy MiB\n");
    return a.kv.empty() ? 2 : 0;
  }
  char name[256];
  int cus = 0, khz = 0;
  size_t mem = 0;
  int rc = beam_device_info(name, sizeof name, &cus, &khz, &mem);
  if (rc != BEAM_OK) {
    std::fprintf(stderr, "no usable device: %s\n", beam_last_error());
    return 3;
  }
  if (a.has("info")) {
    std::printf("device %s, %d CUs, %.0f MHz, %.1f GiB, %d tile configurations\n", name, cus, khz / 1e3,
                mem / 1073741824.0, beam_num_configs());
    return 0;
  }
  if (a.has("run")) return run_tests(a.str("run", "all").empty() ? "all" : a.str("run", "all"));
  if (a.has("bench")) return cli_bench(a);
  if (a.has("tune")) return cli_tune(a);
  if (a.has("copy")) {
    const size_t bytes = (size_t)a.num("copy", 256) << 20;
    DevBuf src(bytes), dst(bytes);
    beam_memset(src.p, 1, bytes);
    for (int i = 0; i < 5; ++i)
      if (beam_memcpy_d2d(dst.p, src.p, bytes) != BEAM_OK) return 1;
    beam_sync(nullptr);
    std::printf("copied %zu MiB device to device, 5 times\n", bytes >> 20);
    return 0;
  }
  std::fprintf(stderr, "nothing to do (try --help)\n");
  return 2;
}
