// C ABI of libbeam_hip.so (declarations and reference citations: include/beam_hip.h).
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <atomic>
#include <chrono>
#include <cstdlib>
#include <mutex>
#include <set>
#include <string>
#include <thread>
#include <vector>

#include <unistd.h>

#include "../../include/beam_hip_debug.h"
#include "aux_kernels.h"
#include "kernel_set.h"
#include "tile_map.h"

using namespace beam;

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof g_err, fmt, ap);
  va_end(ap);
  return code;
}

int hip_fail(hipError_t e, const char* what) {
  return fail(BEAM_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
}

#define BEAM_HIP(call)                                  \
  do {                                                  \
    hipError_t e_ = (call);                             \
    if (e_ != hipSuccess) return hip_fail(e_, #call);   \
  } while (0)

struct Device {
  int status = -1;  // -1 = not probed
  char name[256] = "";
  int cus = 0;
  int clock_khz = 0;
  size_t mem = 0;
};
Device g_dev;
std::mutex g_dev_mu;
// Polls before a waiting thread gives up: of statistics slots in the fused LayerNorm (3-4 us each once the pauses
// between tries have grown: about 60 ms), of a tile's flags in the one-launch split-K (about 1 us each).  What a
// workgroup legitimately waits for is resident with it and at most a tile's K loop behind, so the bound is there
// for a device that other work keeps occupied: giving up then costs milliseconds, and the caller's retry as two
// passes (beam_gemmrc_ln_checked) gives the result.
std::atomic<int> g_ln_spin_limit{16384};
// Nonces of fused GEMM+LayerNorm and one-launch split-K launches: consecutive numbers from a start that differs from process to process
// (memory recycled from another process of this library then holds tags of another sequence).
std::atomic<unsigned> g_ln_nonce{(unsigned)std::chrono::steady_clock::now().time_since_epoch().count() * 2654435761u ^
                                 (unsigned)getpid() * 40503u};

// Split-K workspace of beam_gemmrc_splitk_noalloc: device memory that exists from the moment the library's
// code is loaded on a GPU until the process ends, so the entry point never allocates.  In host code the
// array's name is only a handle for hipGetSymbolAddress; what kernels and copies get is the per-device
// address looked up below (every GPU has its own copy at its own address).
constexpr size_t kScratchPartialBytes = (size_t)16 << 20;                      // the partial sums a call may need
constexpr size_t kScratchBytes = kScratchPartialBytes + ((size_t)256 << 10);  // ... + synchronisation words of the one-launch form
constexpr int kMaxDevices = 64;
void* g_scratch_ptr[kMaxDevices] = {};
std::mutex g_scratch_mu;

}  // namespace

static __device__ __align__(256) unsigned char scratch[kScratchBytes];

namespace {

// Address of `scratch` on the current device (looked up once per device, with that device current).
int scratch_on_current_device(void** out) {
  int dev = -1;
  BEAM_HIP(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices) return fail(BEAM_ERR_UNSUPPORTED, "device index %d beyond %d", dev, kMaxDevices - 1);
  std::lock_guard<std::mutex> lk(g_scratch_mu);
  if (!g_scratch_ptr[dev]) {
    void* ptr = nullptr;
    BEAM_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    if (!ptr) return fail(BEAM_ERR_HIP, "hipGetSymbolAddress returned a null address for the scratch array");
    g_scratch_ptr[dev] = ptr;
  }
  *out = g_scratch_ptr[dev];
  return BEAM_OK;
}

const std::vector<KernelSet>& kernel_sets() {
  static const std::vector<KernelSet> sets = [] {
    std::vector<KernelSet> v;
#define BEAM_PUSH(BM, BN, TM, TN) v.push_back(kernel_set_##BM##x##BN##_##TM##x##TN());
    BEAM_FOR_EACH_SET(BEAM_PUSH)
#undef BEAM_PUSH
    return v;
  }();
  return sets;
}

const KernelSet* find_set(const beam_tile_cfg& c) {
  for (const KernelSet& k : kernel_sets())
    if (k.block_m == c.block_m && k.block_n == c.block_n && k.wave_m == c.wave_m && k.wave_n == c.wave_n)
      return &k;
  return nullptr;
}

// Raster group height (tile rows that share one sweep over the columns): measured best is 4 for the
// tiles that run one workgroup per CU (8192^3: +1.7% over 8; 16384 x 16384 x 2048: +28%) and 8 for the
// smaller ones, which run two or more per CU.
constexpr int default_group_m(int block_m, int block_n) { return block_m * block_n >= 256 * 128 ? 4 : 8; }
// Largest K: the buffer descriptor of a 256-row operand tile, (255 * K + K) * 2 bytes, must stay below the
// out-of-range offset the kernels use for masked chunks (kOobOffset).
constexpr int kMaxK = (int)((kOobOffset / 512u) & ~7u) - 8;
static_assert((unsigned long long)kMaxK * 512ull < kOobOffset && kMaxK % 8 == 0, "descriptor range");

// Elements of a side-job array: its byte size must stay below the out-of-range offset the kernels use.
constexpr long long kMaxSideElems = (long long)(kOobOffset / 16) * 8;

// Validates a gemmrc problem.  *generic is set when it is well formed but outside what the tiled kernels take
// (rows of A / B that are not multiples of 16 bytes, i.e. K % 8 != 0; operands not 16-byte or output not
// 8-byte aligned; K beyond the descriptor range): such problems run on the plain kernel of aux_kernels.hip.
int check_problem(const void* A, const void* B, const void* C, int M, int N, int K, int dtype, bool* generic) {
  *generic = false;
  if (M < 0 || N < 0 || K < 0) return fail(BEAM_ERR_INVALID, "negative dimension (M=%d N=%d K=%d)", M, N, K);
  if (dtype != BEAM_F16 && dtype != BEAM_BF16) return fail(BEAM_ERR_UNSUPPORTED, "dtype %d: only fp16 (0) and bf16 (1)", dtype);
  if (M == 0 || N == 0) return BEAM_OK;
  if (!C) return fail(BEAM_ERR_INVALID, "null output pointer");
  if (K > 0 && (!A || !B)) return fail(BEAM_ERR_INVALID, "null input pointer");
  if (((uintptr_t)A | (uintptr_t)B | (uintptr_t)C) & 1) return fail(BEAM_ERR_INVALID, "A, B and C must be aligned to their 16-bit elements");
  if ((size_t)M * (size_t)N >= ((size_t)1 << 40)) return fail(BEAM_ERR_UNSUPPORTED, "M*N too large");
  if ((M + 63) / 64 > 65535) return fail(BEAM_ERR_UNSUPPORTED, "M=%d too large", M);
  *generic = K > kMaxK || K % 8 != 0 || ((((uintptr_t)A | (uintptr_t)B) & 15) != 0) || (((uintptr_t)C & 7) != 0);
  return BEAM_OK;
}

// Slices for `tiles` output tiles when the caller leaves the choice to the library: as many as make
// one full round of workgroups (tiles * slices = CUs), at least 4 K tiles each.  Measured at
// 256 x 256 x 32768: 16 tiles x 16 slices 15.1 us, x 24 (one and a half rounds, what the reference's
// rule gives: beam_slice_heuristic) 19.8 us, x 32 17.6 us; 8 tiles x 32 slices 14.2 us, x 16 17.0 us.
int auto_slices(long tiles, int K, int cus) {
  if (tiles * 2 > cus) return 1;
  const int ktiles = (K + kBK - 1) / kBK;
  long s = cus / (tiles < 1 ? 1 : tiles);
  if (s > ktiles / 4) s = ktiles / 4;
  if (s > 64) s = 64;  // the reduction reads every slice: 64 x 64 x 32768 takes 9.1 us with 64 slices, 11.4 with 128
  // Half a round of workgroups with 16 K tiles each beats a full round of shorter slices (every slice pays its
  // pipeline fill and adds M x N partial sums): 128 x 128 x 32768 takes 8.5 us in 32 slices, 9.6 in 64;
  // 128 x 256 x 8192 7.8 us in 16, 7.9 in 32.
  const long half_round = (cus / 2 + tiles - 1) / (tiles < 1 ? 1 : tiles);
  const long want = ktiles / 16 > half_round ? ktiles / 16 : half_round;
  if (s > want) s = want;
  return s < 1 ? 1 : (int)s;
}

int choose_default(int M, int N, int K, int split_req, beam_tile_cfg* cfg, int* split_k);

// split_req: -1 the caller cannot run K slices (no workspace); 0 it can, and leaves the number to
// the library; > 0 it asks for that many.  The default tile is chosen for that situation.
// w4_ok: the caller has a form of the 4-wavefront kernel (gemm_w4.h); for the others the library's own choice
// of that tile means the 8-wavefront 256 x 256 tile.
int resolve_cfg(const beam_tile_cfg* in, int M, int N, int K, beam_tile_cfg* out, const KernelSet** ks,
                int split_req = -1, bool w4_ok = false) {
  if (in) {
    *out = *in;
  } else {
    int s;
    int rc = choose_default(M, N, K, split_req, out, &s);
    if (rc) return rc;
    if (!w4_ok && out->block_m == 256 && out->block_n == 256 && out->wave_m == 128 && out->wave_n == 128) out->wave_n = 64;
  }
  if (out->pipeline < 0 || out->pipeline > 2) return fail(BEAM_ERR_UNSUPPORTED, "pipeline %d: 0 (3 A + 2 B LDS slots), 1 (2 + 2) or 2 (deep)", out->pipeline);
  if (out->group_m <= 0) out->group_m = default_group_m(out->block_m, out->block_n);
  *ks = find_set(*out);
  if (!*ks)
    return fail(BEAM_ERR_UNSUPPORTED, "no kernel for workgroup tile %dx%d / wavefront tile %dx%d", out->block_m,
                out->block_n, out->wave_m, out->wave_n);
  return BEAM_OK;
}

GemmParams base_params(const void* A, const void* B, int M, int N, int K, const beam_tile_cfg& c) {
  GemmParams p;
  std::memset(&p, 0, sizeof p);
  p.A = A;
  p.B = B;
  p.M = M;
  p.N = N;
  p.K = K;
  p.tiles_m = (M + c.block_m - 1) / c.block_m;
  p.tiles_n = (N + c.block_n - 1) / c.block_n;
  p.k_slice = ((K + kBK - 1) / kBK) * kBK;
  if (p.k_slice == 0) p.k_slice = kBK;
  p.splits = 1;
  p.group_m = c.group_m;
  p.divs = make_tile_divs(p.tiles_m, p.tiles_n, p.group_m);
  return p;
}

size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

// ---- host data generation -------------------------------------------------------------

inline uint64_t mix64(uint64_t x) {  // splitmix64 finaliser
  x += 0x9E3779B97F4A7C15ull;
  x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
  x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
  return x ^ (x >> 31);
}

inline uint64_t draw(uint64_t seed, uint64_t tensor_id, uint64_t i) {
  return mix64(mix64(seed + 0x632BE59BD9B4E019ull * (tensor_id + 1)) + i);
}

inline uint32_t f32_bits(float f) {
  uint32_t u;
  std::memcpy(&u, &f, 4);
  return u;
}

inline uint16_t to_bf16_bits(float f) {
  uint32_t x = f32_bits(f);
  if ((x & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((x >> 16) | 0x40u);
  return (uint16_t)((x + 0x7fffu + ((x >> 16) & 1u)) >> 16);
}

inline uint16_t to_f16_bits(float f) {
  // Round the significand to 11 bits in float arithmetic, then repack.
  const uint32_t x = f32_bits(f);
  const uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
  const uint32_t ax = x & 0x7fffffffu;
  if (ax > 0x7f800000u) return (uint16_t)(sign | 0x7e00u);
  if (ax >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);
  float a;
  std::memcpy(&a, &ax, 4);
  if (ax < 0x38800000u) {
    // subnormal half: a / 2^-24 rounded to nearest even integer
    const float scaled = a * 16777216.0f;
    const float r = std::nearbyintf(scaled);  // default rounding mode = to nearest even
    return (uint16_t)(sign | (uint16_t)r);
  }
  uint32_t r = ax + 0xfffu + ((ax >> 13) & 1u);  // RN-even at bit 13
  return (uint16_t)(sign | ((r - 0x38000000u) >> 13));
}

template <typename F>
void parallel_for(size_t n, F f) {
  unsigned hw = std::thread::hardware_concurrency();
  unsigned nt = hw == 0 ? 4 : (hw > 16 ? 16 : hw);
  if (n < (1u << 16)) nt = 1;
  std::vector<std::thread> th;
  const size_t chunk = (n + nt - 1) / nt;
  for (unsigned t = 0; t < nt; ++t) {
    const size_t lo = t * chunk, hi = lo + chunk < n ? lo + chunk : n;
    if (lo >= hi) break;
    th.emplace_back([=] { f(lo, hi); });
  }
  for (auto& t : th) t.join();
}

}  // namespace

extern "C" {

const char* beam_last_error(void) { return g_err; }

int beam_init(void) {
  std::lock_guard<std::mutex> lk(g_dev_mu);
  if (g_dev.status >= 0) return g_dev.status == BEAM_OK ? BEAM_OK : fail(g_dev.status, "device probe failed earlier");
  int n = 0;
  hipError_t e = hipGetDeviceCount(&n);
  if (e != hipSuccess || n == 0) {
    g_dev.status = BEAM_ERR_HIP;
    return fail(BEAM_ERR_HIP, "no HIP device (%s)", e == hipSuccess ? "count is zero" : hipGetErrorString(e));
  }
  hipDeviceProp_t prop;
  e = hipGetDeviceProperties(&prop, 0);
  if (e != hipSuccess) {
    g_dev.status = BEAM_ERR_HIP;
    return hip_fail(e, "hipGetDeviceProperties");
  }
  std::snprintf(g_dev.name, sizeof g_dev.name, "%s (%s)", prop.name, prop.gcnArchName);
  g_dev.cus = prop.multiProcessorCount;
  g_dev.clock_khz = prop.clockRate;
  g_dev.mem = prop.totalGlobalMem;
  if (std::strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
    g_dev.status = BEAM_ERR_DEVICE;
    return fail(BEAM_ERR_DEVICE, "device 0 is %s; this library holds gfx950 code only", prop.gcnArchName);
  }
  g_dev.status = BEAM_OK;
  void* ignored;
  return scratch_on_current_device(&ignored);  // the no-allocation entry point's memory, looked up at set-up
}

int beam_device_info(char* name, int len, int* compute_units, int* clock_khz, size_t* mem_bytes) {
  int rc = beam_init();
  if (rc != BEAM_OK && rc != BEAM_ERR_DEVICE) return rc;
  if (name && len > 0) std::snprintf(name, (size_t)len, "%s", g_dev.name);
  if (compute_units) *compute_units = g_dev.cus;
  if (clock_khz) *clock_khz = g_dev.clock_khz;
  if (mem_bytes) *mem_bytes = g_dev.mem;
  return rc;
}

int beam_num_configs(void) { return (int)kernel_sets().size(); }

int beam_get_config(int index, beam_tile_cfg* out) {
  if (!out || index < 0 || index >= beam_num_configs()) return fail(BEAM_ERR_INVALID, "config index %d out of range", index);
  const KernelSet& k = kernel_sets()[index];
  out->block_m = k.block_m;
  out->block_n = k.block_n;
  out->wave_m = k.wave_m;
  out->wave_n = k.wave_n;
  out->pipeline = 0;
  out->group_m = default_group_m(out->block_m, out->block_n);
  return BEAM_OK;
}

int beam_slice_heuristic(int tiles, int compute_units) {
  if (tiles < 1) tiles = 1;
  const float units = (float)compute_units;
  int s = 1;
  if ((float)tiles < units) {
    s = (int)((units - 1.0f) / (float)tiles + 1.0f);
    float waves = (float)s * (float)tiles / units;
    float rem = waves - (float)(int)waves;
    while (rem < 0.5f) {
      ++s;
      waves = (float)s * (float)tiles / units;
      rem = waves - (float)(int)waves;
    }
  }
  return s;
}

int beam_default_config(int M, int N, int K, beam_tile_cfg* cfg, int* split_k) {
  return choose_default(M, N, K, split_k ? 0 : -1, cfg, split_k);
}

}  // extern "C"

namespace {

int choose_default(int M, int N, int K, int split_req, beam_tile_cfg* cfg, int* split_k) {
  if (!cfg) return fail(BEAM_ERR_INVALID, "null cfg");
  const int cus = g_dev.cus > 0 ? g_dev.cus : 256;
  auto tiles = [&](int bm, int bn) { return (long)((M + bm - 1) / bm) * ((N + bn - 1) / bn); };
  // A small cost model picks the tile: every CU works through ceil(tiles / CUs) workgroups, `occ` of
  // them at a time (what LDS allows); a workgroup costs a fixed start-up / epilogue time plus its flops
  // at the per-CU rate of its tile shape, which is higher when several workgroups share the CU.  The
  // rates (TFLOP/s per CU, alone / with a full CU) and fixed costs (us) are fits to timings of all
  // compiled tiles on 39 shapes from 512^3 to 8192^3 (square, skinny and short-K) on an MI355X:
  // the pick is within 0.8% of the best tile on average, 6.7% at worst (tile-count thresholds:
  // 6% and 76%).  The 224- and 192-row tiles are there for what 256 rows divide badly: 3072^3 is
  // 0.75 of a round of 192 x 256 tiles against 0.56 of a round of 256 x 256 ones (49.5 against
  // 58.6 us), 7168^3 is 3.5 rounds of 224 x 256 tiles against 3.06 (546 against 613 us).
  struct Candidate {
    beam_tile_cfg cfg;
    int occ;
    double alone, full, fixed;
  };
  static const Candidate kCandidates[] = {
      {{256, 256, 128, 64, 0, default_group_m(256, 256)}, 1, 6.04, 6.04, 8.0},
      {{224, 256, 112, 64, 0, default_group_m(224, 256)}, 1, 5.95, 5.95, 8.0},
      {{192, 256, 96, 64, 0, default_group_m(192, 256)}, 1, 5.22, 5.22, 8.0},
      {{256, 128, 64, 64, 0, default_group_m(256, 128)}, 1, 4.99, 4.99, 6.0},
      {{128, 256, 64, 64, 0, default_group_m(128, 256)}, 1, 4.8, 4.8, 6.0},
      {{128, 128, 64, 64, 0, default_group_m(128, 128)}, 2, 3.8, 4.4, 3.42},
      {{128, 128, 64, 32, 2, default_group_m(128, 128)}, 1, 4.05, 4.05, 4.0},
      {{128, 64, 64, 32, 0, default_group_m(128, 64)}, 2, 2.6, 3.4, 3.5},
      {{128, 64, 64, 32, 2, default_group_m(128, 64)}, 1, 3.2, 3.2, 4.2},
      {{64, 64, 32, 32, 0, default_group_m(64, 64)}, 4, 1.87, 2.9, 2.7},
      {{64, 64, 32, 32, 2, default_group_m(64, 64)}, 1, 2.4, 2.4, 4.0},
      {{64, 128, 32, 64, 0, default_group_m(64, 128)}, 2, 3.15, 3.4, 3.5},
      {{64, 128, 32, 64, 2, default_group_m(64, 128)}, 1, 3.3, 3.3, 4.0},
  };
  // With a workspace at hand the deep-pipeline candidates are priced with their K slices: the
  // slices' workgroups fill the CUs, and the reduction costs a launch plus reading the partial sums.
  beam_tile_cfg c = kCandidates[0].cfg;
  int c_split = 1;
  double best_us = 1e300;
  for (const Candidate& k : kCandidates) {
    const long t = tiles(k.cfg.block_m, k.cfg.block_n);
    int s = 1;
    if (k.cfg.pipeline == 2 && split_req >= 0) {
      const int ktiles = (K + kBK - 1) / kBK;
      s = split_req == 0 ? auto_slices(t, K, cus) : (split_req < ktiles ? split_req : (ktiles > 0 ? ktiles : 1));
    }
    const long load = (t * s + cus - 1) / cus;  // workgroups per CU
    const long conc = load < k.occ ? load : k.occ;
    const double rate = k.occ == 1 ? k.alone : k.alone + (k.full - k.alone) * (double)(conc - 1) / (k.occ - 1);
    const double mflop = 2.0e-6 * k.cfg.block_m * k.cfg.block_n * (double)K / s;
    double us = (double)((load + k.occ - 1) / k.occ) * k.fixed + (double)load * mflop / rate;
    // the partial sums are written through to memory and read back (about 4 TB/s each way), and the reducing
    // workgroups start behind the multiplying ones
    if (s > 1) us += 2.0 + (double)s * M * N * 4.0 / 2.0e6;
    if (us < best_us) {
      best_us = us;
      c = k.cfg;
      c_split = s;
    }
  }
  *cfg = c;
  // From one full round of workgroups on, the 256 x 256 tile runs as four wavefronts of 128 x 128 (the kernel of
  // gemm_w4.h; 8192^3 fp16, same machine, in turn: 1490-1515 against 1455-1465 TFLOP/s) where that kernel's
  // shape conditions hold.
  if (c_split == 1 && c.block_m == 256 && c.block_n == 256 && tiles(256, 256) >= cus && K % kBK == 0 && K >= kW4MinK && N % 8 == 0 &&
      N <= (1 << 21)) {
    cfg->wave_m = 128;
    cfg->wave_n = 128;
  }
  if (split_req < 0 && tiles(c.block_m, c.block_n) < cus / 2 && K >= 2048)
    cfg->pipeline = 2;  // few workgroups per CU: a long prefetch queue keeps HBM busy
  // K slices on at most half the CUs: every workgroup has the memory system of two CUs to itself, the long
  // queue's prologue costs more than it hides (64 x 128 x 65536 in 64 slices: 8.9 against 9.9 us), and the
  // reducing workgroups of the one-launch form start on the idle CUs at once.
  if (c_split > 1 && tiles(c.block_m, c.block_n) * c_split <= cus / 2) cfg->pipeline = 0;
  if (split_k) *split_k = c_split;
  return BEAM_OK;
}

}  // namespace

extern "C" {

int beam_gemmrc(const void* A, const void* B, void* C, int M, int N, int K, int dtype,
                const beam_tile_cfg* cfg, void* stream) {
  bool generic;
  int rc = check_problem(A, B, C, M, N, K, dtype, &generic);
  if (rc) return rc;
  if (M == 0 || N == 0) return BEAM_OK;
  if ((rc = beam_init())) return rc;
  hipStream_t st = (hipStream_t)stream;
  if (K == 0) {
    BEAM_HIP(launch_zero_u16(C, (size_t)M * N, st));
    return BEAM_OK;
  }
  if (generic) {  // whatever tile was named: the tiled kernels cannot take this problem
    BEAM_HIP(launch_generic_gemm(A, B, C, M, N, K, dtype, false, false, st));
    return BEAM_OK;
  }
  beam_tile_cfg c;
  const KernelSet* ks;
  if ((rc = resolve_cfg(cfg, M, N, K, &c, &ks, -1, true))) return rc;
  GemmParams p = base_params(A, B, M, N, K, c);
  p.C = C;
  const long tiles = (long)p.tiles_m * p.tiles_n;
  const int cus = g_dev.cus > 0 ? g_dev.cus : 256;
  // The 256 x 256 tile of four 128 x 128 wavefronts has a kernel of its own (gemm_w4.h), built for problems
  // of a round of workgroups or more: one workgroup per CU walks its tiles with the operand ring running
  // through the tile boundaries.  It is what the tile {256, 256, 128, 128} means wherever its preconditions
  // hold (elsewhere that tile is the 4-wavefront member of the gemm_kernel.h family), and what
  // beam_default_config names from one full round of workgroups on.
  const bool w4_fits = c.pipeline == 0 && K % kBK == 0 && K >= kW4MinK && N % 8 == 0 && ((uintptr_t)C & 15) == 0 && N <= (1 << 21);
  const bool w4_named = c.block_m == 256 && c.block_n == 256 && c.wave_m == 128 && c.wave_n == 128;
  if (w4_named && !w4_fits && !cfg) {  // the library's own choice, but C is only 8-byte aligned: the 8-wavefront tile
    c.wave_m = 128;
    c.wave_n = 64;
    if ((rc = resolve_cfg(&c, M, N, K, &c, &ks))) return rc;
  }
  if (w4_fits && w4_named) {
    // Non-temporal stores of C pay when C is larger than the 256 MB last-level cache (and the K loops
    // are not so short that the writes are the bound).
    p.c_streaming = (size_t)M * N * 2 >= ((size_t)256 << 20) && K >= 1024;
    BEAM_HIP(launch_gemm_w4(p, dtype, dim3((unsigned)(tiles < cus ? tiles : cus), 1, 1), st));
    return BEAM_OK;
  }
  // More than one round of workgroups of another large tile: one workgroup per CU walks the tiles and
  // loads the next one's first operand tiles while it stores the current one (kEpiStoreLoop).
  // That kernel stores 16 bytes per lane through a buffer descriptor and has no short K tile.
  // Against one workgroup per tile, same machine: 16384 x 16384 x 2048 822 against 841 us,
  // 8192 x 8192 x 512 71 against 74.5 us, 8192 x 8192 x 2048 205 against 207 us, 8192^3 no difference.
  GemmLauncher loop = c.pipeline == 0 ? ks->launch[dtype][kEpiStoreLoop][0] : nullptr;
  if (loop && tiles > cus && K % kBK == 0 && N % 8 == 0 && ((uintptr_t)C & 15) == 0 && N <= (1 << 21)) {
    // Non-temporal stores of C pay when C is larger than the 256 MB last-level cache (and the K loops
    // are not so short that the writes are the bound): 16384 x 16384 x 2048 +2.5%, x 4096 +1.2%; an
    // 8192 x 8192 output (134 MB) is absorbed by that cache and loses 0.5-3% with them.
    p.c_streaming = (size_t)M * N * 2 >= ((size_t)256 << 20) && K >= 1024;
    BEAM_HIP(loop(p, dim3((unsigned)cus, 1, 1), st));
    return BEAM_OK;
  }
  BEAM_HIP(ks->launch[dtype][kEpiStore][c.pipeline](p, dim3((unsigned)tiles, 1, 1), st));
  return BEAM_OK;
}

int beam_matmul_nn(const void* A, const void* B, void* C, int M, int N, int K, int dtype, const beam_tile_cfg* cfg,
                   void* stream) {
  bool generic;
  int rc = check_problem(A, B, C, M, N, K, dtype, &generic);
  if (rc) return rc;
  if (M == 0 || N == 0) return BEAM_OK;
  if ((rc = beam_init())) return rc;
  hipStream_t st = (hipStream_t)stream;
  if (K == 0) {
    BEAM_HIP(launch_zero_u16(C, (size_t)M * N, st));
    return BEAM_OK;
  }
  // rows of B ([K][N]) that are not multiples of 16 bytes, or more than a descriptor spans: the plain kernel
  if (generic || N % 8 != 0 || N > (1 << 24)) {
    BEAM_HIP(launch_generic_gemm(A, B, C, M, N, K, dtype, true, false, st));
    return BEAM_OK;
  }
  beam_tile_cfg c;
  const KernelSet* ks;
  if ((rc = resolve_cfg(cfg, M, N, K, &c, &ks, -1, true))) return rc;
  if (!cfg) {
    // The library's choice is priced for B as [N][K].  In this layout a B fragment is two LDS reads, and the tiles
    // whose wavefronts are 64 columns wide pay for it: eight wavefronts of 64 x 32 instead of four of 64 x 64
    // (768 x 3072 x 768: 8.3 against 12.7 us; 2048 x 2048 x 512: 7.9 against 10.0), and 128 x 64 tiles of 64 x 32
    // instead of 64 x 128 tiles of 32 x 64 where that does not make more tiles (256 x 8192 x 8192: 57 against 71).
    auto tiles_of = [&](int bm, int bn) { return (long)((M + bm - 1) / bm) * ((N + bn - 1) / bn); };
    beam_tile_cfg alt = c;
    if (c.block_m == 128 && c.block_n == 128 && c.wave_m == 64 && c.wave_n == 64) {
      alt.wave_n = 32;
    } else if (c.block_m == 64 && c.block_n == 128 && c.wave_m == 32 && c.wave_n == 64 && tiles_of(128, 64) <= tiles_of(64, 128)) {
      alt.block_m = 128, alt.block_n = 64, alt.wave_m = 64, alt.wave_n = 32;
    }
    const KernelSet* alt_ks = nullptr;
    if ((alt.wave_n != c.wave_n) && resolve_cfg(&alt, M, N, K, &alt, &alt_ks) == BEAM_OK) c = alt, ks = alt_ks;
  }
  // The 4-wavefront kernel, as in beam_gemmrc; the K tile's offset into B is a 32-bit scalar there.
  const bool w4_fits = c.pipeline == 0 && K % kBK == 0 && K >= kW4MinK && ((uintptr_t)C & 15) == 0 && N <= (1 << 21) &&
                       (size_t)K * N * 2 < ((size_t)1 << 31);
  const bool w4_named = c.block_m == 256 && c.block_n == 256 && c.wave_m == 128 && c.wave_n == 128;
  if (w4_named && !w4_fits && !cfg) {
    c.wave_m = 128;
    c.wave_n = 64;
    if ((rc = resolve_cfg(&c, M, N, K, &c, &ks))) return rc;
  }
  GemmParams p = base_params(A, B, M, N, K, c);
  p.C = C;
  if (w4_fits && w4_named) {
    const long tiles = (long)p.tiles_m * p.tiles_n;
    const int cus = g_dev.cus > 0 ? g_dev.cus : 256;
    p.c_streaming = (size_t)M * N * 2 >= ((size_t)256 << 20) && K >= 1024;
    BEAM_HIP(launch_gemm_w4_kmajor(p, dtype, dim3((unsigned)(tiles < cus ? tiles : cus), 1, 1), st));
    return BEAM_OK;
  }
  BEAM_HIP(ks->launch_kmajor[dtype][c.pipeline](p, dim3((unsigned)(p.tiles_m * p.tiles_n), 1, 1), st));
  return BEAM_OK;
}

int beam_silu(const void* X, void* Y, long long count, int dtype, void* stream) {
  if (count < 0) return fail(BEAM_ERR_INVALID, "negative element count %lld", count);
  if (dtype != BEAM_F16 && dtype != BEAM_BF16) return fail(BEAM_ERR_UNSUPPORTED, "dtype %d: only fp16 (0) and bf16 (1)", dtype);
  if (count == 0) return BEAM_OK;
  if (!X || !Y) return fail(BEAM_ERR_INVALID, "null elementwise pointer");
  if (((uintptr_t)X | (uintptr_t)Y) & 15) return fail(BEAM_ERR_UNSUPPORTED, "X and Y must be 16-byte aligned");
  int rc = beam_init();
  if (rc) return rc;
  BEAM_HIP(launch_silu(X, Y, (size_t)count, dtype, (hipStream_t)stream));
  return BEAM_OK;
}

int beam_parallel_gemmrc_silu(const void* A, const void* B, void* C, int M, int N, int K, const void* X, void* Y,
                              long long count, int dtype, const beam_tile_cfg* cfg, void* stream) {
  bool generic;
  int rc = check_problem(A, B, C, M, N, K, dtype, &generic);
  if (rc) return rc;
  if (count < 0) return fail(BEAM_ERR_INVALID, "negative element count %lld", count);
  if (count > 0) {
    if (!X || !Y) return fail(BEAM_ERR_INVALID, "null elementwise pointer");
    if (((uintptr_t)X | (uintptr_t)Y) & 15) return fail(BEAM_ERR_UNSUPPORTED, "X and Y must be 16-byte aligned");
    if (count > kMaxSideElems)
      return fail(BEAM_ERR_UNSUPPORTED, "count=%lld exceeds %lld elements (one buffer descriptor)", count, kMaxSideElems);
  }
  if (M == 0 || N == 0 || K == 0 || generic) {  // no (tiled) K loop to hide anything in: the two halves run one after the other
    if ((rc = beam_gemmrc(A, B, C, M, N, K, dtype, cfg, stream))) return rc;
    return beam_silu(X, Y, count, dtype, stream);
  }
  if ((rc = beam_init())) return rc;
  beam_tile_cfg c;
  const KernelSet* ks;
  if ((rc = resolve_cfg(cfg, M, N, K, &c, &ks))) return rc;
  if (!cfg && c.pipeline == 2) c.pipeline = 0;  // the default for split-K-shaped problems
  if (c.pipeline == 2) return fail(BEAM_ERR_UNSUPPORTED, "the side job runs with pipeline 0 or 1");
  GemmParams p = base_params(A, B, M, N, K, c);
  p.C = C;
  p.side_x = X;
  p.side_y = Y;
  p.side_count = count;
  const long long wgs = (long long)p.tiles_m * p.tiles_n;
  const long long per_pass = wgs * ks->threads;  // units one K tile of the whole grid covers
  // The narrowest unit with which the job still ends inside the K loop: the work is then spread
  // evenly over the tiles instead of crowding the first ones.  A job longer than the loop keeps
  // 16-byte units and finishes after the GEMM's epilogue.
  const long long k_tiles = ((long long)K + kBK - 1) / kBK;
  p.side_width = 16;
  for (int w = 4; w < 16; w *= 2) {
    const long long units = (count >> 3) * (16 / w);
    if ((units + per_pass - 1) / per_pass <= k_tiles) {
      p.side_width = w;
      break;
    }
  }
  p.side_iters = (int)(((count >> 3) * (16 / p.side_width) + per_pass - 1) / per_pass);
  BEAM_HIP(ks->launch[dtype][kEpiStoreSide][c.pipeline](p, dim3((unsigned)wgs, 1, 1), (hipStream_t)stream));
  return BEAM_OK;
}

static int custom_fixed(int bm, int bn, int tm, int tn, const void* A, const void* B, void* C, int M,
                        int N, int K, void* stream) {
  beam_tile_cfg c = {bm, bn, tm, tn, 0, 0};
  return beam_gemmrc(A, B, C, M, N, K, BEAM_F16, &c, stream);
}

int beam_custom_gemmrc_128x128(const void* A, const void* B, void* C, int M, int N, int K, void* stream) {
  return custom_fixed(128, 128, 64, 64, A, B, C, M, N, K, stream);
}
int beam_custom_gemmrc_128x256(const void* A, const void* B, void* C, int M, int N, int K, void* stream) {
  return custom_fixed(128, 256, 64, 64, A, B, C, M, N, K, stream);
}
int beam_custom_gemmrc_256x128(const void* A, const void* B, void* C, int M, int N, int K, void* stream) {
  return custom_fixed(256, 128, 64, 64, A, B, C, M, N, K, stream);
}

// Workspace of a split-K call: fp32 partial sums [split_k][M][N], then (256-byte aligned) the synchronisation
// words of the one-launch form.  A workspace that only holds the partial sums still works: two launches.
static size_t splitk_partial_bytes(int M, int N, int split_k) {
  return (size_t)split_k * (size_t)M * (size_t)N * sizeof(float);
}
size_t beam_splitk_workspace_bytes(int M, int N, int split_k) {
  if (M <= 0 || N <= 0 || split_k <= 0) return 0;
  return align_up(splitk_partial_bytes(M, N, split_k), 256) + (size_t)sk_sync_bytes(M, N, split_k);
}

// 1: the fused GEMM+LayerNorm of the 4-wavefront kernel always runs one workgroup per tile (beam_set_ln_walk)
static std::atomic<int> g_ln_no_walk{[] {
  const char* e = getenv("BEAM_LN_WALK");
  return e && *e == '0' ? 1 : 0;
}()};

// 1: the one-launch split-K runs without reducing workgroups where its multiplying workgroups fit one round of the
// CUs; each of them reduces its share of its tile (beam_dbg_set_splitk_self_reduce: a measurement, off by default)
static std::atomic<int> g_splitk_self_reduce{0};

// 0: one launch where it applies, 1: always the partial kernel followed by the reduce kernel
static std::atomic<int> g_splitk_two_launches{[] {
  const char* e = getenv("BEAM_SPLITK_TWO_LAUNCHES");
  return e && *e && *e != '0' ? 1 : 0;
}()};

int beam_set_splitk_two_launches(int on) {
  g_splitk_two_launches.store(on != 0);
  return BEAM_OK;
}

static int effective_split(int M, int N, int K, const beam_tile_cfg& c, int split_k) {
  const int ktiles = (K + kBK - 1) / kBK;
  if (ktiles <= 1) return 1;
  int s = split_k;
  if (s <= 0) {
    const int cus = g_dev.cus > 0 ? g_dev.cus : 256;
    const long t = (long)((M + c.block_m - 1) / c.block_m) * ((N + c.block_n - 1) / c.block_n);
    s = auto_slices(t, K, cus);
  }
  if (s > ktiles) s = ktiles;
  if (s < 1) s = 1;
  const int per = (ktiles + s - 1) / s;
  return (ktiles + per - 1) / per;  // drop slices that would be empty
}

int beam_splitk_effective(int M, int N, int K, const beam_tile_cfg* cfg, int split_k) {
  beam_tile_cfg c;
  const KernelSet* ks;
  if (M <= 0 || N <= 0 || K < 0) return 1;
  if (K % 8 != 0 || K > kMaxK) return 1;  // the plain kernel: no slices
  if (resolve_cfg(cfg, M, N, K, &c, &ks, split_k > 0 ? split_k : 0)) return -1;
  return effective_split(M, N, K, c, split_k);
}

// The once-per-shape line about a slice count the library chose (beam_set_verbose).
static std::atomic<int> g_verbose{[] {
  const char* e = getenv("BEAM_VERBOSE");
  return e && *e && *e != '0' ? 1 : 0;
}()};

int beam_set_verbose(int verbose) {
  g_verbose.store(verbose != 0);
  return BEAM_OK;
}

static void log_split_choice_once(int M, int N, int K, int dtype, const beam_tile_cfg& c, int s) {
  static std::mutex mu;
  static std::set<std::string> seen;
  const long tiles = (long)((M + c.block_m - 1) / c.block_m) * ((N + c.block_n - 1) / c.block_n);
  const int cus = g_dev.cus > 0 ? g_dev.cus : 256;
  char line[256];
  snprintf(line, sizeof line, "split-K [%d,%d,%d] %s: tile %dx%d, %d slices of %d K elements, %ld workgroups = %.2f rounds of %d CUs",
           M, N, K, dtype == BEAM_BF16 ? "bf16" : "fp16", c.block_m, c.block_n, s, split_k_len(K, s), tiles * s,
           (double)(tiles * s) / cus, cus);
  std::lock_guard<std::mutex> lock(mu);
  if (seen.insert(line).second) fprintf(stderr, "[beam] %s\n", line);
}

int beam_gemmrc_splitk(const void* A, const void* B, void* C, int M, int N, int K, int dtype,
                       const beam_tile_cfg* cfg, int split_k, void* ws, size_t ws_bytes, void* stream) {
  bool generic;
  int rc = check_problem(A, B, C, M, N, K, dtype, &generic);
  if (rc) return rc;
  if (M == 0 || N == 0) return BEAM_OK;
  if ((rc = beam_init())) return rc;
  hipStream_t st = (hipStream_t)stream;
  if (K == 0) {
    BEAM_HIP(launch_zero_u16(C, (size_t)M * N, st));
    return BEAM_OK;
  }
  if (generic) {  // one pass of the plain kernel, no slices (beam_splitk_effective says 1 for K % 8 != 0)
    BEAM_HIP(launch_generic_gemm(A, B, C, M, N, K, dtype, false, false, st));
    return BEAM_OK;
  }
  beam_tile_cfg c;
  const KernelSet* ks;
  if ((rc = resolve_cfg(cfg, M, N, K, &c, &ks, split_k > 0 ? split_k : 0))) return rc;
  const int s = effective_split(M, N, K, c, split_k);
  if (split_k <= 0 && g_verbose.load(std::memory_order_relaxed)) log_split_choice_once(M, N, K, dtype, c, s);
  if (s == 1) {  // nothing to reduce: the plain kernel writes C directly
    GemmParams p = base_params(A, B, M, N, K, c);
    p.C = C;
    BEAM_HIP(ks->launch[dtype][kEpiStore][c.pipeline](p, dim3((unsigned)(p.tiles_m * p.tiles_n), 1, 1), st));
    return BEAM_OK;
  }
  const size_t need = splitk_partial_bytes(M, N, s);
  if (!ws || ws_bytes < need)
    return fail(BEAM_ERR_WORKSPACE, "split-K with %d slices needs %zu bytes of workspace, got %zu", s, need, ws_bytes);
  if ((uintptr_t)ws & 15) return fail(BEAM_ERR_UNSUPPORTED, "workspace must be 16-byte aligned");
  GemmParams p = base_params(A, B, M, N, K, c);
  p.ws = (float*)ws;
  p.k_slice = split_k_len(K, s);
  p.splits = s;
  // One launch: the reducing workgroups ride behind the multiplying ones in the same grid.  Needs a tile the
  // form is built for, 16-byte rows of partial sums, at most one flag per lane, a slice that fits one buffer
  // descriptor, and room for the synchronisation words behind the partial sums.
  const GemmLauncher one_launch = ks->launch_partial_fused[dtype][c.pipeline];
  if (one_launch && !g_splitk_two_launches.load(std::memory_order_relaxed) && N % 4 == 0 && s <= 64 &&
      (size_t)M * N <= ((size_t)1 << 28)) {
    // parts of 4 outputs per thread, smaller ones while the reducing workgroups are fewer than the CUs
    const int cus = g_dev.cus > 0 ? g_dev.cus : 256;
    const long tiles = (long)p.tiles_m * p.tiles_n;
    p.sk_out = 4;
    while (p.sk_out > 1 && tiles * sk_parts_per_tile(c.block_m, c.block_n, ks->threads, p.sk_out) < cus) p.sk_out /= 2;
    const long parts = sk_parts_per_tile(c.block_m, c.block_n, ks->threads, p.sk_out);
    const size_t sync_at = align_up(need, 256);
    const size_t sync_bytes = 4 * ((size_t)kSkFlags + (size_t)(tiles * parts) * (size_t)s);
    // Many tiles make many reducing workgroups, and those carry the kernel's LDS allocation: one per CU at a time,
    // round after round behind the last multiplying workgroups.  Beyond two rounds of them the reduce kernel of the
    // two-launch form, which spreads over the CUs at once, is the faster end (2048 x 1024 x 4096 in 2 slices of
    // 128 x 128 tiles: 25.7 against 27.2 us; 1024 x 1024 x 8192 in 4: 25.9 against 24.8 the other way).
    if (ws_bytes >= sync_at + sync_bytes && tiles * parts <= 2l * cus) {
      p.C = C;
      p.sk_sync = (int*)((char*)ws + sync_at);
      p.ln_nonce = g_ln_nonce.fetch_add(1, std::memory_order_relaxed) + 1;
      p.spin_limit = g_ln_spin_limit.load();
      p.sk_self = g_splitk_self_reduce.load(std::memory_order_relaxed) && tiles * s <= cus ? 1 : 0;
      BEAM_HIP(one_launch(p, dim3((unsigned)(tiles * s + (p.sk_self ? 0 : tiles * parts)), 1, 1), st));
      return BEAM_OK;
    }
  }
  BEAM_HIP(ks->launch[dtype][kEpiPartial][c.pipeline](p, dim3((unsigned)(p.tiles_m * p.tiles_n * s), 1, 1), st));
  // Where the workspace has synchronisation words, the reduce kernel marks them "no one-launch call is the latest":
  // a time-out recorded by an earlier one-launch call on this workspace must not be read as this call's.
  const size_t hdr_at = align_up(need, 256);
  int* hdr = ws_bytes >= hdr_at + 4 * (size_t)kSkFlags ? (int*)((char*)ws + hdr_at) : nullptr;
  BEAM_HIP(launch_splitk_reduce((const float*)ws, C, (size_t)M * N, s, dtype, hdr, st));
  return BEAM_OK;
}

int beam_gemmrc_splitk_timed_out(const void* ws, size_t ws_bytes, int M, int N, int split_k_effective, void* stream,
                                 int* timed_out) {
  if (!timed_out || M <= 0 || N <= 0 || split_k_effective < 1) return fail(BEAM_ERR_INVALID, "bad argument");
  *timed_out = 0;
  BEAM_HIP(hipStreamSynchronize((hipStream_t)stream));
  int hdr[4] = {0, 0, 0, 0};
  const size_t sync_at = align_up(splitk_partial_bytes(M, N, split_k_effective), 256);
  // One slice, or a workspace that ends with the partial sums: the call had no waiting workgroups (plain kernel, or
  // partial + reduce kernel), and there are no synchronisation words to read.
  if (!ws || split_k_effective == 1 || ws_bytes < sync_at + sizeof hdr) return BEAM_OK;
  BEAM_HIP(hipMemcpy(hdr, (const char*)ws + sync_at, sizeof hdr, hipMemcpyDeviceToHost));
  *timed_out = hdr[kSkMagic] == kSkMagicValue && hdr[kSkLaunchTag] != 0 && hdr[kSkTimeout] == hdr[kSkLaunchTag];
  return BEAM_OK;
}

size_t beam_splitk_noalloc_max_bytes(void) { return kScratchPartialBytes; }

int beam_gemmrc_splitk_noalloc(const void* A, const void* B, void* C, int M, int N, int K, int dtype,
                               const beam_tile_cfg* cfg, int split_k, void* stream) {
  int rc = beam_init();
  if (rc) return rc;
  bool generic = false;
  if ((rc = check_problem(A, B, C, M, N, K, dtype, &generic))) return rc;
  if (M > 0 && N > 0 && K > 0 && !generic) {  // (the plain kernel, one pass, needs no workspace)
    const int s = beam_splitk_effective(M, N, K, cfg, split_k);
    if (s < 0) return BEAM_ERR_UNSUPPORTED;  // the message is already set
    const size_t need = s > 1 ? splitk_partial_bytes(M, N, s) : 0;
    if (need > kScratchPartialBytes)
      return fail(BEAM_ERR_WORKSPACE, "split-K of %d x %d in %d slices needs %zu bytes; the built-in workspace of the "
                  "no-allocation entry point holds %zu (use beam_gemmrc_splitk with a workspace of your own)", M, N, s, need,
                  kScratchPartialBytes);
  }
  void* ws = nullptr;
  if ((rc = scratch_on_current_device(&ws))) return rc;
  return beam_gemmrc_splitk(A, B, C, M, N, K, dtype, cfg, split_k, ws, kScratchBytes, stream);
}

// Fused GEMM+LayerNorm workspace: [header, 256 bytes | (mean, tag) words | (M2, ~tag) words], one word of
// each kind per (row band, column tile, row).  Nothing in it is ever prepared or cleared: every fused launch
// gets a nonce that no earlier launch of this process had, and the kernel takes a statistics word for
// published only if it carries the tag made from that nonce (gemm_kernel.h: ln_launch_tag).  The library keeps
// no state about workspaces on the host either.
static size_t ln_fused_header_bytes() { return 256; }
static size_t ln_fused_set_bytes(size_t tiles_m, size_t tiles_n, int block_m) {
  return align_up(tiles_m * tiles_n * (size_t)block_m * 2 * sizeof(float), 256);
}

static bool ln_fused_applies_on(const beam_tile_cfg& c, const KernelSet& ks, int N, int cus) {
  // The residency argument of the fused kernel (tile_map.h: band_block_tile) is made for 8 XCDs of 32 CUs.
  if (cus != kNumXcd * 32) return false;
  // a band's column tiles are spread over the 8 XCDs; each XCD must hold its share (<= 32) at once,
  // and the band's statistics ((tiles_n + 1) * block_m pairs) are gathered into the kernel's LDS
  const int tiles_n = (N + c.block_n - 1) / c.block_n;
  const int lds = c.pipeline ? ks.lds_bytes_shallow : ks.lds_bytes;
  return tiles_n <= 64 && (size_t)(tiles_n + 1) * c.block_m * 8 <= (size_t)lds;
}
static bool ln_fused_applies(const beam_tile_cfg& c, const KernelSet& ks, int N) { return ln_fused_applies_on(c, ks, N, g_dev.cus); }

static int ln_resolve_mode(int mode, const beam_tile_cfg& c, const KernelSet& ks, int N) {
  if (mode == BEAM_LN_AUTO) return ln_fused_applies(c, ks, N) ? BEAM_LN_FUSED : BEAM_LN_TWOPASS;
  return mode;
}

// GEMM+LayerNorm problems that run on the plain kernels, and the workspace they need (fp32 X).
static bool ln_is_generic(bool gemm_generic, const void* gamma, const void* beta) {
  return gemm_generic || ((((uintptr_t)gamma | (uintptr_t)beta) & 7) != 0);
}
static size_t ln_generic_need(int M, int N) { return align_up((size_t)M * N * sizeof(float), 256); }

// Bytes for tile `c` in `mode` (already resolved: two-pass or fused).
static size_t ln_workspace_need(int M, int N, const beam_tile_cfg& c, int mode) {
  const size_t tiles_m = (size_t)(M + c.block_m - 1) / c.block_m;
  const size_t tiles_n = (size_t)(N + c.block_n - 1) / c.block_n;
  if (mode == BEAM_LN_FUSED) return ln_fused_header_bytes() + 2 * ln_fused_set_bytes(tiles_m, tiles_n, c.block_m);
  return align_up((size_t)M * N * sizeof(float), 256) + align_up((size_t)M * tiles_n * 2 * sizeof(float), 256);
}

// The tile a GEMM+LayerNorm call runs with: the caller's, or the library's; never the deep pipeline.
// For the one-kernel form (mode AUTO or FUSED on a device it runs on) the library does not take the plain GEMM's
// tile: every workgroup ends with the epilogue's chain of latencies, so a round of workgroups costs a fixed time
// that grows with the tile, and rounds count in whole numbers -- of bands, since a band's tiles wait for each other.
// The model is that sentence: rounds x (fixed + flops of a tile / rate), rates (TFLOP/s per CU) and fixed costs (us)
// fitted by least squares to the timings of every tile on 34 shapes (beam/ln_tile_timings.json: the pick is within
// 1.5% of the best tile in the geometric mean, 16% at worst).
struct LnCandidate {
  beam_tile_cfg cfg;
  double rate, fixed;
};
// Two candidates share the 256 x 256 tile: the 4-wavefront kernel of gemm_w4.h (the faster K loop; an epilogue in
// which nothing overlaps the vector work of its one wavefront per SIMD) and the 8-wavefront one (two wavefronts per
// SIMD cover each other's waits in the epilogue).  Measured, the first wins by 3-5% where K is 2048 and more and the
// rounds are few (4096^3: 100.3 against 105.6 us), the second by 3-14% where a tile's K loop is short (8192 x 8192 x
// 1024: 146.1 against 150.7 us; 4096 x 16384 x 1024, whose bands are too wide to walk: 166.8 against 190.8).
static const LnCandidate kLnCandidates[] = {
    {{256, 256, 128, 128, 0, 0}, 7.91, 18.17},  // (only where gemm_w4.h's conditions hold)
    {{256, 256, 128, 64, 0, 0}, 7.08, 14.13},
    {{224, 256, 112, 64, 0, 0}, 6.94, 12.35},
    {{192, 256, 96, 64, 0, 0}, 6.66, 11.01},
    {{256, 128, 64, 64, 0, 0}, 5.38, 8.00},
    {{128, 256, 64, 64, 0, 0}, 5.41, 8.17},
    {{128, 128, 64, 32, 0, 0}, 5.05, 6.65},
    {{64, 128, 32, 64, 0, 0}, 3.33, 3.54},
    {{64, 64, 32, 32, 0, 0}, 2.98, 2.76},
};
// The model's pick for a device of `cus` compute units; false if the one-kernel form applies with none of the tiles.
static bool ln_choose_tile(int M, int N, int K, int cus, beam_tile_cfg* out, const KernelSet** out_ks) {
  double best_us = 1e300;
  bool found = false;
  for (const LnCandidate& k : kLnCandidates) {
    beam_tile_cfg c = k.cfg;
    const KernelSet* ks = nullptr;
    const bool w4 = c.wave_m == 128 && c.wave_n == 128;
    if (w4 && !(K % kBK == 0 && K >= kW4MinK && N % 8 == 0)) continue;
    if (resolve_cfg(&c, M, N, K, &c, &ks, -1, w4) != BEAM_OK || !ln_fused_applies_on(c, *ks, N, cus)) continue;
    // (a band's column tiles wait for each other, so a band that straddles two rounds costs both: a round is
    // worth the whole bands it holds)
    const int tiles_m = (M + c.block_m - 1) / c.block_m, tiles_n = (N + c.block_n - 1) / c.block_n;
    const int bands_per_round = cus / tiles_n > 1 ? cus / tiles_n : 1;
    const double rounds = (double)((tiles_m + bands_per_round - 1) / bands_per_round);
    const double us = rounds * (k.fixed + 2.0e-6 * c.block_m * c.block_n * (double)K / k.rate);
    if (us < best_us) {
      best_us = us;
      *out = c;
      *out_ks = ks;
      found = true;
    }
  }
  return found;
}
static int ln_resolve_cfg(const beam_tile_cfg* cfg, int M, int N, int K, int mode, beam_tile_cfg* c, const KernelSet** ks) {
  int rc = resolve_cfg(cfg, M, N, K, c, ks, -1, true);
  if (rc) return rc;
  if (c->pipeline == 2) c->pipeline = 0;  // the deep pipeline exists for the store / split-K kernels only
  if (cfg || mode == BEAM_LN_TWOPASS || g_dev.cus <= 0) return BEAM_OK;
  beam_tile_cfg alt;
  const KernelSet* alt_ks = nullptr;
  if (ln_choose_tile(M, N, K, g_dev.cus, &alt, &alt_ks)) {
    *c = alt;
    *ks = alt_ks;
  }
  return BEAM_OK;
}

// What a GEMM+LayerNorm call does and the workspace it needs: one function, so that the entry point and the
// workspace queries cannot disagree.
//   plain     the problem is outside what the tiled kernels take (K % 8, K beyond a descriptor, operands aligned to
//             an element only): plain GEMM into fp32 X, then a row-wise LayerNorm
//   capturing the stream is being captured: AUTO then means two passes (a replayed graph may share the device with
//             other work, which the fused kernel's residency argument does not cover); an explicit FUSED is honoured
//   wide_io   Y, gamma and beta are 16-byte aligned (the 4-wavefront kernel's vector accesses)
struct LnPlan {
  enum Kind { kPlain, kTwoPass, kFused } kind;
  beam_tile_cfg c;
  const KernelSet* ks;
  bool w4;  // fused, on the kernel of gemm_w4.h
  size_t need;
};
static int ln_plan(int M, int N, int K, const beam_tile_cfg* cfg, int mode, bool plain, bool capturing, bool wide_io, LnPlan* out) {
  out->ks = nullptr;
  out->w4 = false;
  if (plain) {
    out->kind = LnPlan::kPlain;
    out->need = ln_generic_need(M, N);
    return BEAM_OK;
  }
  if (capturing && mode == BEAM_LN_AUTO) mode = BEAM_LN_TWOPASS;
  int rc = ln_resolve_cfg(cfg, M, N, K, mode, &out->c, &out->ks);
  if (rc) return rc;
  beam_tile_cfg& c = out->c;
  if (mode == BEAM_LN_FUSED && !ln_fused_applies(c, *out->ks, N))
    return fail(BEAM_ERR_UNSUPPORTED, "fused LayerNorm: needs a device of %d CUs and at most 64 column tiles (N=%d, block_n=%d, %d CUs)",
                kNumXcd * 32, N, c.block_n, g_dev.cus);
  mode = ln_resolve_mode(mode, c, *out->ks, N);
  // The 256 x 256 tile runs on the kernel of gemm_w4.h where that one's preconditions hold (asked for by
  // name, or as the library's own choice); where they do not, the library's own choice falls back to the
  // 8-wavefront tile of the same shape.
  const bool w4_fits = mode == BEAM_LN_FUSED && c.pipeline == 0 && c.block_m == 256 && c.block_n == 256 && K % kBK == 0 &&
                       K >= kW4MinK && N % 8 == 0 && N <= (1 << 21) && wide_io;
  if (!cfg && !w4_fits && c.block_m == 256 && c.block_n == 256 && c.wave_m == 128 && c.wave_n == 128) {
    c.wave_n = 64;
    if ((rc = resolve_cfg(&c, M, N, K, &c, &out->ks))) return rc;
  }
  out->w4 = w4_fits && c.wave_m == 128 && c.wave_n == 128;
  out->kind = mode == BEAM_LN_FUSED ? LnPlan::kFused : LnPlan::kTwoPass;
  out->need = ln_workspace_need(M, N, c, mode);
  return BEAM_OK;
}

// Enough for beam_gemmrc_ln_ex(M, N, K, cfg, mode) on operands aligned as the tiled kernels need them.  AUTO covers
// both forms it can resolve to (one kernel eagerly, two passes under stream capture and as the retry of
// beam_gemmrc_ln_checked), which also covers the plain path.
size_t beam_gemmrc_ln_workspace_bytes_for(int M, int N, int K, const beam_tile_cfg* cfg, int mode) {
  if (M <= 0 || N <= 0 || K < 0) return 0;
  if (K % 8 != 0 || K > kMaxK) return ln_generic_need(M, N);
  (void)beam_init();  // AUTO depends on the device
  LnPlan eager, captured;
  if (ln_plan(M, N, K, cfg, mode, false, false, true, &eager)) return 0;
  if (mode != BEAM_LN_AUTO) return eager.need;
  if (ln_plan(M, N, K, cfg, mode, false, true, true, &captured)) return eager.need;
  return eager.need > captured.need ? eager.need : captured.need;
}

// Enough for any call with these M, N, cfg and mode: every K, every alignment, captured or not.
size_t beam_gemmrc_ln_workspace_bytes_ex(int M, int N, const beam_tile_cfg* cfg, int mode) {
  if (M <= 0 || N <= 0) return 0;
  size_t need = ln_generic_need(M, N);  // K % 8 != 0, operands aligned to an element only
  auto take = [&](size_t n) { need = n > need ? n : need; };
  // a given tile does not depend on K
  if (cfg) {
    take(beam_gemmrc_ln_workspace_bytes_for(M, N, 64, cfg, mode));
    return need;
  }
  // Without a tile the library picks one from (M, N, K), and K is not known here: the largest need over
  // every tile it can pick, in every form `mode` can resolve to.
  (void)beam_init();
  for (int i = 0; i < beam_num_configs(); ++i) {
    beam_tile_cfg c;
    const KernelSet* ks;
    if (beam_get_config(i, &c) || resolve_cfg(&c, M, N, 64, &c, &ks)) continue;
    take(ln_workspace_need(M, N, c, ln_resolve_mode(mode, c, *ks, N)));
    if (mode == BEAM_LN_AUTO) take(ln_workspace_need(M, N, c, BEAM_LN_TWOPASS));
  }
  return need;
}

size_t beam_gemmrc_ln_workspace_bytes(int M, int N, const beam_tile_cfg* cfg) {
  return beam_gemmrc_ln_workspace_bytes_ex(M, N, cfg, BEAM_LN_AUTO);
}

size_t beam_dbg_ln_plan_bytes(int M, int N, int K, const beam_tile_cfg* cfg, int mode, int plain, int capturing, int wide_io) {
  LnPlan plan;
  if (M <= 0 || N <= 0 || K < 0 || ln_plan(M, N, K, cfg, mode, plain != 0 || K % 8 != 0 || K > kMaxK, capturing != 0, wide_io != 0, &plan)) return 0;
  return plan.need;
}

int beam_dbg_set_splitk_self_reduce(int on) {
  g_splitk_self_reduce.store(on != 0);
  return BEAM_OK;
}

int beam_set_ln_walk(int on) {
  g_ln_no_walk.store(on ? 0 : 1);
  return BEAM_OK;
}

int beam_dbg_assume_compute_units(int compute_units) {
  std::lock_guard<std::mutex> lk(g_dev_mu);
  if (g_dev.status == BEAM_OK) return fail(BEAM_ERR_INVALID, "a device has been probed: its own CU count stands");
  g_dev.cus = compute_units;
  return BEAM_OK;
}

int beam_gemmrc_ln_ex(const void* A, const void* B, const void* gamma, const void* beta, float eps, void* Y,
                      int M, int N, int K, int dtype, const beam_tile_cfg* cfg, int mode, void* ws,
                      size_t ws_bytes, void* stream) {
  bool generic;
  int rc = check_problem(A, B, Y, M, N, K, dtype, &generic);
  if (rc) return rc;
  if (M == 0 || N == 0) return BEAM_OK;
  if (!gamma || !beta) return fail(BEAM_ERR_INVALID, "null gamma/beta");
  if (((uintptr_t)gamma | (uintptr_t)beta) & 1) return fail(BEAM_ERR_INVALID, "gamma and beta must be aligned to their 16-bit elements");
  if (!(eps >= 0.0f)) return fail(BEAM_ERR_INVALID, "eps must be >= 0");
  if (mode < BEAM_LN_AUTO || mode > BEAM_LN_FUSED) return fail(BEAM_ERR_INVALID, "unknown LayerNorm mode %d", mode);
  if ((rc = beam_init())) return rc;
  hipStream_t st = (hipStream_t)stream;
  hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
  if (st != nullptr) (void)hipStreamIsCapturing(st, &capturing);
  LnPlan plan;
  if ((rc = ln_plan(M, N, K, cfg, mode, ln_is_generic(generic, gamma, beta), capturing != hipStreamCaptureStatusNone,
                    (((uintptr_t)Y | (uintptr_t)gamma | (uintptr_t)beta) & 15) == 0, &plan)))
    return rc;
  const size_t need = plan.need;
  if (!ws || ws_bytes < need)
    return fail(BEAM_ERR_WORKSPACE, "GEMM+LayerNorm needs %zu bytes of workspace, got %zu", need, ws_bytes);
  if (plan.kind == LnPlan::kPlain) {
    // What the tiled kernels cannot take: the plain GEMM into fp32 X, then a row-wise LayerNorm (whatever mode was named).
    if ((uintptr_t)ws & 15) return fail(BEAM_ERR_UNSUPPORTED, "workspace must be 16-byte aligned");
    if (K == 0) BEAM_HIP(launch_fill_floats((float*)ws, (size_t)M * N, 0.0f, st));
    else BEAM_HIP(launch_generic_gemm(A, B, ws, M, N, K, dtype, false, true, st));
    BEAM_HIP(launch_ln_rows((const float*)ws, gamma, beta, Y, M, N, eps, dtype, st));
    return BEAM_OK;
  }
  if ((uintptr_t)ws & 255) return fail(BEAM_ERR_UNSUPPORTED, "workspace must be 256-byte aligned");
  const beam_tile_cfg& c = plan.c;
  const KernelSet* ks = plan.ks;
  GemmParams p = base_params(A, B, M, N, K, c);
  // K == 0: the kernels run with an empty K range and produce x = 0, i.e. y = beta.
  if (plan.kind == LnPlan::kFused) {
    p.C = Y;
    // Launches that share a workspace must be ordered (same stream): overlapping ones would race on the sets.
    const size_t set_bytes = ln_fused_set_bytes(p.tiles_m, p.tiles_n, c.block_m);
    float* sets = (float*)((char*)ws + ln_fused_header_bytes());
    // A recorded launch repeats its arguments on every replay: the counter in the header then makes the tag new.
    if (capturing != hipStreamCaptureStatusNone) BEAM_HIP(launch_ln_replay_bump((int*)ws, st));
    p.ln_nonce = g_ln_nonce.fetch_add(1, std::memory_order_relaxed) + 1;
    p.stats = sets;
    p.next_stats = (float*)((char*)sets + set_bytes);
    p.timeout_flag = (int*)ws;
    p.gamma = gamma;
    p.beta = beta;
    p.eps = eps;
    p.spin_limit = g_ln_spin_limit.load();
    // band groups: XCD x owns group_n columns of group_m bands; 8 * group_n covers a whole band and
    // group_m * group_n workgroups fit the 32 CUs of an XCD even at one workgroup per CU
    // ... or, when a band is short enough, whole bands per XCD (tile_map.h: band_xcd_tile)
    //     if that fills every XCD, takes no more rounds of workgroups than the spread order and
    //     streams no more operand panels through an XCD's L2 per round (bands + columns it touches;
    //     measured: 16384 x 2048 x 2048, 4 + 8 against 32 + 1 panels, 112 against 120 us;
    //     8192 x 8192 x 4096, 1 + 32 against 8 + 4, 419 against 400 us; 4096^3, 18 either way, 104.1
    //     against 104.8 us)
    // ... or, where those two orders' padding costs rounds of workgroups (20 column tiles are 3 per XCD on
    //     seven XCDs and none on the eighth: 3000 x 5000 x 2000 in 256 x 256 tiles puts 36 workgroups on six
    //     XCDs of 32 CUs), band after band with no padding: id = band * tiles_n + column, which the hardware's
    //     round-robin deals out evenly.
    // All three keep a band's workgroups together in id order, so a launch that gets only part of the device
    // still finishes band by band.  (The plain kernels' raster order streams fewer operand bytes into the L2s
    // when the whole grid is one round -- 4096^3: 204 against 303 MB, in the same time -- but loses exactly that.)
    unsigned grid;
    p.group_n = (p.tiles_n + kNumXcd - 1) / kNumXcd;
    p.group_m = 32 / p.group_n;
    if (p.group_m > p.tiles_m) p.group_m = p.tiles_m;
    const int bx = p.tiles_n <= 32 ? 32 / p.tiles_n : 0;
    const int rounds_spread = (p.tiles_m + p.group_m - 1) / p.group_m;
    const bool whole_bands = bx > 0 && p.tiles_m >= kNumXcd * bx && (p.tiles_m + kNumXcd * bx - 1) / (kNumXcd * bx) <= rounds_spread &&
                             bx + p.tiles_n <= p.group_m + p.group_n;
    const int rounds_grouped = whole_bands ? (p.tiles_m + kNumXcd * bx - 1) / (kNumXcd * bx) : rounds_spread;
    const long per_xcd = ((long)p.tiles_m * p.tiles_n + kNumXcd - 1) / kNumXcd;
    if ((per_xcd + 31) / 32 < rounds_grouped) {
      p.group_n = -1;
      grid = (unsigned)(p.tiles_m * p.tiles_n);
    } else if (whole_bands) {
      p.group_n = 0;
      p.group_m = bx;
      grid = (unsigned)band_xcd_grid(p.tiles_m, p.tiles_n, bx);
    } else {
      grid = (unsigned)band_block_grid(p.tiles_m, p.group_m, p.group_n);
    }
    // the band orders' divisors as multipliers (tile_map.h: band_order_divs)
    p.divs = band_order_divs(p.tiles_n, p.group_m, p.group_n);
    if (plan.w4) {
      // More ids than CUs: one workgroup per CU walks the ids w, w + CUs, ... of the same order, with the next
      // tile's first operand tiles arriving while the band's statistics are exchanged (gemm_w4.h says why no
      // chain of waits closes: a band's ids lie within fewer than 256 of each other in all three orders).  The
      // walking form keeps the epilogue's scratch inside the two LDS slots the operand ring leaves free, which
      // holds a band of up to 32 column tiles; wider bands keep one workgroup per tile.
      p.ln_ids = (int)grid;
      const unsigned cus = (unsigned)g_dev.cus;
      const bool walk = grid > cus && p.tiles_n <= kW4LnCompactTiles && !g_ln_no_walk.load(std::memory_order_relaxed);
      BEAM_HIP(launch_gemm_w4_ln(p, dtype, dim3(walk ? cus : grid, 1, 1), st));
      return BEAM_OK;
    }
    BEAM_HIP(ks->launch[dtype][kEpiLnFused][c.pipeline](p, dim3(grid, 1, 1), st));
    return BEAM_OK;
  }
  p.ws = (float*)ws;
  p.stats = (float*)((char*)ws + align_up((size_t)M * N * sizeof(float), 256));
  BEAM_HIP(ks->launch[dtype][kEpiLnStats][c.pipeline](p, dim3((unsigned)(p.tiles_m * p.tiles_n), 1, 1), st));
  BEAM_HIP(launch_ln_apply(p.ws, p.stats, gamma, beta, Y, M, N, p.tiles_n, c.block_n, eps, dtype, st));
  return BEAM_OK;
}

int beam_gemmrc_ln(const void* A, const void* B, const void* gamma, const void* beta, float eps, void* Y,
                   int M, int N, int K, int dtype, const beam_tile_cfg* cfg, void* ws, size_t ws_bytes,
                   void* stream) {
  return beam_gemmrc_ln_ex(A, B, gamma, beta, eps, Y, M, N, K, dtype, cfg, BEAM_LN_AUTO, ws, ws_bytes, stream);
}

int beam_gemmrc_ln_checked(const void* A, const void* B, const void* gamma, const void* beta, float eps, void* Y,
                           int M, int N, int K, int dtype, const beam_tile_cfg* cfg, void* ws, size_t ws_bytes,
                           void* stream, int* fell_back) {
  if (fell_back) *fell_back = 0;
  hipStream_t st = (hipStream_t)stream;
  hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
  if (st != nullptr) (void)hipStreamIsCapturing(st, &capturing);
  // (captured: AUTO is two passes, which wait for nothing; a stream being captured cannot be waited for anyway)
  int rc = beam_gemmrc_ln_ex(A, B, gamma, beta, eps, Y, M, N, K, dtype, cfg, BEAM_LN_AUTO, ws, ws_bytes, stream);
  if (rc || capturing != hipStreamCaptureStatusNone || M == 0 || N == 0) return rc;
  bool generic;
  (void)check_problem(A, B, Y, M, N, K, dtype, &generic);
  LnPlan plan;
  if (ln_plan(M, N, K, cfg, BEAM_LN_AUTO, ln_is_generic(generic, gamma, beta), false,
              (((uintptr_t)Y | (uintptr_t)gamma | (uintptr_t)beta) & 15) == 0, &plan) || plan.kind != LnPlan::kFused)
    return BEAM_OK;  // nothing in the call waits for anything
  int timed_out = 0;
  if ((rc = beam_gemmrc_ln_timed_out(ws, stream, &timed_out))) return rc;
  if (!timed_out) return BEAM_OK;
  if (fell_back) *fell_back = 1;
  if ((rc = beam_gemmrc_ln_ex(A, B, gamma, beta, eps, Y, M, N, K, dtype, cfg, BEAM_LN_TWOPASS, ws, ws_bytes, stream))) return rc;
  BEAM_HIP(hipStreamSynchronize(st));
  return BEAM_OK;
}

int beam_gemmrc_ln_workspace_reset(const void* ws) {
  if (!ws) return fail(BEAM_ERR_INVALID, "null workspace");
  // Forgets a recorded time-out (never needed).  The replay counter behind these words stays: it is part of the tag
  // of captured launches, and a counter that went back could hand a replay the tag of an earlier one, whose
  // statistics words would then pass for published.
  static_assert(kLnHdrTimeout < 3 && kLnHdrMagic < 3 && kLnHdrLaunchTag < 3 && kLnHdrReplay == 3, "header words");
  BEAM_HIP(hipMemset(const_cast<void*>(ws), 0, 3 * sizeof(int)));
  return BEAM_OK;
}

int beam_set_ln_spin_limit(int polls) {
  if (polls < -1) return fail(BEAM_ERR_INVALID, "spin limit must be >= -1");
  g_ln_spin_limit.store(polls);
  return BEAM_OK;
}

int beam_gemmrc_ln_timed_out(const void* ws, void* stream, int* timed_out) {
  if (!ws || !timed_out) return fail(BEAM_ERR_INVALID, "null argument");
  BEAM_HIP(hipStreamSynchronize((hipStream_t)stream));
  int hdr[4] = {0, 0, 0, 0};
  BEAM_HIP(hipMemcpy(hdr, ws, sizeof hdr, hipMemcpyDeviceToHost));
  // the header speaks of a fused launch at all, and the launch that gave up is the latest one
  *timed_out = hdr[kLnHdrMagic] == kLnMagic && hdr[kLnHdrLaunchTag] != 0 && hdr[kLnHdrTimeout] == hdr[kLnHdrLaunchTag];
  return BEAM_OK;
}

// BEAM_OP_PROBE_SPLITK_LOADS: the launch of beam_gemmrc_splitk's partial kernel, resolved the same way.
static int probe_splitk_loads(const beam_problem* q, const beam_tile_cfg* cfg, hipStream_t st) {
  bool generic;
  int rc = check_problem(q->A, q->B, q->C, q->M, q->N, q->K, q->dtype, &generic);
  if (rc) return rc;
  if ((rc = beam_init())) return rc;
  if (generic || q->dtype != BEAM_F16 || q->M == 0 || q->N == 0 || q->K == 0)
    return fail(BEAM_ERR_UNSUPPORTED, "the load probe is built for fp16 problems of the tiled kernels");
  beam_tile_cfg c;
  const KernelSet* ks;
  if ((rc = resolve_cfg(cfg, q->M, q->N, q->K, &c, &ks, q->split_k > 0 ? q->split_k : 0))) return rc;
  const bool built = c.pipeline == 2 && c.block_m == 64 && ((c.block_n == 128 && c.wave_m == 32 && c.wave_n == 64) ||
                                                            (c.block_n == 64 && c.wave_m == 32 && c.wave_n == 32));
  if (!built) return fail(BEAM_ERR_UNSUPPORTED, "the load probe is built for the deep 64x128 (wave 32x64) and 64x64 (wave 32x32) tiles");
  const int s = effective_split(q->M, q->N, q->K, c, q->split_k);
  GemmParams p = base_params(q->A, q->B, q->M, q->N, q->K, c);
  p.ws = (float*)q->ws;  // never written
  p.k_slice = split_k_len(q->K, s);
  p.splits = s;
  BEAM_HIP(launch_probe_splitk_loads(p, c.block_m, c.block_n, dim3((unsigned)(p.tiles_m * p.tiles_n * s), 1, 1), st));
  return BEAM_OK;
}

int beam_bench(int op, const beam_problem* q, const beam_tile_cfg* cfg, int warmup, int iters, void* stream,
               float* avg_ms) {
  if (!q || !avg_ms || iters < 1 || warmup < 0) return fail(BEAM_ERR_INVALID, "bad bench arguments");
  auto once = [&]() -> int {
    switch (op) {
      case BEAM_OP_GEMM:
        return beam_gemmrc(q->A, q->B, q->C, q->M, q->N, q->K, q->dtype, cfg, stream);
      case BEAM_OP_SPLITK:
        return beam_gemmrc_splitk(q->A, q->B, q->C, q->M, q->N, q->K, q->dtype, cfg, q->split_k, q->ws,
                                  q->ws_bytes, stream);
      case BEAM_OP_GEMM_LN:
        return beam_gemmrc_ln_ex(q->A, q->B, q->gamma, q->beta, q->eps, q->C, q->M, q->N, q->K, q->dtype, cfg, q->ln_mode,
                                 q->ws, q->ws_bytes, stream);
      case BEAM_OP_GEMM_SILU:
        return beam_parallel_gemmrc_silu(q->A, q->B, q->C, q->M, q->N, q->K, q->side_x, q->side_y, q->side_count,
                                         q->dtype, cfg, stream);
      case BEAM_OP_MATMUL_NN:
        return beam_matmul_nn(q->A, q->B, q->C, q->M, q->N, q->K, q->dtype, cfg, stream);
      case BEAM_OP_SILU:
        return beam_silu(q->side_x, q->side_y, q->side_count, q->dtype, stream);
      case BEAM_OP_PROBE_EMPTY:
      case BEAM_OP_PROBE_EMPTY_PAIR: {
        int rc = beam_init();
        if (rc) return rc;
        BEAM_HIP(launch_empty(256, 256, (hipStream_t)stream));
        if (op == BEAM_OP_PROBE_EMPTY_PAIR) BEAM_HIP(launch_empty(1024, 64, (hipStream_t)stream));
        return BEAM_OK;
      }
      case BEAM_OP_PROBE_SPLITK_LOADS:
        return probe_splitk_loads(q, cfg, (hipStream_t)stream);
      case BEAM_OP_PROBE_LN_APPLY: {
        // the second kernel of a two-pass GEMM+LayerNorm alone, on the fp32 X and statistics a two-pass call left in ws
        int rc = beam_init();
        if (rc) return rc;
        LnPlan plan;
        if ((rc = ln_plan(q->M, q->N, q->K, cfg, BEAM_LN_TWOPASS, q->K % 8 != 0 || q->K > kMaxK, false, true, &plan))) return rc;
        if (plan.kind != LnPlan::kTwoPass || !q->ws || q->ws_bytes < plan.need) return fail(BEAM_ERR_WORKSPACE, "needs the workspace of a two-pass call");
        const float* stats = (const float*)((const char*)q->ws + align_up((size_t)q->M * q->N * sizeof(float), 256));
        BEAM_HIP(launch_ln_apply((const float*)q->ws, stats, q->gamma, q->beta, q->C, q->M, q->N, (q->N + plan.c.block_n - 1) / plan.c.block_n,
                                 plan.c.block_n, q->eps, q->dtype, (hipStream_t)stream));
        return BEAM_OK;
      }
      default:
        return fail(BEAM_ERR_INVALID, "unknown op %d", op);
    }
  };
  hipStream_t st = (hipStream_t)stream;
  for (int i = 0; i < warmup; ++i) {
    int rc = once();
    if (rc) return rc;
  }
  hipEvent_t e0, e1;
  BEAM_HIP(hipEventCreate(&e0));
  BEAM_HIP(hipEventCreate(&e1));
  int rc = BEAM_OK;
  hipError_t he = hipEventRecord(e0, st);
  for (int i = 0; i < iters && rc == BEAM_OK && he == hipSuccess; ++i) rc = once();
  if (he == hipSuccess) he = hipEventRecord(e1, st);
  if (he == hipSuccess) he = hipEventSynchronize(e1);
  float ms = 0.0f;
  if (he == hipSuccess) he = hipEventElapsedTime(&ms, e0, e1);
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  if (rc) return rc;
  if (he != hipSuccess) return hip_fail(he, "event timing");
  *avg_ms = ms / (float)iters;
  return BEAM_OK;
}

int beam_probe_mfma(int dtype, int mfma_shape, int data, int passes, int warmup, int iters, void* stream, float* avg_ms,
                    double* flop_per_launch) {
  if (!avg_ms || iters < 1 || warmup < 0 || passes < 1) return fail(BEAM_ERR_INVALID, "bad probe arguments");
  if (dtype != BEAM_F16 && dtype != BEAM_BF16) return fail(BEAM_ERR_UNSUPPORTED, "dtype %d: only fp16 (0) and bf16 (1)", dtype);
  if (mfma_shape != BEAM_MFMA_16X16X32 && mfma_shape != BEAM_MFMA_32X32X16) return fail(BEAM_ERR_INVALID, "unknown MFMA shape %d", mfma_shape);
  if (data != BEAM_PROBE_DATA_NORMAL && data != BEAM_PROBE_DATA_ZEROS) return fail(BEAM_ERR_INVALID, "unknown data kind %d", data);
  int rc = beam_init();
  if (rc) return rc;
  const int cus = g_dev.cus > 0 && g_dev.cus <= 1024 ? g_dev.cus : 256;
  hipStream_t st = (hipStream_t)stream;
  for (int i = 0; i < warmup; ++i) BEAM_HIP(launch_probe_mfma(dtype, mfma_shape, cus, passes, data == BEAM_PROBE_DATA_ZEROS, st));
  hipEvent_t e0, e1;
  BEAM_HIP(hipEventCreate(&e0));
  BEAM_HIP(hipEventCreate(&e1));
  hipError_t he = hipEventRecord(e0, st);
  for (int i = 0; i < iters && he == hipSuccess; ++i) he = launch_probe_mfma(dtype, mfma_shape, cus, passes, data == BEAM_PROBE_DATA_ZEROS, st);
  if (he == hipSuccess) he = hipEventRecord(e1, st);
  if (he == hipSuccess) he = hipEventSynchronize(e1);
  float ms = 0.0f;
  if (he == hipSuccess) he = hipEventElapsedTime(&ms, e0, e1);
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  if (he != hipSuccess) return hip_fail(he, "matrix-core probe");
  *avg_ms = ms / (float)iters;
  if (flop_per_launch) *flop_per_launch = (double)cus * 4.0 * (double)passes * 1024.0 * 1024.0;
  return BEAM_OK;
}

int beam_stream_create(void** stream) {
  if (!stream) return fail(BEAM_ERR_INVALID, "null stream pointer");
  int rc = beam_init();
  if (rc) return rc;
  hipStream_t s;
  BEAM_HIP(hipStreamCreate(&s));  // default priority
  *stream = s;
  return BEAM_OK;
}

int beam_stream_destroy(void* stream) {
  BEAM_HIP(hipStreamDestroy((hipStream_t)stream));
  return BEAM_OK;
}

int beam_graph_begin_capture(void* stream) {
  if (!stream) return fail(BEAM_ERR_INVALID, "the default stream cannot be captured");
  BEAM_HIP(hipStreamBeginCapture((hipStream_t)stream, hipStreamCaptureModeThreadLocal));
  return BEAM_OK;
}

int beam_graph_end_capture(void* stream, void** graph_exec) {
  if (!graph_exec) return fail(BEAM_ERR_INVALID, "null graph pointer");
  hipGraph_t g = nullptr;
  BEAM_HIP(hipStreamEndCapture((hipStream_t)stream, &g));
  hipGraphExec_t e = nullptr;
  hipError_t err = hipGraphInstantiate(&e, g, nullptr, nullptr, 0);
  (void)hipGraphDestroy(g);
  if (err != hipSuccess) return hip_fail(err, "hipGraphInstantiate");
  *graph_exec = e;
  return BEAM_OK;
}

int beam_graph_launch(void* graph_exec, void* stream) {
  BEAM_HIP(hipGraphLaunch((hipGraphExec_t)graph_exec, (hipStream_t)stream));
  return BEAM_OK;
}

int beam_graph_destroy(void* graph_exec) {
  BEAM_HIP(hipGraphExecDestroy((hipGraphExec_t)graph_exec));
  return BEAM_OK;
}

int beam_event_create(void** event) {
  if (!event) return fail(BEAM_ERR_INVALID, "null event");
  hipEvent_t e;
  BEAM_HIP(hipEventCreate(&e));
  *event = (void*)e;
  return BEAM_OK;
}
int beam_event_record(void* event, void* stream) {
  if (!event) return fail(BEAM_ERR_INVALID, "null event");
  BEAM_HIP(hipEventRecord((hipEvent_t)event, (hipStream_t)stream));
  return BEAM_OK;
}
int beam_event_elapsed_ms(void* start, void* stop, float* ms) {
  if (!start || !stop || !ms) return fail(BEAM_ERR_INVALID, "null event");
  BEAM_HIP(hipEventSynchronize((hipEvent_t)stop));
  BEAM_HIP(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
  return BEAM_OK;
}
int beam_event_destroy(void* event) {
  if (event) BEAM_HIP(hipEventDestroy((hipEvent_t)event));
  return BEAM_OK;
}

int beam_malloc(void** dptr, size_t bytes) {
  if (!dptr) return fail(BEAM_ERR_INVALID, "null dptr");
  *dptr = nullptr;
  if (bytes == 0) return BEAM_OK;
  BEAM_HIP(hipMalloc(dptr, bytes));
  return BEAM_OK;
}
int beam_free(void* dptr) {
  if (dptr) BEAM_HIP(hipFree(dptr));
  return BEAM_OK;
}
int beam_memcpy_h2d(void* dst, const void* src_host, size_t bytes) {
  if (bytes) BEAM_HIP(hipMemcpy(dst, src_host, bytes, hipMemcpyHostToDevice));
  return BEAM_OK;
}
int beam_memcpy_d2h(void* dst_host, const void* src, size_t bytes) {
  if (bytes) BEAM_HIP(hipMemcpy(dst_host, src, bytes, hipMemcpyDeviceToHost));
  return BEAM_OK;
}
int beam_memcpy_d2d(void* dst, const void* src, size_t bytes) {
  if (bytes) BEAM_HIP(hipMemcpy(dst, src, bytes, hipMemcpyDeviceToDevice));
  return BEAM_OK;
}
int beam_memset(void* dptr, int byte, size_t bytes) {
  if (bytes) BEAM_HIP(hipMemset(dptr, byte, bytes));
  return BEAM_OK;
}
int beam_sync(void* stream) {
  BEAM_HIP(hipStreamSynchronize((hipStream_t)stream));
  return BEAM_OK;
}

int beam_host_fill_uniform(void* dst_host, size_t n, int dtype, uint64_t seed, uint64_t tensor_id) {
  if (!dst_host && n) return fail(BEAM_ERR_INVALID, "null destination");
  if (dtype != BEAM_F16 && dtype != BEAM_BF16) return fail(BEAM_ERR_UNSUPPORTED, "dtype %d", dtype);
  uint16_t* out = (uint16_t*)dst_host;
  parallel_for(n, [=](size_t lo, size_t hi) {
    for (size_t i = lo; i < hi; ++i) {
      const uint64_t r = draw(seed, tensor_id, i);
      const float v = (float)(r >> 40) * (1.0f / 8388608.0f) - 1.0f;  // 24 bits -> [-1, 1)
      out[i] = dtype == BEAM_BF16 ? to_bf16_bits(v) : to_f16_bits(v);
    }
  });
  return BEAM_OK;
}

int beam_host_fill_normal(void* dst_host, size_t n, int dtype, uint64_t seed, uint64_t tensor_id, float mean,
                          float scale) {
  if (!dst_host && n) return fail(BEAM_ERR_INVALID, "null destination");
  if (dtype != BEAM_F16 && dtype != BEAM_BF16) return fail(BEAM_ERR_UNSUPPORTED, "dtype %d", dtype);
  uint16_t* out = (uint16_t*)dst_host;
  parallel_for(n, [=](size_t lo, size_t hi) {
    for (size_t i = lo; i < hi; ++i) {
      const uint64_t r = draw(seed, tensor_id, i);
      const double u1 = ((double)(r >> 40) + 1.0) * (1.0 / 16777216.0);      // (0, 1]
      const double u2 = (double)((r >> 8) & 0xffffffull) * (1.0 / 16777216.0);  // [0, 1)
      const double z = std::sqrt(-2.0 * std::log(u1)) * std::cos(6.283185307179586476925 * u2);
      const float v = (float)((double)mean + (double)scale * z);
      out[i] = dtype == BEAM_BF16 ? to_bf16_bits(v) : to_f16_bits(v);
    }
  });
  return BEAM_OK;
}

int beam_dbg_tile_of_workgroup(int wg, int tiles_m, int tiles_n, int group_m, int* tm, int* tn) {
  if (tiles_m < 1 || tiles_n < 1 || group_m < 1 || wg < 0 || wg >= tiles_m * tiles_n || !tm || !tn)
    return fail(BEAM_ERR_INVALID, "bad rasterisation query");
  const TileDivs dv = make_tile_divs(tiles_m, tiles_n, group_m);
  const TileCoord t = tile_of_workgroup(wg, tiles_m, tiles_n, group_m, dv);
  *tm = t.tm;
  *tn = t.tn;
  return BEAM_OK;
}

int beam_dbg_tile_of_workgroup_by_division(int wg, int tiles_m, int tiles_n, int group_m, int* tm, int* tn) {
  if (tiles_m < 1 || tiles_n < 1 || group_m < 1 || wg < 0 || wg >= tiles_m * tiles_n || !tm || !tn)
    return fail(BEAM_ERR_INVALID, "bad rasterisation query");
  const TileCoord t = tile_of_workgroup(wg, tiles_m, tiles_n, group_m);
  *tm = t.tm;
  *tn = t.tn;
  return BEAM_OK;
}

unsigned beam_dbg_fast_div(unsigned n, unsigned d) { return fast_div(n, make_fast_div(d)); }

int beam_dbg_band_xcd_tile(int wg, int tiles_m, int tiles_n, int bx, int* tm, int* tn) {
  if (tiles_m < 1 || tiles_n < 1 || bx < 1 || wg < 0 || wg >= band_xcd_grid(tiles_m, tiles_n, bx) || !tm || !tn)
    return fail(BEAM_ERR_INVALID, "bad rasterisation query");
  const TileCoord t = band_xcd_tile(wg, tiles_m, tiles_n, bx);
  *tm = t.tm;
  *tn = t.tn;
  return BEAM_OK;
}

int beam_dbg_band_xcd_grid(int tiles_m, int tiles_n, int bx) { return band_xcd_grid(tiles_m, tiles_n, bx); }

int beam_dbg_lds_offset(int row, int chunk) { return lds_offset(row, chunk); }

int beam_dbg_kmajor_lds_offset(int k, int n, int block_n) { return kmajor_lds_offset(k, n, block_n); }

int beam_dbg_ln_default_config(int M, int N, int K, int compute_units, beam_tile_cfg* cfg) {
  if (!cfg || M <= 0 || N <= 0 || K <= 0) return fail(BEAM_ERR_INVALID, "bad argument");
  const KernelSet* ks = nullptr;
  return ln_choose_tile(M, N, K, compute_units, cfg, &ks) ? BEAM_OK : BEAM_ERR_UNSUPPORTED;
}

int beam_dbg_w4_kmajor_swizzle(int k) { return w4_kmajor_swizzle(k); }

int beam_dbg_w4_kmajor_read_offset(int wn, int b, int g, int e, int q) { return w4_kmajor_read_offset(wn, b, g, e, q); }

int beam_dbg_band_block_tile(int wg, int tiles_m, int tiles_n, int gb, int gc, int* tm, int* tn) {
  if (tiles_m < 1 || tiles_n < 1 || gb < 1 || gc < 1 || wg < 0 || wg >= band_block_grid(tiles_m, gb, gc) || !tm || !tn)
    return fail(BEAM_ERR_INVALID, "bad band-block query");
  const TileCoord t = band_block_tile(wg, tiles_m, tiles_n, gb, gc);
  *tm = t.tm;
  *tn = t.tn;
  return BEAM_OK;
}

int beam_dbg_band_block_grid(int tiles_m, int gb, int gc) { return band_block_grid(tiles_m, gb, gc); }

int beam_dbg_band_order_tile(int id, int tiles_m, int tiles_n, int group_m, int group_n, int* tm, int* tn) {
  if (tiles_m < 1 || tiles_n < 1 || group_m < 1 || id < 0 || !tm || !tn) return fail(BEAM_ERR_INVALID, "bad band-order query");
  const TileCoord t = band_order_tile(id, tiles_m, tiles_n, group_m, group_n, band_order_divs(tiles_n, group_m, group_n));
  *tm = t.tm;
  *tn = t.tn;
  return BEAM_OK;
}

}  // extern "C"
