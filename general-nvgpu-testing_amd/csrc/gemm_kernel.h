// Tiled gemmrc macro-kernel for gfx950 (MI355X, CDNA4).
//
//   C[m][n] = round_to_16bit( sum_k float(A[m][k]) * float(B[n][k]) )
//
// A is M x K row-major, B is N x K row-major (i.e. a column-major K x N operand), C is
// M x N row-major; accumulation is fp32 on the matrix cores.  This is the operation of the
// reference's custom kernels (cuda/cute_kernels/cute_gemm_128x128.cu:14-191,
// cute_gemm_128x256.cu:17-194; layouts cuda/cute_kernels/main.cc:29-40; fp32 accumulate
// :90; round-to-nearest output :183) rebuilt for 64-wide wavefronts:
//
//   * one workgroup owns a BM x BN tile of C; WAVES_M x WAVES_N wavefronts each own a
//     (BM/WAVES_M) x (BN/WAVES_N) sub-tile made of 16x16 MFMA blocks
//     (v_mfma_f32_16x16x32_{f16,bf16}: 32 K elements per instruction -- on random data it
//     draws measurably less power per flop than the 32x32x16 shape, and this part is power
//     limited long before it is issue limited);
//   * K is walked in tiles of 64 elements; an LDS slot holds one operand tile as rows of 128
//     bytes whose 16-byte chunks are XOR-swizzled (tile_map.h): the 1 KiB-per-wavefront fills
//     and the ds_read_b128 fragment reads are both bank-conflict free;
//   * global -> LDS goes through buffer loads that write LDS directly (no VGPR staging);
//     rows past the matrix edge are outside the buffer descriptor and never touch memory;
//   * A has AST slots and B has BST slots (3 + 2 for the 256x256 tile = all 160 KiB of LDS).
//     While tile h feeds the MFMAs, B tile h+BST-1 and A tile h+AST-1 are in flight, their
//     loads issued one at a time between rows of MFMAs so the vector-memory path (64 B/clk)
//     never sees a burst; one s_barrier per K tile;
//   * fragments are software pipelined one 32-wide step ahead, both operands double buffered
//     in registers; the reads of the next step are issued in the first rows of the current
//     one, between that row's MFMAs, and every row is closed by a scheduling fence, so the
//     order written here is the order executed;
//   * with two wavefronts per SIMD only the older wavefront of each pair issues loads (the
//     hardware lets it win the matrix pipe, so it has time to spare; the younger one is the
//     critical path of every K tile);
//   * B may also be stored [K][N] (B_KMAJOR): its tiles are staged as they lie in memory and
//     transposed on the way into registers by ds_read_b64_tr_b16;
//   * the MFMA is issued with B as the first operand, so every lane ends up with 4
//     consecutive columns of one output row per block: a row's statistics reduce over the
//     lane's own registers first, fp32 output is stored 16 bytes at a time, and 16-bit output
//     takes one trip through the (by then idle) LDS so that it leaves as whole rows of the
//     wavefront's sub-tile, 16 bytes per lane.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "elementwise.h"
#include "tile_map.h"

namespace beam {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x2 __attribute__((ext_vector_type(2)));

template <typename T>
struct ElemTraits;

template <>
struct ElemTraits<_Float16> {
  using vec8 = f16x8;
  using vec4 = f16x4;
  static __device__ __forceinline__ f32x4 mfma(vec8 a, vec8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
};

template <>
struct ElemTraits<__bf16> {
  using vec8 = bf16x8;
  using vec4 = bf16x4;
  static __device__ __forceinline__ f32x4 mfma(vec8 a, vec8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
};

// What the kernel does with the fp32 accumulators.
enum Epilogue : int {
  kEpiStore = 0,    // round to 16-bit and store C
  kEpiPartial = 1,  // store fp32 partial sums of this K slice into the split-K workspace
  kEpiLnStats = 2,  // store fp32 X and per-(row, column-tile) mean / M2 for LayerNorm
  kEpiLnFused = 3,  // LayerNorm in the epilogue: tiles of a row band exchange statistics only
  kEpiStoreSide = 4,  // kEpiStore plus an independent elementwise job (SiLU) streamed through the K loop
  // kEpiStore for a grid smaller than the tile count: a workgroup walks the tiles id, id + grid, ...
  // and has the first operand tiles of the next one in flight while it stores the current one
  kEpiStoreLoop = 5,
  // Measurement only (beam_bench's BEAM_OP_PROBE_SPLITK_LOADS; not in the launch tables): the K loop of
  // kEpiPartial with its global->LDS loads and fragment reads but without MFMAs, and nothing stored.
  // What such a launch costs is the floor that the loads of a split-K launch shape set by themselves.
  kEpiProbeLoads = 6,
  // Split-K in one launch (own launch table, small tiles only): kEpiPartial with its partial sums written
  // through to memory, followed in the same grid by reducing workgroups that add the slices of a tile in
  // slice order as soon as all of them have signalled (splitk_reduce_part_of below).
  kEpiPartialFused = 7,
};
constexpr int kNumEpilogues = 6;  // epilogues of the launch tables

struct GemmParams {
  const void* A;
  const void* B;
  void* C;       // 16-bit [M][N]                                  (kEpiStore)
  float* ws;     // fp32 [splits][M][N] (kEpiPartial) or fp32 [M][N] (kEpiLnStats)
  float* stats;  // fp32 [M][tiles_n][2] = (mean, M2) over the tile's columns (kEpiLnStats)
                 // kEpiLnFused: 8-byte words [tiles_m][tiles_n][BM] = (mean, tag of the launch that wrote it)
  float* next_stats;    // kEpiLnFused: 8-byte words [tiles_m][tiles_n][BM] = (M2, ~tag)
  // kEpiLnFused: the workspace header (tile_map.h: kLnHdr*); never has to be initialised
  int* timeout_flag;
  unsigned ln_nonce;    // kEpiLnFused, kEpiPartialFused: a number no earlier launch of this process had (ln_launch_tag, sk_launch_tag)
  const void* gamma;    // 16-bit [N]                                                   (kEpiLnFused)
  const void* beta;     // 16-bit [N]
  float eps;
  int spin_limit;       // polls (of statistics slots / of a tile's flags) before a waiting thread gives up
  int M, N, K;
  int tiles_m, tiles_n;
  int k_slice;   // K elements per split-K slice, a multiple of kBK
  int splits;    // number of K slices (1 = no split); the grid holds tiles_m * tiles_n * splits workgroups
  int group_m;   // rasterisation group height in tiles (fused LayerNorm: bands per band group)
  int group_n;   // fused LayerNorm: columns of a band group owned by one XCD; 0: whole bands, group_m of them, per XCD;
                 // -1: band after band, workgroup id = band * tiles_n + column (no padding)
  int ln_ids;    // fused LayerNorm on the kernel of gemm_w4.h: ids of that order, padding included; the grid may be smaller
                 // (a workgroup then walks the ids blockIdx, blockIdx + gridDim, ...)
  TileDivs divs; // the tile maps' divisors as multipliers (tile_map.h), made by the host from tiles_m, tiles_n, group_m
  // Side job (kEpiStoreSide): y[i] = silu(x[i]) over a flat 16-bit array.  The whole 8-element
  // groups of the array are cut into units of side_width bytes (16, 8 or 4), dealt out in
  // contiguous runs of side_iters * threads units per workgroup, `threads` units per K tile; the
  // last side_count % 8 elements are done by workgroup 0.  The host picks the narrowest unit with
  // which the job still fits into the K loop, so that every tile carries an equal, small share.
  const void* side_x;
  void* side_y;
  long long side_count;  // elements
  int side_iters;        // K tiles' worth of units per workgroup
  int side_width;        // bytes per unit
  int c_streaming;       // kEpiStoreLoop: store C non-temporal
  // kEpiPartialFused: word kSkTimeout, then from word kSkFlags on one flag per (tile, part of the tile, slice);
  // behind the partial sums in the caller's workspace.  Never has to be initialised (see sk_launch_tag).
  int* sk_sync;
  int sk_out;  // kEpiPartialFused: outputs per thread of a reducing workgroup (4, 2 or 1)
  // kEpiPartialFused, measurement only: 1 = no reducing workgroups; the multiplying workgroup of (tile, slice s)
  // reduces parts s, s + splits, ... of its tile itself.  Every multiplying workgroup must then be resident at once.
  int sk_self;
};

// ---- statistics exchange of the fused GEMM+LayerNorm (both K loops: this file's and gemm_w4.h's) ----------
// A tile publishes, per row, two 8-byte words: (mean, tag) and (M2, ~tag), each with one device-scope atomic
// store.  Such stores go straight through the XCD-private L2 to memory and the device-scope loads of the
// gather come straight from it, so the exchange needs no cache-wide write-back / invalidate (a
// __threadfence() per workgroup costs tens of microseconds here).  `tag` is different for every launch: the
// host hands every fused launch a fresh nonce, and a launch recorded in a graph, whose arguments repeat, is
// preceded by a one-thread kernel that moves on a counter in the workspace header.  A word that does not carry
// the launch's tag is "not published yet", whatever it holds: memory never used before, statistics of an
// earlier launch or of another shape, or somebody else's data.  So a workspace needs no preparation, no
// clearing between launches and no state on the host.  (A stray word passes for published with probability
// 2^-32 per word, and both words of a row have to.)
__device__ __forceinline__ unsigned ln_launch_tag(const GemmParams& p) {
  unsigned x = p.ln_nonce + (unsigned)p.timeout_flag[kLnHdrReplay] * 0x9E3779B1u;  // uniform: nobody writes it during a launch
  x ^= x >> 16;
  x *= 0x7feb352du;
  x ^= x >> 15;
  x *= 0x846ca68bu;
  x ^= x >> 16;
  return x | 1u;  // never 0: a zeroed header then never reads as "timed out"
}

// Workgroup 0 records which launch the header speaks of.
__device__ __forceinline__ void ln_sign_header(const GemmParams& p, unsigned tag) {
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    p.timeout_flag[kLnHdrMagic] = kLnMagic;
    p.timeout_flag[kLnHdrLaunchTag] = (int)tag;
  }
}

__device__ __forceinline__ void ln_publish(const GemmParams& p, size_t slot, float mean, float m2, unsigned tag) {
  const unsigned long long w0 = (unsigned long long)__float_as_uint(mean) | ((unsigned long long)tag << 32);
  const unsigned long long w1 = (unsigned long long)__float_as_uint(m2) | ((unsigned long long)(~tag) << 32);
  __hip_atomic_store((unsigned long long*)p.stats + slot, w0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __hip_atomic_store((unsigned long long*)p.next_stats + slot, w1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Gathers the (mean, M2) pairs of slots [first, first + n_slots) into `gathered` (LDS, 8 bytes per slot):
// batches of INFLIGHT slots per thread, the missing part of a batch fetched again (one bounded budget of tries
// per thread) until both words of each of its slots carry the tag.  A thread that runs out of budget raises the
// header's flag and poisons the pairs still missing, so that the rows concerned come out as NaN instead of as
// plausible numbers.
template <int NT, int INFLIGHT = 8>
__device__ __forceinline__ void ln_gather(const GemmParams& p, unsigned tag, size_t first, int n_slots, int tid,
                                          unsigned long long* gathered) {
  const unsigned long long* w0s = (const unsigned long long*)p.stats + first;
  const unsigned long long* w1s = (const unsigned long long*)p.next_stats + first;
  const unsigned not_tag = ~tag;
  int polls = 0;
  for (int q0 = tid; q0 < n_slots; q0 += INFLIGHT * NT) {
    unsigned long long a[INFLIGHT], b[INFLIGHT];
    // A batch is fetched with all its loads in flight at once; what does not carry the launch's tag yet is fetched
    // again, again all of it at once and nothing else, after a pause that grows with the number of tries: a try
    // costs one round trip to memory for the batch, and waiting workgroups do not flood the memory system that
    // the tiles they wait for still need.
    unsigned missing = 0;  // bit u: slot u of the batch is still to be fetched
#pragma unroll
    for (int u = 0; u < INFLIGHT; ++u) missing |= (q0 + u * NT < n_slots) ? (1u << u) : 0u;
    for (;;) {
#pragma unroll
      for (int u = 0; u < INFLIGHT; ++u) {
        if (missing & (1u << u)) {
          a[u] = __hip_atomic_load(w0s + q0 + u * NT, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          b[u] = __hip_atomic_load(w1s + q0 + u * NT, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
      }
      // (a negative limit: treat everything as unpublished -- how the host forces the time-out in a test)
#pragma unroll
      for (int u = 0; u < INFLIGHT; ++u)
        if ((missing & (1u << u)) && (unsigned)(a[u] >> 32) == tag && (unsigned)(b[u] >> 32) == not_tag && p.spin_limit >= 0)
          missing &= ~(1u << u);
      if (missing == 0) break;
      if (++polls > p.spin_limit) {
        p.timeout_flag[kLnHdrTimeout] = (int)tag;
#pragma unroll
        for (int u = 0; u < INFLIGHT; ++u)
          if (missing & (1u << u)) {
            a[u] = 0x7fc00000ull;
            b[u] = 0x7fc00000ull;
          }
        break;
      }
      for (int z = 0; z < (polls < 8 ? polls : 8); ++z) __builtin_amdgcn_s_sleep(8);
    }
#pragma unroll
    for (int u = 0; u < INFLIGHT; ++u) {
      const int q = q0 + u * NT;
      if (q < n_slots) gathered[q] = (a[u] & 0xffffffffull) | (b[u] << 32);
    }
  }
}

// ---- split-K in one launch (kEpiPartialFused) -----------------------------------------------------------
// The grid holds the tiles x slices workgroups of kEpiPartial and, behind them, one reducing workgroup per
// (tile, part).  Workgroups are placed in id order, so a reducing workgroup starts only once every multiplying
// workgroup has been placed (on its own XCD; the other XCDs place theirs whatever a waiting workgroup here does):
// what it waits for always arrives, with any number of rounds and on a device shared with other work.  The
// partial sums leave with device-scope (write-through) stores, and the flag that announces them is stored after
// those have been acknowledged; the reducing workgroup reads flags and sums with device-scope loads, which come
// from memory, not from an XCD-private L2.  A flag counts only if it equals the launch's tag (a hash of a nonce
// that no earlier launch of the process had), so the workspace needs no clearing; the reducer clears the flags it
// has consumed, so a graph replay, whose arguments and therefore tag repeat, starts clean as well.
__device__ __forceinline__ unsigned sk_launch_tag(unsigned nonce) {
  unsigned x = nonce;
  x ^= x >> 16;
  x *= 0x7feb352du;
  x ^= x >> 15;
  x *= 0x846ca68bu;
  x ^= x >> 16;
  return x | 1u;  // never 0: a cleared flag is never "set"
}
constexpr int kAuxDeviceScope = 16;  // sc1: the access is performed at device scope (through the L2, to memory)

// Buffer descriptor word 3 for gfx9-family raw buffers: 32-bit data format, no swizzle.
constexpr int kRsrcFlags = 0x00020000;
// Byte offset that is out of range of every descriptor built here.
constexpr unsigned kOobOffset = 0x7fffff00u;

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, unsigned bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, kRsrcFlags);
}

// 16 bytes of output, written through the L2 to memory (device scope) instead of left dirty in it.  A kernel ends
// only when its dirty lines have been written back; for the one-tile-per-CU kernels, whose stores all come at the
// very end, writing through moves that work under the other workgroups' last K tiles: 1024^3 5.5 -> 5.3 us,
// 2048 x 2048 x 512 7.1 -> 6.5 us, 3072^3 48.0 -> 47.0 us, 2048^3 and outputs of tens of MB unchanged (same machine,
// the two builds in turn; non-temporal stores, tried beside it, lose 8% at 3000 x 5000 x 2000).
// (The wait states behind it: a store of more than 8 bytes reads its data registers over several cycles, and a
// vector instruction that overwrites them must not follow at once.  The compiler keeps that distance for stores it
// emits itself; it does not look into assembly text.)
__device__ __forceinline__ void store_through_16(void* dst, i32x4 v) {
  asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 2" ::"v"(dst), "v"(v) : "memory");
}

// s_waitcnt vmcnt(N) lgkmcnt(0): at most N of this wavefront's buffer loads still in flight,
// all of its LDS reads returned.
template <int N>
__device__ __forceinline__ void wait_vm_and_lds() {
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
  __builtin_amdgcn_s_waitcnt(0x0070 | (N & 15) | ((N >> 4) << 14));
}

// s_waitcnt lgkmcnt(N): at most N of this wavefront's LDS reads still in flight.
template <int N>
__device__ __forceinline__ void wait_lds() {
  static_assert(N >= 0 && N < 16, "lgkmcnt is a 4-bit counter");
  __builtin_amdgcn_s_waitcnt(0xC07F | (N << 8));
}

// Workgroup barrier without the memory fence of __syncthreads(): the fence would wait for
// every outstanding LDS fill (vmcnt(0)) and serialise the pipeline.  The waits the data
// hazards need are issued explicitly by the caller.
__device__ __forceinline__ void bare_barrier() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

// A-slot count of the "deep" pipeline of a tile shape: as many slots as 160 KiB of LDS hold with one
// slot fewer for B, at most 8.  Small tiles get a long prefetch queue this way, which is what a
// split-K workgroup (few tiles in flight per CU, every byte fetched exactly once) needs to keep HBM busy.
constexpr int deep_a_slots(int BM, int BN) {
  int a = 8;
  while (a > 3 && (a * BM + (a - 1) * BN) * kRowBytes > 160 * 1024) --a;
  return a;
}

template <typename T, int BM, int BN, int WAVES_M, int WAVES_N, int EPI, int AST, int BST, bool B_KMAJOR = false>
struct GemmTile {
  using Traits = ElemTraits<T>;
  using vec8 = typename Traits::vec8;
  using vec4 = typename Traits::vec4;

  static constexpr int NW = WAVES_M * WAVES_N;
  static constexpr int NT = NW * 64;
  // Wavefronts that issue the global->LDS loads.  With two wavefronts per SIMD the hardware favours the
  // older one of each pair (wavefronts 0 .. NW/2-1) when both have an MFMA ready, so those finish a K tile
  // early and idle at the barrier while the younger ones are the critical path: the older half therefore
  // issues every load, two wavefronts' worth each, and the younger half none (8192^3: +3.7%; on all-zero
  // data, where the power cap does not hide it, +21%).
  static constexpr int LDW = NW >= 8 ? NW / 2 : NW;
  static constexpr int NTL = LDW * 64;  // threads that issue loads
  static constexpr int TM = BM / WAVES_M;  // wavefront tile
  static constexpr int TN = BN / WAVES_N;
  static constexpr int FM = TM / 16;       // MFMA blocks per wavefront tile
  static constexpr int FN = TN / 16;
  static constexpr int KSTEPS = kBK / 32;  // MFMA K steps per tile (= 2)
  static constexpr int A_BYTES = BM * kRowBytes;
  static constexpr int B_BYTES = BN * kRowBytes;
  static constexpr int B_REGION = AST * A_BYTES;  // A slots first, then B slots
  static constexpr int LDS_BYTES = AST * A_BYTES + BST * B_BYTES;
  static constexpr int LA = (BM * kChunksPerRow) / NTL;  // buffer loads per wavefront per A tile
  static constexpr int LB = (BN * kChunksPerRow) / NTL;
  static constexpr int LOADS = LA + LB;
  static constexpr int ROWS = KSTEPS * FM;                 // rows of MFMAs per K tile
  static constexpr int PER_ROW = (LOADS + ROWS - 1) / ROWS;  // buffer loads issued after each row
  // Loads that may still be in flight when tile h is needed: the A tiles and B tiles beyond h.
  // The side job adds SV buffer stores and SV buffer loads at the end of every K tile of a loader
  // wavefront; the fills a tile waits for were issued min(AST, BST) - 1 tiles earlier.
  static constexpr bool SIDE = (EPI == kEpiStoreSide);
  static constexpr bool LOOP = (EPI == kEpiStoreLoop);
  // global stores of one wavefront per tile when its output leaves as whole rows, 16 bytes per lane
  static constexpr int NST = TM * (TN / 8) / 64;
  static constexpr int SV = NW / LDW;  // side vectors per loader thread per K tile
  static constexpr int WAIT_STEADY =
      (AST - 2) * LA + (BST - 2) * LB + (SIDE ? 2 * SV * ((AST < BST ? AST : BST) - 1) : 0);

  static_assert(KSTEPS == 2, "the step pipeline below is written for two 32-wide steps per tile");
  static_assert(TM % 16 == 0 && TN % 16 == 0, "wavefront tile must be made of 16x16 blocks");
  static_assert((BM * kChunksPerRow) % NTL == 0 && (BN * kChunksPerRow) % NTL == 0,
                "every wavefront must move a whole number of 1 KiB chunks per tile");
  static_assert(AST >= 2 && BST >= 2 && (AST == BST || AST == BST + 1), "slot counts");
  static_assert(LDS_BYTES <= 160 * 1024, "LDS budget of one CU");
  static_assert(WAIT_STEADY < 64, "vmcnt range");
  static_assert(BM * 8 * (4 * WAVES_N + 2) <= LDS_BYTES, "row statistics scratch of the LayerNorm epilogues");

  // Chunk q = i * NTL + tid of an operand tile lives at LDS byte q * 16 of its slot, which is
  // row q / 8, position q % 8; the position holds logical chunk position ^ swizzle_of_row(row).
  static __device__ __forceinline__ unsigned chunk_voffset(int q, int K) {
    const int row = q >> 3;
    const int chunk = (q & 7) ^ swizzle_of_row(row);
    return (unsigned)row * (unsigned)K * 2u + (unsigned)chunk * 16u;
  }

  // kEpiPartialFused: reducing workgroup r = (tile, part).  Waits until the tile's slices have all signalled,
  // adds their partial sums in slice order 0, 1, 2, ... (the order of splitk_reduce_kernel: same bits) and
  // rounds once.  A thread owns OUT = p.sk_out (4, 2 or 1) consecutive columns of one row of the part: the host
  // makes the parts small when there are few tiles, so that the reads spread over many CUs (a CU takes in its
  // share of the partial sums at well under 100 GB/s; 64 workgroups reading 128 KiB each took 2 us).
  template <int OUT>
  static __device__ __forceinline__ void splitk_reduce_part_of(const GemmParams& p, int r) {
    constexpr int P = sk_parts_per_tile(BM, BN, NT, OUT);
    constexpr int PART_ROWS = NT * OUT / BN;
    static_assert(P >= 1 && P <= NT && P * NT * OUT == BM * BN && PART_ROWS * BN == NT * OUT, "parts tile the tile");
    typedef float acc_t __attribute__((ext_vector_type(OUT)));
    typedef T out_t __attribute__((ext_vector_type(OUT)));
    const int tid = threadIdx.x, lane = tid & 63;
    const int t = r / P, q = r - t * P;
    const int tm = t / p.tiles_n, tn = t - tm * p.tiles_n;
    const int M = p.M, N = p.N, S = p.splits;
    const int tag = (int)sk_launch_tag(p.ln_nonce);
    int* flags = p.sk_sync + kSkFlags + (size_t)r * S;
    if (r == 0 && tid == 0) {  // which launch the header speaks of
      p.sk_sync[kSkMagic] = kSkMagicValue;
      p.sk_sync[kSkLaunchTag] = tag;
    }
    // every wavefront polls for itself (S <= 64: one flag per lane); one bounded budget
    bool arrived = false;
    for (int polls = 0; polls <= p.spin_limit; ++polls) {
      const int v = lane < S ? __hip_atomic_load(flags + lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : tag;
      if (__all(v == tag)) {
        arrived = true;
        break;
      }
      __builtin_amdgcn_s_sleep(1);
    }
    // The partial sums are read after the flags, in the hardware (the loop's exit waits for the flags' values) and
    // in the compiler (relaxed atomic loads order nothing by themselves; the loads below must not be hoisted).
    asm volatile("" ::: "memory");
    const int m = tm * BM + q * PART_ROWS + tid / (BN / OUT);
    const int n = tn * BN + (tid % (BN / OUT)) * OUT;
    const bool valid = m < M && n < N;  // N is a multiple of 4: a thread's columns exist together
    const unsigned off = valid ? ((unsigned)m * (unsigned)N + (unsigned)n) * 4u : kOobOffset;
    const unsigned slice_bytes = (unsigned)M * (unsigned)N * 4u;
    auto load = [&](int z) __attribute__((always_inline)) -> acc_t {
      const __amdgpu_buffer_rsrc_t rs = make_rsrc(p.ws + (size_t)z * M * N, slice_bytes);
      if constexpr (OUT == 4) return __builtin_bit_cast(acc_t, __builtin_amdgcn_raw_buffer_load_b128(rs, (int)off, 0, kAuxDeviceScope));
      else if constexpr (OUT == 2) return __builtin_bit_cast(acc_t, __builtin_amdgcn_raw_buffer_load_b64(rs, (int)off, 0, kAuxDeviceScope));
      else return __builtin_bit_cast(acc_t, __builtin_amdgcn_raw_buffer_load_b32(rs, (int)off, 0, kAuxDeviceScope));
    };
    acc_t s = 0.0f;
    int z = 0;
    // batches of 16, 8, 4, 2, 1 slices: the loads of a batch in flight before the first add
    auto batch = [&](auto n_tag) __attribute__((always_inline)) {
      constexpr int NB = decltype(n_tag)::value;
      while (z + NB <= S) {
        acc_t v[NB];
#pragma unroll
        for (int u = 0; u < NB; ++u) v[u] = load(z + u);
        if (z == 0) s = v[0];
        else s += v[0];
#pragma unroll
        for (int u = 1; u < NB; ++u) s += v[u];
        z += NB;
      }
    };
    if constexpr (OUT < 4) batch(std::integral_constant<int, 32>{});
    batch(std::integral_constant<int, 16>{});
    batch(std::integral_constant<int, 8>{});
    batch(std::integral_constant<int, 4>{});
    batch(std::integral_constant<int, 2>{});
    batch(std::integral_constant<int, 1>{});
    __syncthreads();  // every wavefront has seen the flags: they can go
    if (tid < S) __hip_atomic_store(flags + tid, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (!arrived) {  // never on a working device; visible in the data and in the workspace if it happens
      if (tid == 0) p.sk_sync[kSkTimeout] = tag;
      s = __builtin_nanf("");
    }
    if (valid) {
      out_t o;
#pragma unroll
      for (int e = 0; e < OUT; ++e) o[e] = (T)s[e];
      *(out_t*)((T*)p.C + (size_t)m * N + n) = o;
    }
  }

  static __device__ __forceinline__ void run(const GemmParams& p, char* smem) {
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave % WAVES_M;
    const int wn = wave / WAVES_M;

    if constexpr (EPI == kEpiPartialFused) {
      const int multiplying = p.tiles_m * p.tiles_n * p.splits;
      if ((int)blockIdx.x >= multiplying) {  // (uniform)
        const int r = (int)blockIdx.x - multiplying;
        if (p.sk_out == 4) splitk_reduce_part_of<4>(p, r);
        else if (p.sk_out == 2) splitk_reduce_part_of<2>(p, r);
        else splitk_reduce_part_of<1>(p, r);
        return;
      }
    }

    // Fused LayerNorm uses the band-block order, which keeps the workgroups that must exchange
    // statistics resident together -- and, because a band's workgroups have consecutive ids and workgroups are
    // placed in id order, lets a launch that gets only part of the device finish band by band.  Its grid is
    // padded and the surplus workgroups leave here.  (Where the padding would cost a round of workgroups the
    // host asks for the plain band-after-band order, which has the same property and no padding.)
    // Split-K walks (slice, tile) pairs slice by slice, and the XCD remap gives every XCD one
    // contiguous range of pairs: the tiles that read the same K slice of A and B share an L2.
    TileCoord tc;
    int slice = 0;
    if (EPI == kEpiLnFused) {
      tc = p.group_n > 0    ? band_block_tile(blockIdx.x, p.tiles_m, p.tiles_n, p.group_m, p.group_n)
           : p.group_n == 0 ? band_xcd_tile(blockIdx.x, p.tiles_m, p.tiles_n, p.group_m)
                            : TileCoord{(int)blockIdx.x / p.tiles_n, (int)blockIdx.x % p.tiles_n};
      if (tc.tm < 0) return;
    } else if (p.splits > 1) {
      const int tiles = p.tiles_m * p.tiles_n;
      const int pid = xcd_remap(blockIdx.x, tiles * p.splits);
      slice = (int)fast_div((unsigned)pid, p.divs.tiles);
      tc = grouped_tile(pid - slice * tiles, p.tiles_m, p.tiles_n, p.group_m, p.divs);
    } else {
      tc = tile_of_workgroup(blockIdx.x, p.tiles_m, p.tiles_n, p.group_m, p.divs);
    }
    int row0 = tc.tm * BM;
    int col0 = tc.tn * BN;
    const int M = p.M, N = p.N, K = p.K;

    // K range of this slice.
    const int kb = slice * p.k_slice;
    int klen = K - kb;
    if (klen > p.k_slice) klen = p.k_slice;
    if (klen < 0) klen = 0;
    const int kt_full = klen / kBK;
    const int k_tail = klen - kt_full * kBK;         // multiple of 8 (host guarantees K % 8 == 0)
    const int n_tiles = kt_full + (k_tail ? 1 : 0);  // the short tile, if any, is tile 0

    // Buffer descriptors cover exactly the rows of this tile that exist and the K range of
    // this slice; anything else is out of range: reads return zero and touch no memory.
    int rows_a = (M - row0) < BM ? (M - row0) : BM;
    int rows_b = (N - col0) < BN ? (N - col0) : BN;
    const T* a_base = (const T*)p.A + ((size_t)row0 * K + kb);
    // B as [N][K] (rows of K): like A.  B as [K][N] (B_KMAJOR): the tile's columns start at col0 of
    // row kb; a descriptor is made per K tile (load_b) so that it ends with the tile's last row.
    const T* b_base = B_KMAJOR ? (const T*)p.B + ((size_t)kb * N + col0) : (const T*)p.B + ((size_t)col0 * K + kb);
    unsigned bytes_a = klen > 0 ? ((unsigned)(rows_a - 1) * K + klen) * 2u : 0u;
    unsigned bytes_b = klen > 0 ? ((unsigned)(rows_b - 1) * K + klen) * 2u : 0u;
    const __amdgpu_buffer_rsrc_t rsrc_a = make_rsrc(a_base, bytes_a);
    const __amdgpu_buffer_rsrc_t rsrc_b = make_rsrc(b_base, bytes_b);
    // kEpiStoreLoop: the same for the next tile of this workgroup (neither split-K nor the [K][N]
    // layout nor a short K tile exist in that mode: the host sees to it)
    auto set_tile = [&](int id) __attribute__((always_inline)) {
      tc = tile_of_workgroup(id, p.tiles_m, p.tiles_n, p.group_m, p.divs);
      row0 = tc.tm * BM;
      col0 = tc.tn * BN;
      rows_a = (M - row0) < BM ? (M - row0) : BM;
      rows_b = (N - col0) < BN ? (N - col0) : BN;
      a_base = (const T*)p.A + (size_t)row0 * K;
      b_base = (const T*)p.B + (size_t)col0 * K;
      bytes_a = ((unsigned)(rows_a - 1) * K + klen) * 2u;
      bytes_b = ((unsigned)(rows_b - 1) * K + klen) * 2u;
    };

    unsigned voff_a[LA], voff_b[LB];
#pragma unroll
    for (int i = 0; i < LA; ++i) voff_a[i] = chunk_voffset(i * NTL + tid, K);
#pragma unroll
    for (int i = 0; i < LB; ++i) {
      if (B_KMAJOR) {
        // LDS position q of the stage: row k = q / CPR, and the chunk that lives there is position ^ swizzle
        constexpr int CPR = BN / 8;
        const int q = i * NTL + tid;
        const int k = q / CPR;
        const int chunk = (q % CPR) ^ kmajor_swizzle(k, BN);
        voff_b[i] = ((unsigned)k * (unsigned)N + (unsigned)chunk * 8u) * 2u;
      } else {
        voff_b[i] = chunk_voffset(i * NTL + tid, K);
      }
    }

    // First K element (inside the slice) of tile t: the short tile comes first.
    auto tile_koff = [&](int t) { return k_tail ? (t == 0 ? kt_full * kBK : (t - 1) * kBK) : t * kBK; };

    // ---- global -> LDS ------------------------------------------------------------------
    // One buffer load (1 KiB per wavefront) of A tile t / B tile t into its slot.  Tiles past the end
    // of the K range get an empty descriptor: the load is still issued and counted (the pipeline below
    // has no special cases for its last iterations) but touches no memory.
    auto load_a = [&](int i, int t) __attribute__((always_inline)) {
      char* dst = smem + (t % AST) * A_BYTES + wave * 1024 + i * (NTL * 16);
      const __amdgpu_buffer_rsrc_t r = make_rsrc(a_base, t < n_tiles ? bytes_a : 0u);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (__attribute__((address_space(3))) void*)dst, 16,
                                               (int)voff_a[i], tile_koff(t) * 2, 0, 0);
    };
    auto load_b = [&](int i, int t) __attribute__((always_inline)) {
      char* dst = smem + B_REGION + (t % BST) * B_BYTES + wave * 1024 + i * (NTL * 16);
      if (B_KMAJOR) {
        // Rows koff .. koff + kBK of the slice, as many as exist: rows past the end of K and the
        // columns past the last row's end are out of range and read as zeros.  (Columns past N in
        // earlier rows read the next row's data; they only feed output columns that do not exist.)
        const int koff = tile_koff(t);
        int rows = klen - koff;
        if (rows > kBK) rows = kBK;
        const unsigned bytes = (t < n_tiles && rows > 0) ? ((unsigned)(rows - 1) * N + rows_b) * 2u : 0u;
        const __amdgpu_buffer_rsrc_t r = make_rsrc(b_base + (size_t)koff * N, bytes);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (__attribute__((address_space(3))) void*)dst, 16,
                                                 (int)voff_b[i], 0, 0, 0);
      } else {
        const __amdgpu_buffer_rsrc_t r = make_rsrc(b_base, t < n_tiles ? bytes_b : 0u);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (__attribute__((address_space(3))) void*)dst, 16,
                                                 (int)voff_b[i], tile_koff(t) * 2, 0, 0);
      }
    };
    // The short tile goes through registers so that chunks at or past `kvalid` are zero-filled.
    // (A K-major B needs none of this: its rows past the end of K are out of range by themselves.)
    const bool loader = LDW == NW || wave < LDW;
    auto fill_short_tile = [&](int kvalid) __attribute__((always_inline)) {
      if (!loader) return;
      const int koff = tile_koff(0);
      i32x4 ra[LA], rb[LB];
#pragma unroll
      for (int i = 0; i < LA; ++i) {
        const int q = i * NTL + tid;
        const int chunk = (q & 7) ^ swizzle_of_row(q >> 3);
        const unsigned off = (chunk * 8 < kvalid) ? voff_a[i] + (unsigned)koff * 2u : kOobOffset;
        ra[i] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_a, (int)off, 0, 0);
      }
      if (!B_KMAJOR) {
#pragma unroll
        for (int i = 0; i < LB; ++i) {
          const int q = i * NTL + tid;
          const int chunk = (q & 7) ^ swizzle_of_row(q >> 3);
          const unsigned off = (chunk * 8 < kvalid) ? voff_b[i] + (unsigned)koff * 2u : kOobOffset;
          rb[i] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_b, (int)off, 0, 0);
        }
      }
      char* sa = smem + tid * 16;
      char* sb = smem + B_REGION + tid * 16;
#pragma unroll
      for (int i = 0; i < LA; ++i) *(i32x4*)(sa + i * (NTL * 16)) = ra[i];
      if (!B_KMAJOR) {
#pragma unroll
        for (int i = 0; i < LB; ++i) *(i32x4*)(sb + i * (NTL * 16)) = rb[i];
      }
    };

    // ---- LDS -> MFMA fragments ----------------------------------------------------------
    // 16x16x32 operand: lane l supplies row (l & 15), K elements 8*(l>>4) .. +7 of the step.
    int frag_off[KSTEPS];
#pragma unroll
    for (int kk = 0; kk < KSTEPS; ++kk) frag_off[kk] = lds_offset(lane & 15, 4 * kk + (lane >> 4));
    const int a_wave_off = wm * TM * kRowBytes;
    const int b_wave_off = B_KMAJOR ? 0 : wn * TN * kRowBytes;
    // K-major B: a fragment (16 columns x 32 rows of k) is two transposing 8-byte reads.  In the
    // 16-lane group g = lane >> 4, lane 4*e + q points at row k = 8*g + e (+4 for the second read),
    // columns 4*q .. 4*q + 3 of the block; the read hands lane i of the group column i of rows
    // 8*g .. 8*g + 3: the same register contents as the 16-byte read of the [N][K] layout.
    int bfrag_off[FN];
    if (B_KMAJOR) {
#pragma unroll
      for (int j = 0; j < FN; ++j)
        bfrag_off[j] = kmajor_lds_offset(8 * (lane >> 4) + ((lane >> 2) & 3), wn * TN + j * 16 + 4 * (lane & 3), BN);
    }
    // The transposing reads are inline assembly: given the intrinsic, the compiler orders every
    // LDS read it can see behind all outstanding global->LDS fills (vmcnt(0)), which would
    // serialise the pipeline.  Results of inline assembly are not tracked by the compiler's
    // wait-count insertion, so the step below waits for them explicitly.
    auto read_b_fragment = [&](const char* sb, int j) __attribute__((always_inline)) -> vec8 {
      if constexpr (B_KMAJOR) {
        const unsigned addr = (unsigned)(size_t)(__attribute__((address_space(3))) const char*)(sb + bfrag_off[j]);
        vec4 lo, hi;
        asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(lo) : "v"(addr));
        asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(hi) : "v"(addr), "n"(4 * BN * 2));
        return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
      } else {
        return *(const vec8*)(sb + j * 16 * kRowBytes);
      }
    };

    f32x4 acc[FM][FN];
    auto zero_acc = [&]() __attribute__((always_inline)) {
#pragma unroll
      for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
          for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.0f;
    };

    // Fragments: both operands are double-buffered in registers (set 0 / set 1).  While the MFMAs
    // of one step consume one set, the LDS reads of the next step fill the other.  They start as
    // zeros so that the very first step of the pipeline multiplies nothing.
    vec8 fa0[FM], fa1[FM], fb0[FN], fb1[FN];
    auto zero_fragments = [&]() __attribute__((always_inline)) {
#pragma unroll
      for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          fa0[i][e] = 0;
          fa1[i][e] = 0;
        }
#pragma unroll
      for (int j = 0; j < FN; ++j)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          fb0[j][e] = 0;
          fb1[j][e] = 0;
        }
    };

    // ---- side job: state and pieces ------------------------------------------------------
    // side_buf holds the units loaded during the previous K tile; step 1 pushes them through silu
    // in place, a pair of elements at a time on evenly spaced MFMA rows, and they are stored at the
    // end of the tile, right before the load of the next units.  Units outside this workgroup's
    // run get an offset outside the descriptor: the load returns zeros and the store is dropped.
    // Only the loader wavefronts do this work, SV units each.  They are the older wavefront of
    // their SIMD, win the arbitration for the matrix core and reach the barrier of every tile with
    // some hundred cycles to spare, while the younger ones set the pace of the loop: arithmetic
    // given to the older wavefront fills that slack, the same arithmetic in the younger one
    // lengthens the tile.
    const unsigned side_bytes = SIDE ? (unsigned)((p.side_count >> 3) << 4) : 0u;
    const __amdgpu_buffer_rsrc_t rsrc_sx = make_rsrc(p.side_x, side_bytes);
    const __amdgpu_buffer_rsrc_t rsrc_sy = make_rsrc(p.side_y, side_bytes);
    const unsigned side_v0 = SIDE ? ((unsigned)blockIdx.x * (unsigned)p.side_iters * NT + tid) : 0u;
    int side_buf[SV][4];  // pairs of elements: x when loaded, overwritten pair by pair with silu(x)
#pragma unroll
    for (int s = 0; s < SV; ++s) {
#pragma unroll
      for (int e = 0; e < 4; ++e) side_buf[s][e] = 0;
    }
    // W: bytes per unit (compile time inside each version of the loop).  The host picks wide units
    // only for an array that is large beside the GEMM; its traffic is then marked non-temporal
    // (auxiliary bit 1), so that lines written once do not push the GEMM's operands out of the L2:
    // 900 -> 866 us for 8192^3 carrying 256 Mi elements.  A small array (4-byte units) is better
    // left in the cache, for whoever reads y next.
    auto side_offset = [&](int it, int s, int W) __attribute__((always_inline)) {  // thread tid of the loaders owns units tid + s * NTL of a tile
      return (it >= 0 && it < p.side_iters) ? (side_v0 + (unsigned)it * NT + (unsigned)s * NTL) * (unsigned)W : kOobOffset;
    };
    auto side_load = [&](int it, auto w_tag) __attribute__((always_inline)) {
      constexpr int W = decltype(w_tag)::value;
      constexpr int AUX = W >= 8 ? 2 : 0;
#pragma unroll
      for (int s = 0; s < SV; ++s) {
        const int off = (int)side_offset(it, s, W);
        if constexpr (W == 16) {
          const i32x4 v = __builtin_amdgcn_raw_buffer_load_b128(rsrc_sx, off, 0, AUX);
#pragma unroll
          for (int e = 0; e < 4; ++e) side_buf[s][e] = v[e];
        } else if constexpr (W == 8) {
          const i32x2 v = __builtin_amdgcn_raw_buffer_load_b64(rsrc_sx, off, 0, AUX);
          side_buf[s][0] = v[0];
          side_buf[s][1] = v[1];
        } else {
          side_buf[s][0] = __builtin_amdgcn_raw_buffer_load_b32(rsrc_sx, off, 0, AUX);
        }
      }
    };
    auto side_store = [&](int it, auto w_tag) __attribute__((always_inline)) {
      constexpr int W = decltype(w_tag)::value;
      constexpr int AUX = W >= 8 ? 2 : 0;
#pragma unroll
      for (int s = 0; s < SV; ++s) {
        const int off = (int)side_offset(it, s, W);
        const int* o = side_buf[s];
        if constexpr (W == 16) __builtin_amdgcn_raw_buffer_store_b128(i32x4{o[0], o[1], o[2], o[3]}, rsrc_sy, off, 0, AUX);
        else if constexpr (W == 8) __builtin_amdgcn_raw_buffer_store_b64(i32x2{o[0], o[1]}, rsrc_sy, off, 0, AUX);
        else __builtin_amdgcn_raw_buffer_store_b32(o[0], rsrc_sy, off, 0, AUX);
      }
    };
    auto side_pair = [&](int e) __attribute__((always_inline)) {  // pair e of every unit this thread holds
#pragma unroll
      for (int s = 0; s < SV; ++s) {
        typedef T pair_t __attribute__((ext_vector_type(2)));
        const pair_t x = __builtin_bit_cast(pair_t, side_buf[s][e]);
        const pair_t y = {silu_16<T>(x[0]), silu_16<T>(x[1])};
        side_buf[s][e] = __builtin_bit_cast(int, y);
      }
    };

    // One pipeline step = FM rows of FN MFMAs on the fragments in (fa_cur, fb_cur).  The FM + FN
    // LDS reads of the next step's fragments (from sa, sb into fa_nxt, fb_nxt; B first, it is
    // needed by the next step's very first MFMA) are issued at the head of the first READ_ROWS
    // rows, so the last of them has a row or more of MFMA time to land before the step ends; each
    // row also carries its share of the tile's buffer loads.  A scheduling fence closes every row:
    // left alone, the compiler sinks the reads to the end of the step and re-uses fragment
    // registers across the two sets, and the step then starts by waiting for its own reads.
    //   ROW0: index of the step's first row inside the tile (the loads are dealt out row by row).
    auto step = [&](const char* sa, const char* sb, vec8(&fa_cur)[FM], vec8(&fa_nxt)[FM], vec8(&fb_cur)[FN],
                    vec8(&fb_nxt)[FN], int h, auto row0_tag, auto ld_tag, auto w_tag) __attribute__((always_inline)) {
      constexpr int ROW0 = decltype(row0_tag)::value;
      constexpr bool LD = decltype(ld_tag)::value;
      constexpr int SIDE_PAIRS = decltype(w_tag)::value / 4;  // pairs of elements per side unit
      constexpr int READS = FM + FN;
      constexpr int READ_ROWS = FM * FN >= 64 ? FM / 2 : (FM > 1 ? FM - 1 : 1);
      constexpr int PER_READ_ROW = (READS + READ_ROWS - 1) / READ_ROWS;
#pragma unroll
      for (int i = 0; i < FM; ++i) {
#pragma unroll
        for (int u = 0; u < PER_READ_ROW; ++u) {
          const int r = i * PER_READ_ROW + u;
          if (i < READ_ROWS && r < READS) {
            if (r < FN) fb_nxt[r] = read_b_fragment(sb, r);
            else fa_nxt[r - FN] = *(const vec8*)(sa + (r - FN) * 16 * kRowBytes);
          }
        }
        if constexpr (B_KMAJOR) {
          // Row 0: everything the previous step read must have arrived; only the transposing reads
          // issued just above (two per B fragment of this row) may still be in flight.  The row's A
          // fragment reads are not counted: the scheduler may place them on either side of this wait,
          // and counting one that ends up behind it would let a read of the previous step slip through.
          if (i == 0) {
            constexpr int B_NOW = PER_READ_ROW < FN ? PER_READ_ROW : FN;
            constexpr int NOW = 2 * B_NOW;
            wait_lds<(NOW < 15 ? NOW : 15)>();
            // ... and the MFMAs must not be moved above that wait: tie their B operands to it.
#pragma unroll
            for (int j = 0; j < FN; ++j) asm volatile("" : "+v"(fb_cur[j]));
          }
        }
#pragma unroll
        for (int jj = 0; jj < FN; ++jj) {
          // With two wavefronts per SIMD the rows walk the B fragments boustrophedon: consecutive
          // MFMAs then always share one operand (fewer input toggles: about 2% more throughput under
          // the power cap in a register-only loop, 1% here).  A wavefront that has its SIMD to itself
          // loses 5-7% that way (measured), so 4-wavefront tiles keep the plain order.
          const int j = (NW >= 8 && (i & 1)) ? FN - 1 - jj : jj;
          if constexpr (EPI == kEpiProbeLoads) asm volatile("" ::"v"(fb_cur[j]), "v"(fa_cur[i]));  // fragments stay live
          else acc[i][j] = Traits::mfma(fb_cur[j], fa_cur[i], acc[i][j]);
        }
        if constexpr (SIDE && LD && ROW0 != 0) {  // step 1: this row's share of the side vectors
          // pairs are dealt to every (FM / SIDE_PAIRS)-th row, or several to a row of a short step
          constexpr int EVERY = FM >= SIDE_PAIRS ? FM / SIDE_PAIRS : 1;
          constexpr int PER = FM >= SIDE_PAIRS ? 1 : (SIDE_PAIRS + FM - 1) / FM;
          if (i % EVERY == 0 && h < p.side_iters) {  // uniform: tiles past the workgroup's run carry nothing
#pragma unroll
            for (int u = 0; u < PER; ++u)
              if ((i / EVERY) * PER + u < SIDE_PAIRS) side_pair((i / EVERY) * PER + u);
          }
        }
#pragma unroll
        for (int u = 0; u < PER_ROW; ++u) {
          const int l = (ROW0 + i) * PER_ROW + u;  // B first: it is needed one tile sooner
          if constexpr (LD) {
            if (l < LB) load_b(l, h + BST - 1);
            else if (l < LOADS) load_a(l - LB, h + AST - 1);
          }
        }
        // Inside the row: MFMA, LDS read, MFMA, LDS read, MFMA, the rest of the reads, buffer load, the
        // remaining MFMAs.  A read or load issued between two MFMAs costs no matrix-core time (an MFMA
        // occupies its issue port for a quarter of its 16 cycles), whereas in front of the row it delays
        // the row's first MFMA: +1 to 3% on most tiles.  The 128x128 wavefront tile (a lone wavefront per
        // SIMD, 8 MFMAs a row) loses 13% with it and keeps reads-first.
        if constexpr (FN >= 4 && FM * FN < 64) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
          __builtin_amdgcn_sched_group_barrier(0x020, PER_ROW, 0);
          __builtin_amdgcn_sched_group_barrier(0x008, FN - 3, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    };

    // One K tile h: make it visible to every wavefront, then two steps.  Step 0 multiplies the
    // second half of tile h-1 (set 1) while reading the first half of tile h into set 0; step 1
    // multiplies set 0 while reading the second half of tile h into set 1.
    bool stores_pending = false;  // kEpiStoreLoop: a store epilogue precedes the tile being started
    auto tile_body = [&](int h, auto ld_tag, auto w_tag) __attribute__((always_inline)) {
      // my fills of tile h have landed; my reads of tile h-1 are done
      if constexpr (!decltype(ld_tag)::value) {
        wait_lds<0>();  // a wavefront that loads nothing has no fills to wait for
      } else if constexpr (LOOP) {
        // the first tile after a store epilogue: that epilogue's NST stores are younger than the fills
        if (h == 0 && stores_pending) wait_vm_and_lds<WAIT_STEADY + NST>();
        else wait_vm_and_lds<WAIT_STEADY>();
      } else {
        wait_vm_and_lds<WAIT_STEADY>();
      }
      bare_barrier();  // ... and so have everyone else's: the slots of tile h-1 are free
      const char* sa = smem + (h % AST) * A_BYTES + a_wave_off;
      const char* sb = smem + B_REGION + (h % BST) * B_BYTES + b_wave_off;
      // per-step offset of the B fragments: a swizzled chunk of the row, or 32 rows of k
      const int sb0 = B_KMAJOR ? 0 : frag_off[0];
      const int sb1 = B_KMAJOR ? 32 * BN * 2 : frag_off[1];
      step(sa + frag_off[0], sb + sb0, fa1, fa0, fb1, fb0, h, std::integral_constant<int, 0>{}, ld_tag, w_tag);
      step(sa + frag_off[1], sb + sb1, fa0, fa1, fb0, fb1, h, std::integral_constant<int, FM>{}, ld_tag, w_tag);
      if constexpr (SIDE && decltype(ld_tag)::value) {
        side_store(h, w_tag);
        side_load(h + 1, w_tag);
      }
    };

    // Prologue: A tiles 0 .. AST-2 and B tiles 0 .. BST-2, oldest first (tile 0 is what the first
    // wait of the loop is about).  A short tile 0 goes through registers instead.
    auto issue_prologue = [&]() __attribute__((always_inline)) {
      if (k_tail) fill_short_tile(k_tail);
#pragma unroll
      for (int s = 0; s < (loader ? AST - 1 : 0); ++s) {
        if (!(s == 0 && k_tail)) {
#pragma unroll
          for (int i = 0; i < LA; ++i) load_a(i, s);
        }
        if (s < BST - 1 && (B_KMAJOR || !(s == 0 && k_tail))) {
#pragma unroll
          for (int i = 0; i < LB; ++i) load_b(i, s);
        }
      }
    };
    using W16 = std::integral_constant<int, 16>;
    using W8 = std::integral_constant<int, 8>;
    using W4 = std::integral_constant<int, 4>;
    auto k_loop_and_drain = [&]() __attribute__((always_inline)) {
      // two straight-line versions of the loop, with and without the loads: a branch around every load
      // would cut each row of MFMAs into several scheduling regions
      // (and the side job one version per unit width: the unit's elements are dealt to rows at compile time)
      if constexpr (SIDE) {
        if (!loader) {
          for (int h = 0; h < n_tiles; ++h) tile_body(h, std::false_type{}, W16{});
        } else if (p.side_width == 16) {
          for (int h = 0; h < n_tiles; ++h) tile_body(h, std::true_type{}, W16{});
        } else if (p.side_width == 8) {
          for (int h = 0; h < n_tiles; ++h) tile_body(h, std::true_type{}, W8{});
        } else {
          for (int h = 0; h < n_tiles; ++h) tile_body(h, std::true_type{}, W4{});
        }
      } else if constexpr (LDW == NW) {
        for (int h = 0; h < n_tiles; ++h) tile_body(h, std::true_type{}, W16{});
      } else if (loader) {
        for (int h = 0; h < n_tiles; ++h) tile_body(h, std::true_type{}, W16{});
      } else {
        for (int h = 0; h < n_tiles; ++h) tile_body(h, std::false_type{}, W16{});
      }
      wait_vm_and_lds<0>();  // the empty fills of the last iterations must be gone before LDS is reused
      // Drain: the second half of the last tile is in set 1.
      if constexpr (B_KMAJOR) {
#pragma unroll
        for (int j = 0; j < FN; ++j) asm volatile("" : "+v"(fb1[j]));
      }
#pragma unroll
      for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j) {
          if constexpr (EPI == kEpiProbeLoads) asm volatile("" ::"v"(fb1[j]), "v"(fa1[i]));
          else acc[i][j] = Traits::mfma(fb1[j], fa1[i], acc[i][j]);
        }
    };
    // The first operand tiles are on their way before anything else is set up: accumulators and fragments are
    // cleared while they travel (a workgroup lives 3-5 us at 512^3 and 1024^3; every 0.1 us in front of its first
    // load is 2-3% of it).
    if (n_tiles > 0) issue_prologue();
    zero_acc();
    zero_fragments();
    if (n_tiles > 0) {
      if (SIDE && loader) {
        side_store(-1, W4{});  // dropped; keeps the number of side operations per tile uniform
        if (p.side_width == 16) side_load(0, W16{});
        else if (p.side_width == 8) side_load(0, W8{});
        else side_load(0, W4{});
      }
      if constexpr (!LOOP) k_loop_and_drain();
    }

    // ---- per-row statistics of the tile (LayerNorm epilogues) -------------------------------
    // A row's BN columns are spread over WAVES_N wavefronts x 4 lane groups (lane >> 4); every lane
    // reduces its own FN*4 values to (mean, M2) in registers, drops the pair into LDS, and one
    // thread per row merges the 4*WAVES_N pairs in a fixed order with Chan's update: no cross-lane
    // shuffles (they go through the LDS crossbar one at a time) and no cancellation.
    // Result: row_stats[rl] = (mean, M2) over the tile's valid columns, for rl in [0, BM).
    // A row of `part` is padded by one pair: its stride in 4-byte words is then twice an odd number, so
    // the 32 lanes of a pass (consecutive rows, one 8-byte pair each) fall on 32 different bank pairs,
    // both when the lanes drop their pairs and when one thread per row walks its row.
    auto tile_row_stats = [&](float* part /* [BM][4*WAVES_N + 1][2] */, float* row_stats /* [BM][2] */) {
      constexpr int SLOTS = 4 * WAVES_N;
      constexpr int PITCH = SLOTS + 1;  // pairs per row of `part`
      const int n_lane0 = col0 + wn * TN + 4 * (lane >> 4);  // first column of this lane
      const bool full = (col0 + BN <= N);
#pragma unroll
      for (int i = 0; i < FM; ++i) {
        float s = 0.0f, m2 = 0.0f, mean;
        if (full) {
#pragma unroll
          for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int e = 0; e < 4; ++e) s += acc[i][j][e];
          mean = s * (1.0f / (float)(FN * 4));
#pragma unroll
          for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const float d = acc[i][j][e] - mean;
              m2 += d * d;
            }
        } else {
          int cnt = 0;
#pragma unroll
          for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int e = 0; e < 4; ++e)
              if (n_lane0 + j * 16 + e < N) {
                s += acc[i][j][e];
                ++cnt;
              }
          mean = cnt > 0 ? s / (float)cnt : 0.0f;
#pragma unroll
          for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int e = 0; e < 4; ++e)
              if (n_lane0 + j * 16 + e < N) {
                const float d = acc[i][j][e] - mean;
                m2 += d * d;
              }
        }
        const int rl = wm * TM + i * 16 + (lane & 15);
        const int slot = wn * 4 + (lane >> 4);
        part[(rl * PITCH + slot) * 2 + 0] = mean;
        part[(rl * PITCH + slot) * 2 + 1] = m2;
      }
      __syncthreads();
      for (int rl = tid; rl < BM; rl += NT) {
        float mean = 0.0f, m2 = 0.0f, n_acc = 0.0f;
        if (full) {
          // every slot covers FN * 4 columns: the mean of the slot means, then M2 about it -- the same
          // merge as below for equal counts, in the same fixed order, without its divisions
          float mw[SLOTS], qw[SLOTS];
#pragma unroll
          for (int slot = 0; slot < SLOTS; ++slot) {
            mw[slot] = part[(rl * PITCH + slot) * 2 + 0];
            qw[slot] = part[(rl * PITCH + slot) * 2 + 1];
            mean += mw[slot];
          }
          mean *= 1.0f / (float)SLOTS;
#pragma unroll
          for (int slot = 0; slot < SLOTS; ++slot) {
            const float d = mw[slot] - mean;
            m2 += qw[slot] + (float)(FN * 4) * d * d;
          }
          row_stats[rl * 2 + 0] = mean;
          row_stats[rl * 2 + 1] = m2;
          continue;
        }
#pragma unroll
        for (int slot = 0; slot < SLOTS; ++slot) {
          // valid columns of this (wavefront, lane group): 4 per 16-wide block, clipped at N
          int cnt = FN * 4;
          if (!full) {
            cnt = 0;
            const int n0 = col0 + (slot >> 2) * TN + 4 * (slot & 3);
#pragma unroll
            for (int j = 0; j < FN; ++j) {
              int c = N - (n0 + j * 16);
              cnt += c < 0 ? 0 : (c > 4 ? 4 : c);
            }
            if (cnt == 0) continue;
          }
          const float mw = part[(rl * PITCH + slot) * 2 + 0];
          const float qw = part[(rl * PITCH + slot) * 2 + 1];
          const float nb = (float)cnt;
          const float tot = n_acc + nb;
          const float delta = mw - mean;
          mean += delta * (nb / tot);
          m2 += qw + delta * delta * (n_acc * nb / tot);
          n_acc = tot;
        }
        row_stats[rl * 2 + 0] = mean;
        row_stats[rl * 2 + 1] = m2;
      }
      __syncthreads();  // `part` may be reused by the caller from here on
    };

    // ---- epilogue ---------------------------------------------------------------------
    // acc[i][j][e]: row m = row0 + wm*TM + i*16 + (lane & 15),
    //               col n = col0 + wn*TN + j*16 + 4*(lane>>4) + e.
    const int m_base = row0 + wm * TM + (lane & 15);
    const int n_base = col0 + wn * TN + 4 * (lane >> 4);
    const bool vec_ok = (N % 4) == 0;

    // 16-bit output through LDS, so that a store instruction writes whole rows of the wavefront's
    // sub-tile (TN columns = TN / 8 lanes of 16 bytes each) instead of 16 rows x 32 bytes: the
    // direct stores cost 3% at 4096^3 and 5% at 16384 x 16384 x 2048.  Each wavefront uses a
    // private region of (TM / HALVES) rows of TN * 2 bytes behind the first RESERVED bytes of LDS;
    // the caller has made sure that LDS is free (a barrier).
    // Layout of a region (measured with the bank-conflict counter): an 8-byte write is served 16
    // lanes (= the 16 rows of a block, one column group) at a time out of 32 banks, so the 16 rows
    // must land in 16 different 8-byte slots of a 128-byte window.  A row's 16-byte chunks are
    // XORed with the row number (3 bits; 2 bits and the row's parity where two rows share a
    // window) and rows 8..15 of a block have the two halves of every chunk swapped.  The 16-byte
    // reads run over whole rows (any padding of the rows makes them conflict) and undo both.
    //   row_ctx(i): per-row values of block row i, passed on to value(i, j, ctx) -> 4 outputs.
    auto staged_store = [&](T* C, auto reserved_tag, auto row_ctx, auto value) {
      constexpr int RESERVED = decltype(reserved_tag)::value;
      constexpr int AVAIL = LDS_BYTES - RESERVED;
      constexpr int RB = TN * 2;  // bytes per row
      constexpr int HALVES = NW * TM * RB <= AVAIL ? 1 : (NW * TM * RB <= 2 * AVAIL ? 2 : 4);
      static_assert(NW * (TM / HALVES) * RB <= AVAIL && FM % HALVES == 0 && RESERVED % 128 == 0, "staging area");
      static_assert(RB == 64 || RB == 128 || RB == 256, "row of a wavefront's sub-tile");
      constexpr int FMH = FM / HALVES;  // blocks of 16 rows per pass
      constexpr int LPR = TN / 8;       // lanes per row
      constexpr int RPI = 64 / LPR;     // rows per store instruction
      auto chunk_xor = [](int r) { return RB == 64 ? (r >> 1) & 3 : r & 7; };
      char* stage = smem + RESERVED + wave * (FMH * 16 * RB);
      const bool wide_ok = (N % 8) == 0 && ((size_t)C & 15) == 0;
      const int srow = lane / LPR, schunk = lane % LPR;
      const int wr = lane & 15, wg = lane >> 4;  // writer: row of the block, column group
      const int w_off = wr * RB + (((wg & 1) ^ (wr >> 3)) << 3);
#pragma unroll
      for (int hf = 0; hf < HALVES; ++hf) {
#pragma unroll
        for (int i = 0; i < FMH; ++i) {
          const auto ctx = row_ctx(hf * FMH + i);
#pragma unroll
          for (int j = 0; j < FN; ++j)
            *(vec4*)(stage + i * 16 * RB + w_off + (((2 * j + (wg >> 1)) ^ chunk_xor(wr)) << 4)) = value(hf * FMH + i, j, ctx);
        }
#pragma unroll
        for (int it = 0; it < FMH * 16 / RPI; ++it) {
          const int r = it * RPI + srow;
          vec8 v = *(const vec8*)(stage + r * RB + schunk * 16);
          if ((r >> 3) & 1) v = vec8{v[4], v[5], v[6], v[7], v[0], v[1], v[2], v[3]};
          const int n_st = col0 + wn * TN + (schunk ^ chunk_xor(r)) * 8;
          const int m = row0 + wm * TM + hf * FMH * 16 + r;
          if (m < M) {
            T* dst = C + (size_t)m * N + n_st;
            if (wide_ok && n_st + 7 < N) {
              store_through_16(dst, __builtin_bit_cast(i32x4, v));
            } else if (vec_ok && n_st + 7 < N) {  // C only 8-byte aligned, or N % 8 == 4
              *(vec4*)dst = vec4{v[0], v[1], v[2], v[3]};
              *(vec4*)(dst + 4) = vec4{v[4], v[5], v[6], v[7]};
            } else {
#pragma unroll
              for (int e = 0; e < 8; ++e)
                if (n_st + e < N) dst[e] = v[e];
            }
          }
        }
      }
    };

    if (EPI == kEpiStore || EPI == kEpiStoreSide) {
      T* C = (T*)p.C;
      __syncthreads();  // every wavefront is done with the last tile, and no fill is still landing
      staged_store(C, std::integral_constant<int, 0>{}, [](int) { return 0; },
                   [&](int i, int j, int) {
                     vec4 v;
#pragma unroll
                     for (int e = 0; e < 4; ++e) v[e] = (T)acc[i][j][e];
                     return v;
                   });
      if constexpr (SIDE) {
        // Side vectors beyond the K tiles of this workgroup (a short K loop or a long array), then
        // the elements after the last whole vector.
        // (the host narrows the units only when the job then still fits into the loop: 16-byte units here)
        for (int it = n_tiles; loader && it < p.side_iters; ++it) {
#pragma unroll
          for (int e = 0; e < 4; ++e) side_pair(e);
          side_store(it, std::integral_constant<int, 16>{});
          side_load(it + 1, std::integral_constant<int, 16>{});
        }
        const long long done = (p.side_count >> 3) << 3;
        if (blockIdx.x == 0 && done + tid < p.side_count) {
          const T* x = (const T*)p.side_x;
          T* y = (T*)p.side_y;
          y[done + tid] = silu_16<T>(x[done + tid]);
        }
      }
    } else if constexpr (LOOP) {
      // Walk the tiles id, id + grid, ...  After the K loop of one tile every LDS slot is dead: the
      // first operand tiles of the next one go into the slots they belong to (A 0 .. AST-2, B 0 ..
      // BST-2) right away, and the output is staged in the two slots that stay free, in as many
      // passes as that takes.  The stores leave through a buffer descriptor (rows and columns that
      // do not exist get an offset outside it and are dropped), so every wavefront issues exactly
      // NST of them per tile and the first wait of the next K loop can count them.
      static_assert(!B_KMAJOR && AST >= 3 && BST >= 2 && NW % 2 == 0, "looping store kernel");
      constexpr int RB = TN * 2;
      constexpr int FREE = A_BYTES < B_BYTES ? A_BYTES : B_BYTES;  // bytes of a free slot half the wavefronts share
      constexpr int PASSES = (NW / 2) * TM * RB <= FREE ? 1
                           : (FM % 2 == 0 && (NW / 2) * (TM / 2) * RB <= FREE) ? 2
                           : (FM % 4 == 0 && (NW / 2) * (TM / 4) * RB <= FREE) ? 4 : FM;
      constexpr int FMH = FM / PASSES;
      static_assert(FM % PASSES == 0 && (NW / 2) * FMH * 16 * RB <= FREE, "staging area");
      static_assert(RB == 64 || RB == 128 || RB == 256, "row of a wavefront's sub-tile");
      constexpr int LPR = TN / 8, RPI = 64 / LPR;
      auto chunk_xor = [](int r) { return RB == 64 ? (r >> 1) & 3 : r & 7; };
      T* C = (T*)p.C;
      const int total = p.tiles_m * p.tiles_n;
      int id = blockIdx.x;
      for (;;) {
        k_loop_and_drain();
        __syncthreads();  // every wavefront is done with the last K tile, and no fill is still landing
        // The epilogue's lane constants are recomputed per tile from a value the compiler cannot see
        // through: hoisted out of this loop they would stay live across the K loop, which has no
        // register to spare.
        int ol = lane;
        asm volatile("" : "+v"(ol));
        char* stage = (wave < NW / 2 ? smem + (AST - 1) * A_BYTES + wave * (FMH * 16 * RB)
                                     : smem + B_REGION + (BST - 1) * B_BYTES + (wave - NW / 2) * (FMH * 16 * RB));
        const int srow = ol / LPR, schunk = ol % LPR;
        const int wr = ol & 15, wg = ol >> 4;
        const int w_off = wr * RB + (((wg & 1) ^ (wr >> 3)) << 3);
        const int s_row0 = row0, s_col0 = col0, s_rows = rows_a, s_cols = rows_b;
        id += gridDim.x;
        const bool more = id < total;  // uniform
        if (more) {
          set_tile(id);
          issue_prologue();
        }
        const __amdgpu_buffer_rsrc_t rsrc_c =
            make_rsrc(C + ((size_t)s_row0 * N + s_col0), ((unsigned)(s_rows - 1) * N + s_cols) * 2u);
        // Non-temporal stores when the host asks for them (an output larger than the last-level cache:
        // its lines then do not push operand panels out of the L2).  Two copies of the loop, not a
        // branch per store: the reads of a pass stay batched ahead of its stores.
        auto store_tile = [&](auto aux_tag) __attribute__((always_inline)) {
        constexpr int AUX = decltype(aux_tag)::value;
#pragma unroll
        for (int ps = 0; ps < PASSES; ++ps) {
#pragma unroll
          for (int i = 0; i < FMH; ++i) {
#pragma unroll
            for (int j = 0; j < FN; ++j) {
              vec4 v;
#pragma unroll
              for (int e = 0; e < 4; ++e) v[e] = (T)acc[ps * FMH + i][j][e];
              *(vec4*)(stage + i * 16 * RB + w_off + (((2 * j + (wg >> 1)) ^ chunk_xor(wr)) << 4)) = v;
            }
          }
#pragma unroll
          for (int it = 0; it < FMH * 16 / RPI; ++it) {
            const int r = it * RPI + srow;
            vec8 v = *(const vec8*)(stage + r * RB + schunk * 16);
            if ((r >> 3) & 1) v = vec8{v[4], v[5], v[6], v[7], v[0], v[1], v[2], v[3]};
            const int tr = wm * TM + ps * FMH * 16 + r;                    // row inside the tile
            const int tcn = wn * TN + (schunk ^ chunk_xor(r)) * 8;          // column inside the tile
            const unsigned off = (tr < s_rows && tcn < s_cols) ? ((unsigned)tr * (unsigned)N + (unsigned)tcn) * 2u : kOobOffset;
            __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(i32x4, v), rsrc_c, (int)off, 0, AUX);
          }
        }
        };
        if (p.c_streaming) store_tile(std::integral_constant<int, 2>{});
        else store_tile(std::integral_constant<int, 0>{});
        if (!more) break;
        stores_pending = true;
        zero_acc();
        zero_fragments();
      }
    } else if (EPI == kEpiLnFused) {
      // gamma / beta for this lane's columns: issued now, consumed in step 5
      const T* gamma = (const T*)p.gamma;
      const T* beta = (const T*)p.beta;
      vec4 gv[FN], bv[FN];
#pragma unroll
      for (int j = 0; j < FN; ++j) {
        const int n = n_base + j * 16;
        if (vec_ok && n + 3 < N) {
          gv[j] = *(const vec4*)(gamma + n);
          bv[j] = *(const vec4*)(beta + n);
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const int nn = (n + e < N) ? n + e : N - 1;
            gv[j][e] = gamma[nn];
            bv[j][e] = beta[nn];
          }
        }
      }
      // 1. per-row (mean, M2) over this tile's columns
      __syncthreads();            // every LDS slot is dead; reuse the space
      float* red = (float*)smem;   // [BM][2] tile statistics, later (mean, rstd) of the whole row
      float* part = red + BM * 2;  // [BM][4*WAVES_N + 1][2], then reused as `gathered`
      tile_row_stats(part, red);
      // 2. publish the tile's statistics (ln_publish above: two tagged 8-byte words per row)
      const unsigned tag = ln_launch_tag(p);
      ln_sign_header(p, tag);
      const size_t my_slot = ((size_t)tc.tm * p.tiles_n + tc.tn) * BM;
      // (tile_row_stats left row rl's pair with the thread that publishes it: same rl = tid stride)
      for (int rl = tid; rl < BM; rl += NT) ln_publish(p, my_slot + rl, red[rl * 2 + 0], red[rl * 2 + 1], tag);
      // 3. gather the band's statistics into LDS
      float* gathered = part;  // [tiles_n][BM][2]; tiles_n <= 64 keeps it within the LDS the kernel owns
      ln_gather<NT>(p, tag, (size_t)tc.tm * p.tiles_n * BM, p.tiles_n * BM, tid, (unsigned long long*)gathered);
      __syncthreads();
      // 4. merge in tile order -> (mean, rstd) per row
      const bool even_tiles = (N % BN) == 0;  // every column tile is full: equal weights
      for (int rl = tid; rl < BM; rl += NT) {
        float mean = 0.0f, m2 = 0.0f, n_acc = 0.0f;
        if (even_tiles) {
          for (int t = 0; t < p.tiles_n; ++t) mean += gathered[((size_t)t * BM + rl) * 2 + 0];
          mean *= 1.0f / (float)p.tiles_n;
          for (int t = 0; t < p.tiles_n; ++t) {
            const float d = gathered[((size_t)t * BM + rl) * 2 + 0] - mean;
            m2 += gathered[((size_t)t * BM + rl) * 2 + 1] + (float)BN * d * d;
          }
          red[rl * 2 + 0] = mean;
          red[rl * 2 + 1] = __builtin_amdgcn_rsqf(m2 * (1.0f / (float)N) + p.eps);
          continue;
        }
        for (int t = 0; t < p.tiles_n; ++t) {
          int cw = N - t * BN;
          cw = cw > BN ? BN : cw;
          const float mw = gathered[((size_t)t * BM + rl) * 2 + 0];
          const float qw = gathered[((size_t)t * BM + rl) * 2 + 1];
          const float nb = (float)cw;
          const float tot = n_acc + nb;
          const float delta = mw - mean;
          mean += delta * (nb / tot);
          m2 += qw + delta * delta * (n_acc * nb / tot);
          n_acc = tot;
        }
        red[rl * 2 + 0] = mean;
        red[rl * 2 + 1] = 1.0f / sqrtf(m2 / (float)N + p.eps);
      }
      __syncthreads();
      // 5. normalise the accumulators and store Y (through LDS, behind the row statistics)
      T* Y = (T*)p.C;
      struct RowStat { float mean, rstd; };
      staged_store(Y, std::integral_constant<int, BM * 2 * 4>{},
                   [&](int i) {
                     const int rl = wm * TM + i * 16 + (lane & 15);
                     return RowStat{red[rl * 2 + 0], red[rl * 2 + 1]};
                   },
                   [&](int i, int j, RowStat st) {
                     vec4 v;
#pragma unroll
                     for (int e = 0; e < 4; ++e)
                       v[e] = (T)((acc[i][j][e] - st.mean) * st.rstd * (float)gv[j][e] + (float)bv[j][e]);
                     return v;
                   });
    } else {
      if (EPI == kEpiLnStats) {
        // Per-row statistics over the columns this workgroup owns, from the fp32 accumulators.
        __syncthreads();  // every LDS slot is dead; reuse the space
        float* row_stats = (float*)smem;   // [BM][2]
        float* part = row_stats + BM * 2;  // [BM][4*WAVES_N + 1][2]
        tile_row_stats(part, row_stats);
        for (int rl = tid; rl < BM; rl += NT) {
          const int m = row0 + rl;
          if (m >= M) continue;
          float* st = p.stats + ((size_t)m * p.tiles_n + tc.tn) * 2;
          st[0] = row_stats[rl * 2 + 0];
          st[1] = row_stats[rl * 2 + 1];
        }
      }
      if constexpr (EPI == kEpiProbeLoads) return;
      if constexpr (EPI == kEpiPartialFused) {
        // The slice's partial sums, written through to memory (N is a multiple of 4 and M * N * 4 fits a
        // descriptor: the host sees to it), then the flags of the tile's parts.
        const __amdgpu_buffer_rsrc_t rsrc_w = make_rsrc(p.ws + (size_t)slice * M * N, (unsigned)M * (unsigned)N * 4u);
#pragma unroll
        for (int i = 0; i < FM; ++i) {
          const int m = m_base + i * 16;
#pragma unroll
          for (int j = 0; j < FN; ++j) {
            const int n = n_base + j * 16;
            const unsigned off = (m < M && n < N) ? ((unsigned)m * (unsigned)N + (unsigned)n) * 4u : kOobOffset;
            __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(i32x4, acc[i][j]), rsrc_w, (int)off, 0, kAuxDeviceScope);
          }
        }
        __builtin_amdgcn_s_waitcnt(0);  // this wavefront's stores have been acknowledged by memory ...
        __syncthreads();                // ... and so have everyone's
        const int P = sk_parts_per_tile(BM, BN, NT, p.sk_out);
        if (tid < P) {
          const size_t f = ((size_t)(tc.tm * p.tiles_n + tc.tn) * P + tid) * p.splits + slice;
          __hip_atomic_store(p.sk_sync + kSkFlags + f, (int)sk_launch_tag(p.ln_nonce), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        if (p.sk_self) {  // (uniform)
          const int t = tc.tm * p.tiles_n + tc.tn;
          for (int q = slice; q < P; q += p.splits) {
            if (p.sk_out == 4) splitk_reduce_part_of<4>(p, t * P + q);
            else if (p.sk_out == 2) splitk_reduce_part_of<2>(p, t * P + q);
            else splitk_reduce_part_of<1>(p, t * P + q);
          }
        }
        return;
      }
      // fp32 tile: split-K partial sums of this slice, or X for the normalisation pass.
      float* W = p.ws + (EPI == kEpiPartial ? (size_t)slice * M * N : (size_t)0);
#pragma unroll
      for (int i = 0; i < FM; ++i) {
        const int m = m_base + i * 16;
        if (m >= M) continue;
        float* wrow = W + (size_t)m * N;
#pragma unroll
        for (int j = 0; j < FN; ++j) {
          const int n = n_base + j * 16;
          if (vec_ok && n + 3 < N) {
            *(f32x4*)(wrow + n) = acc[i][j];
          } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
              if (n + e < N) wrow[n + e] = acc[i][j][e];
          }
        }
      }
    }
  }
};

template <typename T, int BM, int BN, int WAVES_M, int WAVES_N, int EPI, int AST, int BST, bool B_KMAJOR = false>
__global__ void __launch_bounds__(WAVES_M* WAVES_N * 64)
    gemmrc_kernel(const GemmParams p) {
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  GemmTile<T, BM, BN, WAVES_M, WAVES_N, EPI, AST, BST, B_KMAJOR>::run(p, smem);
}

}  // namespace beam
