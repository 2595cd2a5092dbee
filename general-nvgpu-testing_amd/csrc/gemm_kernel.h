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
//   * one workgroup owns a BM x BN tile of C, WAVES_M x WAVES_N wavefronts each own a
//     (BM/WAVES_M) x (BN/WAVES_N) sub-tile made of 32x32 MFMA blocks
//     (v_mfma_f32_32x32x16_{f16,bf16}: 16 K elements per instruction);
//   * K is walked in steps of 64 elements; a stage of LDS holds BM + BN rows of 128 bytes,
//     16-byte chunks XOR-swizzled (tile_map.h) so that both the 1 KiB-per-wavefront fills
//     and the ds_read_b128 fragment reads are bank-conflict free;
//   * global -> LDS goes through buffer loads that write LDS directly (no VGPR staging);
//     rows past the matrix edge are outside the buffer descriptor and never touch memory;
//   * two LDS stages: the fill of stage s^1 is in flight while stage s feeds the MFMAs, and
//     fragments are double-buffered in registers so LDS latency hides behind MFMA issue;
//   * the MFMA is issued with B as the first operand, so every lane ends up with 4
//     consecutive columns of one output row per accumulator quad: rows reduce inside a
//     lane (LayerNorm statistics) and stores are 8-byte (16-bit C) or 16-byte (fp32).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "tile_map.h"

namespace beam {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef int i32x4 __attribute__((ext_vector_type(4)));

template <typename T>
struct ElemTraits;

template <>
struct ElemTraits<_Float16> {
  using vec8 = f16x8;
  using vec4 = f16x4;
  static __device__ __forceinline__ f32x16 mfma(vec8 a, vec8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
};

template <>
struct ElemTraits<__bf16> {
  using vec8 = bf16x8;
  using vec4 = bf16x4;
  static __device__ __forceinline__ f32x16 mfma(vec8 a, vec8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
};

// What the kernel does with the fp32 accumulators.
enum Epilogue : int {
  kEpiStore = 0,    // round to 16-bit and store C
  kEpiPartial = 1,  // store fp32 partial sums of this K slice into the split-K workspace
  kEpiLnStats = 2,  // store fp32 X and per-(row, column-tile) mean / M2 for LayerNorm
};

struct GemmParams {
  const void* A;
  const void* B;
  void* C;       // 16-bit [M][N]                                  (kEpiStore)
  float* ws;     // fp32 [splits][M][N] (kEpiPartial) or fp32 [M][N] (kEpiLnStats)
  float* stats;  // fp32 [M][tiles_n][2] = (mean, M2) over the tile's columns (kEpiLnStats)
  int M, N, K;
  int tiles_m, tiles_n;
  int k_slice;   // K elements per blockIdx.z slice, a multiple of kBK
  int group_m;   // rasterisation group height in tiles
};

// Buffer descriptor word 3 for gfx9-family raw buffers: 32-bit data format, no swizzle.
constexpr int kRsrcFlags = 0x00020000;
// Byte offset that is out of range of every descriptor built here.
constexpr unsigned kOobOffset = 0x7fffff00u;

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, unsigned bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, kRsrcFlags);
}

template <typename T, int BM, int BN, int WAVES_M, int WAVES_N, int EPI, bool DIRECT>
struct GemmTile {
  using Traits = ElemTraits<T>;
  using vec8 = typename Traits::vec8;
  using vec4 = typename Traits::vec4;

  static constexpr int NW = WAVES_M * WAVES_N;
  static constexpr int NT = NW * 64;
  static constexpr int TM = BM / WAVES_M;  // wavefront tile
  static constexpr int TN = BN / WAVES_N;
  static constexpr int FM = TM / 32;       // MFMA blocks per wavefront tile
  static constexpr int FN = TN / 32;
  static constexpr int A_BYTES = BM * kRowBytes;
  static constexpr int B_BYTES = BN * kRowBytes;
  static constexpr int STAGE_BYTES = A_BYTES + B_BYTES;
  static constexpr int LDS_BYTES = 2 * STAGE_BYTES;
  static constexpr int LA = (BM * kChunksPerRow) / NT;  // 16-byte chunks per thread per stage
  static constexpr int LB = (BN * kChunksPerRow) / NT;

  static_assert(TM % 32 == 0 && TN % 32 == 0, "wavefront tile must be made of 32x32 blocks");
  static_assert((BM * kChunksPerRow) % NT == 0 && (BN * kChunksPerRow) % NT == 0,
                "every thread must move a whole number of chunks per stage");
  static_assert(LDS_BYTES <= 160 * 1024, "LDS budget of one CU");

  // ---- global -> LDS ------------------------------------------------------------------
  // Chunk q = i * NT + tid of an operand tile lives at LDS byte q * 16 of its stage, which is
  // row q / 8, slot q % 8; the slot holds logical chunk slot ^ swizzle_of_row(row).

  static __device__ __forceinline__ unsigned chunk_voffset(int q, int K) {
    const int row = q >> 3;
    const int chunk = (q & 7) ^ swizzle_of_row(row);
    return (unsigned)row * (unsigned)K * 2u + (unsigned)chunk * 16u;
  }

  static __device__ __forceinline__ void run(const GemmParams& p, char* smem) {
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave % WAVES_M;
    const int wn = wave / WAVES_M;

    const TileCoord tc = tile_of_workgroup(blockIdx.x, p.tiles_m, p.tiles_n, p.group_m);
    const int row0 = tc.tm * BM;
    const int col0 = tc.tn * BN;
    const int M = p.M, N = p.N, K = p.K;

    // K range of this slice.
    const int kb = blockIdx.z * p.k_slice;
    int klen = K - kb;
    if (klen > p.k_slice) klen = p.k_slice;
    if (klen < 0) klen = 0;
    const int kt_full = klen / kBK;
    const int k_tail = klen - kt_full * kBK;         // multiple of 8 (host guarantees K % 8 == 0)
    const int n_tiles = kt_full + (k_tail ? 1 : 0);  // the short tile, if any, is processed FIRST

    // Buffer descriptors cover exactly the rows of this tile that exist and the K range of
    // this slice; anything else is out of range: reads return zero and touch no memory.
    const int rows_a = (M - row0) < BM ? (M - row0) : BM;
    const int rows_b = (N - col0) < BN ? (N - col0) : BN;
    const T* a_base = (const T*)p.A + ((size_t)row0 * K + kb);
    const T* b_base = (const T*)p.B + ((size_t)col0 * K + kb);
    const __amdgpu_buffer_rsrc_t rsrc_a =
        make_rsrc(a_base, klen > 0 ? ((unsigned)(rows_a - 1) * K + klen) * 2u : 0u);
    const __amdgpu_buffer_rsrc_t rsrc_b =
        make_rsrc(b_base, klen > 0 ? ((unsigned)(rows_b - 1) * K + klen) * 2u : 0u);

    unsigned voff_a[LA], voff_b[LB];
#pragma unroll
    for (int i = 0; i < LA; ++i) voff_a[i] = chunk_voffset(i * NT + tid, K);
#pragma unroll
    for (int i = 0; i < LB; ++i) voff_b[i] = chunk_voffset(i * NT + tid, K);

    // Fill of one stage straight into LDS; `koff` = first K element of the tile inside the slice.
    auto fill_direct = [&](int stage, int koff) {
      char* sa = smem + stage * STAGE_BYTES + wave * 1024;
      char* sb = sa + A_BYTES;
#pragma unroll
      for (int i = 0; i < LA; ++i)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(
            rsrc_a, (__attribute__((address_space(3))) void*)(sa + i * (NT * 16)), 16,
            (int)voff_a[i], koff * 2, 0, 0);
#pragma unroll
      for (int i = 0; i < LB; ++i)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(
            rsrc_b, (__attribute__((address_space(3))) void*)(sb + i * (NT * 16)), 16,
            (int)voff_b[i], koff * 2, 0, 0);
    };

    // Fill of one stage through registers, zero-filling chunks at or past `kvalid` elements
    // (used for the short K tile and by the DIRECT=false variant).
    auto fill_staged = [&](int stage, int koff, int kvalid) {
      i32x4 ra[LA], rb[LB];
#pragma unroll
      for (int i = 0; i < LA; ++i) {
        const int q = i * NT + tid;
        const int chunk = (q & 7) ^ swizzle_of_row(q >> 3);
        const unsigned off = (chunk * 8 < kvalid) ? voff_a[i] + (unsigned)koff * 2u : kOobOffset;
        ra[i] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_a, (int)off, 0, 0);
      }
#pragma unroll
      for (int i = 0; i < LB; ++i) {
        const int q = i * NT + tid;
        const int chunk = (q & 7) ^ swizzle_of_row(q >> 3);
        const unsigned off = (chunk * 8 < kvalid) ? voff_b[i] + (unsigned)koff * 2u : kOobOffset;
        rb[i] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_b, (int)off, 0, 0);
      }
      char* sa = smem + stage * STAGE_BYTES + tid * 16;
      char* sb = sa + A_BYTES;
#pragma unroll
      for (int i = 0; i < LA; ++i) *(i32x4*)(sa + i * (NT * 16)) = ra[i];
#pragma unroll
      for (int i = 0; i < LB; ++i) *(i32x4*)(sb + i * (NT * 16)) = rb[i];
    };

    // ---- LDS -> MFMA fragments ----------------------------------------------------------
    // 32x32x16 operand: lane l supplies row (l & 31), K elements 8*(l>>5) .. +7 of the step.
    const int frow = lane & 31;
    int frag_off[4];
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) frag_off[kk] = lds_offset(frow, 2 * kk + (lane >> 5));
    const int a_wave_off = wm * TM * kRowBytes;
    const int b_wave_off = A_BYTES + wn * TN * kRowBytes;

    auto read_frags = [&](int stage, int kk, vec8 (&fa)[FM], vec8 (&fb)[FN]) {
      const char* s = smem + stage * STAGE_BYTES + frag_off[kk];
#pragma unroll
      for (int i = 0; i < FM; ++i) fa[i] = *(const vec8*)(s + a_wave_off + i * 32 * kRowBytes);
#pragma unroll
      for (int j = 0; j < FN; ++j) fb[j] = *(const vec8*)(s + b_wave_off + j * 32 * kRowBytes);
    };

    f32x16 acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
      for (int j = 0; j < FN; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    auto mma = [&](const vec8 (&fa)[FM], const vec8 (&fb)[FN]) {
#pragma unroll
      for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j) acc[i][j] = Traits::mfma(fb[j], fa[i], acc[i][j]);
    };

    // K offset (inside the slice) of tile t: the short tile comes first.
    auto tile_koff = [&](int t) { return k_tail ? (t == 0 ? kt_full * kBK : (t - 1) * kBK) : t * kBK; };

    if (n_tiles > 0) {
      if (k_tail) {
        fill_staged(0, tile_koff(0), k_tail);
      } else if (DIRECT) {
        fill_direct(0, 0);
      } else {
        fill_staged(0, 0, kBK);
      }
      __builtin_amdgcn_s_waitcnt(0);  // vmcnt(0) expcnt(0) lgkmcnt(0)
      __syncthreads();

      vec8 fa0[FM], fb0[FN], fa1[FM], fb1[FN];
      read_frags(0, 0, fa0, fb0);

      for (int t = 0; t < n_tiles; ++t) {
        const int cur = t & 1;
        const int nxt = cur ^ 1;
        const bool has_next = (t + 1 < n_tiles);
        if (DIRECT) {
          if (has_next) fill_direct(nxt, tile_koff(t + 1));
          read_frags(cur, 1, fa1, fb1);
          mma(fa0, fb0);
          read_frags(cur, 2, fa0, fb0);
          mma(fa1, fb1);
          read_frags(cur, 3, fa1, fb1);
          mma(fa0, fb0);
        } else {
          i32x4 ra[LA], rb[LB];
          if (has_next) {
            const int koff = tile_koff(t + 1);
#pragma unroll
            for (int i = 0; i < LA; ++i)
              ra[i] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_a, (int)voff_a[i], koff * 2, 0);
#pragma unroll
            for (int i = 0; i < LB; ++i)
              rb[i] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_b, (int)voff_b[i], koff * 2, 0);
          }
          read_frags(cur, 1, fa1, fb1);
          mma(fa0, fb0);
          read_frags(cur, 2, fa0, fb0);
          mma(fa1, fb1);
          read_frags(cur, 3, fa1, fb1);
          mma(fa0, fb0);
          if (has_next) {
            char* sa = smem + nxt * STAGE_BYTES + tid * 16;
            char* sb = sa + A_BYTES;
#pragma unroll
            for (int i = 0; i < LA; ++i) *(i32x4*)(sa + i * (NT * 16)) = ra[i];
#pragma unroll
            for (int i = 0; i < LB; ++i) *(i32x4*)(sb + i * (NT * 16)) = rb[i];
          }
        }
        // Every wavefront has read all of stage `cur`; the fill of `nxt` has landed.
        __builtin_amdgcn_s_waitcnt(0);
        __syncthreads();
        if (has_next) read_frags(nxt, 0, fa0, fb0);
        mma(fa1, fb1);
      }
    }

    // ---- epilogue ---------------------------------------------------------------------
    // acc[i][j][r]: row m = row0 + wm*TM + i*32 + (lane & 31),
    //               col n = col0 + wn*TN + j*32 + 8*(r/4) + 4*(lane>>5) + (r%4).
    const int m_base = row0 + wm * TM + (lane & 31);
    const int n_base = col0 + wn * TN + 4 * (lane >> 5);
    const bool vec_ok = (N % 4) == 0;

    if (EPI == kEpiStore) {
      T* C = (T*)p.C;
#pragma unroll
      for (int i = 0; i < FM; ++i) {
        const int m = m_base + i * 32;
        if (m >= M) continue;
        T* crow = C + (size_t)m * N;
#pragma unroll
        for (int j = 0; j < FN; ++j) {
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            const int n = n_base + j * 32 + g * 8;
            vec4 v;
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] = (T)acc[i][j][g * 4 + e];
            if (vec_ok && n + 3 < N) {
              *(vec4*)(crow + n) = v;
            } else {
#pragma unroll
              for (int e = 0; e < 4; ++e)
                if (n + e < N) crow[n + e] = v[e];
            }
          }
        }
      }
    } else if (EPI == kEpiPartial) {
      float* W = p.ws + (size_t)blockIdx.z * M * N;
#pragma unroll
      for (int i = 0; i < FM; ++i) {
        const int m = m_base + i * 32;
        if (m >= M) continue;
        float* wrow = W + (size_t)m * N;
#pragma unroll
        for (int j = 0; j < FN; ++j) {
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            const int n = n_base + j * 32 + g * 8;
            f32x4 v;
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] = acc[i][j][g * 4 + e];
            if (vec_ok && n + 3 < N) {
              *(f32x4*)(wrow + n) = v;
            } else {
#pragma unroll
              for (int e = 0; e < 4; ++e)
                if (n + e < N) wrow[n + e] = v[e];
            }
          }
        }
      }
    } else {  // kEpiLnStats
      // Per-row statistics over the columns this workgroup owns, from the fp32 accumulators.
      // A row's TN columns of one wavefront sit in two lanes (l, l^32): reduce in registers,
      // swap once across the half-wavefronts, then combine the WAVES_N wavefronts via LDS
      // with Chan's pairwise update so no precision is lost to cancellation.
      __syncthreads();  // LDS stages are dead; reuse them for the cross-wavefront exchange
      float* red = (float*)smem;  // [BM][WAVES_N][2]
      const int cols_here = (N - col0) < BN ? (N - col0) : BN;
#pragma unroll
      for (int i = 0; i < FM; ++i) {
        float s = 0.0f;
        int cnt = 0;
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int n = n_base + j * 32 + (r / 4) * 8 + (r % 4);
            if (n < N) { s += acc[i][j][r]; ++cnt; }
          }
        s += __shfl_xor(s, 32);
        cnt += __shfl_xor(cnt, 32);
        const float mean = cnt > 0 ? s / (float)cnt : 0.0f;
        float m2 = 0.0f;
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int n = n_base + j * 32 + (r / 4) * 8 + (r % 4);
            if (n < N) { const float d = acc[i][j][r] - mean; m2 += d * d; }
          }
        m2 += __shfl_xor(m2, 32);
        if (lane < 32) {
          const int rl = wm * TM + i * 32 + lane;
          red[(rl * WAVES_N + wn) * 2 + 0] = mean;
          red[(rl * WAVES_N + wn) * 2 + 1] = m2;
        }
      }
      __syncthreads();
      for (int rl = tid; rl < BM; rl += NT) {
        const int m = row0 + rl;
        if (m >= M) continue;
        float mean = 0.0f, m2 = 0.0f, n_acc = 0.0f;
#pragma unroll
        for (int w = 0; w < WAVES_N; ++w) {
          int cw = cols_here - w * TN;
          cw = cw < 0 ? 0 : (cw > TN ? TN : cw);
          if (cw == 0) continue;
          const float mw = red[(rl * WAVES_N + w) * 2 + 0];
          const float qw = red[(rl * WAVES_N + w) * 2 + 1];
          const float nb = (float)cw;
          const float tot = n_acc + nb;
          const float delta = mw - mean;
          mean += delta * (nb / tot);
          m2 += qw + delta * delta * (n_acc * nb / tot);
          n_acc = tot;
        }
        float* st = p.stats + ((size_t)m * p.tiles_n + tc.tn) * 2;
        st[0] = mean;
        st[1] = m2;
      }
      // fp32 X for the normalisation pass.
      float* X = p.ws;
#pragma unroll
      for (int i = 0; i < FM; ++i) {
        const int m = m_base + i * 32;
        if (m >= M) continue;
        float* xrow = X + (size_t)m * N;
#pragma unroll
        for (int j = 0; j < FN; ++j) {
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            const int n = n_base + j * 32 + g * 8;
            f32x4 v;
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] = acc[i][j][g * 4 + e];
            if (vec_ok && n + 3 < N) {
              *(f32x4*)(xrow + n) = v;
            } else {
#pragma unroll
              for (int e = 0; e < 4; ++e)
                if (n + e < N) xrow[n + e] = v[e];
            }
          }
        }
      }
    }
  }
};

template <typename T, int BM, int BN, int WAVES_M, int WAVES_N, int EPI, bool DIRECT>
__global__ void __launch_bounds__(WAVES_M* WAVES_N * 64)
    gemmrc_kernel(const GemmParams p) {
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  GemmTile<T, BM, BN, WAVES_M, WAVES_N, EPI, DIRECT>::run(p, smem);
}

}  // namespace beam
