// Large-problem gemmrc kernel for gfx950: 256 x 256 workgroup tile, four wavefronts of 128 x 128,
// one wavefront per SIMD, accumulators in the 256 accumulation registers, one workgroup per CU
// walking its output tiles with the operand ring running straight through the tile boundaries.
//
// Same operation and layouts as gemm_kernel.h (C = A . B^T, fp32 accumulation, 16-bit output;
// reference: cuda/cute_kernels/cute_gemm_128x256.cu:17-194, its software-pipelined K loop
// :141-167).  What differs from the 8-wavefront tiles and why:
//
//   * a 128 x 128 wavefront tile needs 16 LDS fragment reads per 64 MFMAs instead of 12 per 32: a
//     third fewer LDS bytes per flop, and this part is power limited on real data;
//   * a wavefront alone on its SIMD issues in order, so what it issues between two MFMAs decides
//     whether the matrix core idles.  Measured on this machine with a lone wavefront per SIMD
//     (64 independent v_mfma_f32_16x16x32_f16 per loop pass = 1024 matrix-core cycles): nothing
//     else 1045 cycles per pass; one ds_read_b128 after every 4th MFMA 1057; the same 16 reads
//     in groups of four 1120, all at the head 1129; 8 LDS-direct buffer loads, one after every 8th
//     MFMA, +4; a workgroup barrier per pass +16.  Hence the rule of the loop below: at most ONE
//     memory instruction between two MFMAs, never two in a row;
//   * the MFMAs are inline assembly with the accumulator tied to an accumulation register.  Left to
//     the compiler, 64 live accumulator blocks (all 256 registers) make it rotate blocks through
//     spare registers with v_accvgpr_mov/read/write and wait states inside the loop;
//   * the ring of LDS operand slots (3 for A, 2 for B) never drains: while the last K tiles of one
//     output tile are multiplied, the first K tiles of the workgroup's next output tile are already
//     being fetched, and the finished accumulators are converted and stored row block by row block
//     in the gaps of the next tile's first K tile (whose first MFMAs start from a zero addend
//     instead of from cleared registers).  No LDS staging, no extra barrier, no pipeline refill;
//   * the B fragment of MFMA block b takes rows 32*(b/2) + 8*(r/4) + 4*(b%2) + r%4 (r = lane % 16)
//     of the wavefront's B rows instead of 16*b + r: a lane then holds 8 consecutive output
//     columns per pair of blocks and stores them as one 16-byte access (64 contiguous bytes per
//     output row and instruction).  The B slots use a swizzle made for that row pattern.
//
//   * B stored [K][N] (B_KMAJOR, the layout of matmul(a, b)): a B tile lies in its slot as it lies in
//     memory, 64 rows of k by 256 columns, and a fragment is two transposing 8-byte reads
//     (ds_read_b64_tr_b16) in place of one 16-byte read.  In a transposing read four lanes supply the
//     addresses of the four column groups of a 16-column block, so the same permuted column order costs
//     nothing; to keep those reads free of bank conflicts the two blocks of a pair swap their halves of a
//     lane's 8 columns in the odd lane groups, which the store undoes with four selects (w4_kmajor_*).
//
// Preconditions (the host checks them; anything else takes the kernels of gemm_kernel.h):
// K a multiple of 64 and at least 192, N a multiple of 8, C 16-byte aligned, grid <= number of tiles;
// B_KMAJOR: K * N * 2 below 2^31 (the K tile's byte offset into B is a 32-bit scalar).
#pragma once

#include "gemm_kernel.h"

namespace beam {

// The 64 accumulator blocks of a wavefront live in the accumulation registers a0 .. a255 (block n in
// a[4n : 4n+3]) and are named only inside inline assembly: the compiler never allocates, copies or
// spills them.  (Handed 64 live four-register values that fill the whole file, its allocator starts
// rotating blocks through spare registers and scratch memory.)  The compiler is told once, by a clobber
// list, that these registers are in use; it has no reason to touch them itself as long as the rest of
// the kernel fits the 256 ordinary registers.
template <typename T>
struct W4Mfma;

template <>
struct W4Mfma<_Float16> {
  // block BLK += b x a (b supplies the output columns, a the output rows)
  template <int BLK>
  static __device__ __forceinline__ void fma(f16x8 b, f16x8 a) {
    asm volatile("v_mfma_f32_16x16x32_f16 a[%2:%3], %0, %1, a[%2:%3]" ::"v"(b), "v"(a), "n"(4 * BLK), "n"(4 * BLK + 3));
  }
  // block BLK = b x a: the first K step of an output tile
  template <int BLK>
  static __device__ __forceinline__ void first(f16x8 b, f16x8 a) {
    asm volatile("v_mfma_f32_16x16x32_f16 a[%2:%3], %0, %1, 0" ::"v"(b), "v"(a), "n"(4 * BLK), "n"(4 * BLK + 3));
  }
};

template <>
struct W4Mfma<__bf16> {
  template <int BLK>
  static __device__ __forceinline__ void fma(bf16x8 b, bf16x8 a) {
    asm volatile("v_mfma_f32_16x16x32_bf16 a[%2:%3], %0, %1, a[%2:%3]" ::"v"(b), "v"(a), "n"(4 * BLK), "n"(4 * BLK + 3));
  }
  template <int BLK>
  static __device__ __forceinline__ void first(bf16x8 b, bf16x8 a) {
    asm volatile("v_mfma_f32_16x16x32_bf16 a[%2:%3], %0, %1, 0" ::"v"(b), "v"(a), "n"(4 * BLK), "n"(4 * BLK + 3));
  }
};

// Element REG of the accumulation registers.  The caller keeps matrix-core results at least three MFMAs
// (48 cycles) old before reading them: the compiler cannot insert the wait states it does not know about.
template <int REG>
__device__ __forceinline__ float w4_acc_read() {
  float x;
  asm volatile("v_accvgpr_read_b32 %0, a[%1:%1]" : "=v"(x) : "n"(REG));
  return x;
}

__device__ __forceinline__ void w4_claim_acc_registers() {
  asm volatile("" ::: "a0", "a1", "a2", "a3", "a4", "a5", "a6", "a7", "a8", "a9", "a10", "a11", "a12", "a13", "a14", "a15",
               "a16", "a17", "a18", "a19", "a20", "a21", "a22", "a23", "a24", "a25", "a26", "a27", "a28", "a29", "a30", "a31",
               "a32", "a33", "a34", "a35", "a36", "a37", "a38", "a39", "a40", "a41", "a42", "a43", "a44", "a45", "a46", "a47",
               "a48", "a49", "a50", "a51", "a52", "a53", "a54", "a55", "a56", "a57", "a58", "a59", "a60", "a61", "a62", "a63",
               "a64", "a65", "a66", "a67", "a68", "a69", "a70", "a71", "a72", "a73", "a74", "a75", "a76", "a77", "a78", "a79",
               "a80", "a81", "a82", "a83", "a84", "a85", "a86", "a87", "a88", "a89", "a90", "a91", "a92", "a93", "a94", "a95",
               "a96", "a97", "a98", "a99", "a100", "a101", "a102", "a103", "a104", "a105", "a106", "a107", "a108", "a109",
               "a110", "a111", "a112", "a113", "a114", "a115", "a116", "a117", "a118", "a119", "a120", "a121", "a122", "a123",
               "a124", "a125", "a126", "a127", "a128", "a129", "a130", "a131", "a132", "a133", "a134", "a135", "a136", "a137",
               "a138", "a139", "a140", "a141", "a142", "a143", "a144", "a145", "a146", "a147", "a148", "a149", "a150", "a151",
               "a152", "a153", "a154", "a155", "a156", "a157", "a158", "a159", "a160", "a161", "a162", "a163", "a164", "a165",
               "a166", "a167", "a168", "a169", "a170", "a171", "a172", "a173", "a174", "a175", "a176", "a177", "a178", "a179",
               "a180", "a181", "a182", "a183", "a184", "a185", "a186", "a187", "a188", "a189", "a190", "a191", "a192", "a193",
               "a194", "a195", "a196", "a197", "a198", "a199", "a200", "a201", "a202", "a203", "a204", "a205", "a206", "a207",
               "a208", "a209", "a210", "a211", "a212", "a213", "a214", "a215", "a216", "a217", "a218", "a219", "a220", "a221",
               "a222", "a223", "a224", "a225", "a226", "a227", "a228", "a229", "a230", "a231", "a232", "a233", "a234", "a235",
               "a236", "a237", "a238", "a239", "a240", "a241", "a242", "a243", "a244", "a245", "a246", "a247", "a248", "a249",
               "a250", "a251", "a252", "a253", "a254", "a255");
}

// f(std::integral_constant<int, 0>{}), ..., f(std::integral_constant<int, N - 1>{}): a loop whose index is a
// constant expression in the body (register numbers inside assembly text have to be).
template <int I, int N, typename F>
__device__ __forceinline__ void w4_static_for(F&& f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>{});
    w4_static_for<I + 1, N>(f);
  }
}

// XOR pattern of the 16-byte chunks of a B row in LDS.  A fragment read touches, per 16 lanes, rows
// base + 8*(r/4) + r%4 (+4 for odd blocks), r = 0..15: bits 1, 3 and 4 of the row number take all
// 8 combinations and bit 0 selects the half of the 256-byte bank sweep, so 16 distinct 16-byte slots.
__host__ __device__ inline int w4_swizzle_b(int row) { return (((row >> 3) & 3) << 1) | ((row >> 1) & 1); }
// First B row (inside the wavefront's 128) of MFMA block b, and the row of lane-row r in it.
__host__ __device__ inline int w4_b_row(int b, int r) { return 32 * (b >> 1) + 4 * (b & 1) + 8 * (r >> 2) + (r & 3); }

// (B as [K][N]: the slot layout and the transposing reads' addresses are w4_kmajor_* in tile_map.h.)

// SB, SA: a wavefront issues its 8 loads of the next B tile in gaps 0, SB, 2 SB, ... of step A and its 8
// loads of the A tile after next in gaps 0, SA, ... of step B.  The path from the vector-memory unit into
// LDS moves 64 bytes per cycle and CU, i.e. one 1 KiB load per 64 cycles (4 MFMAs) and wavefront when all
// four issue: loads issued faster than that stall the wavefront, and with it its MFMAs, at issue.
// C_NT: C is stored non-temporal (an output larger than the last-level cache: its lines then do not push
// operand panels out of the caches).
// LN: the fused GEMM+LayerNorm of gemm_kernel.h (kEpiLnFused) with this K loop: output tiles in the band
// order of tile_map.h, and after each tile's K loop the same exchange of per-row (mean, M2) pairs between the
// column tiles of a row band, normalisation in registers, Y stored once.  A workgroup walks the ids
// blockIdx, blockIdx + gridDim, ... of that order: with a grid as large as the order it has one tile, with a
// grid of one workgroup per CU it walks several, and the operand ring then runs through the tile boundary as
// in the plain kernel -- the next tile's first operand tiles arrive while the band's statistics are
// exchanged (walking_layer_norm below says why nobody waits for ever).
// B_KMAJOR: B is stored [K][N].
template <typename T, bool C_NT = false, bool LN = false, int SB = 4, int SA = 8, int G0 = 2, bool B_KMAJOR = false>
struct GemmW4 {
  static_assert(!(LN && B_KMAJOR), "the fused LayerNorm is built for B as [N][K]");
  using Traits = ElemTraits<T>;
  using vec8 = typename Traits::vec8;
  using Mfma = W4Mfma<T>;

  static constexpr int BM = 256, BN = 256;
  static constexpr int NW = 4, NT = 256;
  static constexpr int FM = 8, FN = 8;          // 16 x 16 blocks of a wavefront tile
  static constexpr int SLOT = 256 * kRowBytes;  // one operand tile of 64 K elements: 32 KiB
  static constexpr int AST = 3, BST = 2;
  static constexpr int B_REGION = AST * SLOT;
  static constexpr int LDS_BYTES = (AST + BST) * SLOT;
  static constexpr int LPT = SLOT / (NW * 1024);  // buffer loads per wavefront per operand tile (8)
  static_assert(LDS_BYTES == 160 * 1024 && LPT == 8, "LDS budget");
  static constexpr int B_READS = B_KMAJOR ? 2 * FN : FN;  // LDS reads that make the B fragments of a step
  // What goes into gap m (after MFMA m) of a step: load number k, or fragment read number n (B 0..B_READS-1,
  // then A 0..7; they take the gaps the loads leave free, in order), or nothing (-1).
  // G0: gaps 0 .. G0 - 1 of step A hold nothing but, in the last of them, the wait and the barrier
  static constexpr int load_at(int half, int m) {
    const int s = half == 0 ? SB : SA;
    return (m >= G0 && (m - G0) % s == 0 && (m - G0) / s < LPT) ? (m - G0) / s : -1;
  }
  static constexpr int read_at(int half, int m) {
    if (m < G0 || load_at(half, m) >= 0) return -1;
    int n = 0;
    for (int x = G0; x < m; ++x) n += load_at(half, x) < 0;
    return n < B_READS + FM ? n : -1;
  }
  static constexpr int LAST_B = G0 + (LPT - 1) * SB, LAST_A = G0 + (LPT - 1) * SA;  // gaps of a step's last load
  static constexpr int last_read(int half) {
    int m = 63;
    while (read_at(half, m) < 0) --m;
    return m;
  }
  static constexpr int LAST_READ = last_read(0) > last_read(1) ? last_read(0) : last_read(1);
  static constexpr int kLnStores = FM * FN / 2;  // 16-byte stores per wavefront of a LayerNorm epilogue (32)
  static_assert(LAST_B + 3 < 64 && LAST_A + 3 < 64 && LAST_READ + 2 < LAST_A, "room for the scalar bookkeeping");
  static_assert(load_at(0, LAST_B) == LPT - 1 && load_at(1, LAST_A) == LPT - 1 && LAST_B < 62 && LAST_A < 62, "loads fit a step");

  static __device__ __forceinline__ void run(const GemmParams& p, char* smem) {
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave & 1, wn = wave >> 1;
    const int r = lane & 15, g = lane >> 4;
    const int M = p.M, N = p.N, K = p.K;
    const int n_k = K / kBK;
    const int total_tiles = p.tiles_m * p.tiles_n;
    const int first_tile = blockIdx.x, tile_step = gridDim.x;
    // LN: id of the band order -> tile (tm < 0: the band grids are padded), and the first id from `id` on, in
    // steps of the grid, that is a tile (>= p.ln_ids: none)
    auto ln_next_id = [&](int id, TileCoord* tc) {
      for (; id < p.ln_ids; id += tile_step) {
        *tc = band_order_tile(id, p.tiles_m, p.tiles_n, p.group_m, p.group_n, p.divs);
        if (tc->tm >= 0) break;
      }
      return id;
    };
    int ln_id = 0;
    TileCoord ln_tile{0, 0};
    if constexpr (LN) {
      ln_id = ln_next_id(first_tile, &ln_tile);
      if (ln_id >= p.ln_ids) return;
    }
    // (LN: the number of tiles is found on the way; the streams' descriptors are made from `has_tile` flags)
    const int my_tiles = LN ? 1 : (total_tiles - first_tile + tile_step - 1) / tile_step;
    const int g_total = my_tiles * n_k;  // K tiles this workgroup multiplies

    // ---- global -> LDS -----------------------------------------------------------------------
    // Load i of wavefront w fills bytes [(4 i + w) KiB, + 1 KiB) of a slot = rows 32 i + 8 w .. + 8;
    // lane l writes position l % 8 of row 32 i + 8 w + l / 8 and fetches the chunk that belongs there.
    // (Neither swizzle depends on i; B as [K][N] has its own map below.)  The row goes into the per-lane offset, the K tile into the scalar
    // offset: the hardware checks their sum against the descriptor's size, and a row past the end of a
    // matrix is past it by its per-lane part alone: that check is what keeps such rows from touching memory.
    const int fill_row = 8 * wave + (lane >> 3);
    unsigned voff_a[LPT], voff_b[LPT];
#pragma unroll
    for (int i = 0; i < LPT; ++i) {
      const unsigned row_bytes = (unsigned)(fill_row + 32 * i) * (unsigned)K * 2u;
      voff_a[i] = row_bytes + (unsigned)(((lane & 7) ^ swizzle_of_row(fill_row)) << 4);
      if constexpr (B_KMAJOR) {
        // 1 KiB = rows k, k + 1 of the [K][N] tile, k = 8 i + 2 w; lane l fills position l % 32 of row k + l / 32
        const int k = 8 * i + 2 * wave + (lane >> 5);
        voff_b[i] = ((unsigned)k * (unsigned)N + (unsigned)(((lane & 31) ^ w4_kmajor_swizzle(k)) << 3)) * 2u;
      } else {
        voff_b[i] = row_bytes + (unsigned)(((lane & 7) ^ w4_swizzle_b(fill_row)) << 4);
      }
    }

    // Operand rows of the workgroup's j-th output tile as (address, bytes) of a buffer descriptor; empty
    // past its last tile: such loads are issued and counted like any other and touch no memory.
    auto tile_coord = [&](int j) { return tile_of_workgroup(first_tile + j * tile_step, p.tiles_m, p.tiles_n, p.group_m, p.divs); };
    auto rows_of_a = [&](int j, TileCoord tc) {
      if (j >= my_tiles) return make_rsrc(p.A, 0u);
      const int row0 = tc.tm * BM;
      const int rows = (M - row0) < BM ? (M - row0) : BM;
      return make_rsrc((const T*)p.A + (size_t)row0 * K, (unsigned)rows * (unsigned)K * 2u);
    };
    auto rows_of_b = [&](int j, TileCoord tc) {
      if (j >= my_tiles) return make_rsrc(p.B, 0u);
      const int col0 = tc.tn * BN;
      const int rows = (N - col0) < BN ? (N - col0) : BN;
      // [K][N]: the tile's columns of all K rows (the range check counts the scalar offset, which holds the K
      // tile here, together with the per-lane one).  Columns past the tile's last one read the next row's data,
      // past the last row's end nothing: they only feed output columns that do not exist.
      if constexpr (B_KMAJOR) return make_rsrc((const T*)p.B + col0, ((unsigned)(K - 1) * (unsigned)N + (unsigned)rows) * 2u);
      return make_rsrc((const T*)p.B + (size_t)col0 * K, (unsigned)rows * (unsigned)K * 2u);
    };
    // A load stream: the operand rows of the output tile it is at (a finished buffer descriptor), the K
    // tile inside them (byte offset in a row) and the ring slot (byte offset in LDS, plus this wavefront's
    // KiB) its next loads go to.  The streams run ahead of the multiplication, across the boundaries of
    // output tiles.  Advancing one is a handful of scalar selects (no branch), dealt out over a few gaps
    // between MFMAs like everything else.
    struct Stream {
      __amdgpu_buffer_rsrc_t rows;
      int koff;
      int lds;
    };
    // bytes from one K tile to the next and to the end of K, per operand
    const int a_step = kBK * 2, a_end = K * 2;
    const int b_step = B_KMAJOR ? kBK * N * 2 : kBK * 2, b_end = B_KMAJOR ? K * N * 2 : K * 2;
    // The LDS address of an LDS-direct load comes from M0.  The compiler's own sequence for the builtin
    // is "write M0, one wait state, load" in one place; here M0 is written one gap ahead of the load, so
    // the MFMA between them is the wait state and no gap holds more than one scalar and one memory
    // instruction.  The loads are therefore invisible to the compiler's wait-count bookkeeping; every wait
    // for them in this kernel is an explicit s_waitcnt vmcnt.
    auto set_load_target = [&](const Stream& st, auto i_tag) __attribute__((always_inline)) {
      // (the add writes the scalar condition bit: without that in the clobber list the compiler keeps a compare's
      // result alive across this statement and selects on the add's carry instead)
      asm volatile("s_add_u32 m0, %0, %1" ::"s"(st.lds), "n"(decltype(i_tag)::value * 4096) : "memory", "scc");
    };
    auto load_tile_part = [&](const Stream& st, unsigned voff) __attribute__((always_inline)) {
      asm volatile("buffer_load_dwordx4 %0, %1, %2 offen lds" ::"v"(voff), "s"(st.rows), "s"(st.koff) : "memory");
    };
    // (in `part`s of two or three scalar instructions, one part per gap; part < 0: all of them)
    bool wrap_a = false, wrap_b = false;
    auto advance = [&](Stream& st, bool& wrap, __amdgpu_buffer_rsrc_t next, int ring_begin, int ring_end, int k_step, int k_end, int part) __attribute__((always_inline)) {
      if (part == 0 || part < 0) {
        const int lds = st.lds + SLOT;
        st.lds = lds == ring_end + wave * 1024 ? ring_begin + wave * 1024 : lds;
      }
      if (part == 1 || part < 0) {
        const int k = st.koff + k_step;
        wrap = k == k_end;
        st.koff = wrap ? 0 : k;
      }
      if (part == 2 || part < 0) st.rows = wrap ? next : st.rows;
    };

    // ---- LDS -> fragments ----------------------------------------------------------------------
    // 16x16x32 operand: lane supplies row r of the block, K elements 8 g .. 8 g + 7 of the 32-wide step.
    int a_off[2], b_off[2];
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      a_off[kk] = lds_offset(wm * 128 + r, 4 * kk + g);
      const int brow = wn * 128 + w4_b_row(0, r);
      b_off[kk] = brow * kRowBytes + (((4 * kk + g) ^ w4_swizzle_b(brow)) << 4);
    }
    // [K][N]: where this lane points in a transposing read of block b = 2 pair + parity (first read, first half)
    int bt_off[2][FN / 2];
    if constexpr (B_KMAJOR) {
#pragma unroll
      for (int par = 0; par < 2; ++par)
#pragma unroll
        for (int pair = 0; pair < FN / 2; ++pair) bt_off[par][pair] = w4_kmajor_read_offset(wn, 2 * pair + par, g, (lane >> 2) & 3, lane & 3);
    }
    auto read_b_transposed = [&](const char* sb, int half, int n) __attribute__((always_inline)) {
      // read n of a step: rows +0 (n even) or +4 (n odd) of block n / 2, in the K tile's half `half`
      typedef short i16x4 __attribute__((ext_vector_type(4)));
      const char* at = sb + bt_off[(n >> 1) & 1][n >> 2] + half * (32 * 512) + (n & 1) * (4 * 512);
      return __builtin_bit_cast(i32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) i16x4*)at));
    };

    w4_claim_acc_registers();  // block (i, b) of the wavefront tile is accumulator block 8 i + b
    // Fragments, double buffered: set 0 holds the first 32 K elements of a tile, set 1 the second.
    vec8 fa0[FM], fa1[FM], fb0[FN], fb1[FN];
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        fa0[i][e] = 0;
        fa1[i][e] = 0;
        fb0[i][e] = 0;
        fb1[i][e] = 0;
      }

    // ---- output --------------------------------------------------------------------------------
    // acc[i][b][e]: row 128 wm + 16 i + r, column 128 wn + 32 (b / 2) + 8 g + 4 (b % 2) + e of the tile.
    // A pair of blocks is one 16-byte store per lane through a descriptor of row blocks i .. 7 of the
    // tile's part of C (per row block, because only the per-lane offset is range checked): rows that do
    // not exist fall outside it, columns that do not exist get an offset outside it.
    struct OutTile {
      char* base;  // first element of the tile in C
      int bytes;   // from there to the end of the tile's last valid row
      unsigned voff[FN / 2];
    };
    auto out_tile_of = [&](int j, TileCoord tc) {
      OutTile o;
      if (j < 0 || j >= my_tiles) {
        o.base = (char*)p.C;
        o.bytes = 0;
#pragma unroll
        for (int q = 0; q < FN / 2; ++q) o.voff[q] = kOobOffset;
        return o;
      }
      const int row0 = tc.tm * BM, col0 = tc.tn * BN;
      const int rows = (M - row0) < BM ? (M - row0) : BM;
      const int cols = (N - col0) < BN ? (N - col0) : BN;
      o.base = (char*)((T*)p.C + ((size_t)row0 * N + col0));
      o.bytes = ((rows - 1) * N + cols) * 2;
#pragma unroll
      for (int q = 0; q < FN / 2; ++q) {
        const int col = wn * 128 + 32 * q + 8 * g;
        o.voff[q] = col < cols ? ((unsigned)(wm * 128 + r) * (unsigned)N + (unsigned)col) * 2u : kOobOffset;
      }
      return o;
    };
    OutTile out = out_tile_of(-1, TileCoord{0, 0});  // the tile whose accumulators are being stored
    // LAST: the stores after the workgroup's last K loop.  Nothing hides them, and a kernel ends only when its
    // dirty lines have left the L2: those go through it to memory at once (device-scope stores; 4096^3, one tile
    // per workgroup: 98.9 -> 96.5 us, fused LayerNorm 105.7 -> 103.7 us).  The stores of earlier tiles lie under
    // the next tile's MFMAs and stay plain (written through, 8192^3 loses 0.2%).
    auto store_pair = [&](auto i_tag, auto q_tag, auto last_tag) __attribute__((always_inline)) {
      constexpr int i = decltype(i_tag)::value, q = decltype(q_tag)::value;
      constexpr int AUX = C_NT ? 2 : (decltype(last_tag)::value ? kAuxDeviceScope : 0);
      constexpr int R0 = 4 * (8 * i + 2 * q);  // first register of block (i, 2 q); block (i, 2 q + 1) follows
      vec8 v;
      v[0] = (T)w4_acc_read<R0 + 0>();
      v[1] = (T)w4_acc_read<R0 + 1>();
      v[2] = (T)w4_acc_read<R0 + 2>();
      v[3] = (T)w4_acc_read<R0 + 3>();
      v[4] = (T)w4_acc_read<R0 + 4>();
      v[5] = (T)w4_acc_read<R0 + 5>();
      v[6] = (T)w4_acc_read<R0 + 6>();
      v[7] = (T)w4_acc_read<R0 + 7>();
      i32x4 w = __builtin_bit_cast(i32x4, v);
      if constexpr (B_KMAJOR) {  // odd lane groups hold the two blocks' columns the other way round
        const i32x4 s = {w[2], w[3], w[0], w[1]};
        w = (g & 1) ? s : w;
      }
      const int skip = i * 16 * N * 2;  // bytes of the row blocks above this one
      const int left = out.bytes - skip;
      const __amdgpu_buffer_rsrc_t rsrc = make_rsrc(out.base + skip, left > 0 ? (unsigned)left : 0u);
      __builtin_amdgcn_raw_buffer_store_b128(w, rsrc, (int)out.voff[q], 0, AUX);
    };

    // ---- one K tile ------------------------------------------------------------------------------
    // Step A multiplies the second half of the previous K tile (set 1) while the first half of this
    // one is read into set 0 and B of the next K tile is fetched; step B multiplies set 0 while the
    // second half is read into set 1 and A of the K tile after next is fetched.  Every MFMA is
    // followed by at most one memory instruction and a scheduling fence.
    // FIRST: this is the first K tile of an output tile.  Step A then completes the previous output
    // tile row block by row block; each pair of its blocks is converted and stored a little later
    // (three MFMAs after the row's last one at the earliest: results of the matrix core must not be
    // read sooner, and the compiler does not see the inline-assembly MFMAs), always before step B
    // overwrites it.
    Stream ld_a, ld_b;         // where the next A / B loads go
    __amdgpu_buffer_rsrc_t next_a, next_b;  // operand rows of the output tile after the one the streams are at
    int rd_a = 0, rd_b = B_REGION;  // slots (byte offsets) of the K tile being multiplied
    // LN, FIRST: the accumulators hold nothing that step A could complete (the previous tile was finished and
    // stored by its epilogue; set 1 is stale), so step A issues no MFMA -- a one-cycle no-op stands in for each,
    // which also keeps the wait state between a write of M0 and the load that uses it.  after_epilogue: the
    // youngest memory operations of this wavefront are then the 32 stores of that epilogue, not loads.
    bool after_epilogue = false;
    auto k_tile = [&](auto first_tag) __attribute__((always_inline)) {
      constexpr bool FIRST = decltype(first_tag)::value;
      const char* sa = smem + rd_a;
      const char* sb = smem + rd_b;
      w4_static_for<0, 128>([&](auto gap_tag) __attribute__((always_inline)) {
        constexpr int gap = decltype(gap_tag)::value;
        constexpr int half = gap >> 6, m = gap & 63;
        // row blocks in turn, the B fragments forwards and backwards alternately: consecutive MFMAs always
        // share one operand (fewer input toggles; this part is power limited)
        constexpr int i = m >> 3, b = (i & 1) ? 7 - (m & 7) : (m & 7);
        constexpr int blk = 8 * i + b;
        if constexpr (half == 0 && LN && FIRST) asm volatile("s_nop 0");
        else if constexpr (half == 0) Mfma::template fma<blk>(fb1[b], fa1[i]);
        else if constexpr (FIRST) Mfma::template first<blk>(fb0[b], fa0[i]);
        else Mfma::template fma<blk>(fb0[b], fa0[i]);
        // the gap
        if constexpr (gap == G0 - 1) {
          // Two MFMAs of the previous K tile are in the matrix core's queue while the wavefronts meet.
          // my fills of this K tile have landed (the youngest 8 are A of the next one) ...
          if constexpr (LN && FIRST) {
            if (after_epilogue) wait_vm_and_lds<kLnStores>();
            else wait_vm_and_lds<LPT>();
          } else {
            wait_vm_and_lds<LPT>();
          }
          bare_barrier();          // ... everyone's have, and everyone is done reading the slots refilled below
        }
        constexpr int ld = load_at(half, m), rd = read_at(half, m);
        constexpr int ld_next = m + 1 < 64 ? load_at(half, m + 1) : -1;
        if constexpr (ld_next >= 0) {
          if constexpr (half == 0) set_load_target(ld_b, std::integral_constant<int, ld_next>{});
          else set_load_target(ld_a, std::integral_constant<int, ld_next>{});
        }
        if constexpr (ld >= 0) {
          if constexpr (half == 0) load_tile_part(ld_b, voff_b[ld]);
          else load_tile_part(ld_a, voff_a[ld]);
        } else if constexpr (rd >= 0 && rd < B_READS) {
          if constexpr (B_KMAJOR) {
            const i32x2 v = read_b_transposed(sb, half, rd);  // K elements 0..3 (even read) or 4..7 of the lane's 8
            vec8& f = half == 0 ? fb0[rd >> 1] : fb1[rd >> 1];
            i32x4 w = __builtin_bit_cast(i32x4, f);
            w[2 * (rd & 1)] = v[0];
            w[2 * (rd & 1) + 1] = v[1];
            f = __builtin_bit_cast(vec8, w);
          } else {
            const vec8 v = *(const vec8*)(sb + b_off[half] + (rd >> 1) * 4096 + (rd & 1) * 512);
            if constexpr (half == 0) fb0[rd] = v;
            else fb1[rd] = v;
          }
        } else if constexpr (rd >= B_READS) {
          const vec8 v = *(const vec8*)(sa + a_off[half] + (rd - B_READS) * 2048);
          if constexpr (half == 0) fa0[rd - B_READS] = v;
          else fa1[rd - B_READS] = v;
        }
        // scalar bookkeeping, a few instructions per gap: the B stream moves on after its last load, ...
        if constexpr (half == 0 && m > LAST_B && m <= LAST_B + 3) advance(ld_b, wrap_b, next_b, B_REGION, LDS_BYTES, b_step, b_end, m - LAST_B - 1);
        // ... the read slots once the last fragment read of the K tile is out, the A stream after its last load
        if constexpr (half == 1 && m == LAST_READ + 1) rd_a = rd_a + SLOT == B_REGION ? 0 : rd_a + SLOT;
        if constexpr (half == 1 && m == LAST_READ + 2) rd_b = rd_b + SLOT == LDS_BYTES ? B_REGION : rd_b + SLOT;
        if constexpr (half == 1 && m > LAST_A && m <= LAST_A + 3) advance(ld_a, wrap_a, next_a, 0, B_REGION, a_step, a_end, m - LAST_A - 1);
        if constexpr (FIRST && !LN && gap >= 10 && gap < 10 + 8 * FM && ((gap - 10) & 1) == 0) {
          // pair q of row block i goes into gap 10 + 8 i + 2 q
          store_pair(std::integral_constant<int, (gap - 10) / 8>{}, std::integral_constant<int, ((gap - 10) / 2) % 4>{}, std::false_type{});
        }
        __builtin_amdgcn_sched_barrier(0);
      });
    };

    auto load_whole_tile = [&](const Stream& st, const unsigned(&voff)[LPT]) __attribute__((always_inline)) {
      w4_static_for<0, LPT>([&](auto i_tag) __attribute__((always_inline)) {
        set_load_target(st, i_tag);
        asm volatile("s_nop 0");  // the wait state between the write of M0 and its use
        load_tile_part(st, voff[decltype(i_tag)::value]);
      });
    };
    // Prologue: A and B of K tile 0, A of K tile 1 (oldest first: the first wait is about tile 0).
    auto prologue = [&](__amdgpu_buffer_rsrc_t rows_a0, __amdgpu_buffer_rsrc_t rows_b0) __attribute__((always_inline)) {
      next_a = rows_a0;  // (never used: K >= 3 tiles, so no stream wraps before the loops below set them)
      next_b = rows_b0;
      ld_a = Stream{rows_a0, 0, wave * 1024};
      ld_b = Stream{rows_b0, 0, B_REGION + wave * 1024};
      load_whole_tile(ld_a, voff_a);
      load_whole_tile(ld_b, voff_b);
      advance(ld_a, wrap_a, next_a, 0, B_REGION, a_step, a_end, -1);
      advance(ld_b, wrap_b, next_b, B_REGION, LDS_BYTES, b_step, b_end, -1);
      load_whole_tile(ld_a, voff_a);
      advance(ld_a, wrap_a, next_a, 0, B_REGION, a_step, a_end, -1);
    };
    // The second half of a tile's last K tile is in set 1.
    auto drain = [&]() __attribute__((always_inline)) {
      w4_static_for<0, 64>([&](auto m_tag) __attribute__((always_inline)) {
        constexpr int m = decltype(m_tag)::value;
        Mfma::template fma<m>(fb1[m & 7], fa1[m >> 3]);
      });
      asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
    };

    if constexpr (LN) {
      TileCoord tc = ln_tile;
      prologue(rows_of_a(0, tc), rows_of_b(0, tc));
      // Scratch of the epilogue: compact (inside the two operand slots the ring leaves free at a tile boundary)
      // when a band has at most kLnCompactTiles column tiles, else all of LDS -- the host then gives every
      // workgroup one tile, and nothing is in flight when the K loop ends.
      const bool compact = p.tiles_n <= kLnCompactTiles;
      for (;;) {
        // The streams move on to the workgroup's next tile while this one is multiplied, as in the plain kernel.
        TileCoord tc_next = tc;
        const int next_id = ln_next_id(ln_id + tile_step, &tc_next);
        const bool has_next = next_id < p.ln_ids;  // (uniform)
        next_a = rows_of_a(has_next ? 0 : 1, tc_next);
        next_b = rows_of_b(has_next ? 0 : 1, tc_next);
        k_tile(std::true_type{});
        for (int h = 1; h < n_k; ++h) k_tile(std::false_type{});
        // Behind a workgroup's last tile the streams' fills are empty (they touch no memory and return at once): they
        // are waited for here, so that nothing is on its way into LDS when the epilogue reuses it or the kernel ends.
        // In front of a further tile the fills are that tile's first operand tiles, and nobody waits for them yet.
        if (!has_next) wait_vm_and_lds<0>();
        drain();
        out = out_tile_of(0, tc);
        // After K tile h: rd_a / rd_b are the slots of K tile h + 1 (the next tile's first, already there or on
        // its way, like A of the one after it); the slots K tile h was in are free until the next K loop's first
        // loads, which come behind a barrier that every wavefront reaches only after its epilogue.
        const int free_a = rd_a == 0 ? B_REGION - SLOT : rd_a - SLOT;
        const int free_b = rd_b == B_REGION ? B_REGION + SLOT : B_REGION;
        layer_norm_epilogue(p, smem, tc, out, compact, free_a, free_b);
        if (!has_next) break;
        ln_id = next_id;
        tc = tc_next;
        after_epilogue = true;
      }
    } else if (g_total > 0) {
      TileCoord tc_cur = tile_coord(0);
      prologue(rows_of_a(0, tc_cur), rows_of_b(0, tc_cur));
      for (int j = 0; j < my_tiles; ++j) {
        // The streams move on to tile j + 1 while tile j is multiplied: A in its last but one K tile,
        // B in its last.  With K = 3 tiles that is this very K tile, so the rows come first.
        const TileCoord tc_j = tc_cur;
        tc_cur = tile_coord(j + 1 < my_tiles ? j + 1 : j);
        next_a = rows_of_a(j + 1, tc_cur);
        next_b = rows_of_b(j + 1, tc_cur);
        k_tile(std::true_type{});
        out = out_tile_of(j, tc_j);  // from here on the accumulators belong to tile j
        for (int h = 1; h < n_k; ++h) k_tile(std::false_type{});
      }
      // Drain, then the last tile's output.
      wait_vm_and_lds<0>();
      drain();
      w4_static_for<0, FM * FN / 2>([&](auto o_tag) __attribute__((always_inline)) {
        constexpr int o = decltype(o_tag)::value;
        store_pair(std::integral_constant<int, o / 4>{}, std::integral_constant<int, o % 4>{}, std::true_type{});
      });
    }
  }

  // ---- LayerNorm over the row band (LN) -------------------------------------------------------------
  // The same five steps as the kEpiLnFused epilogue of gemm_kernel.h, for this kernel's accumulator layout:
  // row block i of a lane is 32 values (blocks 8 i .. 8 i + 7) of row 128 wm + 16 i + r, in the four groups of
  // 8 columns 128 wn + 32 q + 8 g; a row of the tile is spread over 4 lane groups x 2 wavefronts = 8 slots.
  // Thread t owns row t of the tile in steps 2 to 4 (256 threads, 256 rows).
  //
  // Scratch.  compact: the operand ring keeps running through the tile boundary, so three of the five LDS slots
  // hold the next tile's first operand tiles (landed or in flight) and only the two slots of the K tile just
  // multiplied are free: the lane partials (18 KiB) go into the free A slot, behind the 2 KiB that will hold the
  // rows' final (mean, rstd); the pairs of the band's column tiles (2 KiB per tile: 8 bytes per row) are gathered
  // into the free B slot (tiles 0 .. 15) and, the lane partials being dead by then, into the free A slot from its
  // start (tiles 16 .. 31).  A thread only ever touches its own row's 8 bytes of each of those 2 KiB, and it writes
  // its row's (mean, rstd) when it has merged its pairs, so the last 2 KiB may lie where tile 16's pairs were.
  // Hence kLnCompactTiles = 32.  Otherwise (up to 64 column tiles) all of LDS is used: the caller has made sure
  // that nothing is in flight and that no tile follows.
  //
  // Why nobody waits for ever when workgroups walk several tiles (one workgroup per CU, all resident): ids of the
  // band order that are 256 apart belong to one workgroup, which takes them in rising order and publishes a
  // tile's statistics before it waits for anything.  The tiles of one band lie within fewer than 256 consecutive
  // ids in each of the three orders (a band group of the padded orders is at most 8 x 32 ids; a band of the plain
  // order at most 64).  If tile T1 waits for T2 of its band, and T2 has not started because its workgroup is
  // still waiting at an earlier tile T3, then id(T3) <= id(T2) - 256 < id(T1): every such step leads to a strictly
  // smaller id, so no chain of waits returns to where it began, and the smallest id in any chain waits only for
  // tiles whose K loops are running or done.
  static constexpr int kLnCompactTiles = 32;
  template <typename OutTileT>
  static __device__ __forceinline__ void layer_norm_epilogue(const GemmParams& p, char* smem, TileCoord tc, const OutTileT& out,
                                                             bool compact, int free_a, int free_b) {
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave & 1, wn = wave >> 1;
    const int r = lane & 15, g = lane >> 4;
    const int N = p.N;
    const int col0 = tc.tn * BN;
    constexpr int SLOTS = 8, PITCH = SLOTS + 1;  // (a row of `part` is padded by one pair: see gemm_kernel.h)
    // Every barrier here is a bare one behind a wait for this wavefront's LDS accesses only: __syncthreads() would
    // also wait for the next tile's operand loads in flight.  The wait is assembly with a memory clobber: given the
    // s_waitcnt builtin, the compiler is free to sink the LDS stores in front of it to behind it (it sees no
    // dependence), and the other wavefronts then read what has not been written yet.
    auto lds_barrier = [&]() __attribute__((always_inline)) {
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      bare_barrier();
    };
    // gamma / beta of this lane's four column groups: issued now, used in step 5
    bool q_valid[4];
    vec8 gv[4], bv[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int n = col0 + wn * 128 + 32 * q + 8 * g;
      q_valid[q] = n < N;  // N is a multiple of 8: a group of 8 columns exists whole or not at all
      gv[q] = *(const vec8*)((const T*)p.gamma + (q_valid[q] ? n : 0));
      bv[q] = *(const vec8*)((const T*)p.beta + (q_valid[q] ? n : 0));
    }
    const int my_cols = 8 * ((int)q_valid[0] + (int)q_valid[1] + (int)q_valid[2] + (int)q_valid[3]);
    const bool full = col0 + BN <= N;
    bare_barrier();  // every wavefront is done with the slots of the last K tile (its fragments are in registers)
    float* red = (float*)(smem + (compact ? free_a : 0));  // [BM][2]: (mean, rstd) of the whole row, written in step 4
    float* part = red + BM * 2;                             // [BM][PITCH][2] lane partials
    // The pairs of this thread's row, one per column tile of the band, 2 KiB apart: tiles 0 .. n0 - 1 from g0 on,
    // the others from g1 on.
    const int n0 = compact ? (p.tiles_n < 16 ? p.tiles_n : 16) : p.tiles_n;
    const int n1 = p.tiles_n - n0;
    float* g0 = (compact ? (float*)(smem + free_b) : part) + tid * 2;
    float* g1 = red + tid * 2;
    constexpr int GP = BM * 2;  // floats from one tile's pairs to the next
    // 1. per-lane (mean, M2) over the lane's columns of each of its rows, dropped into LDS.  Two copies of the loop,
    //    chosen once per tile: a full tile (every column exists) needs no masks, and masks written as selects cost
    //    two instructions more per value (1757 against 1030 vector instructions per lane and tile).
    auto lane_stats = [&](auto full_tag) __attribute__((always_inline)) {
      constexpr bool FULL = decltype(full_tag)::value;
      w4_static_for<0, FM>([&](auto i_tag) __attribute__((always_inline)) {
        constexpr int i = decltype(i_tag)::value;
        float x[32];
        w4_static_for<0, 32>([&](auto t_tag) __attribute__((always_inline)) {
          constexpr int t = decltype(t_tag)::value;
          x[t] = w4_acc_read<4 * (8 * i) + t>();  // block 8 i + t / 4, element t % 4
        });
        float sum = 0.0f, m2 = 0.0f;
#pragma unroll
        for (int t = 0; t < 32; ++t) sum += (FULL || q_valid[t >> 3]) ? x[t] : 0.0f;
        const float mean = FULL ? sum * (1.0f / 32.0f) : (my_cols > 0 ? sum / (float)my_cols : 0.0f);
#pragma unroll
        for (int t = 0; t < 32; ++t) {
          const float d = x[t] - mean;
          if constexpr (FULL) m2 += d * d;
          else m2 += q_valid[t >> 3] ? d * d : 0.0f;
        }
        const int rl = wm * 128 + 16 * i + r;
        part[(rl * PITCH + wn * 4 + g) * 2 + 0] = mean;
        part[(rl * PITCH + wn * 4 + g) * 2 + 1] = m2;
      });
    };
    if (full) lane_stats(std::true_type{});  // (uniform)
    else lane_stats(std::false_type{});
    lds_barrier();
    // 2. one thread per row merges the 8 slots in a fixed order (Chan's update) ...
    const int rl = tid;
    float mean = 0.0f, m2 = 0.0f, n_acc = 0.0f;
    if (full) {
      // every slot covers 32 columns: the mean of the slot means, then M2 about it -- the merge below for
      // equal counts, in the same fixed order, without its divisions
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
        m2 += qw[slot] + 32.0f * d * d;
      }
    }
#pragma unroll
    for (int slot = 0; slot < (full ? 0 : SLOTS); ++slot) {
      int cnt = 0;
#pragma unroll
      for (int q = 0; q < 4; ++q) cnt += (col0 + (slot >> 2) * 128 + 32 * q + 8 * (slot & 3) < N) ? 8 : 0;
      if (cnt == 0) continue;
      const float mw = part[(rl * PITCH + slot) * 2 + 0];
      const float qw = part[(rl * PITCH + slot) * 2 + 1];
      const float nb = (float)cnt;
      const float tot = n_acc + nb;
      const float delta = mw - mean;
      mean += delta * (nb / tot);
      m2 += qw + delta * delta * (n_acc * nb / tot);
      n_acc = tot;
    }
    // ... and publishes the tile's pair (gemm_kernel.h: ln_publish, two tagged 8-byte words per row)
    const unsigned tag = ln_launch_tag(p);
    ln_sign_header(p, tag);
    ln_publish(p, ((size_t)tc.tm * p.tiles_n + tc.tn) * BM + rl, mean, m2, tag);
    lds_barrier();  // `part` is free again
    // 3. gather the pairs of this thread's row from the band's column tiles into LDS, 16 tiles' worth in flight at
    //    once, fetching again -- boundedly -- what does not carry the launch's tag yet (the protocol of
    //    gemm_kernel.h's ln_gather).  The tile's own pair comes back through memory like the others'.  What the
    //    gather costs is a round trip to memory (1.3 us) plus the spread of the band's tiles, whose CUs run at clocks
    //    several percent apart: 2.6 us for a band of 16 tiles, 5 us for one of 32, with 8 or 16 in flight alike.  (32
    //    in flight need 128 registers, and the compiler then parks values in accumulation registers, i.e. in the
    //    accumulators: the codegen test watches for that.)
    {
      const unsigned long long* w0s = (const unsigned long long*)p.stats + (size_t)tc.tm * p.tiles_n * BM + rl;
      const unsigned long long* w1s = (const unsigned long long*)p.next_stats + (size_t)tc.tm * p.tiles_n * BM + rl;
      const unsigned not_tag = ~tag;
      constexpr int INFLIGHT = 16;
      int polls = 0;
      for (int t0 = 0; t0 < p.tiles_n; t0 += INFLIGHT) {
        unsigned long long a[INFLIGHT], b[INFLIGHT];
        unsigned missing = 0;  // bit u: column tile t0 + u is still to be fetched
#pragma unroll
        for (int u = 0; u < INFLIGHT; ++u) {
          a[u] = 0;
          b[u] = 0;
          missing |= (t0 + u < p.tiles_n) ? (1u << u) : 0u;  // (the tile's own pair comes back like the others')
        }
        while (missing != 0) {
#pragma unroll
          for (int u = 0; u < INFLIGHT; ++u) {
            if (missing & (1u << u)) {
              a[u] = __hip_atomic_load(w0s + (size_t)(t0 + u) * BM, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
              b[u] = __hip_atomic_load(w1s + (size_t)(t0 + u) * BM, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
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
          const int t = t0 + u;
          if (t < p.tiles_n) {
            float* at = t < n0 ? g0 + t * GP : g1 + (t - n0) * GP;
            at[0] = __uint_as_float((unsigned)a[u]);
            at[1] = __uint_as_float((unsigned)b[u]);
          }
        }
      }
    }
    // (the pairs a thread merges are the ones it stored itself: no barrier in between)
    // 4. merge in tile order -> (mean, rstd) of the whole row.  The pairs come back from LDS eight at a time, every
    //    read of a batch issued before the first is used (a loop that waits for one read per step is bound by the
    //    latency of each), and none of them conditional (the compiler turns a conditional read into a branch): a
    //    batch that reaches past the last tile reads the last tile again, with weight zero.
    mean = 0.0f;
    m2 = 0.0f;
    n_acc = 0.0f;
    const bool even_tiles = (N % BN) == 0;  // every column tile is full: equal weights
    constexpr int CH = 8;
    float mw[CH], qw[CH];
    // tiles t0 .. t0 + CH - 1 of the region that starts at `base` and holds n tiles
    auto load_batch = [&](const float* base, int n, int t0, bool with_m2) __attribute__((always_inline)) {
#pragma unroll
      for (int u = 0; u < CH; ++u) {
        const int t = t0 + u < n ? t0 + u : n - 1;  // (uniform)
        mw[u] = base[t * GP];
        if (with_m2) qw[u] = base[t * GP + 1];
      }
    };
    // the two regions in tile order: (g0, n0 tiles, first tile 0), (g1, n1 tiles, first tile n0)
    if (even_tiles) {
#pragma unroll
      for (int reg = 0; reg < 2; ++reg) {
        const float* base = reg == 0 ? g0 : g1;
        const int n = reg == 0 ? n0 : n1;
        for (int t0 = 0; t0 < n; t0 += CH) {
          load_batch(base, n, t0, false);
#pragma unroll
          for (int u = 0; u < CH; ++u) mean += t0 + u < n ? mw[u] : 0.0f;
        }
      }
      mean *= 1.0f / (float)p.tiles_n;
#pragma unroll
      for (int reg = 0; reg < 2; ++reg) {
        const float* base = reg == 0 ? g0 : g1;
        const int n = reg == 0 ? n0 : n1;
        for (int t0 = 0; t0 < n; t0 += CH) {
          load_batch(base, n, t0, true);
#pragma unroll
          for (int u = 0; u < CH; ++u) {
            const float d = mw[u] - mean;
            m2 += t0 + u < n ? qw[u] + (float)BN * d * d : 0.0f;
          }
        }
      }
    } else {
#pragma unroll
      for (int reg = 0; reg < 2; ++reg) {
        const float* base = reg == 0 ? g0 : g1;
        const int n = reg == 0 ? n0 : n1;
        for (int t0 = 0; t0 < n; t0 += CH) {
          load_batch(base, n, t0, true);
#pragma unroll
          for (int u = 0; u < CH; ++u) {
            if (t0 + u < n) {  // (uniform)
              int cw = N - ((reg == 0 ? 0 : n0) + t0 + u) * BN;
              cw = cw > BN ? BN : cw;
              const float nb = (float)cw;
              const float tot = n_acc + nb;
              const float delta = mw[u] - mean;
              mean += delta * (nb / tot);
              m2 += qw[u] + delta * delta * (n_acc * nb / tot);
              n_acc = tot;
            }
          }
        }
      }
    }
    red[rl * 2 + 0] = mean;
    red[rl * 2 + 1] = even_tiles ? __builtin_amdgcn_rsqf(m2 * (1.0f / (float)N) + p.eps) : 1.0f / sqrtf(m2 / (float)N + p.eps);
    lds_barrier();
    // 5. normalise the accumulators and store Y: a pair of blocks is one 16-byte store per lane.  The stores go
    //    through the L2 to memory at once: nothing hides those of a workgroup's last tile, and a kernel ends only
    //    when its dirty lines have left the L2 (4096^3, one tile per workgroup: 105.7 -> 103.7 us); under a next
    //    tile's K loop the kind of store measures the same.  One copy of this code for every tile, whatever
    //    follows it: two instantiations of the same source need not round alike (the compiler fuses the last
    //    multiply-add with the conversion to 16 bits in one place and not in another, which differs on ties), and
    //    a workgroup that walks its tiles must give the bits of one that has a single tile.
    constexpr int AUX = kAuxDeviceScope;
    w4_static_for<0, FM>([&](auto i_tag) __attribute__((always_inline)) {
      constexpr int i = decltype(i_tag)::value;
      const int row = wm * 128 + 16 * i + r;
      const float row_mean = red[row * 2 + 0], rstd = red[row * 2 + 1];
      const int skip = i * 16 * N * 2;
      const int left = out.bytes - skip;
      const __amdgpu_buffer_rsrc_t rsrc = make_rsrc(out.base + skip, left > 0 ? (unsigned)left : 0u);
      w4_static_for<0, 4>([&](auto q_tag) __attribute__((always_inline)) {
        constexpr int q = decltype(q_tag)::value;
        vec8 v;
        w4_static_for<0, 8>([&](auto e_tag) __attribute__((always_inline)) {
          constexpr int e = decltype(e_tag)::value;
          v[e] = (T)((w4_acc_read<4 * (8 * i + 2 * q) + e>() - row_mean) * rstd * (float)gv[q][e] + (float)bv[q][e]);
        });
        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(i32x4, v), rsrc, (int)out.voff[q], 0, AUX);
      });
    });
    // (the reads of `red` above are behind the next K loop's first barrier only in program order: a wavefront must
    // have them before the loads behind that barrier overwrite the slot)
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  }
};

template <typename T, bool C_NT = false, bool LN = false, int SB = 4, int SA = 8, int G0 = 2, bool B_KMAJOR = false>
__global__ void __launch_bounds__(256) gemmrc_w4_kernel(const GemmParams p) {
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  GemmW4<T, C_NT, LN, SB, SA, G0, B_KMAJOR>::run(p, smem);
}

}  // namespace beam
