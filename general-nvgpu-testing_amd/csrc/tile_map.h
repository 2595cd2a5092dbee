// Integer index maps shared by device kernels and host-side checks.
//
// Everything here is plain integer arithmetic, callable from host and device, so the
// host can verify (by brute force) that each map is a bijection and that the LDS
// layout is bank-conflict free before any kernel is launched.
//
// Reference counterparts:
//   * workgroup -> tile rasterisation ("mtile" grouping):
//       cuda/cute_kernels/cute_gemm_128x128.cu:22-33, cute_gemm_128x256.cu:26-37
//   * shared-memory XOR swizzle of 16-byte chunks:
//       cuda/cute_kernels/cute_gemm_128x128.cu:55-65  (Swizzle<3,3,3>)
#pragma once

#define BEAM_HD __host__ __device__ inline

namespace beam {

// K extent (elements) of one LDS stage: 64 x 2 bytes = 128 bytes = 8 chunks of 16 bytes.
constexpr int kBK = 64;
constexpr int kRowBytes = kBK * 2;
constexpr int kChunksPerRow = 8;
// MI355X: 8 accelerator complex dies, workgroups are dispatched to them round-robin.
constexpr int kNumXcd = 8;

// XOR pattern applied to the 16-byte chunk index of an LDS row.
// LDS has 64 banks of 4 bytes (256 bytes per bank sweep) and rows are 128 bytes, so two
// consecutive rows share a sweep; 16 consecutive rows of the same logical chunk land on
// 16 distinct 16-byte slots when the chunk is XORed with (row >> 1) & 7.
BEAM_HD int swizzle_of_row(int row) { return (row >> 1) & 7; }

// Byte offset inside a stage of logical (row, chunk) after swizzling.
BEAM_HD int lds_offset(int row, int chunk) {
  return row * kRowBytes + ((chunk ^ swizzle_of_row(row)) << 4);
}

// B stored K-major ("NN" layout, B[K][N]): a stage holds kBK rows of block_n 16-bit columns
// (block_n / 8 chunks of 16 bytes per row).  Fragments are fetched with the transposing read
// ds_read_b64_tr_b16: in one 32-lane pass the lanes touch 8 different rows k (k & 3 and bit 3 of
// k vary), 32 contiguous bytes in each, so the 32-byte segment index is XORed with a 3-bit code
// of exactly those bits of k (2 bits when a row is only 128 bytes and two rows share a bank sweep).
// The XOR is applied to the chunk index, shifted left by one.
BEAM_HD int kmajor_swizzle(int k, int block_n) {
  const int code = block_n >= 128 ? ((k & 3) | (((k >> 3) & 1) << 2)) : (((k >> 1) & 1) | (((k >> 3) & 1) << 1));
  return code << 1;
}

// Byte offset inside a K-major stage of element (k, n), n a multiple of 4.
BEAM_HD int kmajor_lds_offset(int k, int n, int block_n) {
  return k * block_n * 2 + ((((n >> 3) ^ kmajor_swizzle(k, block_n))) << 4) + ((n & 7) << 1);
}

// The 4-wavefront kernel (gemm_w4.h) with B as [K][N]: XOR pattern of the 16-byte chunks of a k row (512 bytes)
// in LDS.  A transposing read of block b has, per 32 lanes, lane 4 e + q of group g (g = 0, 1) at row 8 g + e, chunk 4 (b / 2) + q, 8-byte half
// (b ^ q) % 2: bits 0, 2 and 3 of the code spread the 8 rows, q's bit 1 and the half do the rest, 32 distinct
// 8-byte bank pairs.  (Bits 2 and 5 of k stay out of it: the second read of a fragment, 4 rows on, and the
// second half of a K tile, 32 rows on, are constant offsets from the first.)
BEAM_HD int w4_kmajor_swizzle(int k) { return (k & 1) | (((k >> 1) & 1) << 2) | (((k >> 3) & 1) << 3); }
// Byte offset in a [K][N] slot of the 8 bytes that lane (g, e, q) of a transposing read of block b supplies
// (wn: the wavefront's half of the tile's columns; first read of the first half of the K tile).
BEAM_HD int w4_kmajor_read_offset(int wn, int b, int g, int e, int q) {
  const int k = 8 * g + e;
  return k * 512 + (((16 * wn + 4 * (b >> 1) + q) ^ w4_kmajor_swizzle(k)) << 4) + (((b ^ q) & 1) << 3);
}

// Words of the fused GEMM+LayerNorm workspace header (256 bytes in front of the two arrays of statistics
// words).  Nothing in it has to be initialised: every fused launch carries a tag that no earlier launch had,
// a statistics word counts as published only if it carries that tag, and the header words say which launch
// wrote them.
constexpr int kLnHdrTimeout = 0;    // tag of a launch in which a workgroup gave up waiting for a band's statistics
constexpr int kLnHdrMagic = 1;      // kLnMagic once a fused launch has run on this workspace
constexpr int kLnHdrLaunchTag = 2;  // tag of the latest launch
constexpr int kLnHdrReplay = 3;     // counter that a one-thread kernel moves on in front of a captured launch, whose
                                    // kernel arguments repeat from replay to replay; part of the tag
constexpr int kLnMagic = 0x4c4e3033;

// Split-K in one launch: the synchronisation words behind the partial sums in the workspace.  The first words
// say which launch ran last and whether one of its reducing workgroups gave up waiting (never initialised: the
// words name the launch they speak of); from word kSkFlags on there is one
// flag per (tile, part, slice): the workgroup of (tile, slice) sets the flags of all the tile's parts to the
// launch's tag once its partial sums are in memory, the workgroup that reduces (tile, part) waits for its
// `splits` flags and clears them again.  A part is what one reducing workgroup adds up: 4, 2 or 1 outputs per
// thread (the fewer the tiles, the smaller the parts, so that many CUs share the reading).
constexpr int kSkTimeout = 0;    // tag of a launch in which a reducing workgroup gave up waiting
constexpr int kSkMagic = 1;      // kSkMagicValue once a one-launch split-K has run on this workspace
constexpr int kSkLaunchTag = 2;  // tag of the latest launch
constexpr int kSkMagicValue = 0x534b3031;
constexpr int kSkFlags = 64;
__host__ __device__ constexpr int sk_parts_per_tile(int block_m, int block_n, int threads, int out) {
  return block_m * block_n / (threads * out);
}
// Bytes of synchronisation words that are enough for any tile the one-launch form is built for (up to 128 x 128;
// a part is at least 256 outputs, and the tiles cover at most (M + 127) x (N + 127) outputs).
__host__ __device__ constexpr unsigned long long sk_sync_bytes(int M, int N, int splits) {
  return 4ull * (kSkFlags + ((unsigned long long)(M + 127) * (unsigned long long)(N + 127) / 256ull + 1ull) * (unsigned long long)splits);
}

struct TileCoord {
  int tm;  // tile index along M
  int tn;  // tile index along N
};

// Workgroup id -> linear tile id such that the workgroups living on one XCD (ids congruent
// modulo 8) own one contiguous range of tile ids. Bijection on [0, total).
BEAM_HD int xcd_remap(int wg, int total) {
  const int base = total / kNumXcd;
  const int rem = total % kNumXcd;
  const int xcd = wg % kNumXcd;
  const int local = wg / kNumXcd;
  return xcd * base + (xcd < rem ? xcd : rem) + local;
}

// Division of a number below 2^31 by a divisor known on the host: one multiply-high and a shift in the kernel
// instead of the ~25 instructions (and a round trip through the vector unit's reciprocal) of a division by a
// run-time value.  Three of those in a row stood between a workgroup's start and its first load: 0.15 us of
// a 1024^3 launch's 5.3.  mul = ceil(2^(31 + ceil(log2 d)) / d), shift = ceil(log2 d) - 1; d = 1: mul = 0.
struct FastDiv {
  unsigned mul;
  unsigned shift;
};
BEAM_HD FastDiv make_fast_div(unsigned d) {
  FastDiv f = {0u, 0u};
  if (d <= 1u) return f;
  unsigned lg = 0;
  while ((1ull << lg) < d) ++lg;  // ceil(log2 d), >= 1
  const unsigned long long p2 = 1ull << (31 + lg);
  f.mul = (unsigned)((p2 + d - 1) / d);
  f.shift = lg - 1;
  return f;
}
BEAM_HD unsigned fast_div(unsigned n, FastDiv f) {
  return f.mul == 0u ? n : (unsigned)(((unsigned long long)n * f.mul) >> 32) >> f.shift;
}
// The divisors of a launch's tile maps (made once on the host, passed with the kernel's arguments).
struct TileDivs {
  FastDiv group;      // group_m * tiles_n: tiles per group of tile rows
  FastDiv rows;       // group_m: tile rows of a full group
  FastDiv rows_last;  // tile rows of the last, short group (= rows when tiles_m is a multiple of group_m)
  FastDiv tiles;      // tiles_m * tiles_n (split-K: workgroup -> slice)
};
BEAM_HD TileDivs make_tile_divs(int tiles_m, int tiles_n, int group_m) {
  TileDivs d;
  const int g = group_m < 1 ? 1 : group_m;
  d.group = make_fast_div((unsigned)(g * tiles_n));
  d.rows = make_fast_div((unsigned)g);
  const int last = tiles_m % g;
  d.rows_last = make_fast_div((unsigned)(last ? last : g));
  d.tiles = make_fast_div((unsigned)(tiles_m * tiles_n));
  return d;
}

// Linear tile id -> (tm, tn): groups of `group_m` tile rows, M fastest inside a group, so
// that workgroups with neighbouring ids reuse the same B panel and a small set of A panels
// out of the XCD-private L2.
BEAM_HD TileCoord grouped_tile(int pid, int tiles_m, int tiles_n, int group_m) {
  const int gsize = group_m * tiles_n;
  const int g = pid / gsize;
  const int first_m = g * group_m;
  const int rows = (tiles_m - first_m) < group_m ? (tiles_m - first_m) : group_m;
  const int within = pid - g * gsize;
  TileCoord t;
  t.tm = first_m + within % rows;
  t.tn = within / rows;
  return t;
}

// Order for kernels whose tiles of one row band cooperate (fused LayerNorm): a workgroup may wait for
// the other column tiles of its band, so all of them must be resident at the same time.  The grid is
// cut into band groups of `gb` bands; inside a band group XCD x owns the `gc` columns
// [x*gc, (x+1)*gc) of every band, i.e. a gb x gc block of tiles (good L2 reuse of both operands), and
// 8*gc >= tiles_n, so one band group is exactly what the 8 XCDs hold at once (gb*gc <= CUs per XCD).
// Every XCD walks the band groups in the same order, and the hardware dispatches the workgroups of an
// XCD in id order: the earliest unfinished band group is always fully resident, hence no deadlock.
// Inside its block an XCD takes band after band (columns fastest): a launch that shares the device with
// another then holds whole bands plus at most one partial band per XCD, and the CUs that the whole bands
// free are enough to complete the partial ones.  (Bands fastest, the first form of this order, left two
// launches on two streams with a part of *every* band of a group each: they waited for each other until
// the driver's time slicing, seconds later, or the poll budget ended it.)
// The grid is padded (8 * band_groups * gb * gc workgroups); ids that fall outside the tile grid
// return tm = -1 and the workgroup exits at once.
BEAM_HD TileCoord band_block_tile(int wg, int tiles_m, int tiles_n, int gb, int gc) {
  const int xcd = wg % kNumXcd;
  const int local = wg / kNumXcd;
  const int per_group = gb * gc;
  const int bg = local / per_group;
  const int within = local - bg * per_group;
  TileCoord t;
  t.tm = bg * gb + within / gc;
  t.tn = xcd * gc + within % gc;
  if (t.tm >= tiles_m || t.tn >= tiles_n) t.tm = -1;
  return t;
}

// Number of workgroups of that padded grid.
BEAM_HD int band_block_grid(int tiles_m, int gb, int gc) {
  return kNumXcd * ((tiles_m + gb - 1) / gb) * gb * gc;
}

// The same contract with whole bands on one XCD, for bands short enough (tiles_n * bx <= CUs per
// XCD): XCD x holds bands (g * 8 + x) * bx .. + bx - 1 in round g, band after band (columns
// fastest, for the reason given above).  The XCDs of one part
// run at clocks that differ by several percent under a matrix-core load (measured: the same tiles
// take 5% longer on some XCDs than on others), so a band spread over all XCDs waits for the slowest
// of them; a band inside one XCD finishes together.  L2 traffic is the same as for band_block_tile
// (bx A panels + tiles_n B panels per XCD and round, against gb + gc).
BEAM_HD TileCoord band_xcd_tile(int wg, int tiles_m, int tiles_n, int bx) {
  const int xcd = wg % kNumXcd;
  const int local = wg / kNumXcd;
  const int per_group = bx * tiles_n;
  const int g = local / per_group;
  const int within = local - g * per_group;
  TileCoord t;
  t.tm = (g * kNumXcd + xcd) * bx + within / tiles_n;
  t.tn = within % tiles_n;
  if (t.tm >= tiles_m) t.tm = -1;
  return t;
}

BEAM_HD int band_xcd_grid(int tiles_m, int tiles_n, int bx) {
  const int bands_per_round = kNumXcd * bx;
  return ((tiles_m + bands_per_round - 1) / bands_per_round) * bands_per_round * tiles_n;
}

BEAM_HD TileCoord tile_of_workgroup(int wg, int tiles_m, int tiles_n, int group_m) {
  return grouped_tile(xcd_remap(wg, tiles_m * tiles_n), tiles_m, tiles_n, group_m);
}

// The same maps with the divisions done by multiplication (what the kernels call; a host test walks both over
// every workgroup of many grids).
BEAM_HD TileCoord grouped_tile(int pid, int tiles_m, int tiles_n, int group_m, const TileDivs& dv) {
  const int gsize = group_m * tiles_n;
  const int g = (int)fast_div((unsigned)pid, dv.group);
  const int first_m = g * group_m;
  const bool short_group = tiles_m - first_m < group_m;
  const int rows = short_group ? tiles_m - first_m : group_m;
  const int within = pid - g * gsize;
  TileCoord t;
  t.tn = (int)fast_div((unsigned)within, short_group ? dv.rows_last : dv.rows);
  t.tm = first_m + within - t.tn * rows;
  return t;
}
BEAM_HD TileCoord tile_of_workgroup(int wg, int tiles_m, int tiles_n, int group_m, const TileDivs& dv) {
  return grouped_tile(xcd_remap(wg, tiles_m * tiles_n), tiles_m, tiles_n, group_m, dv);
}

// The three workgroup orders of the fused GEMM+LayerNorm as one map with its divisions done by multiplication (what
// the kernels call; a host test walks it against the defining functions above over every id of many grids).
//   group_n > 0: band_block_tile with gb = group_m, gc = group_n;  group_n == 0: band_xcd_tile with bx = group_m;
//   group_n < 0: band after band, id = band * tiles_n + column, no padding.
BEAM_HD TileDivs band_order_divs(int tiles_n, int group_m, int group_n) {
  TileDivs d;
  const int g = group_m < 1 ? 1 : group_m;
  d.group = make_fast_div((unsigned)(g * (group_n > 0 ? group_n : tiles_n)));  // ids of one XCD per band group
  d.rows = make_fast_div((unsigned)(group_n > 0 ? group_n : (tiles_n < 1 ? 1 : tiles_n)));  // columns of an XCD's block
  d.rows_last = d.rows;
  d.tiles = make_fast_div((unsigned)(tiles_n < 1 ? 1 : tiles_n));
  return d;
}
BEAM_HD TileCoord band_order_tile(int id, int tiles_m, int tiles_n, int group_m, int group_n, const TileDivs& dv) {
  TileCoord t;
  if (group_n < 0) {
    t.tm = (int)fast_div((unsigned)id, dv.tiles);
    t.tn = id - t.tm * tiles_n;
    return t;
  }
  const int xcd = id % kNumXcd;
  const int local = id / kNumXcd;
  const int per_group = group_m * (group_n > 0 ? group_n : tiles_n);
  const int bg = (int)fast_div((unsigned)local, dv.group);
  const int within = local - bg * per_group;
  const int cols = group_n > 0 ? group_n : tiles_n;
  const int band = (int)fast_div((unsigned)within, dv.rows);  // within / cols
  const int col = within - band * cols;
  if (group_n > 0) {
    t.tm = bg * group_m + band;
    t.tn = xcd * group_n + col;
  } else {
    t.tm = (bg * kNumXcd + xcd) * group_m + band;
    t.tn = col;
  }
  if (t.tm >= tiles_m || t.tn >= tiles_n) t.tm = -1;
  return t;
}

// K range [begin, end) of split slice `z` out of `splits`: every slice gets the same whole
// number of kBK-wide K tiles (the last ones may be short or empty). Matches the CUTLASS
// partitioning the reference relies on (cuda/cutlass_kernels/cutlass_gemmrc_splitk.cu:95-99).
BEAM_HD int split_k_len(int K, int splits) {
  const int ktiles = (K + kBK - 1) / kBK;
  return ((ktiles + splits - 1) / splits) * kBK;
}

}  // namespace beam
