// Index math shared by the gfx950 GEMM kernels and the host-side layout simulator.
//
// Everything here is a pure function of small integers, usable from host and device code.
// The kernels move operand tiles from HBM into LDS with 16-byte direct-to-LDS buffer loads
// (one wave instruction deposits 64 lanes x 16 B = 1 KiB of contiguous LDS), read the
// K-contiguous operand with 16-byte LDS reads and the N-contiguous operand with the gfx950
// LDS transpose reads, and feed 32x32 MFMA blocks.  The functions below say, for every lane,
// which global 16-byte chunk it fetches, where that chunk lives in LDS, and which LDS address
// a lane presents when it assembles an MFMA operand.
//
// Conventions
//   ES     element size in bytes (2 for bf16/fp16, 1 for fp8)
//   chunk  16 bytes = CE elements (8 or 16)
//   "row tile"   an operand tile stored as [rows][BK elements], K contiguous  (A, or B given as B^T)
//   "col tile"   an operand tile stored as [BK rows (k)][BN elements], N contiguous (row-major B)
#pragma once

#if defined(__HIPCC__)
#define IRIS_HD __host__ __device__ __forceinline__
#else
#define IRIS_HD inline
#endif

namespace iris_layout {

constexpr int kChunkBytes = 16;
constexpr int kWave = 64;
constexpr int kDmaBytes = kWave * kChunkBytes;  // LDS bytes written by one wave-level load

// ---------------------------------------------------------------------------------------------
// Row tile: [rows][RB bytes], RB = BK*ES in {64, 128}.  16-byte chunks are XOR-swizzled so that
// 16 lanes reading the same logical chunk of 16 consecutive rows touch 16 distinct 16-byte
// bank groups (one full sweep of the 64 four-byte banks).
// ---------------------------------------------------------------------------------------------
template <int RB>
struct RowTile {
  static_assert(RB == 64 || RB == 128 || RB == 256, "row bytes must be 64, 128 or 256");
  static constexpr int kChunksPerRow = RB / kChunkBytes;
  static constexpr int kRowsPer256 = (256 / RB) > 0 ? (256 / RB) : 1;

  IRIS_HD static int swizzle(int row) { return (row / kRowsPer256) % kChunksPerRow; }
  // LDS byte offset of logical chunk c of a row.
  IRIS_HD static int lds_offset(int row, int c) { return row * RB + ((c ^ swizzle(row)) * kChunkBytes); }
  // Inverse used by the loader: LDS byte offset (multiple of 16) -> (row, logical chunk).
  IRIS_HD static void from_lds(int off, int& row, int& c) {
    row = off / RB;
    c = ((off % RB) / kChunkBytes) ^ swizzle(row);
  }
};

// ---------------------------------------------------------------------------------------------
// Col tile: [BK rows][RB bytes], RB = BN*ES >= 256 (16-bit) or >= 128 (8-bit).  LDS serves a
// transpose read one half-wave (32 lanes x 8 bytes = 256 bytes = all 64 banks) at a time.  A half-wave
// touches 4 k-rows x 64 contiguous bytes (16-bit) or 8 k-rows x 32 bytes (8-bit); the other half-wave
// reads the same columns 8 (32) k-rows further down.  XOR-ing the index of that 64- (32-) byte block
// with the k-row puts the rows of a half-wave on distinct blocks of a 256-byte bank line.  When a
// 256-byte bank line holds two tile rows (RB = 128) the row parity already separates them and the
// XOR uses k-row / 2.  (Rotating 32-byte blocks by k-row % 8 for 16-bit data, as an earlier layout
// did, is conflict-free per 16 lanes but lets rows 2i and 2i+1 of a half-wave share a block: the
// hardware counted bank conflicts on half of the cycles of these reads.)
// ---------------------------------------------------------------------------------------------
template <int RB, int ES>
struct ColTile {
  static_assert(ES == 1 || ES == 2, "element size must be 1 or 2 bytes");
  static constexpr int kChunksPerRow = RB / kChunkBytes;
  static constexpr int kBlockChunks = (ES == 2) ? 4 : 2;        // 16-byte chunks per swizzled block
  static constexpr int kRowsPerLine = RB >= 256 ? 1 : 256 / RB;  // tile rows per 256-byte bank line
  static constexpr int kSwRows = ((ES == 2) ? 4 : 8) / kRowsPerLine;
  static_assert(kChunksPerRow >= kSwRows * kBlockChunks, "tile row too short for the swizzle");

  IRIS_HD static int swizzle(int krow) { return ((krow / kRowsPerLine) % kSwRows) * kBlockChunks; }
  IRIS_HD static int lds_offset(int krow, int c) { return krow * RB + ((c ^ swizzle(krow)) * kChunkBytes); }
  IRIS_HD static void from_lds(int off, int& krow, int& c) {
    krow = off / RB;
    c = ((off % RB) / kChunkBytes) ^ swizzle(krow);
  }
};

// ---------------------------------------------------------------------------------------------
// MFMA 32x32 operand lanes.  For v_mfma_f32_32x32x16_{bf16,f16} lane l supplies, for row (or
// column) l%32, the 8 k-values 8*(l/32)..+7 of the 16-wide k-slice; for the 8-bit 32x32x64 form
// it supplies the 32 k-values 32*(l/32)..+31.  Only the pairing of A and B k-slots matters for
// the product, so both operands simply use the same rule.
// ---------------------------------------------------------------------------------------------

// 16-bit, K-contiguous operand: one 16-byte read per 32x32x16 MFMA.
//   row  = block_row0 + lane%32 ; chunk = kk*2 + lane/32        (kk = k-slice of 16 within the tile)
IRIS_HD int frag16_row(int lane) { return lane % 32; }
IRIS_HD int frag16_chunk(int lane, int kk) { return kk * 2 + lane / 32; }

// 8-bit, K-contiguous operand: two 16-byte reads per 32x32x64 MFMA (h = 0,1).
IRIS_HD int frag8_chunk(int lane, int kk, int h) { return kk * 4 + 2 * (lane / 32) + h; }

// LDS transpose read, 16-bit (ds_read_b64_tr_b16).  Within each 16-lane group, lane p presents
// the address of 4 consecutive n at k-row p/4, n = 4*(p%4); it receives, for n = p, the 4 k-rows.
// For read j (0,1) of the k-slice kk, lane l of the wave addresses:
IRIS_HD int tr16_krow(int lane, int kk, int j) {
  int g = lane / 16, p = lane % 16;
  return kk * 16 + 8 * (g / 2) + 4 * j + p / 4;
}
IRIS_HD int tr16_ncol(int lane) {  // first of 4 consecutive n, relative to the 32-wide block
  int g = lane / 16, p = lane % 16;
  return 16 * (g % 2) + 4 * (p % 4);
}

// LDS transpose read, 8-bit (ds_read_b64_tr_b8).  Lane p of a 16-lane group presents 8
// consecutive n at k-row p/2, n = 8*(p%2); it receives, for n = p, the 8 k-rows.
// For read r (0..3) of the 64-wide k-slice kk:
IRIS_HD int tr8_krow(int lane, int kk, int r) {
  int g = lane / 16, p = lane % 16;
  return kk * 64 + 32 * (g / 2) + 8 * r + p / 2;
}
IRIS_HD int tr8_ncol(int lane) {
  int g = lane / 16, p = lane % 16;
  return 16 * (g % 2) + 8 * (p % 2);
}

// Accumulator of D = X * Y for the 32x32 MFMA: register i (0..15) of lane l holds
//   D[row = 8*(i/4) + 4*(l/32) + i%4][col = l%32].
// The kernels issue mfma(Bfrag, Afrag) so that D rows run along n and columns along m: every
// lane then owns 4 consecutive n for one m, which packs into one 8-byte LDS write.
IRIS_HD int acc_row(int lane, int i) { return 8 * (i / 4) + 4 * (lane / 32) + (i % 4); }
IRIS_HD int acc_col(int lane) { return lane % 32; }

// ---------------------------------------------------------------------------------------------
// Tile order.  Workgroup b of a launch lands on XCD b % num_xcd (round-robin dispatch).  Tiles
// are first put in a grouped order (group_m tile-rows at a time, walking down the group's
// column before moving right) and each XCD is handed one contiguous span of that order, so the
// tiles that share A row-panels and B column-panels meet in the same L2.
// ---------------------------------------------------------------------------------------------
IRIS_HD void grouped_tile(int idx, int tiles_m, int tiles_n, int group_m, int& tm, int& tn) {
  int per_group = group_m * tiles_n;
  int g = idx / per_group;
  int first_m = g * group_m;
  int rows = tiles_m - first_m < group_m ? tiles_m - first_m : group_m;
  int r = idx - g * per_group;
  tm = first_m + r % rows;
  tn = r / rows;
}

// Position in the grouped order of the it-th tile processed by workgroup `wg` of `nwg`.
// Returns -1 when that workgroup has no it-th tile.
IRIS_HD int xcd_tile_index(int wg, int nwg, int it, int total, int num_xcd) {
  if (nwg % num_xcd != 0 || nwg < num_xcd) {  // plain round-robin
    long idx = (long)wg + (long)it * nwg;
    return idx < total ? (int)idx : -1;
  }
  int xcd = wg % num_xcd;
  int local = wg / num_xcd;
  int wg_per_xcd = nwg / num_xcd;
  int span = (total + num_xcd - 1) / num_xcd;
  long in_span = (long)local + (long)it * wg_per_xcd;
  if (in_span >= span) return -1;
  long idx = (long)xcd * span + in_span;
  return idx < total ? (int)idx : -1;
}

// ---------------------------------------------------------------------------------------------
// Flag tiles (the reference's BLOCK_SIZE_M x BLOCK_SIZE_N tiles) and their owners.
// ---------------------------------------------------------------------------------------------
IRIS_HD int cdiv(int a, int b) { return (a + b - 1) / b; }

// Owner of flag tile t under interleaved (two-shot all-reduce) distribution.
IRIS_HD int owner_interleaved(int t, int world) { return t % world; }

// Owner of flag tile t under contiguous (reduce-scatter) distribution: each rank takes
// total/world tiles, the last rank also the remainder.
IRIS_HD int owner_contiguous(int t, int total, int world) {
  int per = total / world;
  if (per == 0) return world - 1;
  int o = t / per;
  return o < world - 1 ? o : world - 1;
}

// How many kernel macro-tiles (KM x KN) overlap flag tile (fm, fn) of size (FM x FN) in an
// M x N matrix.  A flag is raised by the last of them to finish.
IRIS_HD int macro_tiles_over_flag_tile(int fm, int fn, int FM, int FN, int KM, int KN, int M, int N) {
  int r0 = fm * FM, r1 = (fm + 1) * FM < M ? (fm + 1) * FM : M;
  int c0 = fn * FN, c1 = (fn + 1) * FN < N ? (fn + 1) * FN : N;
  int nm = (r1 - 1) / KM - r0 / KM + 1;
  int nn = (c1 - 1) / KN - c0 / KN + 1;
  return nm * nn;
}

// ---------------------------------------------------------------------------------------------
// Tail policy of the 256x256 tile: how the tiles of a partly filled last round are split along K.
//
// An XCD's `wgs` workgroups meet `left` (< wgs) tiles in the last round.  When at most half of them
// would get a tile, workgroup h < left HELPS tile h: the tile's MAIN workgroup (the last `left`
// workgroups of the XCD) multiplies the K steps [0, main_steps) and owns the epilogue, the helper
// multiplies [main_steps, nsteps) and passes its fp32 accumulators on as a partial sum.  Helpers beyond
// `left` stay idle.
// All mains walk K from step 0 at the same pace and all helpers from main_steps, as the whole tiles of
// the earlier rounds do, so the operand panels they share keep meeting in the XCD's L2.  What was measured
// and left out (bf16, one rank, kernel time whole -> split):
//   - the textbook scheme, the round's K steps cut into equal consecutive shares: every workgroup sits at
//     another K offset and the operand traffic from the last-level cache grows ninefold
//     (8192 x 1792 x 4096, 28 of 32 tiles left: 116 -> 154 us);
//   - several helpers per tile: the main adds their partial sums one after the other
//     (5120 x 3840 x 4096, 6 of 32 left, four helpers each: 187 -> 192 us; one helper each: 186 -> 163);
//   - a helper serving several tiles in a row when more than half of the round is filled
//     (4096 x 2880 x 4096, 24 of 32 left, three tiles per helper: 91 -> 102 us).
// main_steps balances the main's work (its steps, then `gather_cost` steps' worth of loading the partial
// sum) against the helper's (its steps, `pass_cost` steps' worth of pipeline fill and storing the partial
// sum).  per_tile = 0 means: do not split (nothing to gain).  With both costs at 0 (a test setting) every
// round of at least 4 K steps that can be split is split.
// ---------------------------------------------------------------------------------------------
struct SplitPlan {
  int per_tile;     // helper pieces per tile (0: tiles stay whole)
  int per_helper;   // tiles a helper serves
  int main_steps;   // K steps [0, main_steps) stay with the main
  int piece_steps;  // K steps of a helper piece (the last piece of a tile may be shorter)
};
// In K steps of the 256x256 tile (about 0.75 us each), from time stamps inside a split launch
// (8192 x 2880 x 4096 bf16): a helper's 256 KiB of partial sums are stored and acknowledged 4.7 us after
// its last K step, and the next tile's first operands land 3 us later; the main has the partial sum in
// its staged tile 6 us after the helper's flag went up, 4.5 us more than staging alone takes.
constexpr int kSplitGatherCost = 8;
constexpr int kSplitPassCost = 10;

IRIS_HD SplitPlan split_plan(int left, int wgs, int nsteps, int gather_cost = kSplitGatherCost, int pass_cost = kSplitPassCost) {
  SplitPlan s = {0, 1, nsteps, 0};
  const int helpers = wgs - left;
  if (left <= 0 || helpers <= 0 || nsteps < 4) return s;
  if (helpers < left) return s;  // more than half of the round is filled
  const int n = 1, m = 1;
  // main_steps + n * gather = m * ((nsteps - main_steps) / n + pass)
  long num = (long)m * nsteps + (long)n * m * pass_cost - (long)n * n * gather_cost;
  int main_steps = (int)(num / (n + m));
  if (main_steps < 1) main_steps = 1;
  if (main_steps > nsteps - n) return s;        // every helper piece needs a step
  const int piece = (nsteps - main_steps + n - 1) / n;
  // The round as its slowest workgroup sees it, in K steps; a split that does not beat a whole tile is none.
  const int main_cost = main_steps + n * gather_cost;
  const int helper_cost = m * (piece + pass_cost);
  if ((main_cost > helper_cost ? main_cost : helper_cost) >= nsteps) return s;
  s.per_tile = n;
  s.per_helper = m;
  s.main_steps = main_steps;
  s.piece_steps = piece;
  return s;
}
// K steps the slowest workgroup of the round spends, split or not (what the launch code compares).
IRIS_HD int split_round_steps(const SplitPlan& s, int nsteps, int gather_cost = kSplitGatherCost, int pass_cost = kSplitPassCost) {
  if (s.per_tile == 0) return nsteps;
  const int main_cost = s.main_steps + s.per_tile * gather_cost;
  const int helper_cost = s.per_helper * (s.piece_steps + pass_cost);
  return main_cost > helper_cost ? main_cost : helper_cost;
}

// What workgroup `local` (0 .. wgs-1) of an XCD does in the split round as its `served`-th item (0, 1, ...).
// Returns false when it has nothing (more) to do.  Otherwise tile j (0 .. left-1) of the round, the K
// steps [k_begin, k_end), and
//   kind 0: a whole tile (the plan does not split),
//   kind 1: a helper piece - the accumulators go to partial-sum slot `slot`,
//   kind 2: the main's piece - the partial sum in slot `slot` is added before the epilogue (partners = 1).
// Slots count from 0 within the XCD (all below wgs).  Helpers are the first
// wgs - left workgroups, mains the last `left`.
IRIS_HD bool split_item(const SplitPlan& s, int left, int wgs, int nsteps, int local, int served,
                        int& j, int& k_begin, int& k_end, int& kind, int& partners, int& slot) {
  const int helpers = wgs - left;
  k_begin = 0; k_end = nsteps; kind = 0; partners = 0; slot = 0;
  if (local >= helpers) {  // main
    if (served > 0) return false;
    j = local - helpers;
    if (s.per_tile > 0) {
      kind = 2;
      k_end = s.main_steps;
      const int pieces = (nsteps - s.main_steps + s.piece_steps - 1) / s.piece_steps;
      partners = pieces < s.per_tile ? pieces : s.per_tile;
      slot = j * s.per_tile;
    }
    return true;
  }
  if (s.per_tile == 0 || served >= s.per_helper) return false;
  int piece = 1;
  if (s.per_helper > 1) {
    j = local * s.per_helper + served;
  } else {
    j = local % left;
    piece = 1 + local / left;
  }
  k_begin = s.main_steps + (piece - 1) * s.piece_steps;
  if (j >= left || piece > s.per_tile || k_begin >= nsteps) return false;
  k_end = k_begin + s.piece_steps < nsteps ? k_begin + s.piece_steps : nsteps;
  kind = 1;
  slot = j * s.per_tile + piece - 1;
  return true;
}

// The 32x32 small-output kernel addresses A from the operand's first row (of the slot that holds it) and
// the peers' aux tiles from the buffer's first element, with 32-bit byte offsets into a buffer resource
// of 2^31 bytes: an offset at or beyond 2^31 would read zeros.  True when every offset the kernel can
// form stays below that: a_rows rows of A (the rows one slot holds) with a stride of s_am elements of es
// bytes and K elements per row; M x N outputs of 2-byte elements with a row stride of s_cm elements.
// Launches that fail the test take the tiled kernels, which rebase their resources per tile.
IRIS_HD bool decode_offsets_fit(long long a_rows, long long s_am, long long K, int es, long long M, long long s_cm, long long N) {
  const long long limit = 1ll << 31;
  const long long a_last = (a_rows - 1) * s_am * es + K * es;  // one past the last byte of A
  const long long c_last = ((M - 1) * s_cm + N) * 2;            // ... of aux / C
  return a_rows > 0 && s_am >= 0 && s_cm >= 0 && a_last < limit && c_last < limit;
}

}  // namespace iris_layout
