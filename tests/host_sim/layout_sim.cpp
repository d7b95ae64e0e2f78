// Host-side check of iris_amd/csrc/layout.h: replays, on the CPU, what the gfx950 kernels do with the
// index functions - direct-to-LDS deposits, 16-byte fragment reads, LDS transpose reads - and checks
// that every MFMA operand slot receives the element the kernel assumes, that the LDS swizzles are
// bijections without bank conflicts inside a 16-lane group, and that the tile orders and flag-tile
// counts are exact.  The transpose-read semantics used here (within each 16-lane group, output lane i
// element e comes from input lane 4e + i/4, element i%4 for 16-bit data; input lane 2e + i/8, byte
// i%8 for 8-bit data) were measured on an MI355X.
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <set>
#include <vector>

#include "layout.h"

using namespace iris_layout;

static int failures = 0;
#define CHECK(cond, ...)                         \
  do {                                           \
    if (!(cond)) {                               \
      if (failures < 20) { printf("FAIL %s:%d: ", __FILE__, __LINE__); printf(__VA_ARGS__); printf("\n"); } \
      ++failures;                                \
    }                                            \
  } while (0)

// ---- swizzle bijection + bank spread -------------------------------------------------------------
template <int RB>
void check_row_tile(int rows) {
  using T = RowTile<RB>;
  std::set<int> seen;
  for (int r = 0; r < rows; ++r)
    for (int c = 0; c < T::kChunksPerRow; ++c) {
      int off = T::lds_offset(r, c);
      CHECK(off >= 0 && off < rows * RB && off % 16 == 0, "row tile offset out of range");
      CHECK(seen.insert(off).second, "row tile offset reused");
      int r2, c2;
      T::from_lds(off, r2, c2);
      CHECK(r2 == r && c2 == c, "row tile inverse mismatch RB=%d r=%d c=%d", RB, r, c);
    }
  // 16 lanes reading the same logical chunk of 16 consecutive rows: 16 distinct 16-byte bank groups
  for (int r0 = 0; r0 + 16 <= rows; r0 += 16)
    for (int c = 0; c < T::kChunksPerRow; ++c) {
      std::set<int> banks;
      for (int i = 0; i < 16; ++i) banks.insert((T::lds_offset(r0 + i, c) % 256) / 16);
      CHECK(banks.size() == 16, "row tile RB=%d bank conflict at rows %d.., chunk %d (%zu groups)", RB, r0, c, banks.size());
    }
}

template <int RB, int ES>
void check_col_tile(int krows) {
  using T = ColTile<RB, ES>;
  std::set<int> seen;
  for (int k = 0; k < krows; ++k)
    for (int c = 0; c < T::kChunksPerRow; ++c) {
      int off = T::lds_offset(k, c);
      CHECK(off >= 0 && off < krows * RB, "col tile offset out of range");
      CHECK(seen.insert(off).second, "col tile offset reused");
      int k2, c2;
      T::from_lds(off, k2, c2);
      CHECK(k2 == k && c2 == c, "col tile inverse mismatch");
    }
}

// ---- simulate loader + fragment reads for one operand tile -----------------------------------------
// Element identity: (row-or-k, col) packed in an int; the simulated LDS stores one id per element.
struct Lds {
  std::vector<int> id;  // per byte/ES element slot
  int es;
  Lds(int bytes, int es_) : id(bytes / es_, -1), es(es_) {}
  int& at(int byte_off) { return id[byte_off / es]; }
};

// K-contiguous operand (A, or B^T): tile [rows][BK], fragment lanes per frag16_*/frag8_*.
template <int RB, int ES>
void sim_row_operand(int rows, int nwaves) {
  using T = RowTile<RB>;
  const int CE = 16 / ES, BK = RB / ES;
  Lds lds(rows * RB, ES);
  // loader: wave w, instruction i deposits 1 KiB at (w + i*nwaves)*1024; lane l its 16 bytes
  const int ninstr = rows * RB / kDmaBytes;
  for (int q = 0; q < ninstr; ++q)
    for (int lane = 0; lane < 64; ++lane) {
      int off = q * kDmaBytes + lane * 16, row, c;
      T::from_lds(off, row, c);
      for (int e = 0; e < CE; ++e) lds.at(off + e * ES) = row * 4096 + (c * CE + e);  // global (row, k)
    }
  for (int x : lds.id) CHECK(x >= 0, "row operand: LDS element never written");
  // fragment reads: block of 32 rows starting at r0, every k-slice
  const int KM = ES == 2 ? 16 : 64;
  for (int r0 = 0; r0 + 32 <= rows; r0 += 32)
    for (int kk = 0; kk < BK / KM; ++kk)
      for (int lane = 0; lane < 64; ++lane) {
        const int nfrag = ES == 2 ? 1 : 2;
        for (int h = 0; h < nfrag; ++h) {
          int c = ES == 2 ? frag16_chunk(lane, kk) : frag8_chunk(lane, kk, h);
          int off = T::lds_offset(r0 + frag16_row(lane), c);
          for (int e = 0; e < CE; ++e) {
            int got = lds.at(off + e * ES);
            // MFMA slot: row lane%32, k = kk*KM + (KM/2)*(lane/32) + h*CE + e
            int want = (r0 + lane % 32) * 4096 + kk * KM + (KM / 2) * (lane / 32) + h * CE + e;
            CHECK(got == want, "row operand ES=%d lane %d kk %d: got (%d,%d) want (%d,%d)", ES, lane, kk, got / 4096, got % 4096, want / 4096, want % 4096);
          }
        }
      }
}

// N-contiguous operand (row-major B): tile [BK][BN], transpose reads.
template <int RB, int ES>
void sim_col_operand(int BK) {
  using T = ColTile<RB, ES>;
  const int CE = 16 / ES, BN = RB / ES;
  Lds lds(BK * RB, ES);
  const int ninstr = BK * RB / kDmaBytes;
  for (int q = 0; q < ninstr; ++q)
    for (int lane = 0; lane < 64; ++lane) {
      int off = q * kDmaBytes + lane * 16, k, c;
      T::from_lds(off, k, c);
      for (int e = 0; e < CE; ++e) lds.at(off + e * ES) = k * 4096 + (c * CE + e);  // global (k, n)
    }
  for (int x : lds.id) CHECK(x >= 0, "col operand: LDS element never written");
  const int KM = ES == 2 ? 16 : 64;
  const int per_read = ES == 2 ? 4 : 8;     // elements a lane contributes / receives per transpose read
  const int nreads = ES == 2 ? 2 : 4;
  for (int n0 = 0; n0 + 32 <= BN; n0 += 32)
    for (int kk = 0; kk < BK / KM; ++kk)
      for (int rd = 0; rd < nreads; ++rd) {
        // every lane presents an address; the hardware redistributes within 16-lane groups
        int addr[64];
        std::set<int> banks_by_group[2];  // LDS serves a transpose read one half-wave (256 bytes) at a time
        for (int lane = 0; lane < 64; ++lane) {
          int krow = ES == 2 ? tr16_krow(lane, kk, rd) : tr8_krow(lane, kk, rd);
          int n = n0 + (ES == 2 ? tr16_ncol(lane) : tr8_ncol(lane));
          addr[lane] = T::lds_offset(krow, n / CE) + (n % CE) * ES;
          for (int b = 0; b < 8; b += 4) banks_by_group[lane / 32].insert(((addr[lane] + b) % 256) / 4);
        }
        for (int g = 0; g < 2; ++g)
          CHECK(banks_by_group[g].size() == 64, "col operand ES=%d RB=%d: bank conflict in half-wave %d (%zu banks)", ES, RB, g, banks_by_group[g].size());
        for (int lane = 0; lane < 64; ++lane) {
          int grp = lane / 16, i = lane % 16;
          for (int e = 0; e < per_read; ++e) {
            int src_lane = grp * 16 + (ES == 2 ? 4 * e + i / 4 : 2 * e + i / 8);
            int src_elem = ES == 2 ? i % 4 : i % 8;
            int got = lds.at(addr[src_lane] + src_elem * ES);
            // MFMA slot of lane: n = lane%32, k = kk*KM + (KM/2)*(lane/32) + rd*per_read + e
            int want = (kk * KM + (KM / 2) * (lane / 32) + rd * per_read + e) * 4096 + n0 + lane % 32;
            CHECK(got == want, "col operand ES=%d lane %d kk %d read %d elem %d: got (k%d,n%d) want (k%d,n%d)", ES, lane, kk, rd, e,
                  got / 4096, got % 4096, want / 4096, want % 4096);
          }
        }
      }
}

// ---- accumulator layout: every (n, m) of a 32x32 block owned exactly once -----------------------------
void check_acc_layout() {
  std::set<int> seen;
  for (int lane = 0; lane < 64; ++lane)
    for (int i = 0; i < 16; ++i) {
      int r = acc_row(lane, i), c = acc_col(lane);
      CHECK(r >= 0 && r < 32 && c >= 0 && c < 32, "acc index range");
      CHECK(seen.insert(r * 32 + c).second, "acc element owned twice");
      if (i % 4) CHECK(acc_row(lane, i) == acc_row(lane, i - 1) + 1, "acc rows of a register quad must be consecutive");
    }
  CHECK(seen.size() == 1024, "acc layout must cover the block");
}

// ---- tile orders ---------------------------------------------------------------------------------------
void check_tile_orders() {
  for (int tm = 1; tm <= 40; tm += 3)
    for (int tn = 1; tn <= 40; tn += 5)
      for (int g : {1, 2, 4, 8, 16}) {
        std::set<int> seen;
        for (int idx = 0; idx < tm * tn; ++idx) {
          int a, b;
          grouped_tile(idx, tm, tn, g, a, b);
          CHECK(a >= 0 && a < tm && b >= 0 && b < tn, "grouped_tile out of range tm=%d tn=%d g=%d idx=%d -> (%d,%d)", tm, tn, g, idx, a, b);
          seen.insert(a * tn + b);
        }
        CHECK((int)seen.size() == tm * tn, "grouped_tile is not a bijection tm=%d tn=%d g=%d", tm, tn, g);
      }
  for (int total : {1, 7, 8, 10, 224, 255, 256, 257, 1000, 2048})
    for (int nwg : {1, 5, 8, 16, 224, 256})
      for (int xcd : {1, 8}) {
        std::map<int, int> count;
        for (int wg = 0; wg < nwg; ++wg) {
          bool ended = false;
          for (int it = 0; it < total + 2; ++it) {
            int idx = xcd_tile_index(wg, nwg, it, total, xcd);
            if (idx < 0) { ended = true; continue; }
            CHECK(!ended, "xcd_tile_index resumed after it ended (total=%d nwg=%d)", total, nwg);
            CHECK(idx < total, "xcd_tile_index out of range");
            count[idx]++;
          }
        }
        CHECK((int)count.size() == total, "xcd_tile_index misses tiles: total=%d nwg=%d xcd=%d covered=%zu", total, nwg, xcd, count.size());
        for (auto& kv : count) CHECK(kv.second == 1, "tile %d processed %d times", kv.first, kv.second);
      }
}

// The order launches that stream whole tiles use: the grouped order dealt out workgroup by workgroup
// (xcd_tile_index with one "XCD"), optionally started `rotate` positions in (the reduce-scatter starts
// at the rank's own band of rows).  Every tile exactly once; and with groups of g rows, XCD x (workgroup
// index modulo 8) of a full first round meets 1/g of the round's tile rows and g/8 of its tile columns.
void check_dealt_order() {
  struct Case { int tm, tn, g, nwg, rotate; };
  for (Case c : {Case{16, 16, 2, 256, 0}, Case{64, 32, 2, 256, 0}, Case{32, 16, 2, 256, 2 * 16 * 5}, Case{32, 16, 2, 512, 2 * 16 * 15},
                 Case{7, 23, 2, 168, 46}, Case{32, 8, 4, 256, 0}}) {
    const int total = c.tm * c.tn;
    std::vector<int> count(total, 0);
    for (int wg = 0; wg < c.nwg; ++wg)
      for (int it = 0;; ++it) {
        int idx = xcd_tile_index(wg, c.nwg, it, total, 1);
        if (idx < 0) break;
        idx += c.rotate;
        if (idx >= total) idx -= total;
        CHECK(idx >= 0 && idx < total, "dealt order out of range");
        count[idx]++;
      }
    for (int t = 0; t < total; ++t) CHECK(count[t] == 1, "dealt order: tile %d taken %d times (tm=%d tn=%d)", t, count[t], c.tm, c.tn);
  }
  // 16 x 16 tiles, groups of two rows, 256 workgroups on 8 XCDs: each XCD sees 8 of the 16 tile rows and 4 of the 16 tile columns
  for (int xcd = 0; xcd < 8; ++xcd) {
    std::set<int> rows, cols;
    for (int wg = xcd; wg < 256; wg += 8) {
      int a, b;
      grouped_tile(xcd_tile_index(wg, 256, 0, 256, 1), 16, 16, 2, a, b);
      rows.insert(a);
      cols.insert(b);
    }
    CHECK(rows.size() == 8 && cols.size() == 4, "dealt order: XCD %d meets %zu tile rows and %zu tile columns", xcd, rows.size(), cols.size());
  }
}

// ---- flag tiles ----------------------------------------------------------------------------------------
void check_flag_counts() {
  struct Case { int M, N, FM, FN, KM, KN; };
  for (Case c : {Case{4096, 4096, 256, 64, 256, 256}, Case{1024, 1024, 512, 512, 128, 128}, Case{1024, 1024, 384, 200, 128, 128},
                 Case{100, 72, 32, 24, 64, 64}, Case{257, 129, 64, 64, 64, 64}, Case{1000, 600, 96, 96, 256, 256}}) {
    int ftm = cdiv(c.M, c.FM), ftn = cdiv(c.N, c.FN);
    for (int fm = 0; fm < ftm; ++fm)
      for (int fn = 0; fn < ftn; ++fn) {
        std::set<int> macro;
        for (int m = fm * c.FM; m < (fm + 1) * c.FM && m < c.M; ++m)
          for (int n = fn * c.FN; n < (fn + 1) * c.FN && n < c.N; n += 1) macro.insert((m / c.KM) * 100000 + n / c.KN);
        int got = macro_tiles_over_flag_tile(fm, fn, c.FM, c.FN, c.KM, c.KN, c.M, c.N);
        CHECK(got == (int)macro.size(), "macro_tiles_over_flag_tile(%d,%d) = %d, brute force %zu", fm, fn, got, macro.size());
      }
  }
  for (int world : {1, 2, 3, 4, 8})
    for (int total : {1, 4, 7, 40, 64, 2048}) {
      int per = total / world;
      for (int t = 0; t < total; ++t) {
        int want = -1;
        for (int r = 0; r < world; ++r) {
          int s = r * per, e = (r == world - 1) ? total : s + per;
          if (t >= s && t < e) want = r;
        }
        CHECK(owner_contiguous(t, total, world) == want, "owner_contiguous(%d,%d,%d)", t, total, world);
        CHECK(owner_interleaved(t, world) == t % world, "owner_interleaved");
      }
    }
}

// The rule that keeps launches away from the 32x32 kernel when its 32-bit offsets would not reach.
void check_decode_offsets() {
  CHECK(decode_offsets_fit(32, 1024, 1024, 1, 32, 8192, 8192), "decode shape 32 x 8192 x 1024 fp8");
  CHECK(decode_offsets_fit(16384, 4096, 4096, 2, 16384, 32, 32), "tall output, 128 MiB of A");
  CHECK(!decode_offsets_fit(16384, 65536, 65536, 2, 16384, 32, 32), "16384 x 65536 bf16 is 2 GiB of A");
  CHECK(decode_offsets_fit(16384, 65536, 65536, 1, 16384, 32, 32), "the same in fp8 is 1 GiB");
  CHECK(!decode_offsets_fit(2048, 1 << 20, 512, 2, 2048, 32, 32), "padded A rows: 2048 rows of 2 MiB");
  CHECK(decode_offsets_fit(1023, 1 << 20, 512, 2, 1023, 32, 32), "1023 rows of 2 MiB end below 2 GiB");
  CHECK(!decode_offsets_fit(1025, 1 << 20, 512, 2, 1025, 32, 32), "1025 rows of 2 MiB do not");
  CHECK(!decode_offsets_fit(64, 512, 512, 2, 16385, 1 << 16, 32), "strided C view: 16385 rows of 128 KiB");
  CHECK(decode_offsets_fit(64, 512, 512, 2, 16384, 1 << 15, 32), "16384 rows of 64 KiB end below 2 GiB");
  CHECK(!decode_offsets_fit(0, 512, 512, 2, 64, 64, 64), "no rows");
}

// The tail policy: for every (tiles left in the last round, workgroups, K steps) the items of all
// workgroups must cover every K step of every tile exactly once, helpers must come before the mains that
// wait for them, slots must be distinct and within the XCD's share of the workspace, the main must expect
// exactly the partial sums that get written, in ascending K order, and the predicted round must never
// be longer than a whole tile.
void check_split_plan() {
  for (int wgs : {4, 32, 38})
    for (int left = 1; left < wgs; ++left)
      for (int nsteps : {1, 3, 4, 5, 10, 11, 43, 128, 129, 256, 1000})
      for (int costs = 0; costs < 2; ++costs) {  // planned with the measured costs, and with none (the test setting)
        const int gc = costs ? kSplitGatherCost : 0, pc = costs ? kSplitPassCost : 0;
        const SplitPlan s = split_plan(left, wgs, nsteps, gc, pc);
        CHECK(split_round_steps(s, nsteps, gc, pc) < nsteps || s.per_tile == 0, "split round not shorter than a tile: %d %d %d", left, wgs, nsteps);
        std::vector<std::vector<int>> covered(left, std::vector<int>(nsteps, 0));
        std::vector<int> slot_writer(wgs, -1), slot_begin(wgs, -1);
        std::vector<int> expects(left, 0), first_slot(left, 0), main_end(left, nsteps);
        for (int local = 0; local < wgs; ++local)
          for (int served = 0;; ++served) {
            int j, kb, ke, kind, partners, slot;
            if (!split_item(s, left, wgs, nsteps, local, served, j, kb, ke, kind, partners, slot)) break;
            CHECK(served < 64, "a workgroup never runs out of items");
            if (served >= 64) break;
            CHECK(j >= 0 && j < left && kb >= 0 && kb < ke && ke <= nsteps, "item out of range: %d %d %d wg %d", left, wgs, nsteps, local);
            for (int k = kb; k < ke; ++k) covered[j][k]++;
            if (kind == 1) {
              CHECK(local < wgs - left, "helper among the mains");
              CHECK(slot >= 0 && slot < wgs && slot_writer[slot] < 0, "slot %d reused or out of range (%d %d %d)", slot, left, wgs, nsteps);
              if (slot >= 0 && slot < wgs) { slot_writer[slot] = j; slot_begin[slot] = kb; }
            } else {
              CHECK(local >= wgs - left && kb == 0, "main among the helpers");
              CHECK((kind == 2) == (s.per_tile > 0), "kind of the main's item");
              expects[j] = partners; first_slot[j] = slot; main_end[j] = ke;
            }
          }
        for (int j = 0; j < left; ++j) {
          bool once = true;
          for (int k = 0; k < nsteps; ++k) once = once && covered[j][k] == 1;
          CHECK(once, "K steps of tile %d not covered exactly once (%d %d %d)", j, left, wgs, nsteps);
          int prev = main_end[j];
          for (int i = 0; i < expects[j]; ++i) {
            const int sl = first_slot[j] + i;
            CHECK(sl < wgs && slot_writer[sl] == j && slot_begin[sl] == prev, "main %d expects a partial sum nobody writes (%d %d %d)", j, left, wgs, nsteps);
            if (sl < wgs && slot_writer[sl] == j) prev = slot_begin[sl] + s.piece_steps;
          }
          int written = 0;
          for (int sl = 0; sl < wgs; ++sl) written += slot_writer[sl] == j;
          CHECK(written == expects[j], "tile %d: %d partial sums written, %d expected (%d %d %d)", j, written, expects[j], left, wgs, nsteps);
        }
      }
  // worked examples (32 workgroups per XCD).  More than half of the round filled: the tiles stay whole
  CHECK(split_plan(28, 32, 128).per_tile == 0 && split_plan(28, 32, 1024).per_tile == 0 && split_plan(17, 32, 1024).per_tile == 0,
        "a round that is more than half full stays whole");
  const SplitPlan h = split_plan(16, 32, 256);  // half a round: one helper per tile, about equal halves
  CHECK(h.per_tile == 1 && h.per_helper == 1 && h.main_steps == 129 && h.piece_steps == 127, "plan for 16/32/256: %d %d %d %d", h.per_tile, h.per_helper, h.main_steps, h.piece_steps);
  CHECK(split_round_steps(h, 256) == 137, "round of 16/32/256");
  const SplitPlan q = split_plan(6, 32, 256);   // a fifth of a round: still one helper per tile, twenty stay idle
  CHECK(q.per_tile == 1 && q.per_helper == 1 && q.main_steps == h.main_steps, "plan for 6/32/256: %d %d %d %d", q.per_tile, q.per_helper, q.main_steps, q.piece_steps);
  CHECK(split_plan(16, 32, 16).per_tile == 0, "16 K steps: the partial sum costs more than it saves");
}

int main() {
  check_row_tile<64>(256);
  check_row_tile<128>(256);
  check_row_tile<256>(64);
  check_col_tile<512, 2>(32);
  check_col_tile<256, 2>(32);
  check_col_tile<256, 1>(64);
  check_col_tile<128, 1>(64);
  sim_row_operand<64, 2>(256, 8);   // bf16/fp16 A tile 256 x 32
  sim_row_operand<64, 2>(128, 4);
  sim_row_operand<64, 1>(256, 8);   // fp8 A tile 256 x 64
  sim_col_operand<512, 2>(32);      // bf16 B tile 32 x 256
  sim_col_operand<256, 2>(32);      // bf16 B tile 32 x 128
  sim_col_operand<256, 1>(64);      // fp8 B tile 64 x 256
  sim_col_operand<128, 1>(64);      // fp8 B tile 64 x 128
  check_acc_layout();
  check_tile_orders();
  check_dealt_order();
  check_flag_counts();
  check_decode_offsets();
  check_split_plan();
  if (failures) { printf("%d check(s) failed\n", failures); return 1; }
  printf("layout_sim: all checks passed\n");
  return 0;
}
