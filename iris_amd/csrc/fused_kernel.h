// The MFMA kernel of libiris_hip (fused_mfma_kernel) with the types it shares with the generic
// kernel (FusedParams, the flag helpers), its tile shapes and its launch code.  The kernel is
// instantiated for 3 input types x 4 tile shapes x 2 operand layouts (plus the one-round builds);
// each input type is compiled in a translation unit of its own (iris_hip_mfma_<type>.hip), which
// instantiates dispatch_mfma_in<IN> below, so that the build can compile them side by side.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include <atomic>
#include <type_traits>

#include "iris_hip.h"
#include "layout.h"
#include "device_util.h"
#include "host_common.h"

using namespace iris_layout;

#define LDS_AS __attribute__((address_space(3)))

// Stages of the slot-sum pipeline of the eight-wave tile (see reduce_chunks).
#ifndef IRIS_HIP_EPILOGUE_DEPTH
#define IRIS_HIP_EPILOGUE_DEPTH 2
#endif

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;
typedef __attribute__((ext_vector_type(2))) int i32x2_t;
typedef __attribute__((ext_vector_type(4))) int i32x4_t;
typedef __attribute__((ext_vector_type(8))) int i32x8_t;
typedef __attribute__((ext_vector_type(4))) short i16x4_t;
typedef __attribute__((ext_vector_type(2))) unsigned u32x2_t;
typedef __attribute__((ext_vector_type(4))) unsigned u32x4_t;

enum { EPI_STORE = 0, EPI_ONE_SHOT = 1, EPI_TWO_SHOT = 2, EPI_REDUCE_SCATTER = 3, EPI_ALL_GATHER = 4, EPI_ATOMIC = 5 };

// Epilogues that publish aux + flags and then reduce over the slots.
__host__ __device__ inline bool epi_has_flags(int epi) { return epi == EPI_ONE_SHOT || epi == EPI_TWO_SHOT || epi == EPI_REDUCE_SCATTER; }
enum { GATHER_NONE = 0, GATHER_K = 1, GATHER_M = 2 };

struct FusedParams {
  const char* A;
  const char* B;
  char* C;
  char* aux;
  int* locks;
  const char* bias;
  int M, N, K;
  int K_local;  // K extent held by one source slot (== K unless gathered along K)
  int M_local;  // rows held by one source slot when gathered along M
  int gather;
  long long s_am, s_ak, s_bk, s_bn, s_cm, s_cn, s_bias;  // element strides
  const long long* heap_bases;
  int rank, world;
  int flag_bm, flag_bn;
  int epi;
  int acc_mode;
  int all_owners;
  int sum_peers;
  int bias_dtype;
  float scale;
  long long spin_limit;
  int* status;
  int tiles_m, tiles_n, group_m, num_xcd;
  // Tile order: 0 gives every XCD one contiguous span of the grouped order (tiles that share operand
  // panels share an L2), 1 deals the grouped order out workgroup by workgroup (the chip works on one
  // contiguous band of rows at a time; launches that stream the peers' tiles, see dispatch_mfma_in).
  int interleave;
  int tile_rotate;  // with interleave: the workgroups start this many positions into the grouped order (and wrap)
  int group_m_spans;  // host only: the group height to use if the launch falls back to spans (split tiles)
  int row_offset;  // all-gather: first row of this rank's block in the gathered output
  // Heap bases as kernel arguments (slots 0..7), valid when hb_in_args is set: the host knew the contents
  // of the context tensor (iris_hip_register_context), which spares the kernels a dependent scalar load
  // on the way to the peers' flags and tiles.
  long long hb_arg[8];
  int hb_in_args;
  // Split tiles (see the STREAMK builds of fused_mfma_kernel): one slot of partial sums and one flag per
  // workgroup, and the value a flag takes in this launch.  NULL / 0 when the launch does not split tiles.
  char* sk_partials;
  int* sk_flags;
  int sk_epoch;
  int sk_gather_cost, sk_pass_cost;  // the costs the host planned the split with (iris_layout::split_plan)
  int no_workspace_alloc;  // host only: the caller must not trigger an allocation (split tiles need one)
#ifdef IRIS_HIP_PHASE_STAMPS
  unsigned long long* stamps;  // diagnostic build: rows of 16 time stamps (see PHASE_STAMP)
  long long stamp_rows;        // rows the buffer holds; rows beyond it are not written
#endif
};

// Diagnostic build (-DIRIS_HIP_PHASE_STAMPS): thread 0 of every workgroup records the constant-rate
// 100 MHz counter at the phase boundaries of its first eight tiles, into row it * gridDim.x + blockIdx.x
// of p.stamps (16 slots per row, slot i):
//   0 kernel entry, 1 first operands in LDS, 2 K loop done, 3 tile staged in LDS, 4 phase-1 stores
//   issued, 5 phase-1 stores acknowledged, 6 own flags raised and peers' flags seen, 7 phase-2 stores
//   issued, 8 last store acknowledged.  The regular build compiles the macro away.
#ifdef IRIS_HIP_PHASE_STAMPS
#define PHASE_STAMP(i)                                                                         \
  do {                                                                                         \
    if (p.stamps && threadIdx.x == 0 && it < 8 && (long long)it * gridDim.x + blockIdx.x < p.stamp_rows)     \
      p.stamps[((long long)it * gridDim.x + blockIdx.x) * 16 + (i)] = wall_clock64();                       \
  } while (0)
#else
#define PHASE_STAMP(i) \
  do {                 \
  } while (0)
#endif

// ------------------------------------------------------------------------------------------------
// Small device helpers
// ------------------------------------------------------------------------------------------------

__device__ __forceinline__ int owner_of(int epi, int t, int total, int world, int rank) {
  if (epi == EPI_TWO_SHOT) return owner_interleaved(t, world);
  if (epi == EPI_REDUCE_SCATTER) return owner_contiguous(t, total, world);
  return rank;
}

// Raise the flags of the flag tiles covered by the macro tile at (m0, n0) of KM x KN elements.
// Must be called by every thread of the workgroup after the workgroup's aux stores have completed
// (vmcnt(0)) and a workgroup barrier.
// WRITTEN_THROUGH = false: the aux stores were ordinary stores (dirty lines in L2), so the flag is
//   raised with system-scope release, which writes the L2 back first.
// WRITTEN_THROUGH = true: the aux stores were system-scope write-through stores (store16_system) that
//   have been acknowledged, so the data is already where a peer reads it and a relaxed system-scope
//   flag store after them is enough; this spares one whole-L2 write-back per workgroup (measured 5-11 %
//   of the fused launch).
template <int KM, int KN, int NT, bool WRITTEN_THROUGH>
__device__ __forceinline__ void raise_flags(const FusedParams& p, int m0, int n0, int tid) {
  const int m1 = min(m0 + KM, p.M), n1 = min(n0 + KN, p.N);
  const int ftn = cdiv(p.N, p.flag_bn);
  const int fm_lo = m0 / p.flag_bm, fm_hi = (m1 - 1) / p.flag_bm;
  const int fn_lo = n0 / p.flag_bn, fn_hi = (n1 - 1) / p.flag_bn;
  const int nfn = fn_hi - fn_lo + 1;
  const int nft = (fm_hi - fm_lo + 1) * nfn;
  for (int i = tid; i < nft; i += NT) {
    const int fm = fm_lo + i / nfn, fn = fn_lo + i % nfn;
    int* flag = p.locks + (fm * ftn + fn);
    const int needed = macro_tiles_over_flag_tile(fm, fn, p.flag_bm, p.flag_bn, KM, KN, p.M, p.N);
    bool last = true;
    if (needed > 1) {
      // Arrivals are counted in steps of 2 so that the flag never reads 1 before the last one.
      int old = WRITTEN_THROUGH ? __hip_atomic_fetch_add(flag, 2, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM)
                                : __hip_atomic_fetch_add(flag, 2, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_SYSTEM);
      last = ((old >> 1) + 1) == needed;
    }
    if (last) {
      if (WRITTEN_THROUGH) __hip_atomic_exchange(flag, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
      else __hip_atomic_exchange(flag, 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
    }
  }
}

// Wait until the peers' flags of every flag tile this workgroup reduces are 1.
template <int KM, int KN, int NT>
__device__ __forceinline__ void wait_peer_flags(const FusedParams& p, int m0, int n0, int tid) {
  const int m1 = min(m0 + KM, p.M), n1 = min(n0 + KN, p.N);
  const int ftn = cdiv(p.N, p.flag_bn);
  const int ftotal = cdiv(p.M, p.flag_bm) * ftn;
  const int fm_lo = m0 / p.flag_bm, fm_hi = (m1 - 1) / p.flag_bm;
  const int fn_lo = n0 / p.flag_bn, fn_hi = (n1 - 1) / p.flag_bn;
  const int nfn = fn_hi - fn_lo + 1;
  const int nft = (fm_hi - fm_lo + 1) * nfn;
  const int items = nft * p.world;
  bool waited = false;
  for (int i = tid; i < items; i += NT) {
    const int r = i % p.world;
    const int f = i / p.world;
    if (r == p.rank) continue;
    const int t = (fm_lo + f / nfn) * ftn + fn_lo + f % nfn;
    if (!p.all_owners && owner_of(p.epi, t, ftotal, p.world, p.rank) != p.rank) continue;
    const int* flag = (const int*)slot_ptr(p.heap_bases, p.locks + t, p.rank, r);
    // Relaxed system-scope polls (they bypass the caches) and one acquire fence once the flag is up: an
    // acquire per poll would invalidate the XCD's L2 on every turn of the wait, under the feet of every
    // workgroup that is still multiplying or storing.
    long long polls = 0;
    while (__hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM) != 1) {
      if (p.spin_limit > 0 && ++polls >= p.spin_limit) {
        // A plain system-scope store (one status code, every writer stores the same word): the word
        // may live in pinned host memory.
        if (p.status) __hip_atomic_store(p.status, IRIS_HIP_STATUS_SPIN_TIMEOUT, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        break;
      }
      __builtin_amdgcn_s_sleep(8);
    }
    waited = true;
  }
  if (waited) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "");
}

// One look at the peers' flags that wait_peer_flags would wait for, without waiting: true when
// every flag this thread looked at was already 1, in which case the thread has also passed an
// acquire fence at system scope.  A workgroup barrier must follow before anybody reads the peers' data.
template <int KM, int KN, int NT>
__device__ __forceinline__ bool probe_peer_flags(const FusedParams& p, int m0, int n0, int tid) {
  const int m1 = min(m0 + KM, p.M), n1 = min(n0 + KN, p.N);
  const int ftn = cdiv(p.N, p.flag_bn);
  const int ftotal = cdiv(p.M, p.flag_bm) * ftn;
  const int fm_lo = m0 / p.flag_bm, fm_hi = (m1 - 1) / p.flag_bm;
  const int fn_lo = n0 / p.flag_bn, fn_hi = (n1 - 1) / p.flag_bn;
  const int nfn = fn_hi - fn_lo + 1;
  const int nft = (fm_hi - fm_lo + 1) * nfn;
  const int items = nft * p.world;
  bool up = true, looked = false;
  for (int i = tid; i < items; i += NT) {
    const int r = i % p.world;
    const int f = i / p.world;
    if (r == p.rank) continue;
    const int t = (fm_lo + f / nfn) * ftn + fn_lo + f % nfn;
    if (!p.all_owners && owner_of(p.epi, t, ftotal, p.world, p.rank) != p.rank) continue;
    const int* flag = (const int*)slot_ptr(p.heap_bases, p.locks + t, p.rank, r);
    up = up && (__hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM) == 1);
    looked = true;
  }
  // Only the threads that looked at a flag invalidate the caches (as only the polling threads do in
  // wait_peer_flags): the caches are the compute unit's, and an invalidation per wave of every
  // workgroup costs more than the probe saves.
  if (looked && up) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "");
  return up;
}

// ------------------------------------------------------------------------------------------------
// MFMA kernel configuration
// ------------------------------------------------------------------------------------------------
enum { IN_BF16 = 0, IN_F16 = 1, IN_FP8 = 2 };

template <int IN_, int BM_, int BN_, int BK_, int WM_, int WN_, int STAGES_, bool B_KCONTIG_>
struct MfmaCfg {
  static constexpr int IN = IN_;
  static constexpr int ES = (IN_ == IN_FP8) ? 1 : 2;
  static constexpr int CE = kChunkBytes / ES;           // elements per 16-byte chunk
  static constexpr int KM = (IN_ == IN_FP8) ? 64 : 16;  // k per MFMA
  static constexpr int BM = BM_, BN = BN_, BK = BK_, STAGES = STAGES_;
  static constexpr bool B_KCONTIG = B_KCONTIG_;
  static constexpr int WM = WM_, WN = WN_, NW = WM_ * WN_, NT = 64 * NW;
  static constexpr int TM = BM / WM, TN = BN / WN;  // per-wave block
  static constexpr int MB = TM / 32, NB = TN / 32;  // 32x32 MFMA blocks per wave
  static constexpr int KSLICES = BK / KM;
  static constexpr int NFRAG = (IN_ == IN_FP8) ? 2 : 1;   // 16-byte pieces per operand fragment
  static constexpr int RBA = BK * ES;                        // bytes per A tile row
  static constexpr int RBB = B_KCONTIG ? BK * ES : BN * ES;  // bytes per B tile row
  static constexpr int A_BYTES = BM * RBA;
  static constexpr int B_BYTES = B_KCONTIG ? BN * RBB : BK * RBB;
  static constexpr int STAGE_BYTES = A_BYTES + B_BYTES;
  static constexpr int LA = A_BYTES / kDmaBytes / NW;  // direct-to-LDS loads per thread per K step
  static constexpr int LB = B_BYTES / kDmaBytes / NW;
  static constexpr int RING_BYTES = STAGES * STAGE_BYTES;
  // Epilogue staging: the whole output tile in 16-bit elements.  The accumulator-layout writes put one
  // row per lane, so rows must not start on the same LDS banks.  The four-wave tiles pad every row by 16
  // bytes and stage over the (dead) operand ring from its start.  The eight-wave tile has no LDS to
  // spare for padding: it XORs the 16-byte chunk index with the row instead, and stages above the first
  // ring slot, which leaves that slot free to take the first K step of the workgroup's NEXT tile while
  // this tile's epilogue is still streaming (160 KiB = one ring slot + the staged tile).
  static constexpr bool STAGE_SWIZZLED = (NW == 8);
  static constexpr int STAGE_OFF = STAGE_SWIZZLED ? STAGE_BYTES : 0;
  static constexpr int TROW = STAGE_SWIZZLED ? BN * 2 : BN * 2 + 16;
  static constexpr int TILE_BYTES = BM * TROW;
  static constexpr int SMEM_BYTES = RING_BYTES > STAGE_OFF + TILE_BYTES ? RING_BYTES : STAGE_OFF + TILE_BYTES;
  static_assert(SMEM_BYTES <= 160 * 1024, "LDS budget of a gfx950 CU");
  static_assert(!STAGE_SWIZZLED || ((BN / 8) & (BN / 8 - 1)) == 0, "chunk swizzle needs a power-of-two row");
  // LDS byte offset of byte `b` of row `row` of the staged tile.
  __host__ __device__ static constexpr int stage_offset(int row, int b) {
    if (STAGE_SWIZZLED) return STAGE_OFF + row * TROW + ((((b >> 4) ^ row) & (BN / 8 - 1)) << 4) + (b & 15);
    return row * TROW + b;
  }
  // Four-wave tiles whose ring fits twice into a CU's LDS run two workgroups per CU, so that the
  // memory round trips of one workgroup's epilogue hide behind the other's K loop.
  static constexpr int WG_PER_CU = (NW == 4 && SMEM_BYTES <= 80 * 1024) ? 2 : 1;
  static constexpr int WAVES_PER_SIMD = WG_PER_CU * NW / 4;
  static_assert(NT % (BN / 8) == 0 && BM % (NT / (BN / 8)) == 0, "epilogue pass shape");
  static_assert(A_BYTES % (kDmaBytes * NW) == 0 && B_BYTES % (kDmaBytes * NW) == 0, "tile/loader mismatch");
  static_assert(BK % KM == 0 && TM % 32 == 0 && TN % 32 == 0, "tile/MFMA mismatch");
  static_assert(STAGES >= 3, "the ring needs at least three slots");
  static_assert((STAGES - 2) * (LA + LB) <= 63, "vmcnt field too small for this prefetch depth");
};

template <int IN>
struct OutOf { using type = OutBF16; };
template <>
struct OutOf<IN_F16> { using type = OutF16; };

// s_waitcnt vmcnt(n) with the other counters left unconstrained (gfx9 encoding).
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  __builtin_amdgcn_s_waitcnt((N & 0xF) | ((N >> 4) << 14) | (0x7 << 4) | (0xF << 8));
}

// The same with lgkmcnt(0): every LDS read of this wave has returned as well.
template <int N>
__device__ __forceinline__ void wait_vmcnt_lgkm0() {
  __builtin_amdgcn_s_waitcnt((N & 0xF) | ((N >> 4) << 14) | (0x7 << 4));
}

constexpr unsigned kInvalidOffset = 0x80000000u;

// Buffer resource words for a raw buffer (stride 0) over [base, base + 2^31).  Bounds are enforced
// per lane by the callers: an invalid lane presents offset 0x80000000, which is past num_records
// and therefore loads zero.
__device__ __forceinline__ i32x4_t make_rsrc_words(unsigned long long b) {
  i32x4_t r;
  r.x = __builtin_amdgcn_readfirstlane((int)(unsigned)b);
  r.y = __builtin_amdgcn_readfirstlane((int)(unsigned)(b >> 32));
  r.z = 0x7FFFFFFF;
  r.w = 0x00020000;
  return r;
}

// One wave-wide 16-byte direct-to-LDS load: lane l deposits global bytes [voff + soff, +16) of the
// buffer at LDS address lds_base + 16*l.  Written as inline assembly so that the compiler's
// wait-count pass does not serialise LDS reads behind loads that target other ring slots; the
// kernel orders them itself with wait_vmcnt() and workgroup barriers.
__device__ __forceinline__ void dma16(i32x4_t rsrc, unsigned lds_base, unsigned voff, unsigned soff) {
  asm volatile("s_mov_b32 m0, %0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
               :
               : "s"(lds_base), "v"(voff), "s"(rsrc), "s"(soff)
               : "memory");
}

// 16-byte store that is written through to memory at system scope (sc0 sc1): once vmcnt reports it
// done, every agent that reads the address with a coherent load sees it, without an L2 write-back.
__device__ __forceinline__ void store16_system(char* p, u32x4_t v) {
  asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1" : : "v"(p), "v"(v) : "memory");
}

// The same for data that the next instructions overwrite with VALU results (accumulator reads, say):
// a store of more than 8 bytes is still fetching its data registers for the last lanes when the next
// instruction issues, and a VALU write to them in that slot reaches memory for those lanes.  The
// compiler pads this hazard between instructions it can see; it cannot see into the asm statement, so
// the wait states are part of it.
__device__ __forceinline__ void store16_system_of_valu_data(char* p, u32x4_t v) {
  asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1\n\ts_nop 1" : : "v"(p), "v"(v) : "memory");
}

// Read one accumulator register.  The "a" constraint keeps the MFMA results in the accumulation
// registers until the epilogue consumes them, instead of copying all of them to VGPRs at once.
__device__ __forceinline__ float acc_read(float a) {
  float v;
  asm("v_accvgpr_read_b32 %0, %1" : "=v"(v) : "a"(a));
  return v;
}

__device__ __forceinline__ unsigned lds_address(const void* p) {
  return (unsigned)(unsigned long long)(LDS_AS const char*)p;
}

template <class CFG>
struct MfmaAcc {
  f32x16_t v[CFG::MB][CFG::NB];
};

// Operand fragments of one k-slice for a wave's block.
template <class CFG>
struct Frags {
  i32x4_t a[CFG::MB][CFG::NFRAG];
  i32x4_t b[CFG::NB][CFG::NFRAG];
};

// One 32x32 MFMA with the operands in the order (B fragment, A fragment): the accumulator then
// holds D[n][m], i.e. each lane owns 4 consecutive n for one m.
template <int IN, int NF>
__device__ __forceinline__ f32x16_t mfma_block(const i32x4_t (&a)[NF], const i32x4_t (&b)[NF], f32x16_t c) {
  if constexpr (IN == IN_BF16) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, b[0]),
                                                   __builtin_bit_cast(bf16x8_t, a[0]), c, 0, 0, 0);
  } else if constexpr (IN == IN_F16) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, b[0]),
                                                  __builtin_bit_cast(f16x8_t, a[0]), c, 0, 0, 0);
  } else {
    i32x8_t av, bv;
    av.lo = a[0]; av.hi = a[1];
    bv.lo = b[0]; bv.hi = b[1];
    // cbsz = blgp = 0 selects e4m3 for both operands; zero scale operands select the unscaled
    // instruction (v_mfma_f32_32x32x64_f8f6f4).
    return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(bv, av, c, 0, 0, 0, 0, 0, 0);
  }
}

constexpr int kMaxCachedSlots = 8;  // heap bases kept in registers; larger worlds re-load them

// A 64-bit value that is the same in every lane, moved to scalar registers.
__device__ __forceinline__ unsigned long long uniform64(unsigned long long x) {
  const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)x), hi = __builtin_amdgcn_readfirstlane((unsigned)(x >> 32));
  return ((unsigned long long)hi << 32) | lo;
}

// A copy of the kernel's argument block with every field materialised in registers at this point: the
// empty asm statements use the values, so their loads are issued together, up front.  Left to itself the
// compiler loads each field next to its first use and waits for it there, which put some twenty
// dependent scalar round trips in front of the first operand load of a launch.
__device__ __forceinline__ FusedParams pin_kernel_arguments(const FusedParams& a) {
  FusedParams q = a;
  asm volatile("" : "+s"(q.A), "+s"(q.B), "+s"(q.C), "+s"(q.aux), "+s"(q.locks), "+s"(q.bias), "+s"(q.heap_bases),
               "+s"(q.status), "+s"(q.spin_limit));
  asm volatile("" : "+s"(q.s_am), "+s"(q.s_ak), "+s"(q.s_bk), "+s"(q.s_bn), "+s"(q.s_cm), "+s"(q.s_cn), "+s"(q.s_bias));
  asm volatile("" : "+s"(q.M), "+s"(q.N), "+s"(q.K), "+s"(q.K_local), "+s"(q.M_local), "+s"(q.gather), "+s"(q.rank),
               "+s"(q.world), "+s"(q.flag_bm), "+s"(q.flag_bn), "+s"(q.epi), "+s"(q.acc_mode), "+s"(q.all_owners),
               "+s"(q.sum_peers), "+s"(q.bias_dtype), "+s"(q.scale));
  asm volatile("" : "+s"(q.tiles_m), "+s"(q.tiles_n), "+s"(q.group_m), "+s"(q.num_xcd), "+s"(q.row_offset),
               "+s"(q.hb_in_args));
  asm volatile("" : "+s"(q.hb_arg[0]), "+s"(q.hb_arg[1]), "+s"(q.hb_arg[2]), "+s"(q.hb_arg[3]), "+s"(q.hb_arg[4]),
               "+s"(q.hb_arg[5]), "+s"(q.hb_arg[6]), "+s"(q.hb_arg[7]));
#ifdef IRIS_HIP_PHASE_STAMPS
  asm volatile("" : "+s"(q.stamps), "+s"(q.stamp_rows));
#endif
  return q;
}

// The same for the tiled kernel, limited to what it needs before its first operand load (it has no
// registers to spare for holding the epilogue's arguments across the K loop).
__device__ __forceinline__ FusedParams pin_loader_arguments(const FusedParams& a) {
  FusedParams q = a;
  asm volatile("" : "+s"(q.A), "+s"(q.B), "+s"(q.s_am), "+s"(q.s_bk), "+s"(q.s_bn), "+s"(q.M), "+s"(q.N), "+s"(q.K),
               "+s"(q.K_local), "+s"(q.M_local), "+s"(q.gather), "+s"(q.rank), "+s"(q.world), "+s"(q.tiles_m),
               "+s"(q.tiles_n), "+s"(q.group_m), "+s"(q.num_xcd));
  return q;
}


// ------------------------------------------------------------------------------------------------
// MFMA kernel
// ------------------------------------------------------------------------------------------------
// ONE_ROUND: the launch has a workgroup for every tile, so a workgroup handles at most one.  The
// tile loop is then known to run once, which lets the compiler drop everything it otherwise carries
// from tile to tile (measured: 1.2 us of a 9 us launch on decode-sized problems).
//
// STREAMK (eight-wave tile only): the tail policy for tile counts that do not fill the last round of
// workgroups (iris_layout::split_plan has the scheme).  Inside every XCD's span of tiles, the tiles of
// the full rounds are handed out whole, as in the other builds.  In the last round the workgroups that
// would find no tile help the others: a helper multiplies a piece of a tile's K steps, stores its fp32
// accumulators to the piece's slot of p.sk_partials (write-through) and sets the slot's flag to
// p.sk_epoch; the tile's main workgroup multiplies the first K steps, waits for its helpers' flags, adds
// their partial sums in ascending piece order and runs the ordinary epilogue.  Helpers are the XCD's
// first workgroups and never wait, mains wait only for helpers - workgroups with lower indices, which
// the hardware dispatches first - so the waits end whatever part of the grid is resident.
template <class CFG, bool ONE_ROUND, bool STREAMK = false>
__global__ void __launch_bounds__(CFG::NT, CFG::WAVES_PER_SIMD) fused_mfma_kernel(const FusedParams p_in) {
  static_assert(!STREAMK || (CFG::NW == 8 && !ONE_ROUND), "split tiles: eight-wave tile, looping build");
  using Out = typename OutOf<CFG::IN>::type;
  using ATile = RowTile<CFG::RBA>;
  constexpr int ES = CFG::ES, CE = CFG::CE, BM = CFG::BM, BN = CFG::BN, BK = CFG::BK;
  constexpr int MB = CFG::MB, NB = CFG::NB, TM = CFG::TM, TN = CFG::TN, NW = CFG::NW, NT = CFG::NT;
  constexpr bool PINGPONG = CFG::NW == 8;
  constexpr int STAGES = CFG::STAGES, LA = CFG::LA, LB = CFG::LB, NFRAG = CFG::NFRAG, KS = CFG::KSLICES;

  extern __shared__ __attribute__((aligned(1024))) char smem[];

  const FusedParams q_args = pin_loader_arguments(p_in);  // the loaders' kernel arguments, fetched in one batch
  const FusedParams& p = q_args;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / CFG::WN, wn = wave % CFG::WN;

  // Heap bases of the first slots, read once (scalar loads) before the kernel stores anything.
  unsigned long long hb[kMaxCachedSlots];
  if (p.hb_in_args) {  // kernel arguments when the host knew them
#pragma unroll
    for (int r = 0; r < kMaxCachedSlots; ++r) hb[r] = (unsigned long long)p.hb_arg[r];
  } else if (p.heap_bases) {  // else independent loads behind one branch (indices clamped to the world size)
#pragma unroll
    for (int r = 0; r < kMaxCachedSlots; ++r) hb[r] = (unsigned long long)p.heap_bases[min(r, p.world - 1)];
  } else {
#pragma unroll
    for (int r = 0; r < kMaxCachedSlots; ++r) hb[r] = 0ull;
  }
#pragma unroll
  for (int r = 0; r < kMaxCachedSlots; ++r) hb[r] = uniform64(hb[r]);  // scalar registers, whichever branch ran
  unsigned long long hb_own = 0ull;
  if (p.rank < kMaxCachedSlots) {
#pragma unroll
    for (int r = 0; r < kMaxCachedSlots; ++r) hb_own = (r == p.rank) ? hb[r] : hb_own;
  } else {
    hb_own = uniform64((unsigned long long)p.heap_bases[p.rank]);
  }
  auto heap_base = [&](int r) -> unsigned long long {
    unsigned long long v = 0;
    if (r < kMaxCachedSlots) {
#pragma unroll
      for (int q = 0; q < kMaxCachedSlots; ++q) v = (r == q) ? hb[q] : v;
    } else {
      v = (unsigned long long)p.heap_bases[r];
    }
    return v;
  };
  // Address in slot r of own-slot address `own`.
  auto in_slot = [&](unsigned long long own, int r) -> unsigned long long { return heap_base(r) + (own - hb_own); };

  // ---- loader descriptors (tile independent) ---------------------------------------------------
  // A: row tile [BM][RBA].
  int la_row[LA], la_k[LA];
  unsigned la_off[LA];
#pragma unroll
  for (int i = 0; i < LA; ++i) {
    int row, c;
    ATile::from_lds((wave + i * NW) * kDmaBytes + lane * kChunkBytes, row, c);
    la_row[i] = row;
    la_k[i] = c * CE;
    la_off[i] = (unsigned)(row * p.s_am * ES + c * kChunkBytes);
  }
  // B: col tile [BK][BN*ES] (row-major B) or row tile [BN][RBA] (B given K-contiguous).
  int lb_row[LB], lb_col[LB];  // col tile: (k row, n element); row tile: (n row, k element)
  unsigned lb_off[LB];
#pragma unroll
  for (int i = 0; i < LB; ++i) {
    int row, c;
    const int off = (wave + i * NW) * kDmaBytes + lane * kChunkBytes;
    if constexpr (CFG::B_KCONTIG) {
      RowTile<CFG::RBB>::from_lds(off, row, c);
      lb_off[i] = (unsigned)(row * p.s_bn * ES + c * kChunkBytes);
    } else {
      ColTile<CFG::RBB, ES>::from_lds(off, row, c);
      lb_off[i] = (unsigned)(row * p.s_bk * ES + c * kChunkBytes);
    }
    lb_row[i] = row;
    lb_col[i] = c * CE;
  }

  // ---- fragment read offsets (relative to the slot's A / B region) -------------------------------
  int fa_off[KS][NFRAG];
#pragma unroll
  for (int kk = 0; kk < KS; ++kk)
#pragma unroll
    for (int h = 0; h < NFRAG; ++h) {
      const int c = (CFG::IN == IN_FP8) ? frag8_chunk(lane, kk, h) : frag16_chunk(lane, kk);
      fa_off[kk][h] = ATile::lds_offset(wm * TM + frag16_row(lane), c);
    }
  // B operand: K-contiguous B reads exactly like A; row-major B uses transpose reads.
  constexpr int NTR = (CFG::IN == IN_FP8) ? 1 : 2;  // distinct swizzles among the transpose reads
  int fb_off[CFG::B_KCONTIG ? KS : NB][CFG::B_KCONTIG ? NFRAG : NTR];
  if constexpr (CFG::B_KCONTIG) {
#pragma unroll
    for (int kk = 0; kk < KS; ++kk)
#pragma unroll
      for (int h = 0; h < NFRAG; ++h) {
        const int c = (CFG::IN == IN_FP8) ? frag8_chunk(lane, kk, h) : frag16_chunk(lane, kk);
        fb_off[kk][h] = RowTile<CFG::RBB>::lds_offset(wn * TN + frag16_row(lane), c);
      }
  } else {
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
      for (int j = 0; j < NTR; ++j) {
        int krow, n;
        if constexpr (CFG::IN == IN_FP8) {
          krow = tr8_krow(lane, 0, 0);
          n = wn * TN + nb * 32 + tr8_ncol(lane);
        } else {
          krow = tr16_krow(lane, 0, j);
          n = wn * TN + nb * 32 + tr16_ncol(lane);
        }
        fb_off[nb][j] = ColTile<CFG::RBB, ES>::lds_offset(krow, n / CE) + (n % CE) * ES;
      }
  }

  // Read the fragments of k-slice kk of ring slot `slot`.
  auto load_frags_b = [&](Frags<CFG>& f, int slot_off, int kk) {  // slot_off: byte offset of the ring slot
    const char* sb = smem + slot_off + CFG::A_BYTES;
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
      if constexpr (CFG::B_KCONTIG) {
#pragma unroll
        for (int h = 0; h < NFRAG; ++h)
          f.b[nb][h] = *(const LDS_AS i32x4_t*)(LDS_AS char*)(sb + fb_off[kk][h] + nb * 32 * CFG::RBB);
      } else if constexpr (CFG::IN == IN_FP8) {
        i32x2_t t[4];
#pragma unroll
        for (int r = 0; r < 4; ++r)
          t[r] = __builtin_amdgcn_ds_read_tr8_b64_v2i32(
              (LDS_AS i32x2_t*)(LDS_AS char*)(sb + fb_off[nb][0] + (kk * 64 + 8 * r) * CFG::RBB));
        f.b[nb][0] = (i32x4_t){t[0].x, t[0].y, t[1].x, t[1].y};
        f.b[nb][NFRAG - 1] = (i32x4_t){t[2].x, t[2].y, t[3].x, t[3].y};
      } else {
        i16x4_t t0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (LDS_AS i16x4_t*)(LDS_AS char*)(sb + fb_off[nb][0] + kk * 16 * CFG::RBB));
        i16x4_t t1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (LDS_AS i16x4_t*)(LDS_AS char*)(sb + fb_off[nb][NTR - 1] + kk * 16 * CFG::RBB));
        i32x2_t u0 = __builtin_bit_cast(i32x2_t, t0), u1 = __builtin_bit_cast(i32x2_t, t1);
        f.b[nb][0] = (i32x4_t){u0.x, u0.y, u1.x, u1.y};
      }
    }
  };
  auto load_frags_a = [&](Frags<CFG>& f, int slot_off, int kk, int mb) {
    const char* sa = smem + slot_off;
#pragma unroll
    for (int h = 0; h < NFRAG; ++h)
      f.a[mb][h] = *(const LDS_AS i32x4_t*)(LDS_AS char*)(sa + fa_off[kk][h] + mb * 32 * CFG::RBA);
  };
  auto load_frags = [&](Frags<CFG>& f, int slot_off, int kk) {
    load_frags_b(f, slot_off, kk);
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) load_frags_a(f, slot_off, kk, mb);
  };

  const int total_tiles = p.tiles_m * p.tiles_n;
  const int nsrc = (p.gather == GATHER_K) ? p.world : 1;
  const int klocal = (p.gather == GATHER_K) ? p.K_local : p.K;
  const int nkb = cdiv(klocal, BK);
  const int nsteps = nsrc * nkb;
  const unsigned smem_base = __builtin_amdgcn_readfirstlane(lds_address(smem));
  const unsigned long long a_own = (unsigned long long)p.A;

  // Split tiles (iris_layout::split_plan): every workgroup first takes its whole tiles, dp_rounds of
  // them at positions dp_first + round * wg_per_xcd of the grouped order; then the last round's tiles,
  // at positions sk_first + j, go to a main and its helpers.  Partial sum slot (and flag) of piece i >= 1
  // of tile j: sk_slot0 + j * per_tile + i - 1.
  enum { ITEM_WHOLE = 0, ITEM_PART = 1, ITEM_OWNER = 2 };  // the kinds of iris_layout::split_item
  int sk_first = 0, sk_left = 0, sk_slot0 = 0, sk_served = 0, dp_first = 0, dp_rounds = 0, dp_it = 0, wg_per_xcd = 1, sk_local = 0;
  SplitPlan plan = {0, 1, nsteps, 0};
  if constexpr (STREAMK) {
    const int xcd = blockIdx.x % p.num_xcd;
    sk_local = blockIdx.x / p.num_xcd;
    wg_per_xcd = gridDim.x / p.num_xcd;
    const int span = cdiv(total_tiles, p.num_xcd);
    const int first = min(xcd * span, total_tiles);
    const int mine = min(span, total_tiles - first);  // tiles of this XCD
    dp_rounds = mine / wg_per_xcd;
    sk_left = mine - dp_rounds * wg_per_xcd;          // tiles of the last, partly filled round
    dp_first = first + sk_local;
    sk_first = first + dp_rounds * wg_per_xcd;
    sk_slot0 = xcd * wg_per_xcd;
    plan = split_plan(sk_left, wg_per_xcd, nsteps, p.sk_gather_cost, p.sk_pass_cost);
  }

  // Looping workgroups of the eight-wave tile fetch the first K step of their next tile into ring slot 0
  // as soon as the K loop of the current tile is over (the staged tile lives above that slot): the loads
  // go out ahead of the epilogue's stores instead of behind them, and their latency - cold operand panels,
  // 2-3 us - passes under the epilogue.
  constexpr bool PREFETCH_NEXT = CFG::STAGE_SWIZZLED && !ONE_ROUND && !STREAMK;
  bool first_step_prefetched = false;
  const int order_xcd = p.interleave ? 1 : p.num_xcd;  // see FusedParams::interleave

  for (int it = 0; ONE_ROUND ? it < 1 : true; ++it) {
    int tidx, k_begin = 0, k_end = nsteps, item = ITEM_WHOLE, partners = 0, slot = 0;
    if constexpr (STREAMK) {
      if (dp_it < dp_rounds) {
        tidx = dp_first + dp_it * wg_per_xcd;
        ++dp_it;
      } else {
        int j;
        if (!split_item(plan, sk_left, wg_per_xcd, nsteps, sk_local, sk_served++, j, k_begin, k_end, item, partners, slot)) break;
        tidx = sk_first + j;
        slot += sk_slot0;
      }
    } else {
      tidx = xcd_tile_index(blockIdx.x, gridDim.x, it, total_tiles, order_xcd);
      if (tidx < 0) break;
      tidx += p.tile_rotate;
      if (tidx >= total_tiles) tidx -= total_tiles;
    }
    PHASE_STAMP(0);
    int tm, tn;
    grouped_tile(tidx, p.tiles_m, p.tiles_n, p.group_m, tm, tn);
    const int m0 = tm * BM, n0 = tn * BN;

    // ---- per-tile loader state ---------------------------------------------------------------
    // Row validity is folded into the per-lane offsets once per tile.
    unsigned a_voff[LA], b_voff[LB];
#pragma unroll
    for (int i = 0; i < LA; ++i) a_voff[i] = (m0 + la_row[i] < p.M) ? la_off[i] : kInvalidOffset;
#pragma unroll
    for (int i = 0; i < LB; ++i) {
      if constexpr (CFG::B_KCONTIG)
        b_voff[i] = (n0 + lb_row[i] < p.N) ? lb_off[i] : kInvalidOffset;
      else
        b_voff[i] = (n0 + lb_col[i] < p.N) ? lb_off[i] : kInvalidOffset;
    }
    // Byte offset of this tile's first A row inside the slot that holds it.
    int a_slot = p.rank;
    long long a_row0 = m0;
    if (p.gather == GATHER_M) {
      a_slot = m0 / p.M_local;
      a_row0 = m0 - (long long)a_slot * p.M_local;
    }
    if (p.gather == GATHER_K) a_slot = k_begin / nkb;  // the source that holds the first K step
    const unsigned long long a_tile_off = (unsigned long long)(a_row0 * p.s_am * ES);
    const i32x4_t rb = make_rsrc_words((unsigned long long)p.B + (unsigned long long)n0 * (CFG::B_KCONTIG ? p.s_bn : 1) * ES);
    i32x4_t ra = make_rsrc_words((p.gather == GATHER_NONE ? a_own : in_slot(a_own, a_slot)) + a_tile_off);

    // Loader position: next K step to issue = (i_src, i_kb), i_step overall.
    int i_step = k_begin, i_src = k_begin / nkb, i_kb = k_begin - (k_begin / nkb) * nkb;

    // The direct-to-LDS loads of one K step, issued one at a time so that the main loop can spread
    // them between its MFMAs (a wave issues in order: a burst of loads right after the barrier would
    // hold back the MFMAs behind it while the memory pipeline absorbs the burst).  Steps past the end
    // load nothing (every lane is out of range and deposits zeros), which keeps the per-thread count
    // of outstanding loads identical on every step.
    struct StepLoads {
      int klim;
      unsigned sa, sb, a_soff, b_soff;
    };
    auto begin_step = [&](int slot_off) {  // slot_off: byte offset of the ring slot to fill
      StepLoads L;
      const bool live = i_step < k_end;
      const int k0 = i_kb * BK;
      L.klim = live ? klocal - k0 : 0;  // k elements of this step that exist
      L.sa = smem_base + slot_off + wave * kDmaBytes;
      L.sb = L.sa + CFG::A_BYTES;
      L.a_soff = (unsigned)(k0 * ES);
      const long long kglob = (long long)i_src * klocal + k0;
      L.b_soff = __builtin_amdgcn_readfirstlane(
          CFG::B_KCONTIG ? (unsigned)(kglob * ES) : (unsigned)(kglob * p.s_bk * ES));
      return L;
    };
    auto load_offset = [&](const StepLoads& L, int j) -> unsigned {  // per-lane offset of load j
      if (j < LA) return (la_k[j] < L.klim) ? a_voff[j] : kInvalidOffset;
      const int i = j - LA;
      const int kpos = CFG::B_KCONTIG ? lb_col[i] : lb_row[i];
      return (kpos < L.klim) ? b_voff[i] : kInvalidOffset;
    };
    auto issue_at = [&](const StepLoads& L, int j, unsigned v) {
      if (j < LA)
        dma16(ra, L.sa + j * NW * kDmaBytes, v, L.a_soff);
      else
        dma16(rb, L.sb + (j - LA) * NW * kDmaBytes, v, L.b_soff);
    };
    auto issue_one = [&](const StepLoads& L, int j) { issue_at(L, j, load_offset(L, j)); };  // j in [0, LA + LB)
    auto end_step = [&]() {
      ++i_step;
      if (++i_kb == nkb) {  // next source slot (gather along K only)
        i_kb = 0;
        ++i_src;
        if (p.gather == GATHER_K && i_src < nsrc) ra = make_rsrc_words(in_slot(a_own, i_src) + a_tile_off);
      }
    };
    auto issue = [&](int slot) {
      const StepLoads L = begin_step(slot * CFG::STAGE_BYTES);
#pragma unroll
      for (int j = 0; j < LA + LB; ++j) issue_one(L, j);
      end_step();
    };

    MfmaAcc<CFG> acc;
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc.v[mb][nb][i] = 0.f;

    // ---- prologue: fill STAGES-1 ring slots, wait for the first ----------------------------------
    // The two-group loop reads a slot in both of its phases and refills it one step later than the
    // single-group loop, so it keeps one step less in flight.
    constexpr int AHEAD = PINGPONG ? STAGES - 2 : STAGES - 1;  // K steps issued before the loop starts
#pragma unroll
    for (int s = 0; s < AHEAD; ++s) {
      if (PREFETCH_NEXT && s == 0 && first_step_prefetched)
        end_step();  // already on its way (or there): only the loader position moves on
      else
        issue(s);
    }
    first_step_prefetched = false;
    wait_vmcnt<(AHEAD - 1) * (LA + LB)>();
    __builtin_amdgcn_s_barrier();
    PHASE_STAMP(1);
    Frags<CFG> fr[KS < 2 ? 2 : KS];  // one set per k-slice (two for the loops that double-buffer)
    if constexpr (!PINGPONG) load_frags(fr[0], 0, 0);

    // ---- main loop ----------------------------------------------------------------------------
    // Invariant at the top of step s: the operands of step s are in LDS and visible to all waves,
    // and the fragments of its first k-slice are in flight.  The step first makes sure step s+1
    // has landed too, so that its first fragments can be fetched while step s still computes.
    // The four-wave tiles have registers to spare and run the loop unrolled over the ring positions,
    // which turns every LDS address of a step into a constant offset (5-10 % on those tiles); the
    // eight-wave tile would spill and keeps the ring position in a register.
    constexpr int RING_UNROLL = (NW == 4) ? STAGES : 1;
    int s = k_begin, ring_pos = 0;
    if constexpr (PINGPONG) {
      // Eight waves, two per SIMD: waves 0-3 and waves 4-7 run half a step apart.  A step is a
      // memory phase (all fragment reads of the step, then the direct-to-LDS loads that refill the
      // slot of the previous step) and a compute phase (nothing but MFMAs), each closed by a
      // workgroup barrier, so that on every SIMD one wave feeds the matrix pipe while the other
      // one has the LDS and memory ports to itself.
      const bool late = wave >= 4;
      if (late) __builtin_amdgcn_s_barrier();
      // The loader position of the common case - a whole K step inside one source - is carried in
      // scalar registers that advance by constants, and its loads need no per-lane k test; partial
      // steps, source changes and the empty steps past the end take the general path.
      const unsigned b_inc = __builtin_amdgcn_readfirstlane(
          CFG::B_KCONTIG ? (unsigned)(BK * ES) : (unsigned)((long long)BK * p.s_bk * ES));
      unsigned a_so = 0, b_so = 0;
      int k_left = 0;
      auto resync = [&]() {
        a_so = (unsigned)(i_kb * BK * ES);
        const long long kglob = (long long)i_src * klocal + (long long)i_kb * BK;
        b_so = __builtin_amdgcn_readfirstlane(
            CFG::B_KCONTIG ? (unsigned)(kglob * ES) : (unsigned)(kglob * p.s_bk * ES));
        k_left = i_step < k_end ? klocal - i_kb * BK : 0;
      };
      resync();
      unsigned rd = 0;                                    // byte offset of the slot this step reads
      unsigned wr = AHEAD * CFG::STAGE_BYTES;             // ... and of the slot it refills
      const unsigned wr_wave = smem_base + wave * kDmaBytes;
      // The fragments of the first half of a step's MFMAs are read in the memory phase, those of the
      // second half between the MFMAs of the first (LDS reads issue in the shadow of an MFMA;
      // direct-to-LDS loads do not, a wave takes some 80 cycles to get one accepted).
      constexpr int NMFMA = KS * MB * NB;
      constexpr bool SPLIT_K = KS >= 2;                    // halves split by k-slice, else by row block
      static_assert(KS == 1 || KS % 2 == 0, "k-slices split in two halves");
      static_assert(MB % 2 == 0, "row blocks split in two halves");
      // Late fragment reads, in pieces: per late k-slice the B fragments, then one row block of A each;
      // with a single slice the upper row blocks of A.
      constexpr int LATE_PIECES = SPLIT_K ? (KS / 2) * (1 + MB) : MB / 2;
      auto late_piece = [&](int pc) {
        if constexpr (SPLIT_K) {
          const int kk = KS / 2 + pc / (1 + MB), q = pc % (1 + MB);
          if (q == 0)
            load_frags_b(fr[kk], rd, kk);
          else
            load_frags_a(fr[kk], rd, kk, q - 1);
        } else {
          load_frags_a(fr[0], rd, 0, MB / 2 + pc);
        }
      };
      for (; s < k_end; ++s) {
        if constexpr (SPLIT_K) {
#pragma unroll
          for (int kk = 0; kk < KS / 2; ++kk) load_frags(fr[kk], rd, kk);
        } else {
          load_frags_b(fr[0], rd, 0);
#pragma unroll
          for (int mb = 0; mb < MB / 2; ++mb) load_frags_a(fr[0], rd, 0, mb);
        }
        __builtin_amdgcn_sched_barrier(0);
        if (k_left >= BK) {
#pragma unroll
          for (int j = 0; j < LA; ++j) dma16(ra, wr_wave + wr + j * NW * kDmaBytes, a_voff[j], a_so);
#pragma unroll
          for (int i = 0; i < LB; ++i)
            dma16(rb, wr_wave + wr + CFG::A_BYTES + i * NW * kDmaBytes, b_voff[i], b_so);
        } else {
          const StepLoads L = begin_step(wr);
#pragma unroll
          for (int j = 0; j < LA + LB; ++j) issue_one(L, j);
        }
        end_step();
        if (i_kb == 0) {
          resync();
        } else {
          a_so += BK * ES;
          b_so += b_inc;
          k_left -= BK;
        }
        // Own early fragment reads done and own loads of step s+1 landed.
        wait_vmcnt_lgkm0<(AHEAD - 1) * (LA + LB)>();
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        // First half of the MFMAs with the late fragment reads spread between them.
#pragma unroll
        for (int i = 0; i < NMFMA / 2; ++i) {
          const int kk = i / (MB * NB), mb = (i / NB) % MB, nb = i % NB;  // one slice: mb < MB/2 here
          acc.v[mb][nb] = mfma_block<CFG::IN, NFRAG>(fr[kk].a[mb], fr[kk].b[nb], acc.v[mb][nb]);
#pragma unroll
          for (int pc = 0; pc < LATE_PIECES; ++pc)
            if (pc * (NMFMA / 2) / LATE_PIECES == i) late_piece(pc);
          __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int i = NMFMA / 2; i < NMFMA; ++i) {
          const int kk = i / (MB * NB), mb = (i / NB) % MB, nb = i % NB;
          acc.v[mb][nb] = mfma_block<CFG::IN, NFRAG>(fr[kk].a[mb], fr[kk].b[nb], acc.v[mb][nb]);
        }
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        rd = rd + CFG::STAGE_BYTES == CFG::RING_BYTES ? 0 : rd + CFG::STAGE_BYTES;
        wr = wr + CFG::STAGE_BYTES == CFG::RING_BYTES ? 0 : wr + CFG::STAGE_BYTES;
      }
      if (!late) __builtin_amdgcn_s_barrier();
    } else
    while (s < k_end) {
#pragma unroll
    for (int u = 0; u < RING_UNROLL; ++u) {
      if (s >= k_end) break;
      ++s;
      const int slot = (RING_UNROLL == 1) ? ring_pos : u;
      // LDS is one coherent memory per CU, so a bare s_barrier (no fence, hence no forced wait for
      // the fragment reads in flight) orders the operand ring between the waves.
      wait_vmcnt<(STAGES - 3) * (LA + LB)>();  // this thread's loads of step s+1 have landed
      __builtin_amdgcn_s_barrier();             // everyone's have; everyone is past step s-1
      int pslot = slot + STAGES - 1;
      if (pslot >= STAGES) pslot -= STAGES;
      const StepLoads L = begin_step(pslot * CFG::STAGE_BYTES);  // refills the slot the previous step used
      const int nslot = slot + 1 == STAGES ? 0 : slot + 1;
      constexpr int NSLOT = KS * MB;          // MFMA groups of a step; the loads are spread over them
      constexpr int NLOAD = LA + LB;
#pragma unroll
      for (int kk = 0; kk < KS; ++kk) {
        if (kk + 1 < KS)
          load_frags(fr[(kk + 1) & 1], slot * CFG::STAGE_BYTES, kk + 1);
        else
          load_frags(fr[(kk + 1) & 1], nslot * CFG::STAGE_BYTES, 0);
        const Frags<CFG>& f = fr[kk & 1];
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
#pragma unroll
          for (int j = 0; j < NLOAD; ++j)
            if (j * NSLOT / NLOAD == kk * MB + mb) issue_one(L, j);
#pragma unroll
          for (int nb = 0; nb < NB; ++nb) acc.v[mb][nb] = mfma_block<CFG::IN, NFRAG>(f.a[mb], f.b[nb], acc.v[mb][nb]);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
      end_step();
      static_assert(KS % 2 == 0 || KS == 1, "fragment double buffer assumes an even slice count");
      if constexpr (KS == 1) {
        // With one slice per step the two buffers alternate across steps.
        Frags<CFG> t = fr[0];
        fr[0] = fr[1];
        fr[1] = t;
      }
      ring_pos = nslot;
    }
    }

    // The ring is reused as epilogue staging: drain the (empty) loads still in flight and make
    // sure every wave has finished reading operands.
    wait_vmcnt<0>();
    __syncthreads();
    PHASE_STAMP(2);

    if constexpr (STREAMK) {
      // Partial sums travel in the accumulators' own layout: 16-byte piece j of thread t at byte
      // (j * NT + t) * 16 of the piece's slot, so that every wave instruction moves 1 KiB.
      constexpr int PIECES = MB * NB * 4;  // 16-byte pieces per thread
      constexpr long long SLOT_BYTES = (long long)PIECES * NT * 16;
      if (item == ITEM_PART) {
        // (The base goes through an empty asm so that the compiler computes the pieces' addresses here, one
        // at a time, instead of keeping all of them in registers from the top of the kernel.)
        unsigned long long slot_base = (unsigned long long)p.sk_partials + (unsigned long long)slot * SLOT_BYTES;
        asm volatile("" : "+s"(slot_base));
        char* const dst = (char*)slot_base + tid * 16;
#pragma unroll
        for (int j = 0; j < PIECES; ++j) {
          const int mb = j / (NB * 4), nb = (j / 4) % NB, q = j % 4;
          u32x4_t v;
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] = __float_as_uint(acc_read(acc.v[mb][nb][4 * q + e]));
          store16_system_of_valu_data(dst + (long long)j * NT * 16, v);
          __builtin_amdgcn_sched_barrier(0);  // one piece at a time: the scheduler would read all 128 registers first
        }
        // Published like an aux tile: stores acknowledged by every wave, then one relaxed flag store.
        wait_vmcnt<0>();
        __syncthreads();
        if (tid == 0) __hip_atomic_store(p.sk_flags + slot, p.sk_epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        PHASE_STAMP(3);
        continue;  // the ring is free (barrier above); no epilogue for a partial sum
      }
      if (item == ITEM_OWNER) {
        if (tid < partners) {
          const int* flag = p.sk_flags + (slot + tid);
          // Relaxed polls and one acquire fence at the end: an acquire load per poll would invalidate the
          // XCD's L2 on every turn while the helpers next door are still storing (measured: their 256 KiB
          // took 25 us that way).
          long long polls = 0;
          while (__hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM) != p.sk_epoch) {
            if (p.spin_limit > 0 && ++polls >= p.spin_limit) {
              if (p.status) __hip_atomic_store(p.status, IRIS_HIP_STATUS_SPIN_TIMEOUT, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
              break;
            }
            __builtin_amdgcn_s_sleep(8);
          }
          __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "");
        }
        __syncthreads();
      }
    }

    if constexpr (PREFETCH_NEXT) {
      int nidx = xcd_tile_index(blockIdx.x, gridDim.x, it + 1, total_tiles, order_xcd);
      if (nidx >= 0) {
        nidx += p.tile_rotate;
        if (nidx >= total_tiles) nidx -= total_tiles;
        int ntm, ntn;
        grouped_tile(nidx, p.tiles_m, p.tiles_n, p.group_m, ntm, ntn);
        const int nm0 = ntm * BM, nn0 = ntn * BN;
        int n_slot = p.rank;
        long long n_row0 = nm0;
        if (p.gather == GATHER_M) {
          n_slot = nm0 / p.M_local;
          n_row0 = nm0 - (long long)n_slot * p.M_local;
        }
        if (p.gather == GATHER_K) n_slot = 0;
        const i32x4_t nra = make_rsrc_words((p.gather == GATHER_NONE ? a_own : in_slot(a_own, n_slot)) + (unsigned long long)(n_row0 * p.s_am * ES));
        const i32x4_t nrb = make_rsrc_words((unsigned long long)p.B + (unsigned long long)nn0 * (CFG::B_KCONTIG ? p.s_bn : 1) * ES);
        const unsigned sa = smem_base + wave * kDmaBytes, sb = sa + CFG::A_BYTES;  // ring slot 0
#pragma unroll
        for (int j = 0; j < LA; ++j) {
          const bool ok = nm0 + la_row[j] < p.M && la_k[j] < klocal;
          dma16(nra, sa + j * NW * kDmaBytes, ok ? la_off[j] : kInvalidOffset, 0u);
        }
#pragma unroll
        for (int i = 0; i < LB; ++i) {
          const bool ok = CFG::B_KCONTIG ? (nn0 + lb_row[i] < p.N && lb_col[i] < klocal) : (nn0 + lb_col[i] < p.N && lb_row[i] < klocal);
          dma16(nrb, sb + i * NW * kDmaBytes, ok ? lb_off[i] : kInvalidOffset, 0u);
        }
        first_step_prefetched = true;
      }
    }

    // ---- epilogue -------------------------------------------------------------------------------
    // The whole output tile is first written to LDS in the output type (the operand ring is dead
    // by now), which frees the accumulators; both phases then stream rows of the tile, 16 bytes per
    // lane and BN*2 contiguous bytes per row, with many loads in flight per thread.
    {
      // Split tiles: 16-byte pieces of a partial sum, in the layout its workgroup stored them in.
      constexpr int PIECES = MB * NB * 4, NBATCH = 4, BATCH = PIECES / NBATCH;
      constexpr long long SLOT_BYTES = (long long)PIECES * NT * 16;
      float badd[MB];
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        badd[mb] = 0.f;
        if (p.bias) {
          const int gm = m0 + wm * TM + mb * 32 + acc_col(lane);
          if (gm < p.M) badd[mb] = load_scalar_as_float(p.bias, (long long)gm * p.s_bias, p.bias_dtype);
        }
      }
      // The lane index as the staging addresses see it goes through an empty asm: with the swizzled layout
      // a lane has one address term per (column block, quarter), and the compiler would otherwise compute
      // them once, ahead of the tile loop, and carry eight more registers through the K loop.
      int lane_s = lane;
      asm volatile("" : "+v"(lane_s));
      // Piece j of the thread: 4 consecutive n of one m, from their fp32 sums to the staged tile.
      auto stage_piece = [&](int j, const float (&sum)[4]) {
        const int mb = j / (NB * 4), nb = (j / 4) % NB, q = j % 4;
        float h[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) h[e] = sum[e] * p.scale + badd[mb];
        u32x2_t w;
        w.x = Out::pack(h[0], h[1]);
        w.y = Out::pack(h[2], h[3]);
        const int trow = wm * TM + mb * 32 + acc_col(lane_s);
        const int tcol = wn * TN + nb * 32 + acc_row(lane_s, 4 * q);
        *(LDS_AS u32x2_t*)(LDS_AS char*)(smem + CFG::stage_offset(trow, tcol * 2)) = w;
      };
      auto own_piece = [&](int j, float (&sum)[4]) {
        const int mb = j / (NB * 4), nb = (j / 4) % NB, q = j % 4;
#pragma unroll
        for (int e = 0; e < 4; ++e) sum[e] = acc_read(acc.v[mb][nb][4 * q + e]);
      };
      bool staged = false;
      if constexpr (STREAMK) {
        if (item == ITEM_OWNER && partners > 0) {
          // own sum + the helper's partial sum, a quarter of the pieces at a time.  (The accumulators are only read: adding into them in place makes the compiler
          // move the whole tile through VGPRs.)
          staged = true;
          unsigned long long base = (unsigned long long)p.sk_partials + (unsigned long long)slot * SLOT_BYTES;
          asm volatile("" : "+s"(base));  // addresses are formed where they are used, not hoisted out of the tile loop
          const char* const src = (const char*)base + tid * 16;
          auto load_batch = [&](u32x4_t (&dst)[BATCH], const char* src, int b) {
#pragma unroll
            for (int i = 0; i < BATCH; ++i)
              dst[i] = __builtin_nontemporal_load((const u32x4_t*)(src + (long long)(b * BATCH + i) * NT * 16));
          };
          {  // the next batch is on its way while this one is staged
            u32x4_t buf[2][BATCH];
            load_batch(buf[0], src, 0);
#pragma unroll
            for (int b = 0; b < NBATCH; ++b) {
              if (b + 1 < NBATCH) load_batch(buf[(b + 1) & 1], src, b + 1);
#pragma unroll
              for (int i = 0; i < BATCH; ++i) {
                float sum[4];
                own_piece(b * BATCH + i, sum);
#pragma unroll
                for (int e = 0; e < 4; ++e) sum[e] += __uint_as_float(buf[b & 1][i][e]);
                stage_piece(b * BATCH + i, sum);
              }
              __builtin_amdgcn_sched_barrier(0);
            }
          }
        }
      }
      if (!staged) {
#pragma unroll
        for (int j = 0; j < PIECES; ++j) {
          float sum[4];
          own_piece(j, sum);
          stage_piece(j, sum);
        }
      }
    }
    __syncthreads();
    PHASE_STAMP(3);

    constexpr int CPR = BN / 8;            // 16-byte chunks per tile row
    constexpr int RPP = NT / CPR;          // tile rows covered by one pass of the workgroup
    constexpr int PASSES = BM / RPP;
    int tid_s = tid;  // as lane_s above: per-thread staging offsets are formed here, not ahead of the tile loop
    asm volatile("" : "+v"(tid_s));
    const int t_row = tid_s / CPR, t_chunk = tid_s % CPR;
    const int gn = n0 + t_chunk * 8;
    const bool col_ok = gn < p.N;
    // LDS offset of this thread's chunk in pass ps: t_pass[ps & 1] + ps * RPP * TROW (the passes are RPP
    // rows apart; with the swizzled layout the chunk's place in the row alternates between two values).
    static_assert(!CFG::STAGE_SWIZZLED || (2 * RPP) % CPR == 0, "the swizzle must repeat every two passes");
    const int t_pass[2] = {CFG::stage_offset(t_row, t_chunk * 16), CFG::stage_offset(t_row + RPP, t_chunk * 16) - RPP * CFG::TROW};

    // Phase 1: C (plain store) or aux (own slot).  When no peer contributes (world of one, or peers
    // switched off) the reduced tile equals the own tile, so C is written in the same pass and
    // phase 2 is skipped.
    const bool flags = epi_has_flags(p.epi);
    const bool solo = flags && (!p.sum_peers || p.world == 1);
    {
      char* const out1 = flags ? p.aux : p.C;
      const int ftn1 = cdiv(p.N, p.flag_bn);
      const int ftotal1 = cdiv(p.M, p.flag_bm) * ftn1;
      const unsigned long long c_base = (unsigned long long)p.C;
      if (p.epi == EPI_ATOMIC) {
        // The tile is added into every rank's C (iris/mem/triton/context.py:689-702) with packed 16-bit
        // atomics of one dword each.  Dword d of a pass belongs to thread d mod NT, so that one wave
        // instruction covers 256 contiguous bytes (two whole lines for the L2's atomic units); with
        // each thread adding the four dwords of its own 16-byte chunk an instruction touched eight
        // lines with eight dwords each, and the launch ran at a quarter of the rate.
        constexpr int DPR = BN / 2;                   // dwords per tile row
        constexpr int DPP = RPP * DPR;                // dwords per pass (= 4 * NT)
        for (int ps = 0; ps < PASSES; ++ps) {
#pragma unroll
          for (int j = 0; j < DPP / NT; ++j) {
            const int d = j * NT + tid;
            const int row = ps * RPP + d / DPR, dc = d % DPR;
            const int gm = m0 + row, gc = n0 + 2 * dc;
            if (gm >= p.M || gc >= p.N) continue;
            const unsigned w = *(const LDS_AS unsigned*)(LDS_AS char*)(smem + CFG::stage_offset(row, dc * 4));
            const long long eoff = ((long long)(gm + p.row_offset) * p.s_cm + gc) * 2;
            for (int pr = 0; pr < p.world; ++pr) atomic_add_packed<Out>((char*)(in_slot(c_base, pr) + eoff), w);
          }
        }
      } else
#pragma unroll 4
      for (int ps = 0; ps < PASSES; ++ps) {
        const int gm = m0 + ps * RPP + t_row;
        const u32x4_t v = *(const LDS_AS u32x4_t*)(LDS_AS char*)(smem + t_pass[ps & 1] + ps * RPP * CFG::TROW);
        if (gm < p.M && col_ok) {
          const long long eoff = ((long long)(gm + p.row_offset) * p.s_cm + gn) * 2;
          if (p.epi == EPI_ALL_GATHER) {
            // the tile goes to every rank's gathered output (iris/mem/triton/context.py:841-864)
            for (int pr = 0; pr < p.world; ++pr) __builtin_nontemporal_store(v, (u32x4_t*)(in_slot(c_base, pr) + eoff));
          } else if (flags) {
            store16_system(out1 + eoff, v);  // aux: read by the peers as soon as the flag is up
          } else {
            __builtin_nontemporal_store(v, (u32x4_t*)(out1 + eoff));
          }
          if (solo) {
            int owner = p.rank;
            if (p.epi != EPI_ONE_SHOT) owner = owner_of(p.epi, (gm / p.flag_bm) * ftn1 + gn / p.flag_bn, ftotal1, p.world, p.rank);
            if (p.all_owners || owner == p.rank) {
              if (p.epi == EPI_TWO_SHOT) {
                for (int pr = 0; pr < p.world; ++pr) __builtin_nontemporal_store(v, (u32x4_t*)(in_slot(c_base, pr) + eoff));
              } else {
                const int dst = p.all_owners ? owner : p.rank;
                __builtin_nontemporal_store(v, (u32x4_t*)(in_slot(c_base, dst) + eoff));
              }
            }
          }
        }
      }
    }

    PHASE_STAMP(4);
    if (flags) {
      // Publish: the aux tile was stored write-through at system scope; every wave waits until its
      // stores are acknowledged, the workgroup meets, and the threads that own flags raise them
      // (no L2 write-back is needed any more).  The peers' flags are polled by one set of threads for
      // the whole workgroup (relaxed loads, one acquire when a flag is up); letting every wave poll
      // and run ahead measured slower.
      // The peers' flags are looked at once while the own stores are still on their way: a thread that
      // found the flags it is responsible for up already - peers that finished first - has their round
      // trip hidden behind that wait and does not poll after the own flags are raised.  Every thread
      // knows only about its own flags; the barrier behind the polling makes it common knowledge.
      const bool up_already = solo ? true : probe_peer_flags<BM, BN, NT>(p, m0, n0, tid);
      wait_vmcnt<0>();
      __syncthreads();
      PHASE_STAMP(5);
      raise_flags<BM, BN, NT, true>(p, m0, n0, tid);
      if (!solo) {
        if (!up_already) wait_peer_flags<BM, BN, NT>(p, m0, n0, tid);
        __syncthreads();
      }
      PHASE_STAMP(6);

      // Phase 2: reduce the flag tiles this rank is responsible for.  The peer loads are issued
      // unconditionally (rows this thread does not reduce read the tile origin instead) and for a
      // compile-time number of peers, so that all loads of a group of passes are in flight
      // together; only the stores are predicated.
      const bool ref_chain = (p.acc_mode == IRIS_HIP_ACC_REFERENCE) && !Out::kFp32SumInReference;
      const unsigned long long aux_own = (unsigned long long)p.aux, c_own = (unsigned long long)p.C;
      const int ftn = cdiv(p.N, p.flag_bn);
      const int ftotal = cdiv(p.M, p.flag_bm) * ftn;
      const int fcol = gn / p.flag_bn;
      const int npeers = p.sum_peers ? p.world - 1 : 0;
      // Peer aux bases in ascending rank order, own rank skipped.
      unsigned long long pb[kMaxCachedSlots - 1];
#pragma unroll
      for (int i = 0; i < kMaxCachedSlots - 1; ++i) pb[i] = (i < p.rank ? hb[i] : hb[i + 1]) + (aux_own - hb_own);
      const long long safe_off = ((long long)m0 * p.s_cm + n0) * 2;  // first element of the tile

      // The peers' tiles are read once and C is written once, so both go past the caches' keep
      // policy (non-temporal): they neither displace the operands nor - what costs more - make the
      // last-level cache write back whatever dirty lines it holds to take them in (measured on the
      // 4096 x 4096 x 1376 bf16 launch with seven peers, after a 256 MB buffer had been zeroed: phase 2
      // 68 -> 39 us; with the peers' tiles already cached the two policies tie for the one-shot variant).
      // Chunks are handed to the threads either over the whole kernel tile (RECT false: thread t
      // takes chunk t of every pass, ownership looked up per chunk) or over one rectangle of it,
      // rows [r0, r1) and `ncw` chunks from column c0, all of which `rect_owner` reduces (RECT true).
      auto reduce_chunks = [&](auto np_tag, auto rect_tag, int r0, int r1, int c0, int ncw, int rect_owner) {
        constexpr int NP = decltype(np_tag)::value;  // peers with cached bases; -1: any number
        constexpr bool RECT = decltype(rect_tag)::value;
        constexpr int NPV = NP > 0 ? NP : 1;
        const int npasses = RECT ? cdiv((r1 - r0) * ncw, NT) : PASSES;
        // One pass of the workgroup: the addresses of this thread's chunk, the peers' chunks requested, the
        // own chunk read from LDS ...
        struct Pass {
          bool active;
          long long eoff;
          int owner;
          u32x4_t own, pv[NPV];
        };
        auto issue = [&](int ps, Pass& st) {
          int gm, gc, lds_off;
          if constexpr (RECT) {
            const unsigned idx = (unsigned)(ps * NT + tid);
            const unsigned row = idx / (unsigned)ncw;
            gm = r0 + (int)row;
            gc = c0 + (int)(idx - row * (unsigned)ncw) * 8;
            st.owner = rect_owner;
            st.active = gm < r1;
            lds_off = st.active ? CFG::stage_offset(gm - m0, (gc - n0) * 2) : CFG::stage_offset(0, 0);
          } else {
            gm = m0 + ps * RPP + t_row;
            gc = gn;
            st.owner = p.rank;
            if (p.epi != EPI_ONE_SHOT) {  // one-shot reduces every tile: no owner arithmetic
              const int t = (gm / p.flag_bm) * ftn + fcol;
              st.owner = owner_of(p.epi, t, ftotal, p.world, p.rank);
            }
            st.active = gm < p.M && col_ok && (p.all_owners || st.owner == p.rank);
            lds_off = t_pass[ps & 1] + ps * RPP * CFG::TROW;
          }
          st.eoff = st.active ? ((long long)gm * p.s_cm + gc) * 2 : safe_off;
          if constexpr (NP > 0) {
#pragma unroll
            for (int i = 0; i < NP; ++i) st.pv[i] = __builtin_nontemporal_load((const u32x4_t*)(pb[i] + st.eoff));
          }
          st.own = *(const LDS_AS u32x4_t*)(LDS_AS char*)(smem + lds_off);
        };
        // ... and its second half: the fp32 sum in ascending rank order from the own value, one cast, the stores.
        auto finish = [&](const Pass& st) {
          float sum[8];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            sum[2 * e] = Out::to_float((unsigned short)(st.own[e] & 0xFFFF));
            sum[2 * e + 1] = Out::to_float((unsigned short)(st.own[e] >> 16));
          }
          auto add_peer = [&](const u32x4_t& v) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              sum[2 * e] += Out::to_float((unsigned short)(v[e] & 0xFFFF));
              sum[2 * e + 1] += Out::to_float((unsigned short)(v[e] >> 16));
            }
            if (ref_chain) {
#pragma unroll
              for (int e = 0; e < 8; ++e) sum[e] = Out::to_float(Out::from_float(sum[e]));
            }
          };
          if constexpr (NP > 0) {
#pragma unroll
            for (int i = 0; i < NP; ++i) add_peer(st.pv[i]);
          } else if constexpr (NP < 0) {
            for (int pr = 0; pr < p.world; ++pr)
              if (pr != p.rank) add_peer(__builtin_nontemporal_load((const u32x4_t*)(in_slot(aux_own, pr) + st.eoff)));
          }
          u32x4_t res;
#pragma unroll
          for (int e = 0; e < 4; ++e) res[e] = Out::pack(sum[2 * e], sum[2 * e + 1]);
          if (st.active) {
            if (p.epi == EPI_TWO_SHOT) {
              __builtin_nontemporal_store(res, (u32x4_t*)(c_own + st.eoff));
              for (int pr = 0; pr < p.world; ++pr)
                if (pr != p.rank) __builtin_nontemporal_store(res, (u32x4_t*)(in_slot(c_own, pr) + st.eoff));
            } else {
              const int dst = p.all_owners ? st.owner : p.rank;
              __builtin_nontemporal_store(res, (u32x4_t*)((dst == p.rank ? c_own : in_slot(c_own, dst)) + st.eoff));
            }
          }
        };
        if constexpr (NW == 8 && NP >= 4 && ONE_ROUND) {
          // Eight-wave tile with many peers, one tile per workgroup: the passes run as a pipeline of DEPTH
          // stages - the loads of the next pass are on their way while one pass is summed and stored - so
          // that the bytes a CU has in flight do not fall to zero between groups of passes (4096 x 4096 x 1376
          // with seven peers: 92.9 -> 90.8 us against groups of two passes; three stages spill and gain
          // nothing more).  Looping workgroups keep the groups: their launches run 1-7 % slower with the
          // pipeline (fp8 16384 x 8192 x 1024: 494 -> 501 us with two stages, 527 with three) - a CU takes
          // no more than about 39 GB/s of such loads however many are in flight, and the steadier stream
          // of one workgroup only takes bandwidth from the others that are streaming at the time.  The
          // four-wave tiles gain nothing from a pipeline of four stages either (-2 to +3 % over ten shapes).
          constexpr int DEPTH = IRIS_HIP_EPILOGUE_DEPTH;
          const int last = RECT ? npasses : min(PASSES, cdiv(p.M - m0, RPP));  // passes below the last row of the matrix are skipped
          Pass st[DEPTH];
#pragma unroll
          for (int d = 0; d < DEPTH; ++d)
            if (d < last) issue(d, st[d]);
          for (int ps = 0; ps < last; ps += DEPTH) {
#pragma unroll
            for (int d = 0; d < DEPTH; ++d) {
              if (ps + d < last) {
                finish(st[d]);
                if (ps + d + DEPTH < last) issue(ps + d + DEPTH, st[d]);
              }
            }
          }
        } else {
          // Passes whose loads are issued together.  Every group is one memory round trip (2 us on a
          // launch of 10-20 us), so the four-wave tiles, which have the registers, take four passes
          // at a time also with seven peers, and groups below the last row of the matrix are skipped.
          constexpr int G0 = (NP >= 4 && NW == 8) ? 2 : 4;
          constexpr int G = G0 < PASSES ? G0 : PASSES;
          static_assert(PASSES % G == 0, "pass grouping");
          for (int pg = 0; pg < npasses; pg += G) {
            if (!RECT && m0 + pg * RPP >= p.M) break;
            Pass st[G];
#pragma unroll
            for (int g = 0; g < G; ++g) issue(pg + g, st[g]);
#pragma unroll
            for (int g = 0; g < G; ++g) finish(st[g]);
          }
        }
      };
      // Variants with tile owners (two-shot, reduce-scatter): only the flag tiles this rank owns are
      // reduced, and a kernel tile may hold none, one or several of them.  When the flag tiles are
      // large enough to keep the workgroup busy, each owned one is streamed as a rectangle by all
      // threads, and a kernel tile without an owned flag tile issues nothing at all; with small flag
      // tiles the threads keep their places in the kernel tile and the stores are predicated.
      auto reduce_tile = [&](auto np_tag) {
        const int m1 = min(m0 + BM, p.M), n1 = min(n0 + BN, p.N);
        const bool by_rect = p.epi != EPI_ONE_SHOT && min(p.flag_bm, BM) * (min(p.flag_bn, BN) / 8) * 2 >= NT;
        if (!by_rect) {
          reduce_chunks(np_tag, std::false_type{}, 0, 0, 0, 0, 0);
          return;
        }
        for (int fr = m0 / p.flag_bm; fr * p.flag_bm < m1; ++fr)
          for (int fc = n0 / p.flag_bn; fc * p.flag_bn < n1; ++fc) {
            const int owner = owner_of(p.epi, fr * ftn + fc, ftotal, p.world, p.rank);
            if (!p.all_owners && owner != p.rank) continue;
            const int r0 = max(m0, fr * p.flag_bm), r1 = min(m1, (fr + 1) * p.flag_bm);
            const int c0 = max(n0, fc * p.flag_bn), c1 = min(n1, (fc + 1) * p.flag_bn);
            reduce_chunks(np_tag, std::true_type{}, r0, r1, c0, (c1 - c0) / 8, owner);
          }
      };
      switch (solo ? -2 : (p.world <= kMaxCachedSlots ? npeers : -1)) {
        case -2: break;  // C was written in phase 1
        case 1: reduce_tile(std::integral_constant<int, 1>{}); break;
        case 3: reduce_tile(std::integral_constant<int, 3>{}); break;
        case 7: reduce_tile(std::integral_constant<int, 7>{}); break;
        default: reduce_tile(std::integral_constant<int, -1>{}); break;
      }
    }
    PHASE_STAMP(7);
#ifdef IRIS_HIP_PHASE_STAMPS
    wait_vmcnt<0>();
    PHASE_STAMP(8);
#endif
    // Staging shares LDS with the operand ring of the next tile: every wave must be done reading it.
    // A bare barrier - __syncthreads() would also wait for this tile's global stores to be
    // acknowledged (1-4 us), which nothing here depends on; they drain behind the next tile's
    // first loads, or behind the end of the kernel.
    __builtin_amdgcn_s_waitcnt((0xF) | (0x3 << 14) | (0x7 << 4));  // lgkmcnt(0), vmcnt and expcnt free
    __builtin_amdgcn_s_barrier();
  }
}

// ------------------------------------------------------------------------------------------------
// Launch of the MFMA kernel
// ------------------------------------------------------------------------------------------------
template <class CFG, bool ONE_ROUND, bool STREAMK = false>
int launch_mfma_grid(const FusedParams& p, int device, int grid, hipStream_t stream) {
  // The dynamic-LDS limit is a per-device attribute of the kernel: set it once on every device used
  // (atomic flags: two host threads may both set it, which is harmless, but neither skips it).
  static std::atomic<bool> attr_set[64];
  if (device < 0 || device >= 64) return iris_host::fail("device index %d out of range", device);
  if (!attr_set[device].load(std::memory_order_acquire)) {
    hipError_t e = hipFuncSetAttribute((const void*)fused_mfma_kernel<CFG, ONE_ROUND, STREAMK>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, CFG::SMEM_BYTES);
    if (e != hipSuccess) return (int)e;
    attr_set[device].store(true, std::memory_order_release);
  }
  hipLaunchKernelGGL((fused_mfma_kernel<CFG, ONE_ROUND, STREAMK>), dim3(grid), dim3(CFG::NT), CFG::SMEM_BYTES, stream, p);
  return (int)hipGetLastError();
}

// Tail policy of the eight-wave tile (the STREAMK builds of the kernel): worth it when the last round of
// workgroups would leave a good part of the chip without a tile for many K steps.  Returns the grid to
// launch (every CU, a multiple of the XCD count) or 0 when tiles are better handed out whole.
//   iris_hip_set_split_tiles(0) / IRIS_HIP_STREAMK=0 never splits, 1 splits whenever the last round is
//   not full and has at least 4 K steps, -1 (default) decides by the rule below.  Results differ from the unsplit launch only in
//   the order of the fp32 sums over K.
template <class CFG>
int split_tile_grid(FusedParams& p, int total, int cu_count) {
  if constexpr (CFG::NW != 8) return 0;
  const int mode = iris_host::split_tile_mode();
  if (mode == 0 || p.no_workspace_alloc || p.num_xcd < 1) return 0;
  const int grid = cu_count - cu_count % p.num_xcd;
  if (grid < p.num_xcd) return 0;
  const int wg_per_xcd = grid / p.num_xcd;
  const int span = cdiv(total, p.num_xcd);     // tiles of an XCD (the last one may have fewer)
  const int left = span % wg_per_xcd;          // tiles of its last, partly filled round
  if (left == 0) return 0;
  const int nsrc = p.gather == GATHER_K ? p.world : 1;
  const int nsteps = nsrc * cdiv(p.gather == GATHER_K ? p.K_local : p.K, CFG::BK);
  // Mode 1 plans without the costs of passing partial sums on: whatever can be split is split.
  p.sk_gather_cost = mode == 1 ? 0 : kSplitGatherCost;
  p.sk_pass_cost = mode == 1 ? 0 : kSplitPassCost;
  const SplitPlan plan = split_plan(left, wg_per_xcd, nsteps, p.sk_gather_cost, p.sk_pass_cost);
  if (plan.per_tile == 0) return 0;
  if (mode == 1 || mode == 2) return grid;  // 2: whatever the plan expects any gain from (a tuning aid)
  // Worth it when the split round is at least 16 K steps (12 us) and an eighth shorter than a whole tile.
  const int steps = split_round_steps(plan, nsteps);
  return (nsteps - steps >= 16 && (nsteps - steps) * 8 >= nsteps) ? grid : 0;
}

template <class CFG>
int launch_mfma(const FusedParams& p, int device, int cu_count, hipStream_t stream, const char* name) {
  const int total = p.tiles_m * p.tiles_n;
  const int cap = cu_count * CFG::WG_PER_CU;
  // A multiple of the XCD count keeps the XCD mapping exact.  Rounded up when the tiles fit in one
  // round (the surplus workgroups find no tile and leave), so that no tile waits for a second round.
  int grid = total < cap ? total : cap;
  if (grid % p.num_xcd) {
    const int up = grid + p.num_xcd - grid % p.num_xcd;
    grid = up <= cap ? up : grid - grid % p.num_xcd;
  }
  if (grid < 1) grid = 1;
  iris_host::set_last_kernel(name);
  const bool uneven_tiles = p.epi == EPI_TWO_SHOT || (p.epi == EPI_REDUCE_SCATTER && !p.all_owners);
  const bool per_tile_launch = uneven_tiles && p.world > 1 && p.sum_peers && total > grid;
  if constexpr (CFG::NW == 8) {
    FusedParams q = p;
    const int sk_grid = per_tile_launch ? 0 : split_tile_grid<CFG>(q, total, cu_count);
    if (sk_grid > 0) {
      q.interleave = 0;  // the plan hands out the last round of every XCD's span
      q.tile_rotate = 0;
      q.group_m = q.group_m_spans;
      constexpr long long slot_bytes = (long long)CFG::MB * CFG::NB * 4 * CFG::NT * 16;
      // No workspace (the stream is being captured before its first split launch, or the device has
      // used up its workspaces): hand the tiles out whole.
      if (iris_host::split_tile_workspace(device, stream, sk_grid, slot_bytes, &q.sk_partials, &q.sk_flags, &q.sk_epoch) == 0) {
        char sk_name[112];
        snprintf(sk_name, sizeof(sk_name), "%s_splitk", name);
        iris_host::set_last_kernel(sk_name);
        return launch_mfma_grid<CFG, false, true>(q, device, sk_grid, stream);
      }
    }
  }
  if (total <= grid) return launch_mfma_grid<CFG, true>(p, device, grid, stream);
  // More tiles than workgroups that fit at once: normally the resident workgroups loop over the tiles.
  // The two-shot all-reduce does better with one workgroup per tile, handed out by the hardware as CUs
  // free up (measured at W = 8: 16384x4096x1376 322 -> 273 us, 8192x8192x2752 461 -> 417 us,
  // 8192x8192x8192 1059 -> 1009 us); the one-shot variant does worse that way (+3-7 %), launches
  // without peers do not care.  The same goes for a reduce-scatter whose rank owns one block of
  // rows: the few tiles that carry the slot sum take half as long again as the others, and a fixed
  // tile-to-workgroup assignment gives some workgroups two of them.
  if (per_tile_launch) {
    int per_tile = total;
    if (per_tile % p.num_xcd) per_tile += p.num_xcd - per_tile % p.num_xcd;
    return launch_mfma_grid<CFG, true>(p, device, per_tile, stream);
  }
  return launch_mfma_grid<CFG, false>(p, device, grid, stream);
}

// Tile shapes of the MFMA kernel (run_fused picks one per launch).
//   big       256x256, 8 waves, 64-byte K steps, 4-slot ring: half the operand bytes per flop of the
//             128x128 tiles; from about half the CUs busy.
//   small     128x128, 4 waves, 128-byte K steps, 4-slot ring: too few big tiles.
//   small2    128x128, 4 waves, 64-byte K steps, 64 KiB ring, two workgroups per CU: more 128x128 tiles
//             than CUs (every tile resident at once instead of a half-empty second round).
//   skinny    64x128, 4 waves, 128-byte K steps, 72 KiB ring, two workgroups per CU: at most 64 rows, or at
//             most two such tiles per CU with a short K.
//   skinny64  64x64, 4 waves of one 32x32 block, 128-byte K steps, 64 KiB ring, two workgroups per CU: at
//             most two such tiles per CU.
// For the small tiles residency - every tile of the output on a CU at once - pays before fat K steps.
enum { TILE_BIG = 0, TILE_SMALL = 1, TILE_SKINNY = 2, TILE_SMALL2 = 3, TILE_DECODE = 4, TILE_SKINNY64 = 5 };
constexpr int tile_bk(int kind, int in) {  // K elements per step
  return (kind == TILE_BIG || kind == TILE_SMALL2 ? 64 : 128) / (in == IN_FP8 ? 1 : 2);
}
template <int IN, bool BKC>
using BigTile = MfmaCfg<IN, 256, 256, tile_bk(TILE_BIG, IN), 2, 4, 4, BKC>;
template <int IN, bool BKC>
using SmallTile = MfmaCfg<IN, 128, 128, tile_bk(TILE_SMALL, IN), 2, 2, 4, BKC>;
template <int IN, bool BKC>
using SkinnyTile = MfmaCfg<IN, 64, 128, tile_bk(TILE_SKINNY, IN), 2, 2, 3, BKC>;
template <int IN, bool BKC>
using Small2Tile = MfmaCfg<IN, 128, 128, tile_bk(TILE_SMALL2, IN), 2, 2, 4, BKC>;
template <int IN, bool BKC>
using Skinny64Tile = MfmaCfg<IN, 64, 64, tile_bk(TILE_SKINNY64, IN), 2, 2, 4, BKC>;

inline int tile_rows(int kind) {
  return kind == TILE_BIG ? 256 : (kind == TILE_SKINNY || kind == TILE_SKINNY64) ? 64 : kind == TILE_DECODE ? 32 : 128;
}
inline int tile_cols(int kind) { return kind == TILE_BIG ? 256 : kind == TILE_DECODE ? 32 : kind == TILE_SKINNY64 ? 64 : 128; }

#include "decode_kernel.h"

template <int IN>
int dispatch_mfma_in(FusedParams& p, int kind, bool bkc, int device, int cu, hipStream_t s) {
  const int bm = tile_rows(kind), bn = tile_cols(kind);
  if (kind == TILE_DECODE) {
    static const char* tnames[3] = {"bf16", "f16", "fp8"};
    char dname[96];
    // More tiles than CUs: half the K per chunk, so that a workgroup's LDS (80 KiB) lets two share a CU
    // and the whole output is in flight at once instead of in two rounds (fp16, eight ranks, 64x8192x512
    // 13.8 -> 9.3 us, 128x4096x4096 27.3 -> 24.5 us).  Also when K is at most two such chunks: every load
    // is in flight from the start either way, and the first MFMA waits for half as many bytes (0.3 us).
    const int kbytes = p.K * (IN == IN_FP8 ? 1 : 2);
    const bool halves = (long long)cdiv(p.M, 32) * cdiv(p.N, 32) > cu || kbytes <= 1024;
    const int chunk = halves ? DecodeCfg<IN, false, 128>::CHUNK : DecodeCfg<IN, false, 256>::CHUNK;
    snprintf(dname, sizeof(dname), "mfma_%s_32x32x%d_%s", tnames[IN], chunk, bkc ? "nt" : "nn");
    if (halves) return bkc ? launch_decode<IN, true, 128>(p, device, s, dname) : launch_decode<IN, false, 128>(p, device, s, dname);
    return bkc ? launch_decode<IN, true, 256>(p, device, s, dname) : launch_decode<IN, false, 256>(p, device, s, dname);
  }
  p.tiles_m = cdiv(p.M, bm);
  p.tiles_n = cdiv(p.N, bn);
  // Group height: tile-rows walked together so that the tiles an XCD works on at one time - its whole
  // span, or one round of it when the span is longer than its resident workgroups - are close to a
  // square (fewest operand panels per L2).
  const int span = cdiv(p.tiles_m * p.tiles_n, p.num_xcd);
  const int resident = (cu / p.num_xcd) * (kind == TILE_BIG || kind == TILE_SMALL ? 1 : 2);
  const bool rounds = span > resident;
  const int at_once = rounds ? resident : span;
  int g = 1;
  while (g * g * 2 <= at_once && g * 2 <= p.tiles_m) g *= 2;
  // Two-shot launches of several rounds (one workgroup per tile, handed out in this order) do better with
  // groups of at most four rows (eight ranks, fp16: 16384x3584x8192 1006 -> 977 us, 8192x8192x2752 441 -> 428).
  if (rounds && p.sum_peers && p.world > 1 && p.epi == EPI_TWO_SHOT) g = g < 4 ? g : 4;
  // A reduce-scatter rank sums the slots only for its own band of rows.  With XCD spans that are
  // close to square that band falls to one or two XCDs, whose CUs then carry all the slow tiles;
  // taller groups spread it over more XCDs at the price of more operand panels per L2
  // (8192 x 4096 x 1376, 8 ranks, seven peers, on one box: 131 us at the default height 8, 114 at
  // 16, 119 at 32; fetched by the L2s: 207, 290 and 443 MB).
  if (p.epi == EPI_REDUCE_SCATTER && !p.all_owners && p.sum_peers && p.world > 1)
    g = g * 2 < p.tiles_m ? g * 2 : p.tiles_m;
  p.interleave = 0;
  p.tile_rotate = 0;
  // Launches whose epilogue streams whole tiles from or to every rank - the one-shot all-reduce with peers
  // spends half its time reading the peers' tiles, matmul_all_gather and the atomic variant write every
  // tile into all slots - want the workgroups that run together to touch long pieces of the same rows
  // (DRAM pages stay open): flat groups of two rows - more for narrow outputs, so that g x tiles_n stays
  // near 32 (64 with two workgroups per CU) and an L2 still sees as few operand panels as with a square
  // span.  When the launch fills at least three quarters of the chip the grouped order is also dealt out
  // workgroup by workgroup instead of in one span per XCD: XCD x then holds the tiles at positions x modulo
  // the XCD count, 1/g of the rows and g/8 of the columns of one band of rows that the whole chip works on.
  // Measured, eight ranks, one box, square spans -> this rule; one-shot: fp8 16384x8192x1024 568 -> 496 us
  // (520 with flat spans), bf16 8192x4096x1376 216 -> 194, 4096x4096x1376 98.0 -> 96.8, 2048x8192x1376
  // 108 -> 99, 2048x4096x1376 (128x128 tiles) 64.6 -> 60.4, 256x4096x4096 (64x64 tiles, chip half full:
  // spans) 39.3 -> 32.2; atomic fp16 8192x4096x1376 566 -> 520; matmul_all_gather fp16 2048x3584x8192
  // 175 -> 168, 512x4096x1376 22.9 -> 21.4.  Dealt out with one-row groups or spans of eight rows are the
  // outliers (+9 % on 1536x6144x2048), and a chip that is little more than half full does better with spans
  // (3072x3072x1024: 67.9 against 70.6).  Two-shot launches lose 3-5 % when dealt out; launches that
  // neither read nor write other ranks' tiles do not care.
  const bool streams_tiles = p.world > 1 && ((p.epi == EPI_ONE_SHOT && p.sum_peers) || p.epi == EPI_ALL_GATHER || p.epi == EPI_ATOMIC);
  if (streams_tiles) {
    const int two_per_cu = !(kind == TILE_BIG || kind == TILE_SMALL);
    g = 2;
    while (g < 8 && g * 2 * p.tiles_n <= (two_per_cu ? 64 : 32)) g *= 2;
    while (g > p.tiles_m && g > 1) g /= 2;
    p.interleave = (long long)p.tiles_m * p.tiles_n * 4 >= (long long)resident * p.num_xcd * 3;
  }
  p.group_m_spans = g;
  // The reduce-scatter with peers is dealt out as well (its launches hand one workgroup per tile to the
  // hardware in this order), starting with the band of rows this rank sums: those tiles take half as long
  // again as the others, so they go first and spread over every XCD (8192x4096x1376, eight ranks, rank 0:
  // 111.8 -> 106.6 us against spans of sixteen rows).
  const bool rs_band = p.epi == EPI_REDUCE_SCATTER && !p.all_owners && p.sum_peers && p.world > 1;
  if (rs_band) {
    p.interleave = 1;
    g = p.tiles_m >= 2 ? 2 : 1;
    const int ftn = cdiv(p.N, p.flag_bn), ftotal = cdiv(p.M, p.flag_bm) * ftn;
    const int band_row = (p.rank * (ftotal / p.world)) / ftn * p.flag_bm / bm;  // first tile row of the rank's band
    p.tile_rotate = band_row / g * g * p.tiles_n;
  }
  static const int forced_order = [] {
    const char* e = getenv("IRIS_HIP_TILE_ORDER");  // "spans" or "dealt": a tuning aid
    return !e ? -1 : (e[0] == 'd' ? 1 : 0);
  }();
  if (forced_order >= 0) p.interleave = forced_order;
  if (!p.interleave) {
    if (rs_band) g = p.group_m_spans;
    p.tile_rotate = 0;
  }
  // IRIS_HIP_GROUP_M overrides the group height (a tuning aid; results do not depend on the tile order).
  static const int forced_group_m = [] { const char* e = getenv("IRIS_HIP_GROUP_M"); return e ? atoi(e) : 0; }();
  if (forced_group_m > 0) {
    g = forced_group_m < p.tiles_m ? forced_group_m : p.tiles_m;
    p.group_m_spans = g;
  }
  p.group_m = g;
  static const char* names[3] = {"bf16", "f16", "fp8"};
  char name[96];
  snprintf(name, sizeof(name), "mfma_%s_%dx%dx%d_%s", names[IN], bm, bn, tile_bk(kind, IN), bkc ? "nt" : "nn");
  switch (kind) {
    case TILE_BIG:
      return bkc ? launch_mfma<BigTile<IN, true>>(p, device, cu, s, name) : launch_mfma<BigTile<IN, false>>(p, device, cu, s, name);
    case TILE_SMALL:
      return bkc ? launch_mfma<SmallTile<IN, true>>(p, device, cu, s, name) : launch_mfma<SmallTile<IN, false>>(p, device, cu, s, name);
    case TILE_SMALL2:
      return bkc ? launch_mfma<Small2Tile<IN, true>>(p, device, cu, s, name) : launch_mfma<Small2Tile<IN, false>>(p, device, cu, s, name);
    case TILE_SKINNY64:
      return bkc ? launch_mfma<Skinny64Tile<IN, true>>(p, device, cu, s, name) : launch_mfma<Skinny64Tile<IN, false>>(p, device, cu, s, name);
    default:
      return bkc ? launch_mfma<SkinnyTile<IN, true>>(p, device, cu, s, name) : launch_mfma<SkinnyTile<IN, false>>(p, device, cu, s, name);
  }
}
