// Stand-alone collectives over the symmetric heap (all-reduce, reduce-scatter): the rank-local part
// of iris/ccl/triton/all_reduce.py and iris/ccl/triton/reduce_scatter.py as one streaming kernel.
//
// These are pure HBM kernels: every output element is the sum of W input elements that sit at the
// same heap offset in W slots.  The kernel walks a flat index space of 16-byte chunks (or single
// elements when the operands are not 16-byte friendly), W loads in flight per chunk and several
// chunks per thread, fp32 sums, one cast, 16-byte stores.
//
// What the reference fixes, and this kernel reproduces element for element:
//   * which tiles a rank reduces (two-shot distributions, iris/ccl/triton/all_reduce.py:620-633),
//   * the grouped tile order that turns a tile id into tile coordinates (:639-644),
//   * the order of the fp32 additions: ascending group index from zero for one-shot (:403-414),
//     cyclic from (j mod comm_sms) mod W for the j-th owned tile of two-shot (:663-669),
//   * where results go: own output (one-shot, reduce-scatter), every rank's output (two-shot),
//     atomic adds into every rank's output (atomic, :212-233).
// How the work is spread over workgroups is free and is chosen for bandwidth, not copied.

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include <type_traits>

#include "iris_hip.h"
#include "layout.h"
#include "device_util.h"
#include "host_common.h"

using namespace iris_layout;

namespace {

enum { CCL_ONE_SHOT = 0, CCL_TWO_SHOT = 1, CCL_REDUCE_SCATTER = 2, CCL_ATOMIC = 3 };

constexpr int kCclThreads = 256;
constexpr int kMaxGroup = 64;  // ranks of one group whose slot offsets are cached in LDS

struct CclParams {
  const char* in;
  char* out;
  int M, N;
  long long s_im, s_in, s_om, s_on;  // element strides
  const long long* heap_bases;
  int group_rank, iris_rank, world, rank_start, rank_stride;
  int mode;
  // Tile grid the ownership and the summation order are defined on.
  int bm, bn, tiles_m, tiles_n, group_m, comm_sms;
  // Owned tiles: ids first_tile + j * tile_stride, j in [0, n_owned).
  int first_tile, tile_stride, n_owned;
  // Work decomposition: a tile is cut into `upt` units (units per tile), `upr` of them per tile row.
  int upr, upt;
  long long total_units;
};

// Tile coordinates of tile id `t` in the grouped order (group_m tile-rows are walked column by
// column before moving on; iris/ccl/triton/all_reduce.py:639-644).
__device__ __forceinline__ void grouped_coords(int t, int tiles_m, int tiles_n, int group_m, int& pm, int& pn) {
  const int per_group = group_m * tiles_n;
  const int g = t / per_group;
  const int first = g * group_m;
  const int gsize = min(tiles_m - first, group_m);
  const int in_group = t - g * per_group;
  pm = first + in_group % gsize;
  pn = in_group / gsize;
}

typedef __attribute__((ext_vector_type(4))) unsigned ccl_u32x4_t;

// 16-byte accesses; NT marks data that is touched once (launches too large to stay in the
// last-level cache), which keeps it from displacing other lines on its way through.
template <bool NT>
__device__ __forceinline__ ccl_u32x4_t load16(const char* p) {
  if constexpr (NT) return __builtin_nontemporal_load((const ccl_u32x4_t*)p);
  else return *(const ccl_u32x4_t*)p;
}
template <bool NT>
__device__ __forceinline__ void store16(char* p, ccl_u32x4_t v) {
  if constexpr (NT) __builtin_nontemporal_store(v, (ccl_u32x4_t*)p);
  else *(ccl_u32x4_t*)p = v;
}

template <class E, int VEC>
struct Chunk;  // VEC elements of type E, moved with one memory instruction

template <class E>
struct Chunk<E, 1> {
  float v[1];
  template <bool NT> __device__ __forceinline__ void load(const char* p) { v[0] = E::load(p); }
  template <bool NT> __device__ __forceinline__ void store(char* p) const { E::store(p, v[0]); }
  __device__ __forceinline__ void atomic_add_to(char* p) const { E::atomic_add(p, v[0]); }
};

template <class E>
struct Chunk<E, 2> {  // two 16-bit elements: the unit of the packed atomics
  float v[2];
  template <bool NT> __device__ __forceinline__ void load(const char* p) {
    const unsigned w = *(const unsigned*)p;
    unsigned short lo = (unsigned short)(w & 0xFFFFu), hi = (unsigned short)(w >> 16);
    v[0] = E::load((const char*)&lo);
    v[1] = E::load((const char*)&hi);
  }
  __device__ __forceinline__ unsigned pack() const {
    unsigned short lo, hi;
    E::store((char*)&lo, v[0]);
    E::store((char*)&hi, v[1]);
    return (unsigned)lo | ((unsigned)hi << 16);
  }
  template <bool NT> __device__ __forceinline__ void store(char* p) const { *(unsigned*)p = pack(); }
  __device__ __forceinline__ void atomic_add_to(char* p) const {
    using Out = typename std::conditional<E::kFp32SumInReference, OutF16, OutBF16>::type;
    atomic_add_packed<Out>(p, pack());
  }
};

template <class E>
struct Chunk<E, 8> {  // eight 16-bit elements
  float v[8];
  template <bool NT> __device__ __forceinline__ void load(const char* p) {
    const ccl_u32x4_t w = load16<NT>(p);
    const unsigned u[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      unsigned short lo = (unsigned short)(u[i] & 0xFFFFu), hi = (unsigned short)(u[i] >> 16);
      v[2 * i] = E::load((const char*)&lo);
      v[2 * i + 1] = E::load((const char*)&hi);
    }
  }
  __device__ __forceinline__ void pack(unsigned (&u)[4]) const {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      unsigned short lo, hi;
      E::store((char*)&lo, v[2 * i]);
      E::store((char*)&hi, v[2 * i + 1]);
      u[i] = (unsigned)lo | ((unsigned)hi << 16);
    }
  }
  template <bool NT> __device__ __forceinline__ void store(char* p) const {
    unsigned u[4];
    pack(u);
    store16<NT>(p, (ccl_u32x4_t){u[0], u[1], u[2], u[3]});
  }
  __device__ __forceinline__ void atomic_add_to(char* p) const {
    unsigned u[4];
    pack(u);
    using Out = typename std::conditional<E::kFp32SumInReference, OutF16, OutBF16>::type;
#pragma unroll
    for (int i = 0; i < 4; ++i) atomic_add_packed<Out>(p + 4 * i, u[i]);
  }
};

template <>
struct Chunk<ElemF32, 4> {
  float v[4];
  template <bool NT> __device__ __forceinline__ void load(const char* p) {
    const ccl_u32x4_t w = load16<NT>(p);
    v[0] = __uint_as_float(w.x); v[1] = __uint_as_float(w.y); v[2] = __uint_as_float(w.z); v[3] = __uint_as_float(w.w);
  }
  template <bool NT> __device__ __forceinline__ void store(char* p) const {
    store16<NT>(p, (ccl_u32x4_t){__float_as_uint(v[0]), __float_as_uint(v[1]), __float_as_uint(v[2]), __float_as_uint(v[3])});
  }
  __device__ __forceinline__ void atomic_add_to(char* p) const {
#pragma unroll
    for (int i = 0; i < 4; ++i) atomicAdd((float*)p + i, v[i]);
  }
};

// E: element traits.  VEC: elements per memory access (1 = any strides).  WCT: compile-time group
// size (0 = run-time loop).  UPT: units (chunks) per thread and iteration.  NT: non-temporal accesses.
template <class E, int VEC, int WCT, int UPT, bool NT>
__global__ void __launch_bounds__(kCclThreads) slot_reduce_kernel(const CclParams p) {
  // Byte offset of every group member's slot relative to the own slot.
  __shared__ long long slot_delta[kMaxGroup];
  for (int i = threadIdx.x; i < p.world && i < kMaxGroup; i += kCclThreads) {
    const int r = p.rank_start + i * p.rank_stride;
    slot_delta[i] = p.heap_bases ? p.heap_bases[r] - p.heap_bases[p.iris_rank] : 0ll;
  }
  __syncthreads();
  auto delta = [&](int i) -> long long {
    if (i < kMaxGroup) return slot_delta[i];
    const int r = p.rank_start + i * p.rank_stride;
    return p.heap_bases[r] - p.heap_bases[p.iris_rank];
  };
  const int W = WCT ? WCT : p.world;
  const bool tiled = (p.mode == CCL_TWO_SHOT || p.mode == CCL_REDUCE_SCATTER);

  const long long span = (long long)gridDim.x * kCclThreads * UPT;
  for (long long base = (long long)blockIdx.x * kCclThreads * UPT; base < p.total_units; base += span) {
    long long in_off[UPT], out_off[UPT];
    int start[UPT];
    bool live[UPT];
#pragma unroll
    for (int u = 0; u < UPT; ++u) {
      const long long g = base + (long long)u * kCclThreads + threadIdx.x;
      live[u] = g < p.total_units;
      const long long gg = live[u] ? g : 0;
      int j, c;  // which owned tile, which unit inside it
      if (p.total_units < (1ll << 31)) {
        j = (int)((unsigned)gg / (unsigned)p.upt);
        c = (int)((unsigned)gg - (unsigned)j * (unsigned)p.upt);
      } else {
        j = (int)(gg / p.upt);
        c = (int)(gg - (long long)j * p.upt);
      }
      int pm, pn;
      if (tiled) {
        grouped_coords(p.first_tile + j * p.tile_stride, p.tiles_m, p.tiles_n, p.group_m, pm, pn);
        start[u] = (j % p.comm_sms) % W;
      } else {
        pm = j / p.tiles_n;
        pn = j - pm * p.tiles_n;
        start[u] = 0;
      }
      const int row = pm * p.bm + c / p.upr;
      const int col = pn * p.bn + (c % p.upr) * VEC;
      live[u] = live[u] && row < p.M && col < p.N;
      in_off[u] = ((long long)row * p.s_im + (long long)col * p.s_in) * E::size;
      out_off[u] = ((long long)row * p.s_om + (long long)col * p.s_on) * E::size;
    }

    if (p.mode == CCL_ATOMIC) {
#pragma unroll
      for (int u = 0; u < UPT; ++u) {
        if (!live[u]) continue;
        Chunk<E, VEC> x;
        x.template load<NT>(p.in + in_off[u]);
        for (int i = 0; i < W; ++i) x.atomic_add_to(p.out + out_off[u] + delta(i));
      }
      continue;
    }

    if constexpr (WCT != 0) {
      // All W x UPT loads are issued before the first add.
      Chunk<E, VEC> x[UPT][WCT];
#pragma unroll
      for (int u = 0; u < UPT; ++u) {
#pragma unroll
        for (int i = 0; i < WCT; ++i) {
          int src = start[u] + i;
          if (src >= WCT) src -= WCT;
          // Dead lanes read the own chunk 0, which always exists.
          x[u][i].template load<NT>(p.in + (live[u] ? in_off[u] + delta(src) : 0ll));
        }
      }
#pragma unroll
      for (int u = 0; u < UPT; ++u) {
        Chunk<E, VEC> acc;
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
          // one-shot starts from +0 (the reference's zero-filled accumulator), two-shot from the
          // first slot's value
          float a = tiled ? x[u][0].v[e] : 0.0f + x[u][0].v[e];
#pragma unroll
          for (int i = 1; i < WCT; ++i) a += x[u][i].v[e];
          acc.v[e] = a;
        }
        if (!live[u]) continue;
        if (p.mode == CCL_TWO_SHOT) {
#pragma unroll
          for (int i = 0; i < WCT; ++i) acc.template store<NT>(p.out + out_off[u] + delta(i));
        } else {
          acc.template store<NT>(p.out + out_off[u]);
        }
      }
    } else {
#pragma unroll
      for (int u = 0; u < UPT; ++u) {
        if (!live[u]) continue;
        Chunk<E, VEC> acc;
        for (int i = 0; i < W; ++i) {
          int src = start[u] + i;
          if (src >= W) src -= W;
          Chunk<E, VEC> x;
          x.template load<NT>(p.in + in_off[u] + delta(src));
#pragma unroll
          for (int e = 0; e < VEC; ++e) acc.v[e] = (i == 0) ? (tiled ? x.v[e] : 0.0f + x.v[e]) : acc.v[e] + x.v[e];
        }
        if (p.mode == CCL_TWO_SHOT) {
          for (int i = 0; i < W; ++i) acc.template store<NT>(p.out + out_off[u] + delta(i));
        } else {
          acc.template store<NT>(p.out + out_off[u]);
        }
      }
    }
  }
}

template <class E, int VEC, int UPT, bool NT>
void launch_for_world(const CclParams& p, int grid, hipStream_t s) {
#define CCL_KERNEL(W, U) hipLaunchKernelGGL((slot_reduce_kernel<E, VEC, W, U, NT>), dim3(grid), dim3(kCclThreads), 0, s, p)
  switch (p.mode == CCL_ATOMIC ? 0 : p.world) {
    case 1: CCL_KERNEL(1, UPT); break;
    case 2: CCL_KERNEL(2, UPT); break;
    case 4: CCL_KERNEL(4, UPT); break;
    case 8: CCL_KERNEL(8, UPT); break;
    default: CCL_KERNEL(0, 1); break;
  }
#undef CCL_KERNEL
}

bool aligned16(const void* q) { return ((uintptr_t)q & 15) == 0; }

int run_ccl(CclParams p, int distribution, int dtype, void* stream) {
  using iris_host::fail;
  iris_host::clear_last_error();
  if (p.M <= 0 || p.N <= 0) return fail("M and N must be positive (got %d, %d)", p.M, p.N);
  if (!p.in || !p.out) return fail("input and output must not be NULL");
  if (p.world < 1 || p.group_rank < 0 || p.group_rank >= p.world)
    return fail("bad group_rank/world_size %d/%d", p.group_rank, p.world);
  if (p.rank_start < 0 || p.rank_stride < 1 || p.iris_rank < 0)
    return fail("bad rank_start/rank_stride/iris_rank %d/%d/%d", p.rank_start, p.rank_stride, p.iris_rank);
  if (p.world > 1 && !p.heap_bases) return fail("heap_bases must not be NULL");
  if (p.bm <= 0 || p.bn <= 0 || p.group_m <= 0 || p.comm_sms <= 0)
    return fail("block sizes, swizzle_size and comm_sms must be positive");
  if (distribution != IRIS_HIP_DISTRIBUTION_STRIDED && distribution != IRIS_HIP_DISTRIBUTION_BLOCK)
    return fail("distribution %d is not 0 (strided) or 1 (block)", distribution);
  const int es = dtype == IRIS_HIP_FP32 ? 4 : (dtype == IRIS_HIP_BF16 || dtype == IRIS_HIP_FP16) ? 2 : 0;
  if (!es) return fail("unsupported element type %d", dtype);

  int device = 0, cu = 0, xcc = 0;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) return (int)e;
  int rc = iris_host::device_facts(device, &cu, &xcc);
  if (rc) return rc;

  const bool tiled = (p.mode == CCL_TWO_SHOT || p.mode == CCL_REDUCE_SCATTER);
  const int vec_full = 16 / es;
  // 16-byte accesses need unit-stride rows that start on 16-byte boundaries in every slot (slots are
  // 4 KiB aligned relative to each other) and tiles that are whole chunks wide.
  bool vec_ok = p.s_in == 1 && p.s_on == 1 && aligned16(p.in) && aligned16(p.out) &&
                (p.s_im * es) % 16 == 0 && (p.s_om * es) % 16 == 0 && p.N % vec_full == 0;
  if (tiled && p.bn % vec_full) vec_ok = false;
  int vec = vec_ok ? vec_full : 1;
  // The atomic variant adds one dword at a time (packed 16-bit pairs, or one float): with a dword per
  // thread a wave instruction covers 256 contiguous bytes, two whole lines for the L2's atomic units;
  // with a 16-byte chunk per thread it touched eight lines with eight dwords each and the launch ran
  // at a third of the rate.
  if (p.mode == CCL_ATOMIC && vec_ok) vec = es == 4 ? 1 : 2;

  if (tiled) {
    p.tiles_m = cdiv(p.M, p.bm);
    p.tiles_n = cdiv(p.N, p.bn);
    const long long total = (long long)p.tiles_m * p.tiles_n;
    if (total >= (1ll << 31)) return fail("too many tiles");
    const int per_rank = (int)((total + p.world - 1) / p.world);
    if (distribution == IRIS_HIP_DISTRIBUTION_STRIDED) {
      p.first_tile = p.group_rank;
      p.tile_stride = p.world;
      const long long remaining = total - p.first_tile;
      p.n_owned = remaining > 0 ? (int)((remaining + p.world - 1) / p.world) : 0;
    } else {
      p.first_tile = (int)((long long)p.group_rank * per_rank);
      p.tile_stride = 1;
      const long long remaining = total - p.first_tile;
      p.n_owned = remaining > 0 ? (int)(remaining < per_rank ? remaining : per_rank) : 0;
    }
  } else {
    // No result depends on the tile grid: stream rows in runs of up to 2048 bytes.
    p.bm = 1;
    p.bn = p.N < 2048 / es ? p.N : 2048 / es;
    if (p.bn % vec) p.bn = vec;  // cannot happen with vec == 1; keeps runs whole chunks otherwise
    p.tiles_m = p.M;
    p.tiles_n = cdiv(p.N, p.bn);
    p.first_tile = 0;
    p.tile_stride = 1;
    const long long total = (long long)p.tiles_m * p.tiles_n;
    if (total >= (1ll << 31)) return fail("tensor too large");
    p.n_owned = (int)total;
  }
  p.upr = cdiv(p.bn, vec);
  if ((long long)p.upr * p.bm >= (1ll << 31)) return fail("block sizes %d x %d are too large", p.bm, p.bn);
  p.upt = p.upr * p.bm;
  p.total_units = (long long)p.n_owned * p.upt;

  hipStream_t s = (hipStream_t)stream;
  char name[96];
  static const char* modes[4] = {"one_shot", "two_shot", "reduce_scatter", "atomic"};
  static const char* types[3] = {"bf16", "f16", "f32"};
  snprintf(name, sizeof(name), "slot_reduce_%s_%s_vec%d", modes[p.mode], types[dtype], vec);
  iris_host::set_last_kernel(name);
  if (p.total_units == 0) return 0;  // this rank owns nothing

  // Launches that move tens of megabytes stream with non-temporal accesses and four chunks per thread:
  // their operands are read once, and lines taken into the last-level cache for them would first have to
  // push out whatever dirty lines it holds (a rank's two-shot share of 8 x 128 MiB after a 256 MB buffer
  // was zeroed: 74 instead of 92 us; reduce-scatter 42 instead of 62 us; 8 x 128 MiB one-shot 5.9
  // instead of 5.1 TB/s).  Cacheable accesses win only when the same operands are still cached from a
  // previous launch (43 against 63 us for the two-shot share), which a collective's inputs - other
  // ranks' fresh results - are not.  Small launches keep cacheable accesses.
  const long long moved = p.total_units * (long long)(vec * es) * (p.world + (p.mode == CCL_TWO_SHOT ? p.world : 1));
  const bool stream_nt = vec > 1 && p.mode != CCL_ATOMIC && moved > (32ll << 20);
  const int upt = stream_nt ? 4 : 2;
  const long long per_wg = (long long)kCclThreads * upt;
  const long long want = (p.total_units + per_wg - 1) / per_wg;
  const long long cap = (long long)cu * 8;
  const int grid = (int)(want < cap ? want : cap);

#define CCL_LAUNCH(E, V)                                       \
  do {                                                         \
    if (stream_nt) launch_for_world<E, V, 4, true>(p, grid, s); \
    else launch_for_world<E, V, 2, false>(p, grid, s);          \
  } while (0)
  if (vec == 2) {  // atomic variant only
    if (dtype == IRIS_HIP_BF16) launch_for_world<ElemBF16, 2, 2, false>(p, grid, s);
    else launch_for_world<ElemF16, 2, 2, false>(p, grid, s);
  }
  else if (dtype == IRIS_HIP_BF16) { if (vec == 8) CCL_LAUNCH(ElemBF16, 8); else CCL_LAUNCH(ElemBF16, 1); }
  else if (dtype == IRIS_HIP_FP16) { if (vec == 8) CCL_LAUNCH(ElemF16, 8); else CCL_LAUNCH(ElemF16, 1); }
  else { if (vec == 4) CCL_LAUNCH(ElemF32, 4); else CCL_LAUNCH(ElemF32, 1); }
#undef CCL_LAUNCH
  return (int)hipGetLastError();
}

bool fits_int(int64_t v) { return v > 0 && v < (1ll << 31); }

int fill_common(CclParams& p, const void* input, void* output, int64_t M, int64_t N, int64_t stride_in_m,
                int64_t stride_in_n, int64_t stride_out_m, int64_t stride_out_n, const int64_t* heap_bases,
                int32_t group_rank, int32_t iris_rank, int32_t world_size, int32_t rank_start, int32_t rank_stride,
                int32_t block_size_m, int32_t block_size_n, int32_t swizzle_size, int32_t comm_sms) {
  if (!fits_int(M) || !fits_int(N)) return iris_host::fail("M and N must be in [1, 2^31)");
  p = CclParams{};
  p.in = (const char*)input;
  p.out = (char*)output;
  p.M = (int)M;
  p.N = (int)N;
  p.s_im = stride_in_m; p.s_in = stride_in_n; p.s_om = stride_out_m; p.s_on = stride_out_n;
  p.heap_bases = (const long long*)heap_bases;
  p.group_rank = group_rank; p.iris_rank = iris_rank; p.world = world_size;
  p.rank_start = rank_start; p.rank_stride = rank_stride;
  p.bm = block_size_m; p.bn = block_size_n; p.group_m = swizzle_size; p.comm_sms = comm_sms;
  return 0;
}

}  // namespace

extern "C" {

int iris_hip_all_reduce(const void* input, void* output, int64_t M, int64_t N, int64_t stride_in_m,
                        int64_t stride_in_n, int64_t stride_out_m, int64_t stride_out_n,
                        const int64_t* heap_bases, int32_t group_rank, int32_t iris_rank, int32_t world_size,
                        int32_t rank_start, int32_t rank_stride, int32_t block_size_m, int32_t block_size_n,
                        int32_t swizzle_size, int32_t comm_sms, int32_t num_xcds, int32_t chunk_size,
                        int32_t variant, int32_t distribution, int32_t dtype, void* stream) {
  (void)num_xcds;
  (void)chunk_size;
  CclParams p;
  int rc = fill_common(p, input, output, M, N, stride_in_m, stride_in_n, stride_out_m, stride_out_n, heap_bases,
                       group_rank, iris_rank, world_size, rank_start, rank_stride, block_size_m, block_size_n,
                       swizzle_size, comm_sms);
  if (rc) return rc;
  switch (variant) {
    case IRIS_HIP_VARIANT_ATOMIC: p.mode = CCL_ATOMIC; break;
    case IRIS_HIP_VARIANT_ONE_SHOT: p.mode = CCL_ONE_SHOT; break;
    case IRIS_HIP_VARIANT_TWO_SHOT: p.mode = CCL_TWO_SHOT; break;
    default: return iris_host::fail("variant %d is not atomic (0), one_shot (2) or two_shot (3)", variant);
  }
  return run_ccl(p, distribution, dtype, stream);
}

int iris_hip_reduce_scatter(const void* input, void* output, int64_t M, int64_t N, int64_t stride_in_m,
                            int64_t stride_in_n, int64_t stride_out_m, int64_t stride_out_n,
                            const int64_t* heap_bases, int32_t group_rank, int32_t iris_rank, int32_t world_size,
                            int32_t rank_start, int32_t rank_stride, int32_t block_size_m, int32_t block_size_n,
                            int32_t swizzle_size, int32_t comm_sms, int32_t num_xcds, int32_t chunk_size,
                            int32_t distribution, int32_t dtype, void* stream) {
  (void)num_xcds;
  (void)chunk_size;
  CclParams p;
  int rc = fill_common(p, input, output, M, N, stride_in_m, stride_in_n, stride_out_m, stride_out_n, heap_bases,
                       group_rank, iris_rank, world_size, rank_start, rank_stride, block_size_m, block_size_n,
                       swizzle_size, comm_sms);
  if (rc) return rc;
  p.mode = CCL_REDUCE_SCATTER;
  return run_ccl(p, distribution, dtype, stream);
}

}  // extern "C"
