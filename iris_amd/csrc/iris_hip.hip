// libiris_hip: gfx950 (MI355X) kernels for the rank-local compute of the fused GEMM+collective
// operators, and the C ABI declared in include/iris_hip.h.
//
// Two kernels implement every operator (the first lives in fused_kernel.h and is compiled in the
// iris_hip_mfma_<type>.hip translation units, the second and the entry points are in this file):
//
//  * fused_mfma_kernel  - persistent tiled GEMM on the 32x32 MFMA blocks of CDNA4.  Operand tiles
//    travel HBM -> LDS with 16-byte direct-to-LDS buffer loads into a ring of STAGES buffers
//    (prefetch distance STAGES-1, one workgroup barrier per K step); the K-contiguous operand is
//    read back with 16-byte LDS reads, the N-contiguous one with LDS transpose reads.  The waves of
//    a workgroup (8 as 2x4 for the 256x256 tile, 4 as 2x2 for the smaller ones) each own a block of
//    fp32 accumulators that stays in the accumulation registers.  Requires 16-byte aligned,
//    unit-stride rows (see mfma_ineligible()).
//  * fused_generic_kernel - a plain 64x64 LDS-tiled kernel on fp32 MFMA for everything else (fp32 data,
//    odd strides, sizes that are not multiples of 8 elements).
//
// The flag-less operators (all_gather_matmul, matmul_all_gather, the atomic all-reduce) store or add
// the tile directly.  The others end in the same epilogue protocol, which follows the reference kernels
// (iris/ops/matmul_all_reduce.py:111-144, iris/ops/matmul_reduce_scatter.py:98-118,
//  iris/mem/triton/context.py:733-764, 801-839, 953-997):
//    1. cast the fp32 tile to the output type and store it to aux in the own slot,
//    2. make those stores visible, then raise the flag of every finished flag tile (the MFMA
//       kernel writes aux through to memory and raises relaxed; the generic kernel raises with release),
//    3. for the flag tiles this rank reduces: wait for the peers' flags, add the peers' aux tiles
//       in ascending rank order, cast once, store to C (own slot; two-shot: every slot).

#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include <atomic>
#include <mutex>
#include <type_traits>
#include <vector>

#include "fused_kernel.h"

// ------------------------------------------------------------------------------------------------
// Generic kernel: 64x64 tile, 256 threads, 4x4 outputs per thread, fp32 FMA.
// ------------------------------------------------------------------------------------------------
constexpr int GT = 64;   // generic tile edge
constexpr int GK = 16;   // generic k step

template <class In, class Out>
__global__ void __launch_bounds__(256) fused_generic_kernel(const FusedParams p) {
  __shared__ float As[GK][GT + 1];
  __shared__ float Bs[GK][GT + 1];
  __shared__ float Cs[GT][GT + 1];
  const int tid = threadIdx.x;
  const int tx = tid % 16, ty = tid / 16;
  // Each of the four waves multiplies one 32x32 quadrant of the tile with fp32 MFMA
  // (v_mfma_f32_32x32x2_f32: lane l supplies A[l % 32][l / 32] and B[l / 32][l % 32] of a 32x2 by 2x32
  // product); inputs of every type are widened to fp32 in LDS first, so products are exact for 16-bit
  // and fp8 data and accumulation is fp32 throughout.
  const int lane = tid & 63, wave = tid >> 6;
  const int qm = (wave >> 1) * 32, qn = (wave & 1) * 32;
  const int total_tiles = p.tiles_m * p.tiles_n;
  const int ftn = cdiv(p.N, p.flag_bn);
  const int ftotal = cdiv(p.M, p.flag_bm) * ftn;
  const int nsrc = (p.gather == GATHER_K) ? p.world : 1;
  const int klocal = (p.gather == GATHER_K) ? p.K_local : p.K;

  for (int tile = blockIdx.x; tile < total_tiles; tile += gridDim.x) {
    const int tm = tile / p.tiles_n, tn = tile % p.tiles_n;
    const int m0 = tm * GT, n0 = tn * GT;
    f32x16_t quad;
#pragma unroll
    for (int r = 0; r < 16; ++r) quad[r] = 0.f;

    // One K step = GK columns of A and rows of B.  The operands of step t+1 are fetched into
    // registers while the MFMAs of step t run, and stored to LDS after them.
    const int ksteps = cdiv(klocal, GK);
    const int nsteps = nsrc * ksteps;
    auto fetch = [&](int step, float (&va)[4], float (&vb)[4]) {
      const int src = step / ksteps, k0 = (step - src * ksteps) * GK;
#pragma unroll
      for (int e = 0; e < 4; ++e) {  // A tile: GT rows x GK k
        const int idx = tid + e * 256;
        const int r = idx / GK, kk = idx % GK;
        const int gm = m0 + r, kl = k0 + kk;
        va[e] = 0.f;
        if (gm < p.M && kl < klocal) {
          int slot = p.rank;
          long long row = gm;
          if (p.gather == GATHER_K) slot = src;
          if (p.gather == GATHER_M) { slot = gm / p.M_local; row = gm - (long long)slot * p.M_local; }
          const char* base = p.gather == GATHER_NONE ? p.A : slot_ptr(p.heap_bases, p.A, p.rank, slot);
          va[e] = In::load(base + (row * p.s_am + (long long)kl * p.s_ak) * In::size);
        }
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) {  // B tile: GK k x GT columns
        const int idx = tid + e * 256;
        const int kk = idx / GT, c = idx % GT;
        const int gn = n0 + c, kl = k0 + kk;
        vb[e] = 0.f;
        if (gn < p.N && kl < klocal) {
          const long long kg = (long long)src * klocal + kl;
          vb[e] = In::load(p.B + (kg * p.s_bk + (long long)gn * p.s_bn) * In::size);
        }
      }
    };
    float va[4], vb[4];
    fetch(0, va, vb);
    for (int step = 0; step < nsteps; ++step) {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int idx = tid + e * 256;
        As[idx % GK][idx / GK] = va[e];
        Bs[idx / GT][idx % GT] = vb[e];
      }
      __syncthreads();
      if (step + 1 < nsteps) fetch(step + 1, va, vb);
#pragma unroll
      for (int kk = 0; kk < GK; kk += 2) {
        const float a = As[kk + (lane >> 5)][qm + (lane & 31)];
        const float b = Bs[kk + (lane >> 5)][qn + (lane & 31)];
        quad = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, quad, 0, 0, 0);
      }
      __syncthreads();
    }
    // Accumulator register r of lane l is element (8*(r/4) + 4*(l/32) + r%4, l%32) of the quadrant;
    // the tile goes through LDS so that the epilogue below can work on 4x4 blocks per thread.
#pragma unroll
    for (int r = 0; r < 16; ++r) Cs[qm + 8 * (r / 4) + 4 * (lane >> 5) + (r % 4)][qn + (lane & 31)] = quad[r];
    __syncthreads();
    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[i][j] = Cs[ty * 4 + i][tx * 4 + j];

    // Own tile, rounded to the output type.
    float own[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int gm = m0 + ty * 4 + i;
      float badd = 0.f;
      if (p.bias && gm < p.M) badd = load_scalar_as_float(p.bias, (long long)gm * p.s_bias, p.bias_dtype);
#pragma unroll
      for (int j = 0; j < 4; ++j) own[i][j] = Out::round(acc[i][j] * p.scale + badd);
    }
    const bool flags = epi_has_flags(p.epi);
    char* const out1 = flags ? p.aux : p.C;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int gm = m0 + ty * 4 + i, gn = n0 + tx * 4 + j;
        if (!(gm < p.M && gn < p.N)) continue;
        const long long eoff = ((long long)(gm + p.row_offset) * p.s_cm + (long long)gn * p.s_cn) * Out::size;
        if (p.epi == EPI_ALL_GATHER) {
          for (int pr = 0; pr < p.world; ++pr) Out::store(slot_ptr(p.heap_bases, p.C, p.rank, pr) + eoff, own[i][j]);
        } else if (p.epi == EPI_ATOMIC) {
          for (int pr = 0; pr < p.world; ++pr) Out::atomic_add(slot_ptr(p.heap_bases, p.C, p.rank, pr) + eoff, own[i][j]);
        } else {
          Out::store(out1 + eoff, own[i][j]);
        }
      }
    if (!flags) continue;

    __atomic_thread_fence(__ATOMIC_RELEASE);
    __syncthreads();
    raise_flags<GT, GT, 256, false>(p, m0, n0, tid);
    if (p.sum_peers && p.world > 1) {
      wait_peer_flags<GT, GT, 256>(p, m0, n0, tid);
      __syncthreads();
    }
    const bool ref_chain = (p.acc_mode == IRIS_HIP_ACC_REFERENCE) && !Out::kFp32SumInReference;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int gm = m0 + ty * 4 + i, gn = n0 + tx * 4 + j;
        if (!(gm < p.M && gn < p.N)) continue;
        const int t = (gm / p.flag_bm) * ftn + gn / p.flag_bn;
        const int owner = owner_of(p.epi, t, ftotal, p.world, p.rank);
        if (!p.all_owners && owner != p.rank) continue;
        const long long eoff = ((long long)gm * p.s_cm + (long long)gn * p.s_cn) * Out::size;
        float sum = own[i][j];
        if (p.sum_peers)
          for (int pr = 0; pr < p.world; ++pr) {
            if (pr == p.rank) continue;
            sum += Out::load(slot_ptr(p.heap_bases, p.aux, p.rank, pr) + eoff);
            if (ref_chain) sum = Out::round(sum);
          }
        if (p.epi == EPI_TWO_SHOT) {
          Out::store(p.C + eoff, sum);
          for (int pr = 0; pr < p.world; ++pr)
            if (pr != p.rank) Out::store(slot_ptr(p.heap_bases, p.C, p.rank, pr) + eoff, sum);
        } else {
          const int dst = p.all_owners ? owner : p.rank;
          Out::store(slot_ptr(p.heap_bases, p.C, p.rank, dst) + eoff, sum);
        }
      }
  }
}

// ------------------------------------------------------------------------------------------------
// Host side
// ------------------------------------------------------------------------------------------------
namespace {

thread_local char g_last_error[512] = "";
thread_local char g_last_kernel[128] = "";

using iris_host::fail;  // defined below, shared with the other translation units

struct DeviceFacts {
  int cu_count = 0;
  int xcc_count = 0;
  int lds_per_block = 0;
  bool ok = false;
};

DeviceFacts g_facts[64];
std::mutex g_facts_mutex;  // entry points may be called from several host threads

int facts_for(int device, DeviceFacts** out) {
  if (device < 0 || device >= 64) return fail("device index %d out of range", device);
  std::lock_guard<std::mutex> lock(g_facts_mutex);
  DeviceFacts& f = g_facts[device];
  if (!f.ok) {
    hipDeviceProp_t prop;
    hipError_t e = hipGetDeviceProperties(&prop, device);
    if (e != hipSuccess) return (int)e;
    f.cu_count = prop.multiProcessorCount;
    f.lds_per_block = (int)prop.sharedMemPerBlock;
    // XCD count as the runtime reports it (the reference asks the same attribute,
    // iris/host/platform/hip.py:218-231); a runtime that does not know the attribute means one XCD.
    int xcc = 0;
    if (hipDeviceGetAttribute(&xcc, hipDeviceAttributeNumberOfXccs, device) != hipSuccess || xcc < 1) {
      (void)hipGetLastError();
      xcc = 1;
    }
    f.xcc_count = xcc;
    f.ok = true;
  }
  *out = &f;
  return 0;
}

int elem_size(int dtype) {
  switch (dtype) {
    case IRIS_HIP_BF16: case IRIS_HIP_FP16: return 2;
    case IRIS_HIP_FP32: return 4;
    case IRIS_HIP_FP8_E4M3: return 1;
  }
  return 0;
}

bool aligned16(const void* p) { return ((uintptr_t)p & 15) == 0; }

// Reasons (if any) the MFMA kernel cannot take these operands.
const char* mfma_ineligible(const FusedParams& p, int in_dtype, int out_dtype, int bm, int bn) {
  if (in_dtype == IRIS_HIP_FP32) return "fp32 inputs";
  const int es = elem_size(in_dtype);
  const int ce = 16 / es;
  const int want_out = (in_dtype == IRIS_HIP_FP16) ? IRIS_HIP_FP16 : IRIS_HIP_BF16;
  if (out_dtype != want_out) return "output type not paired with the input type";
  if (p.s_ak != 1) return "A is not K-contiguous";
  if (p.s_bn != 1 && p.s_bk != 1) return "B has no unit stride";
  if (p.s_cn != 1) return "C is not N-contiguous";
  if (!aligned16(p.A) || !aligned16(p.B) || !aligned16(p.C)) return "base pointers not 16-byte aligned";
  if (p.aux && !aligned16(p.aux)) return "aux not 16-byte aligned";
  if (p.K % ce || p.K_local % ce) return "K not a multiple of 16 bytes";
  if ((p.s_am * es) % 16) return "A rows not 16-byte aligned";
  if (p.s_bn == 1) {
    if (p.N % ce) return "N not a multiple of 16 bytes of B";
    if ((p.s_bk * es) % 16) return "B rows not 16-byte aligned";
  } else {
    if ((p.s_bn * es) % 16) return "B columns not 16-byte aligned";
  }
  if (p.N % 8 || p.s_cm % 8) return "C rows not 16-byte aligned";
  if (p.flag_bn % 8) return "flag tile width not a multiple of 8";
  // 32-bit buffer offsets: per-lane offset + per-step offset must stay below 2^31.
  const long long a_span = (long long)bm * p.s_am * es + (long long)p.K * es;
  const long long b_span = (p.s_bn == 1) ? (long long)p.K * p.s_bk * es + (long long)bn * es
                                         : (long long)bn * p.s_bn * es + (long long)p.K * es;
  if (a_span >= (1ll << 31) || b_span >= (1ll << 31)) return "operand too large for 32-bit tile offsets";
  if (p.gather == GATHER_M && (p.M_local % bm)) return "M_local not a multiple of the tile height";
  return nullptr;
}

template <class In, class Out>
int launch_generic(FusedParams p, int cu_count, hipStream_t stream, const char* name) {
  p.tiles_m = cdiv(p.M, GT);
  p.tiles_n = cdiv(p.N, GT);
  const long long total = (long long)p.tiles_m * p.tiles_n;
  const long long cap = (long long)cu_count * 8;
  const int grid = (int)(total < cap ? total : cap);
  hipLaunchKernelGGL((fused_generic_kernel<In, Out>), dim3(grid < 1 ? 1 : grid), dim3(256), 0, stream, p);
  snprintf(g_last_kernel, sizeof(g_last_kernel), "%s", name);
  return (int)hipGetLastError();
}

// Type pairs the generic kernel is built for (the list of dispatch_generic below).
bool generic_supported(int in_dtype, int out_dtype) {
  switch (in_dtype) {
    case IRIS_HIP_BF16: return out_dtype == IRIS_HIP_BF16 || out_dtype == IRIS_HIP_FP32;
    case IRIS_HIP_FP16: return out_dtype == IRIS_HIP_FP16 || out_dtype == IRIS_HIP_FP32;
    case IRIS_HIP_FP32: return out_dtype == IRIS_HIP_FP32;
    case IRIS_HIP_FP8_E4M3: return out_dtype == IRIS_HIP_BF16 || out_dtype == IRIS_HIP_FP16;
  }
  return false;
}

int dispatch_generic(const FusedParams& p, int in_dtype, int out_dtype, int cu, hipStream_t s) {
#define GEN(I, O, name) return launch_generic<I, O>(p, cu, s, name)
  if (in_dtype == IRIS_HIP_BF16 && out_dtype == IRIS_HIP_BF16) GEN(ElemBF16, ElemBF16, "generic_bf16");
  if (in_dtype == IRIS_HIP_FP16 && out_dtype == IRIS_HIP_FP16) GEN(ElemF16, ElemF16, "generic_f16");
  if (in_dtype == IRIS_HIP_FP32 && out_dtype == IRIS_HIP_FP32) GEN(ElemF32, ElemF32, "generic_f32");
  if (in_dtype == IRIS_HIP_FP8_E4M3 && out_dtype == IRIS_HIP_BF16) GEN(ElemFP8, ElemBF16, "generic_fp8_bf16");
  if (in_dtype == IRIS_HIP_FP8_E4M3 && out_dtype == IRIS_HIP_FP16) GEN(ElemFP8, ElemF16, "generic_fp8_f16");
  if (in_dtype == IRIS_HIP_BF16 && out_dtype == IRIS_HIP_FP32) GEN(ElemBF16, ElemF32, "generic_bf16_f32");
  if (in_dtype == IRIS_HIP_FP16 && out_dtype == IRIS_HIP_FP32) GEN(ElemF16, ElemF32, "generic_f16_f32");
#undef GEN
  return fail("unsupported element types in=%d out=%d", in_dtype, out_dtype);
}

}  // namespace

// Instantiated in iris_hip_mfma_bf16.hip, iris_hip_mfma_f16.hip and iris_hip_mfma_fp8.hip.
extern template int dispatch_mfma_in<IN_BF16>(FusedParams&, int, bool, int, int, hipStream_t);
extern template int dispatch_mfma_in<IN_F16>(FusedParams&, int, bool, int, int, hipStream_t);
extern template int dispatch_mfma_in<IN_FP8>(FusedParams&, int, bool, int, int, hipStream_t);

namespace {

// ------------------------------------------------------------------------------------------------
// Library-owned workspace of iris_hip_matmul_all_reduce_noalloc
// ------------------------------------------------------------------------------------------------
// Layout of the array: [0, 256) a one-rank context (rank 0, world 1, heap base 0: every address
// translates to itself), [256, 256 + 64 KiB) the tile flags, then the aux buffer.
constexpr size_t kScratchContextBytes = 256;
constexpr size_t kScratchFlagBytes = (size_t)IRIS_HIP_NOALLOC_MAX_FLAGS * sizeof(int32_t);
constexpr size_t kScratchAuxOffset = kScratchContextBytes + kScratchFlagBytes;
constexpr size_t kScratchBytes = kScratchAuxOffset + (size_t)IRIS_HIP_NOALLOC_MAX_AUX_BYTES;
static_assert(kScratchAuxOffset % 256 == 0, "aux buffer alignment");

// Device memory of its own on every GPU the library runs on, from module load to process end.  The
// name below is a host-side handle only: device code and HIP calls get the address that
// hipGetSymbolAddress reports for the current device (scratch_for_current_device).
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

void* g_scratch_ptr[64] = {};
std::mutex g_scratch_mutex;

// Address of the scratch array on the current device (looked up once per device).
int scratch_for_current_device(unsigned char** out) {
  int device = 0;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) return (int)e;
  if (device < 0 || device >= 64) return fail("device index %d out of range", device);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[device]) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return (int)e;
    if (!ptr) return fail("the library's workspace has no address on device %d", device);
    g_scratch_ptr[device] = ptr;
  }
  *out = (unsigned char*)g_scratch_ptr[device];
  return 0;
}

// Writes the one-rank context and clears the flags a launch is going to use.  A kernel, not a memset:
// the caller's stream may be under graph capture.
__global__ void __launch_bounds__(256) noalloc_prepare_kernel(long long* context, int* flags, int nflags) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < (int)(kScratchContextBytes / sizeof(long long))) context[i] = (i == 1) ? 1 : 0;  // [rank 0, world 1, base 0, ...]
  if (i < nflags) flags[i] = 0;
}

// ------------------------------------------------------------------------------------------------
// Context tensors whose contents the host has told the library (iris_hip_register_context)
// ------------------------------------------------------------------------------------------------
struct KnownContext {
  const int64_t* device_ptr;
  int rank, world;
  long long bases[kMaxCachedSlots];
};
std::vector<KnownContext> g_contexts;
std::mutex g_contexts_mutex;

// Fill p.hb_arg from the registry when the launch names a registered context tensor with the same
// rank and world size (anything else falls back to loading the bases on the device).
void heap_bases_from_registry(FusedParams& p, const int64_t* context_tensor) {
  p.hb_in_args = 0;
  if (!context_tensor || p.world > kMaxCachedSlots) return;
  std::lock_guard<std::mutex> lock(g_contexts_mutex);
  for (const KnownContext& k : g_contexts) {
    if (k.device_ptr != context_tensor) continue;
    if (k.rank != p.rank || k.world != p.world) return;
    for (int r = 0; r < kMaxCachedSlots; ++r) p.hb_arg[r] = k.bases[r];
    p.hb_in_args = 1;
    return;
  }
}

#ifdef IRIS_HIP_PHASE_STAMPS
unsigned long long* g_stamps = nullptr;  // diagnostic build: where the kernels record their phase stamps
long long g_stamp_rows = 0;              // ... and how many rows of 16 words the buffer holds
#endif

// Launches for the 32x32 kernel (decode_kernel.h): outputs of at most two 32x32 tiles per CU.  Such an
// output is a handful of 128x128 tiles on a handful of CUs, while 32x32 tiles with K split over the waves
// of a workgroup keep the whole chip busy; beyond two tiles per CU the 64x64 tiled kernel is ahead.
bool decode_sized(const FusedParams& p, int cu_count, int in_dtype) {
  if ((long long)cdiv(p.M, 32) * cdiv(p.N, 32) > 2ll * cu_count) return false;
  // ... and whose operands that kernel's 32-bit offsets reach (a tall A with long or padded rows does not
  // qualify: 16384 x 32 outputs of K = 65536 bf16 have 2 GiB of A).
  const long long a_rows = p.gather == GATHER_M ? p.M_local : p.M;
  return decode_offsets_fit(a_rows, p.s_am, p.K_local, in_dtype == IRIS_HIP_FP8_E4M3 ? 1 : 2, p.M + p.row_offset, p.s_cm, p.N);
}
// ... and whose A that kernel can fetch: not gathered, gathered by rows in whole 32-row tiles per slot, or
// gathered along K with every wave's 256 bytes of K inside one slot.
bool decode_gather_ok(const FusedParams& p, int in_dtype) {
  const int es = in_dtype == IRIS_HIP_FP8_E4M3 ? 1 : 2;
  if (p.gather == GATHER_M) return p.M_local % 32 == 0;
  if (p.gather == GATHER_K) return ((long long)p.K_local * es) % 256 == 0;
  return true;
}

// check_only: run every argument check and the kernel choice, launch nothing (0 = the launch would go out).
int run_fused(FusedParams p, int in_dtype, int out_dtype, int path, void* stream, bool check_only = false) {
  g_last_error[0] = 0;
#ifdef IRIS_HIP_PHASE_STAMPS
  p.stamps = g_stamps;
  p.stamp_rows = g_stamp_rows;
#endif
  if (p.M <= 0 || p.N <= 0 || p.K <= 0) return fail("M, N, K must be positive (got %d, %d, %d)", p.M, p.N, p.K);
  if (!p.A || !p.B || !p.C) return fail("A, B and C must not be NULL");
  if (p.world < 1 || p.rank < 0 || p.rank >= p.world) return fail("bad rank/world_size %d/%d", p.rank, p.world);
  if (epi_has_flags(p.epi)) {
    if (!p.aux || !p.locks) return fail("aux_buffer and locks must not be NULL");
    if (p.flag_bm <= 0 || p.flag_bn <= 0) return fail("block sizes must be positive");
  } else {
    p.flag_bm = 256;  // no flags on this path; any valid tile size
    p.flag_bn = 64;
  }
  // Every kernel translates addresses through the heap bases, also with one rank.
  if (!p.heap_bases) return fail("context_tensor must not be NULL");
  heap_bases_from_registry(p, (const int64_t*)p.heap_bases - 2);
  if (elem_size(in_dtype) == 0 || elem_size(out_dtype) == 0 || out_dtype == IRIS_HIP_FP8_E4M3)
    return fail("unsupported element types in=%d out=%d", in_dtype, out_dtype);

  int device = 0;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) return (int)e;
  DeviceFacts* facts = nullptr;
  int rc = facts_for(device, &facts);
  if (rc) return rc;
  p.num_xcd = facts->xcc_count;
  hipStream_t s = (hipStream_t)stream;

  // Tile choice (the tile list in fused_kernel.h has the measurements): the 256x256 tile from about half the
  // CUs busy (cross-over against the 128x128 tiles between 128 and 144 big tiles on 256 CUs) unless the output
  // has at most 64 rows; the latency-oriented 32x32 kernel (decode_kernel.h) for at most two such tiles per CU;
  // 64x64 tiles for at most two of those per CU; 64x128 tiles for at most 64 rows, and for at most two such
  // tiles per CU when K is short; else 128x128 - two workgroups per CU when there are more such tiles than CUs.
  const long long big_tiles = (long long)cdiv(p.M, 256) * cdiv(p.N, 256);
  const bool rows64_ok = !(p.gather == GATHER_M && p.M_local % 64);
  int kind = TILE_SMALL;
  if (big_tiles * 100 >= (long long)facts->cu_count * 53 && !(p.M <= 64 && rows64_ok)) kind = TILE_BIG;
  else if (decode_sized(p, facts->cu_count, in_dtype) && decode_gather_ok(p, in_dtype) && p.world <= 8) kind = TILE_DECODE;
  else if ((long long)cdiv(p.M, 64) * cdiv(p.N, 64) <= 2ll * facts->cu_count && rows64_ok) kind = TILE_SKINNY64;
  else if (rows64_ok && (p.M <= 64 || ((long long)cdiv(p.M, 64) * cdiv(p.N, 128) <= 2ll * facts->cu_count &&
                                       (long long)p.K * elem_size(in_dtype) <= 2048)))
    kind = TILE_SKINNY;
  else if ((long long)cdiv(p.M, 128) * cdiv(p.N, 128) > facts->cu_count) kind = TILE_SMALL2;
  // IRIS_HIP_TILE = big | small | small2 | skinny | skinny64 overrides the choice among the tiled kernels (a tuning
  // aid; results do not depend on the tile shape beyond the order of the fp32 sums over K).
  static const int forced_tile = [] {
    const char* e = getenv("IRIS_HIP_TILE");
    if (!e) return -1;
    if (!strcmp(e, "big")) return (int)TILE_BIG;
    if (!strcmp(e, "small")) return (int)TILE_SMALL;
    if (!strcmp(e, "small2")) return (int)TILE_SMALL2;
    if (!strcmp(e, "skinny")) return (int)TILE_SKINNY;
    if (!strcmp(e, "skinny64")) return (int)TILE_SKINNY64;
    return -1;
  }();
  if (forced_tile >= 0 && kind != TILE_DECODE &&
      !mfma_ineligible(p, in_dtype, out_dtype, tile_rows(forced_tile), tile_cols(forced_tile)))
    kind = forced_tile;  // a tile the operands do not qualify for is not forced
  const char* why = mfma_ineligible(p, in_dtype, out_dtype, tile_rows(kind), tile_cols(kind));
  if (path == IRIS_HIP_PATH_MFMA && why) return fail("MFMA kernel not applicable: %s", why);
  if (path == IRIS_HIP_PATH_GENERIC || why) {
    if (!generic_supported(in_dtype, out_dtype)) return fail("unsupported element types in=%d out=%d", in_dtype, out_dtype);
    return check_only ? 0 : dispatch_generic(p, in_dtype, out_dtype, facts->cu_count, s);
  }
  if (check_only) return 0;

  const bool bkc = (p.s_bn != 1);
  switch (in_dtype) {
    case IRIS_HIP_BF16: rc = dispatch_mfma_in<IN_BF16>(p, kind, bkc, device, facts->cu_count, s); break;
    case IRIS_HIP_FP16: rc = dispatch_mfma_in<IN_F16>(p, kind, bkc, device, facts->cu_count, s); break;
    case IRIS_HIP_FP8_E4M3: rc = dispatch_mfma_in<IN_FP8>(p, kind, bkc, device, facts->cu_count, s); break;
    default: rc = fail("unsupported input type %d", in_dtype);
  }
  return rc;
}

bool fits_int(int64_t v) { return v > 0 && v < (1ll << 31); }

// iris_hip_matmul_all_reduce; check_only stops in front of the launch (see run_fused).
int matmul_all_reduce_impl(const void* A, const void* B, void* C, void* aux_buffer, int32_t* locks,
                               int64_t M, int64_t N, int64_t K,
                               int64_t stride_am, int64_t stride_ak, int64_t stride_bk, int64_t stride_bn,
                               int64_t stride_cm, int64_t stride_cn,
                               const int64_t* context_tensor, int32_t cur_rank, int32_t world_size,
                               int32_t block_size_m, int32_t block_size_n, int32_t block_size_k,
                               int32_t variant, int32_t in_dtype, int32_t out_dtype, float scale,
                               int32_t acc_mode, int64_t spin_limit, int32_t* status, int32_t path,
                               void* stream, bool check_only, bool no_alloc = false) {
  (void)block_size_k;
  if (!fits_int(M) || !fits_int(N) || !fits_int(K)) return fail("M, N, K must be in [1, 2^31)");
  if (variant != IRIS_HIP_VARIANT_ATOMIC && variant != IRIS_HIP_VARIANT_ONE_SHOT && variant != IRIS_HIP_VARIANT_TWO_SHOT)
    return fail("variant %d is not atomic (0), one_shot (2) or two_shot (3)", variant);
  FusedParams p;
  memset(&p, 0, sizeof(p));
  p.A = (const char*)A; p.B = (const char*)B; p.C = (char*)C; p.aux = (char*)aux_buffer; p.locks = locks;
  p.M = (int)M; p.N = (int)N; p.K = (int)K; p.K_local = (int)K; p.gather = GATHER_NONE;
  p.s_am = stride_am; p.s_ak = stride_ak; p.s_bk = stride_bk; p.s_bn = stride_bn;
  p.s_cm = stride_cm; p.s_cn = stride_cn;
  p.heap_bases = context_tensor ? (const long long*)(context_tensor + 2) : nullptr;
  p.rank = cur_rank; p.world = world_size;
  p.flag_bm = block_size_m; p.flag_bn = block_size_n;
  p.epi = variant == IRIS_HIP_VARIANT_ATOMIC ? EPI_ATOMIC : variant == IRIS_HIP_VARIANT_ONE_SHOT ? EPI_ONE_SHOT : EPI_TWO_SHOT;
  p.acc_mode = acc_mode; p.all_owners = 0; p.sum_peers = 1;
  p.scale = scale; p.spin_limit = spin_limit; p.status = status;
  p.no_workspace_alloc = no_alloc ? 1 : 0;
  return run_fused(p, in_dtype, out_dtype, path, stream, check_only);
}

}  // namespace

namespace iris_host {

int fail(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
  va_end(ap);
  return (int)hipErrorInvalidValue;
}

void clear_last_error() { g_last_error[0] = 0; }

void set_last_kernel(const char* name) { snprintf(g_last_kernel, sizeof(g_last_kernel), "%s", name); }

namespace {
struct SplitTileWorkspace {
  int device;
  hipStream_t stream;
  char* partials;
  int* flags;
  int nwg;
  long long slot_bytes;
  unsigned epoch;
};
constexpr int kMaxSplitWorkspacesPerDevice = 8;
std::vector<SplitTileWorkspace> g_split_workspaces;
std::mutex g_split_mutex;
}  // namespace

namespace {
std::atomic<int> g_split_mode{[] { const char* e = getenv("IRIS_HIP_STREAMK"); return e ? atoi(e) : -1; }()};
}
int split_tile_mode() { return g_split_mode.load(std::memory_order_relaxed); }
void set_split_tile_mode(int mode) { g_split_mode.store(mode < 0 ? -1 : (mode > 2 ? 2 : mode), std::memory_order_relaxed); }

int split_tile_workspace(int device, hipStream_t stream, int nwg, long long slot_bytes, char** partials, int** flags, int* epoch) {
  // Never under stream capture: the flag value of a launch is a kernel argument, a replayed launch would
  // meet the flags of its previous replay already at that value and read partial sums before they are
  // written.  (And nothing may be allocated or cleared on a capturing stream.)
  hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &capturing) != hipSuccess || capturing != hipStreamCaptureStatusNone) {
    (void)hipGetLastError();
    return 1;
  }
  std::lock_guard<std::mutex> lock(g_split_mutex);
  int on_device = 0;
  for (SplitTileWorkspace& w : g_split_workspaces) {
    if (w.device != device) continue;
    ++on_device;
    if (w.stream != stream || w.nwg < nwg || w.slot_bytes < slot_bytes) continue;
    w.epoch = w.epoch % 0x7FFFFFFFu + 1;  // 1 .. 2^31 - 1: never the 0 the flags start with
    *partials = w.partials;
    *flags = w.flags;
    *epoch = (int)w.epoch;
    return 0;
  }
  if (on_device >= kMaxSplitWorkspacesPerDevice) return 1;
  // First split launch on this stream.
  SplitTileWorkspace w{device, stream, nullptr, nullptr, nwg, slot_bytes, 1u};
  if (hipMalloc((void**)&w.partials, (size_t)nwg * (size_t)slot_bytes) != hipSuccess) {
    (void)hipGetLastError();
    return 1;
  }
  if (hipMalloc((void**)&w.flags, (size_t)nwg * sizeof(int)) != hipSuccess ||
      hipMemsetAsync(w.flags, 0, (size_t)nwg * sizeof(int), stream) != hipSuccess) {
    (void)hipGetLastError();
    (void)hipFree(w.partials);
    if (w.flags) (void)hipFree(w.flags);
    return 1;
  }
  g_split_workspaces.push_back(w);
  *partials = w.partials;
  *flags = w.flags;
  *epoch = 1;
  return 0;
}

int device_facts(int device, int* cu_count, int* xcc_count) {
  DeviceFacts* f = nullptr;
  const int rc = facts_for(device, &f);
  if (rc) return rc;
  *cu_count = f->cu_count;
  *xcc_count = f->xcc_count;
  return 0;
}

}  // namespace iris_host

extern "C" {

int iris_hip_matmul_all_reduce(const void* A, const void* B, void* C, void* aux_buffer, int32_t* locks,
                               int64_t M, int64_t N, int64_t K,
                               int64_t stride_am, int64_t stride_ak, int64_t stride_bk, int64_t stride_bn,
                               int64_t stride_cm, int64_t stride_cn,
                               const int64_t* context_tensor, int32_t cur_rank, int32_t world_size,
                               int32_t block_size_m, int32_t block_size_n, int32_t block_size_k,
                               int32_t variant, int32_t in_dtype, int32_t out_dtype, float scale,
                               int32_t acc_mode, int64_t spin_limit, int32_t* status, int32_t path,
                               void* stream) {
  return matmul_all_reduce_impl(A, B, C, aux_buffer, locks, M, N, K, stride_am, stride_ak, stride_bk, stride_bn, stride_cm,
                                stride_cn, context_tensor, cur_rank, world_size, block_size_m, block_size_n, block_size_k,
                                variant, in_dtype, out_dtype, scale, acc_mode, spin_limit, status, path, stream, false);
}

int iris_hip_matmul_all_reduce_noalloc(const void* A, const void* B, void* C, int64_t M, int64_t N, int64_t K,
                                       int64_t stride_am, int64_t stride_ak, int64_t stride_bk, int64_t stride_bn,
                                       int64_t stride_cm, int64_t stride_cn,
                                       int32_t block_size_m, int32_t block_size_n, int32_t block_size_k,
                                       int32_t variant, int32_t in_dtype, int32_t out_dtype, float scale,
                                       int32_t path, void* stream) {
  g_last_error[0] = 0;
  if (!fits_int(M) || !fits_int(N) || !fits_int(K)) return fail("M, N, K must be in [1, 2^31)");
  if (variant != IRIS_HIP_VARIANT_ONE_SHOT && variant != IRIS_HIP_VARIANT_TWO_SHOT)
    return fail("variant %d is not one_shot (2) or two_shot (3)", variant);
  if (block_size_m <= 0 || block_size_n <= 0) return fail("block sizes must be positive");
  const int es = elem_size(out_dtype);
  if (es == 0) return fail("unsupported element types in=%d out=%d", in_dtype, out_dtype);
  if (stride_cm < 0 || stride_cn < 0) return fail("negative output strides are not supported");
  if (stride_cm >= (1ll << 40) || stride_cn >= (1ll << 40)) return fail("output strides beyond 2^40 elements are not supported");
  // aux is addressed with C's strides: the bytes it spans and the flags of the tile grid must fit.
  const long long aux_bytes = ((long long)(M - 1) * stride_cm + (long long)(N - 1) * stride_cn + 1) * es;
  const long long nflags = (long long)cdiv((int)M, block_size_m) * cdiv((int)N, block_size_n);
  if (aux_bytes > (long long)IRIS_HIP_NOALLOC_MAX_AUX_BYTES)
    return fail("output of %lld x %lld spans %lld bytes, beyond the %lld bytes of the library's workspace; "
                "use iris_hip_matmul_all_reduce with a caller-owned workspace",
                (long long)M, (long long)N, aux_bytes, (long long)IRIS_HIP_NOALLOC_MAX_AUX_BYTES);
  if (nflags > IRIS_HIP_NOALLOC_MAX_FLAGS)
    return fail("%lld tiles of %d x %d, beyond the %d flags of the library's workspace; use larger block sizes "
                "or iris_hip_matmul_all_reduce with a caller-owned workspace",
                nflags, block_size_m, block_size_n, IRIS_HIP_NOALLOC_MAX_FLAGS);
  unsigned char* base = nullptr;
  int rc = scratch_for_current_device(&base);
  if (rc) return rc;
  long long* context = (long long*)base;
  int32_t* locks = (int32_t*)(base + kScratchContextBytes);
  void* aux = base + kScratchAuxOffset;
  // Every check of the launch itself (types, path, strides) before the prepare kernel goes out: a rejected
  // call enqueues nothing and leaves the workspace alone.
  rc = matmul_all_reduce_impl(A, B, C, aux, locks, M, N, K, stride_am, stride_ak, stride_bk, stride_bn, stride_cm, stride_cn,
                              (const int64_t*)context, 0, 1, block_size_m, block_size_n, block_size_k, variant, in_dtype,
                              out_dtype, scale, IRIS_HIP_ACC_FP32, 0, nullptr, path, stream, true, true);
  if (rc) return rc;
  const int threads = 256;
  const int need = (int)nflags > (int)(kScratchContextBytes / sizeof(long long)) ? (int)nflags : (int)(kScratchContextBytes / sizeof(long long));
  hipLaunchKernelGGL(noalloc_prepare_kernel, dim3((need + threads - 1) / threads), dim3(threads), 0, (hipStream_t)stream,
                     context, locks, (int)nflags);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return (int)e;
  return matmul_all_reduce_impl(A, B, C, aux, locks, M, N, K, stride_am, stride_ak, stride_bk, stride_bn, stride_cm,
                                stride_cn, (const int64_t*)context, 0, 1, block_size_m, block_size_n, block_size_k,
                                variant, in_dtype, out_dtype, scale, IRIS_HIP_ACC_FP32, 0, nullptr, path, stream, false, true);
}

int iris_hip_matmul_reduce_scatter(const void* A, const void* B, void* C, void* aux_buffer, int32_t* locks,
                                   int64_t M, int64_t N, int64_t K,
                                   int64_t stride_am, int64_t stride_ak, int64_t stride_bk, int64_t stride_bn,
                                   int64_t stride_cm, int64_t stride_cn,
                                   const int64_t* context_tensor, int32_t cur_rank, int32_t world_size,
                                   int32_t block_size_m, int32_t block_size_n, int32_t block_size_k,
                                   int32_t all_owners, int32_t sum_peers,
                                   int32_t in_dtype, int32_t out_dtype, float scale, int32_t acc_mode,
                                   int64_t spin_limit, int32_t* status, int32_t path, void* stream) {
  (void)block_size_k;
  if (!fits_int(M) || !fits_int(N) || !fits_int(K)) return fail("M, N, K must be in [1, 2^31)");
  FusedParams p;
  memset(&p, 0, sizeof(p));
  p.A = (const char*)A; p.B = (const char*)B; p.C = (char*)C; p.aux = (char*)aux_buffer; p.locks = locks;
  p.M = (int)M; p.N = (int)N; p.K = (int)K; p.K_local = (int)K; p.gather = GATHER_NONE;
  p.s_am = stride_am; p.s_ak = stride_ak; p.s_bk = stride_bk; p.s_bn = stride_bn;
  p.s_cm = stride_cm; p.s_cn = stride_cn;
  p.heap_bases = context_tensor ? (const long long*)(context_tensor + 2) : nullptr;
  p.rank = cur_rank; p.world = world_size;
  p.flag_bm = block_size_m; p.flag_bn = block_size_n;
  p.epi = EPI_REDUCE_SCATTER;
  p.acc_mode = acc_mode; p.all_owners = all_owners ? 1 : 0; p.sum_peers = sum_peers ? 1 : 0;
  p.scale = scale; p.spin_limit = spin_limit; p.status = status;
  return run_fused(p, in_dtype, out_dtype, path, stream);
}

int iris_hip_all_gather_matmul(const void* A_sharded, const void* B, void* C, const void* bias,
                               int64_t M, int64_t N, int64_t K, int64_t K_local,
                               int64_t stride_am, int64_t stride_ak, int64_t stride_bk, int64_t stride_bn,
                               int64_t stride_cm, int64_t stride_cn, int64_t stride_bias,
                               const int64_t* context_tensor, int32_t cur_rank, int32_t world_size,
                               int32_t block_size_m, int32_t block_size_n, int32_t block_size_k,
                               int32_t gather_dim, int32_t in_dtype, int32_t out_dtype, int32_t bias_dtype,
                               float scale, int32_t path, void* stream) {
  (void)block_size_m; (void)block_size_n; (void)block_size_k;
  if (!fits_int(M) || !fits_int(N) || !fits_int(K) || !fits_int(K_local))
    return fail("M, N, K, K_local must be in [1, 2^31)");
  FusedParams p;
  memset(&p, 0, sizeof(p));
  p.A = (const char*)A_sharded; p.B = (const char*)B; p.C = (char*)C; p.bias = (const char*)bias;
  p.M = (int)M; p.N = (int)N; p.K = (int)K;
  if (gather_dim == IRIS_HIP_GATHER_K) {
    if (K != (int64_t)world_size * K_local)
      return fail("K (%lld) must equal world_size (%d) * K_local (%lld)", (long long)K, world_size, (long long)K_local);
    p.gather = GATHER_K; p.K_local = (int)K_local; p.M_local = (int)M;
  } else if (gather_dim == IRIS_HIP_GATHER_M) {
    if (K_local != K) return fail("gather along M needs K_local == K");
    if (M % world_size) return fail("gather along M needs M divisible by world_size");
    p.gather = GATHER_M; p.K_local = (int)K; p.M_local = (int)(M / world_size);
  } else {
    return fail("gather_dim %d is not 1 (K) or 2 (M)", gather_dim);
  }
  if (bias && elem_size(bias_dtype) < 2) return fail("unsupported bias type %d", bias_dtype);
  p.s_am = stride_am; p.s_ak = stride_ak; p.s_bk = stride_bk; p.s_bn = stride_bn;
  p.s_cm = stride_cm; p.s_cn = stride_cn; p.s_bias = stride_bias; p.bias_dtype = bias_dtype;
  p.heap_bases = context_tensor ? (const long long*)(context_tensor + 2) : nullptr;
  p.rank = cur_rank; p.world = world_size;
  p.epi = EPI_STORE; p.scale = scale;
  return run_fused(p, in_dtype, out_dtype, path, stream);
}

int iris_hip_matmul_all_gather(const void* A, const void* B, void* C_gathered, const void* bias,
                               int64_t M_local, int64_t M, int64_t N, int64_t K,
                               int64_t stride_am, int64_t stride_ak, int64_t stride_bk, int64_t stride_bn,
                               int64_t stride_cm_gathered, int64_t stride_cn_gathered, int64_t stride_bias,
                               const int64_t* context_tensor, int32_t cur_rank, int32_t world_size,
                               int32_t block_size_m, int32_t block_size_n, int32_t block_size_k,
                               int32_t in_dtype, int32_t out_dtype, int32_t bias_dtype, float scale,
                               int32_t path, void* stream) {
  (void)block_size_m; (void)block_size_n; (void)block_size_k;
  if (!fits_int(M_local) || !fits_int(M) || !fits_int(N) || !fits_int(K))
    return fail("M_local, M, N, K must be in [1, 2^31)");
  if (world_size < 1 || M != M_local * world_size)
    return fail("M (%lld) must equal M_local (%lld) * world_size (%d)", (long long)M, (long long)M_local, world_size);
  if (bias && elem_size(bias_dtype) < 2) return fail("unsupported bias type %d", bias_dtype);
  FusedParams p;
  memset(&p, 0, sizeof(p));
  p.A = (const char*)A; p.B = (const char*)B; p.C = (char*)C_gathered; p.bias = (const char*)bias;
  p.M = (int)M_local; p.N = (int)N; p.K = (int)K; p.K_local = (int)K; p.gather = GATHER_NONE;
  p.s_am = stride_am; p.s_ak = stride_ak; p.s_bk = stride_bk; p.s_bn = stride_bn;
  p.s_cm = stride_cm_gathered; p.s_cn = stride_cn_gathered; p.s_bias = stride_bias; p.bias_dtype = bias_dtype;
  p.heap_bases = context_tensor ? (const long long*)(context_tensor + 2) : nullptr;
  p.rank = cur_rank; p.world = world_size;
  p.row_offset = (int)(cur_rank * M_local);
  p.epi = EPI_ALL_GATHER; p.scale = scale;
  return run_fused(p, in_dtype, out_dtype, path, stream);
}

int iris_hip_register_context(const int64_t* context_tensor, const int64_t* host_copy, int32_t num_words) {
  g_last_error[0] = 0;
  if (!context_tensor || !host_copy) return fail("context_tensor and host_copy must not be NULL");
  if (num_words < 3) return fail("a context tensor has at least 3 words (rank, world size, one heap base)");
  const int64_t rank = host_copy[0], world = host_copy[1];
  if (world < 1 || rank < 0 || rank >= world || num_words < 2 + world)
    return fail("bad context contents: rank %lld, world size %lld, %d words", (long long)rank, (long long)world, num_words);
  KnownContext k;
  k.device_ptr = context_tensor;
  k.rank = (int)rank;
  k.world = (int)world;
  for (int r = 0; r < kMaxCachedSlots; ++r) k.bases[r] = r < world ? (long long)host_copy[2 + r] : 0ll;
  std::lock_guard<std::mutex> lock(g_contexts_mutex);
  for (KnownContext& e : g_contexts)
    if (e.device_ptr == context_tensor) {
      e = k;
      return 0;
    }
  g_contexts.push_back(k);
  return 0;
}

int iris_hip_unregister_context(const int64_t* context_tensor) {
  g_last_error[0] = 0;
  std::lock_guard<std::mutex> lock(g_contexts_mutex);
  for (size_t i = 0; i < g_contexts.size(); ++i)
    if (g_contexts[i].device_ptr == context_tensor) {
      g_contexts.erase(g_contexts.begin() + i);
      break;
    }
  return 0;
}

int iris_hip_query(int32_t device, int32_t* cu_count, int32_t* xcc_count, int32_t* lds_bytes_per_block) {
  g_last_error[0] = 0;
  DeviceFacts* f = nullptr;
  int rc = facts_for(device, &f);
  if (rc) return rc;
  if (cu_count) *cu_count = f->cu_count;
  if (xcc_count) *xcc_count = f->xcc_count;
  if (lds_bytes_per_block) *lds_bytes_per_block = f->lds_per_block;
  // Set-up call of the host layer: also look up the no-allocation entry point's workspace address
  // when `device` is the current one, so that its first call has nothing left to resolve.
  int current = -1;
  if (hipGetDevice(&current) == hipSuccess && current == device) {
    unsigned char* unused = nullptr;
    rc = scratch_for_current_device(&unused);
    if (rc) return rc;
  }
  return 0;
}

#ifdef IRIS_HIP_PHASE_STAMPS
// Diagnostic build only: device buffer of `rows` rows of 16 64-bit words, or NULL.  A launch writes row
// it * (number of workgroups) + (workgroup) for the first eight tiles `it` of every workgroup; rows beyond
// the buffer are not written.
void iris_hip_debug_set_stamps(void* device_buffer, long long rows) {
  g_stamps = (unsigned long long*)device_buffer;
  g_stamp_rows = device_buffer ? rows : 0;
}
#endif

void iris_hip_set_split_tiles(int32_t mode) { iris_host::set_split_tile_mode(mode); }

const char* iris_hip_last_error(void) { return g_last_error; }
const char* iris_hip_last_kernel(void) { return g_last_kernel; }
int iris_hip_abi_version(void) { return 5; }

}  // extern "C"
