/*
 * C ABI of libiris_hip.so: hand-written gfx950 (MI355X) kernels for the rank-local compute of the
 * fused GEMM+collective operators of the Iris Python package.
 *
 * The reference package has no native interface: each operator launches a Triton kernel through
 * `iris_launch(kernel_fn, grid, *args, ...)` (iris/host/tracing/kernel_artifacts.py:54-83).  Every
 * entry point below takes the arguments of one such launch, in the same order and with the same
 * meaning, up to and including the three block sizes, followed by a short tail of values the Triton
 * launch gets implicitly (element types, the HIP stream) or that this library adds (scales for fp8
 * inputs, a bound on flag spinning).  The launch arguments after the block sizes are compile-time
 * tuning constants of the Triton kernels and are NOT taken: EVEN_K everywhere (K tails are handled by
 * out-of-range loads), and for the two gather operators GROUP_SIZE_M, NUM_SMS, NUM_XCDS,
 * NUM_K_BLOCKS_LOCAL, USE_BIAS (a NULL bias says the same), EVEN_K and ALLOW_TF32
 * (iris/ops/all_gather_matmul.py:289-295, iris/ops/matmul_all_gather.py:258-262).
 *
 * Conventions
 *   - All data pointers are device pointers.  Strides are in elements, as torch reports them.
 *   - `context_tensor` is the int64 device array built by Iris._build_device_context
 *     (iris/host/iris.py:916-958): [cur_rank, world_size, heap_base_0 .. heap_base_{W-1}, ...].
 *     A pointer p inside slot `cur_rank` names, in slot r, the address
 *     heap_base_r + (p - heap_base_cur_rank)   (iris/mem/triton/context.py:16-27).
 *   - Launches are asynchronous on `stream` (a hipStream_t passed as void*; NULL = default stream).
 *   - Return value: 0 on success, otherwise a hipError_t value.  Argument errors return
 *     hipErrorInvalidValue (1); iris_hip_last_error() then describes the problem.
 *   - The library calls hipMalloc only for the split-tile workspace described at iris_hip_set_split_tiles
 *     (iris_hip_matmul_all_reduce_noalloc never does).  It keeps between calls: device facts (CU count, XCD count, LDS
 *     size) cached per device under a mutex, a once-per-device "attribute set" flag per kernel build
 *     (atomic), the last error and last kernel name per host thread, the contents of context tensors
 *     registered with iris_hip_register_context (under a mutex), and one static device array that
 *     only iris_hip_matmul_all_reduce_noalloc uses.  Entry points may be called from several host threads.
 */
#ifndef IRIS_HIP_H
#define IRIS_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Element types (in_dtype / out_dtype / bias_dtype arguments). */
enum {
  IRIS_HIP_BF16 = 0,
  IRIS_HIP_FP16 = 1,
  IRIS_HIP_FP32 = 2,
  IRIS_HIP_FP8_E4M3 = 3 /* OCP e4m3fn, inputs only; products are multiplied by `scale` */
};

/* All-reduce variants (the strings of FusedConfig.all_reduce_variant, iris/ops/config.py:62), numbered
 * like AllReduceConfig.variant_code (iris/mem/triton/types.py:285-292). */
enum {
  IRIS_HIP_VARIANT_ATOMIC = 0,   /* iris/mem/triton/context.py:689-702 */
  IRIS_HIP_VARIANT_ONE_SHOT = 2, /* iris/mem/triton/context.py:733-764 */
  IRIS_HIP_VARIANT_TWO_SHOT = 3  /* iris/mem/triton/context.py:801-839 */
};

/* How the slot sum is carried (acc_mode). */
enum {
  IRIS_HIP_ACC_FP32 = 0,     /* fp32 running sum, one final cast */
  IRIS_HIP_ACC_REFERENCE = 1 /* the reference rule: fp32 only for fp16 data, else the data type
                                (bf16 sums are re-rounded after every add; context.py:752) */
};

/* Which A rows/columns come from which slot in iris_hip_all_gather_matmul (gather_dim). */
enum {
  IRIS_HIP_GATHER_K = 1, /* reference layout: slot r holds A[:, r*K_local:(r+1)*K_local] */
  IRIS_HIP_GATHER_M = 2  /* slot r holds A[r*M_local:(r+1)*M_local, :]                    */
};

/* Kernel selection (path). */
enum {
  IRIS_HIP_PATH_AUTO = 0,   /* MFMA kernel when the operands qualify, else the generic kernel */
  IRIS_HIP_PATH_MFMA = 1,   /* MFMA kernel or hipErrorInvalidValue */
  IRIS_HIP_PATH_GENERIC = 2 /* generic kernel */
};

/* Codes stored to *status by a kernel. */
enum {
  IRIS_HIP_STATUS_SPIN_TIMEOUT = 1 /* a peer flag did not become 1 within spin_limit polls */
};

/*
 * Fused C = all_reduce(A @ B), rank-local part.
 * Replaces the launch of _fused_matmul_all_reduce_kernel
 * (iris/ops/matmul_all_reduce.py:334-362; kernel :25-145) for VARIANT atomic / one_shot / two_shot.
 *
 * atomic: cast(A @ B) is added atomically into C of every slot (aux_buffer and locks may be NULL).
 *
 * Per flag tile t = pid_m * cdiv(N, block_size_n) + pid_n of block_size_m x block_size_n elements:
 *   aux[tile]   = cast(A @ B)              (own slot)
 *   locks[t]    = 1                        (own slot, after the aux stores are visible)
 *   one_shot:   C[tile] = cast(own + sum_{r != cur_rank, ascending} aux@r[tile]) after locks@r[t] == 1
 *   two_shot:   the same, only if t % world_size == cur_rank, and the result is also stored to
 *               C@r[tile] for every other slot r.
 * aux is addressed with C's strides, as the reference does (matmul_all_reduce.py:128).
 *
 * block_size_k is accepted for signature parity and does not change any result.
 * scale multiplies the fp32 product before the cast (use scale_a*scale_b for fp8, 1.0f otherwise).
 * spin_limit <= 0 spins without bound like the reference; > 0 gives up after that many polls of one
 * flag and stores IRIS_HIP_STATUS_SPIN_TIMEOUT to *status (status may be NULL; device memory or
 * device-visible pinned host memory).
 */
int iris_hip_matmul_all_reduce(const void* A, const void* B, void* C, void* aux_buffer, int32_t* locks,
                               int64_t M, int64_t N, int64_t K,
                               int64_t stride_am, int64_t stride_ak,
                               int64_t stride_bk, int64_t stride_bn,
                               int64_t stride_cm, int64_t stride_cn,
                               const int64_t* context_tensor, int32_t cur_rank, int32_t world_size,
                               int32_t block_size_m, int32_t block_size_n, int32_t block_size_k,
                               int32_t variant,
                               int32_t in_dtype, int32_t out_dtype, float scale, int32_t acc_mode,
                               int64_t spin_limit, int32_t* status, int32_t path, void* stream);

/*
 * iris_hip_matmul_all_reduce for a single rank (world_size 1: C = cast(A @ B), the reference's own
 * single-rank test configuration) WITHOUT a caller-provided workspace and without any allocation.
 *
 * It has no counterpart in the reference, whose operators always allocate their workspace
 * (iris/ops/matmul_all_reduce.py:191-219).  It is for callers that cannot allocate: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  The aux buffer, the tile flags and the
 * one-rank context the kernels need live in a static device array of the library
 * (IRIS_HIP_NOALLOC_MAX_AUX_BYTES + 64 KiB + 256 bytes on every GPU the library runs on, held until the
 * process ends).  The call runs every argument check first (a rejected call enqueues nothing), then
 * launches a small kernel that clears the flags it is going to use and then the same kernels as
 * iris_hip_matmul_all_reduce; it calls no hipMalloc / hipFree.  On first use per device the library looks up
 * the array's address (hipGetSymbolAddress) and, per kernel build, sets the kernel's dynamic-LDS attribute:
 * before capturing calls into a HIP graph, call iris_hip_query() for the device and make one eager call of
 * each shape class that will be captured, so that nothing but kernel launches happens under capture.
 *
 * Limits (hipErrorInvalidValue with a message otherwise): the bytes aux spans with C's strides,
 * ((M-1)*stride_cm + (N-1)*stride_cn + 1) * sizeof(out element), at most IRIS_HIP_NOALLOC_MAX_AUX_BYTES;
 * cdiv(M, block_size_m) * cdiv(N, block_size_n) at most IRIS_HIP_NOALLOC_MAX_FLAGS; variant one_shot or
 * two_shot.  Every call on a GPU uses that GPU's one array: calls that overlap on one GPU (two streams,
 * two threads) race on it and must be ordered by the caller.
 */
#define IRIS_HIP_NOALLOC_MAX_AUX_BYTES (32 * 1024 * 1024)
#define IRIS_HIP_NOALLOC_MAX_FLAGS 16384
int iris_hip_matmul_all_reduce_noalloc(const void* A, const void* B, void* C,
                                       int64_t M, int64_t N, int64_t K,
                                       int64_t stride_am, int64_t stride_ak,
                                       int64_t stride_bk, int64_t stride_bn,
                                       int64_t stride_cm, int64_t stride_cn,
                                       int32_t block_size_m, int32_t block_size_n, int32_t block_size_k,
                                       int32_t variant,
                                       int32_t in_dtype, int32_t out_dtype, float scale,
                                       int32_t path, void* stream);

/*
 * Fused C = reduce_scatter(A @ B), rank-local part.
 * Replaces the launch of _fused_matmul_reduce_scatter_kernel
 * (iris/ops/matmul_reduce_scatter.py:261-288; kernel :25-118; DeviceContext.reduce_scatter
 * iris/mem/triton/context.py:953-997).
 *
 * aux and locks are written for every tile as above.  Flag tile t is owned by
 * min(t / (tiles / world_size), world_size - 1); an owned tile is summed over the slots and stored to
 * C in slot cur_rank at the tile's global coordinates.
 *
 * Two switches that the reference does not have serve a single GPU standing in for all W ranks:
 *   all_owners != 0: the launch reduces every tile and stores tile t into C of slot owner(t).
 *   sum_peers  == 0: peers contribute nothing (their flags are not read, their aux not loaded).
 * The reference behaviour is all_owners = 0, sum_peers = 1.
 */
int iris_hip_matmul_reduce_scatter(const void* A, const void* B, void* C, void* aux_buffer, int32_t* locks,
                                   int64_t M, int64_t N, int64_t K,
                                   int64_t stride_am, int64_t stride_ak,
                                   int64_t stride_bk, int64_t stride_bn,
                                   int64_t stride_cm, int64_t stride_cn,
                                   const int64_t* context_tensor, int32_t cur_rank, int32_t world_size,
                                   int32_t block_size_m, int32_t block_size_n, int32_t block_size_k,
                                   int32_t all_owners, int32_t sum_peers,
                                   int32_t in_dtype, int32_t out_dtype, float scale, int32_t acc_mode,
                                   int64_t spin_limit, int32_t* status, int32_t path, void* stream);

/*
 * Fused C = all_gather(A_sharded) @ B (+ bias[:, None]), rank-local part (pull pattern).
 * Replaces the launch of _fused_all_gather_matmul_kernel
 * (iris/ops/all_gather_matmul.py:266-300; kernel :26-159; DeviceContext.gather
 * iris/mem/triton/context.py:866-888).
 *
 * A_sharded points at the shard in slot cur_rank; the shard of slot r sits at the same heap offset.
 * gather_dim = IRIS_HIP_GATHER_K: A_sharded is M x K_local, K == world_size * K_local, and the
 *   reduction runs over slot 0's columns, then slot 1's, ... (all_gather_matmul.py:94-122).
 * gather_dim = IRIS_HIP_GATHER_M: A_sharded is (M / world_size) x K; output row m uses slot
 *   m / (M / world_size).  K_local must equal K.
 * bias (may be NULL) is a per-row vector of M elements of type bias_dtype, added in fp32 before the
 * cast (all_gather_matmul.py:147-150).
 */
int iris_hip_all_gather_matmul(const void* A_sharded, const void* B, void* C, const void* bias,
                               int64_t M, int64_t N, int64_t K, int64_t K_local,
                               int64_t stride_am, int64_t stride_ak,
                               int64_t stride_bk, int64_t stride_bn,
                               int64_t stride_cm, int64_t stride_cn, int64_t stride_bias,
                               const int64_t* context_tensor, int32_t cur_rank, int32_t world_size,
                               int32_t block_size_m, int32_t block_size_n, int32_t block_size_k,
                               int32_t gather_dim,
                               int32_t in_dtype, int32_t out_dtype, int32_t bias_dtype, float scale,
                               int32_t path, void* stream);

/*
 * Fused C_gathered = all_gather(A @ B (+ bias[:, None])) along rows, rank-local part (scatter pattern).
 * Replaces the launch of _fused_matmul_all_gather_kernel (iris/ops/matmul_all_gather.py:27-105, launch
 * :222-262; DeviceContext.all_gather iris/mem/triton/context.py:841-864).
 *
 * A is M_local x K; the product tile is cast and stored into rows [cur_rank*M_local, (cur_rank+1)*M_local)
 * of C_gathered (M x N, M = M_local * world_size) in EVERY slot.  bias (may be NULL) has M_local elements.
 */
int iris_hip_matmul_all_gather(const void* A, const void* B, void* C_gathered, const void* bias,
                               int64_t M_local, int64_t M, int64_t N, int64_t K,
                               int64_t stride_am, int64_t stride_ak,
                               int64_t stride_bk, int64_t stride_bn,
                               int64_t stride_cm_gathered, int64_t stride_cn_gathered, int64_t stride_bias,
                               const int64_t* context_tensor, int32_t cur_rank, int32_t world_size,
                               int32_t block_size_m, int32_t block_size_n, int32_t block_size_k,
                               int32_t in_dtype, int32_t out_dtype, int32_t bias_dtype, float scale,
                               int32_t path, void* stream);

/* Tile-to-rank distribution of the two-shot collectives (Config.all_reduce_distribution,
 * iris/ccl/config.py:42-43). */
enum {
  IRIS_HIP_DISTRIBUTION_STRIDED = 0, /* rank r owns tiles r, r+W, r+2W, ...                      */
  IRIS_HIP_DISTRIBUTION_BLOCK = 1    /* rank r owns tiles [r*ceil(T/W), min((r+1)*ceil(T/W), T)) */
};

/*
 * Stand-alone all-reduce over the symmetric heap: output = sum over the group's ranks of input,
 * rank-local part.  Replaces the launches in iris/ccl/triton/all_reduce.py:762-956 of
 *   persistent_all_reduce_atomic    (:120-215)  variant IRIS_HIP_VARIANT_ATOMIC
 *   persistent_all_reduce_one_shot  (:345-423)  variant IRIS_HIP_VARIANT_ONE_SHOT
 *   persistent_all_reduce_two_shot  (:574-706)  variant IRIS_HIP_VARIANT_TWO_SHOT
 * with the arguments of those launches, in order, then variant, distribution, element type, stream.
 *
 * input and output are M x N tensors in the slot of `iris_rank` (strides in elements); the copy in
 * the slot of rank q sits at the same heap offset.  The group is the ranks
 * rank_start + i*rank_stride, i in [0, world_size); group_rank is this rank's index in it.
 *   one_shot: every element = cast(fp32 sum of the group's inputs, in group order, starting from 0),
 *             stored to the own output.
 *   two_shot: tile ids run over the block_size_m x block_size_n grid in the grouped order of
 *             swizzle_size tile-rows (all_reduce.py:628-633).  The rank reduces the tiles the
 *             distribution gives it; the j-th of them (j = 0, 1, ...) is summed in fp32 starting at
 *             group index (j mod comm_sms) mod world_size and going round cyclically (:663-669), cast
 *             once, and stored to the output of every rank of the group.
 *   atomic:   the own input is added atomically into the output of every rank of the group
 *             (outputs must have been zeroed; all_reduce.py:83-85).
 * comm_sms takes part in the two-shot summation order as above; the launch itself sizes its grid to
 * the machine.  num_xcds and chunk_size are accepted for signature parity and change no result.
 * dtype is IRIS_HIP_BF16, IRIS_HIP_FP16 or IRIS_HIP_FP32 (input and output alike).
 */
int iris_hip_all_reduce(const void* input, void* output, int64_t M, int64_t N,
                        int64_t stride_in_m, int64_t stride_in_n,
                        int64_t stride_out_m, int64_t stride_out_n,
                        const int64_t* heap_bases,
                        int32_t group_rank, int32_t iris_rank, int32_t world_size,
                        int32_t rank_start, int32_t rank_stride,
                        int32_t block_size_m, int32_t block_size_n, int32_t swizzle_size,
                        int32_t comm_sms, int32_t num_xcds, int32_t chunk_size,
                        int32_t variant, int32_t distribution, int32_t dtype, void* stream);

/*
 * Stand-alone reduce-scatter over the symmetric heap, rank-local part: the two-shot reduction above
 * with the result stored to the own output only.  Replaces the launch of
 * persistent_reduce_scatter_two_shot (iris/ccl/triton/reduce_scatter.py:160-190; kernel :16-140).
 */
int iris_hip_reduce_scatter(const void* input, void* output, int64_t M, int64_t N,
                            int64_t stride_in_m, int64_t stride_in_n,
                            int64_t stride_out_m, int64_t stride_out_n,
                            const int64_t* heap_bases,
                            int32_t group_rank, int32_t iris_rank, int32_t world_size,
                            int32_t rank_start, int32_t rank_stride,
                            int32_t block_size_m, int32_t block_size_n, int32_t swizzle_size,
                            int32_t comm_sms, int32_t num_xcds, int32_t chunk_size,
                            int32_t distribution, int32_t dtype, void* stream);

/*
 * Optional: tell the library what a context tensor holds.  `context_tensor` is the device pointer that
 * later launches pass; `host_copy` points at the same `num_words` int64 words in host memory
 * ([cur_rank, world_size, heap_base_0 .. heap_base_{W-1}, ...], iris/host/iris.py:916-958).  Launches
 * that name a registered context tensor (same pointer, rank and world size, at most 8 ranks) get the
 * heap bases as kernel arguments instead of loading them on the device, which takes a dependent memory
 * round trip (about 1 us) off the path to the peers' flags and tiles; the decode-sized kernel probes
 * the peers' flags ahead of its operand loads only then.  Results do not depend on registration.
 * The contents of a registered tensor must not change, and it must be unregistered before its memory is
 * freed or reused.  No counterpart in the reference (Triton reads the tensor on the device).
 */
int iris_hip_register_context(const int64_t* context_tensor, const int64_t* host_copy, int32_t num_words);
int iris_hip_unregister_context(const int64_t* context_tensor);

/*
 * Tail policy of the 256x256 tile (no counterpart in the reference, whose persistent schedule hands
 * tiles out whole: iris/ops/all_gather_matmul.py:71-79).  When the tile count leaves the last round of
 * workgroups partly empty for many K steps, the K steps of that round's tiles are shared out evenly
 * between all workgroups; a tile that ends up in several shares is summed from fp32 partial sums that
 * travel through a workspace of the library (64 MiB + 1 KiB per (device, stream), allocated with
 * hipMalloc on the stream's first such launch, kept until the process ends, at most 8 per device).
 * Launches on a capturing stream are never split: the flag value that tells this launch's partial sums
 * from the previous launch's is a kernel argument and would repeat on every replay.
 * mode: -1 the library decides per launch (default: when the split round is expected to be at least 16 K
 * steps and an eighth shorter than a whole tile), 0 never split, 1 split whenever the last round is not
 * full and its tiles have at least 4 K steps (a test setting), 2 split whenever any gain is expected (a
 * tuning aid).  The environment variable IRIS_HIP_STREAMK sets the initial mode.  A split launch differs
 * from an unsplit one only in the order of the fp32 sums over K.
 */
void iris_hip_set_split_tiles(int32_t mode);

/*
 * Device facts used by the host layer (reference: get_cu_count / get_num_xcc,
 * iris/host/platform/hip.py:138,218).  Any output pointer may be NULL.
 */
int iris_hip_query(int32_t device, int32_t* cu_count, int32_t* xcc_count, int32_t* lds_bytes_per_block);

/* Text of the last argument error reported on the calling thread ("" if none). */
const char* iris_hip_last_error(void);

/* Name of the kernel configuration the last successful launch on the calling thread used. */
const char* iris_hip_last_kernel(void);

/* ABI version of this header. */
int iris_hip_abi_version(void);

#ifdef __cplusplus
}
#endif

#endif /* IRIS_HIP_H */
