// Small outputs - decode-sized launches (a few rows) and, more generally, outputs of at most two
// 32 x 32 tiles per CU - of every operator: fused_decode_kernel.  The description
// follows the flag-carrying operators; the others leave after the partial tiles have met.
//
// With so few rows the GEMM is a stream of B through the machine (config "fp8, M = 32, N = 8192,
// K = 1024": 8 MB of B, 0.5 GFLOP) and the launch is a chain of memory round trips.  The tiled kernel
// gives such a problem N / 128 workgroups (64 of 256 CUs for N = 8192) and walks K in ring steps; this
// one is built for latency instead:
//   * 32 x 32 output tiles, so N / 32 workgroups (256 for N = 8192) pull B at the same time; the
//     workgroups that share a 128-byte line of B sit on the same XCD;
//   * the four waves split K: in every chunk of 1024 bytes of K each wave owns 256 bytes (512 and 128 in the
//     build the host takes when there are more tiles than CUs - two workgroups then share a CU - or when K
//     is short), loads exactly
//     the operand bytes it multiplies (direct-to-LDS, into a region no other wave touches) and waits for
//     nothing but its own loads - the K phase has no workgroup barrier; problems whose K fits one or two
//     chunks (K <= 2048 bytes with 256-byte shares, 1024 with 128-byte shares) have every operand load in
//     flight from the first instruction on;
//   * a fifth wave multiplies nothing.  Its first instructions, issued while the other four waves still
//     set up their loaders, are probes of the peers' flags (direct-to-LDS, system scope): the oldest loads
//     of the CU.  That matters because a CU's vector memory pipeline returns in order - a probe issued
//     behind the operand loads, by any wave, comes back only after all of them (measured: 4 us instead
//     of 1; scalar loads fare no better, they queue behind the operand stream in L2).  When all flags
//     are already up - the normal case for a rank that is not the first to finish - the helper loads the
//     peers' tiles into LDS while the others multiply, so the slot sum finds them there.  Otherwise the
//     flags are polled after the own tile is published, as in the tiled kernel.  Probing needs the peers'
//     heap bases without a load of their own, i.e. as kernel arguments (FusedParams::hb_in_args);
//   * the four partial accumulators meet in LDS; 256 threads then own one 8-byte piece of the output
//     tile each: scale, cast, aux store (written through), slot sum in ascending rank order and C store
//     (before the flags when the peers' tiles are already there, after them otherwise), flags.
// Results are bit-identical to the tiled kernel's whenever the fp32 sums over K are exact, and within
// fp32 rounding of each other otherwise (the K sum is split four ways here).
#pragma once

typedef __attribute__((ext_vector_type(4))) float f32x4_t;

template <int IN_, bool B_KCONTIG_, int QB_ = 256>
struct DecodeCfg {
  static_assert(QB_ == 128 || QB_ == 256, "a wave owns 128 or 256 bytes of K per chunk");
  static constexpr int IN = IN_;
  static constexpr bool B_KCONTIG = B_KCONTIG_;
  static constexpr int ES = (IN_ == IN_FP8) ? 1 : 2;
  static constexpr int CE = kChunkBytes / ES;
  static constexpr int KM = (IN_ == IN_FP8) ? 64 : 16;   // k per MFMA
  static constexpr int NFRAG = (IN_ == IN_FP8) ? 2 : 1;
  static constexpr int BM = 32, BN = 32, NW = 4;  // NW waves multiply
  static constexpr int NT = 64 * (NW + 1);         // ... and one more probes flags and fetches the peers' tiles
  static constexpr int QB = QB_;                  // bytes of K one wave owns per chunk
  static constexpr int KQ = QB / ES;              // ... in elements
  static constexpr int CHUNK = NW * KQ;           // k elements per chunk of the workgroup
  static constexpr int NSL = KQ / KM;             // MFMAs per wave and chunk
  static constexpr int RBB = B_KCONTIG ? QB : BN * ES;  // bytes per row of a wave's B region
  static constexpr int A_BYTES = BM * QB;         // 8 KiB (4 KiB with 128-byte shares)
  static constexpr int B_BYTES = BN * QB;         // [32 n][QB B] or [KQ k][32 * ES B]
  static constexpr int WAVE_BYTES = A_BYTES + B_BYTES;
  static constexpr int BUF_BYTES = NW * WAVE_BYTES;       // one chunk of the workgroup: 64 KiB (32 KiB)
  static constexpr int LOADS = WAVE_BYTES / kDmaBytes;    // direct-to-LDS loads per wave and chunk: 16 (8)
  static constexpr int RED_STRIDE = 36;                   // floats per row of a partial accumulator
  static constexpr int MAX_PEERS = 7;
  static constexpr int PEER_BYTES = BM * BN * 2;          // one peer's 32 x 32 tile of 16-bit values
  // LDS map: peers' tiles, probe words, one word of workgroup state, then the two operand buffers.
  static constexpr int PEER_AREA = 0;
  static constexpr int PROBE_AREA = PEER_AREA + MAX_PEERS * PEER_BYTES;
  static constexpr int WORD_AREA = PROBE_AREA + MAX_PEERS * 256;
  static constexpr int OPERANDS = WORD_AREA + 256;  // 16 KiB
  static constexpr int SMEM_BYTES = OPERANDS + 2 * BUF_BYTES;  // 144 KiB: one workgroup per CU; 80 KiB: two
  static_assert(BM * RED_STRIDE * 4 <= WAVE_BYTES, "a wave's partial tile reuses its own operand region");
  static_assert(SMEM_BYTES <= 160 * 1024, "LDS budget of a gfx950 CU");
};

// 4-byte direct-to-LDS load at system scope: lane l deposits its dword at lds_base + 4*l (zero when out
// of range).
__device__ __forceinline__ void dma4(i32x4_t rsrc, unsigned lds_base, unsigned voff) {
  asm volatile("s_mov_b32 m0, %0\n\tbuffer_load_dword %1, %2, 0 offen sc0 sc1 lds"
               :
               : "s"(lds_base), "v"(voff), "s"(rsrc)
               : "memory");
}

// 8-byte store written through to memory at system scope (see store16_system).
__device__ __forceinline__ void store8_system(char* p, u32x2_t v) {
  asm volatile("global_store_dwordx2 %0, %1, off sc0 sc1" : : "v"(p), "v"(v) : "memory");
}

// 16-byte direct-to-LDS load at system scope (sc0 sc1): served from where every agent's writes are visible.
__device__ __forceinline__ void dma16_system(i32x4_t rsrc, unsigned lds_base, unsigned voff) {
  asm volatile("s_mov_b32 m0, %0\n\tbuffer_load_dwordx4 %1, %2, 0 offen sc0 sc1 lds"
               :
               : "s"(lds_base), "v"(voff), "s"(rsrc)
               : "memory");
}

template <int IN, bool BKC, int QB>
__global__ void __launch_bounds__(320) fused_decode_kernel(const FusedParams p_in) {
  using CFG = DecodeCfg<IN, BKC, QB>;
  using Out = typename OutOf<IN>::type;
  using ATile = RowTile<CFG::QB>;
  constexpr int ES = CFG::ES, CE = CFG::CE, NFRAG = CFG::NFRAG, LOADS = CFG::LOADS, MAXP = CFG::MAX_PEERS;

  extern __shared__ __attribute__((aligned(1024))) char smem[];
  // Every kernel argument is fetched here, in one batch.  Left to itself the compiler loads each field
  // next to its first use and waits for it there; on this latency-bound kernel that put some twenty
  // dependent scalar round trips (1.7 us) in front of the first operand load.
  const FusedParams q = pin_kernel_arguments(p_in);
  const FusedParams& p = q;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // Tiles are numbered with the row tile running fastest, so that the workgroups that read the same
  // columns of B (and those that share its 128-byte lines) are neighbours and land on one XCD.
  const int tidx = xcd_tile_index(blockIdx.x, gridDim.x, 0, p.tiles_m * p.tiles_n, p.num_xcd);
  if (tidx < 0) return;
#ifdef IRIS_HIP_PHASE_STAMPS
  constexpr int it = 0;  // PHASE_STAMP records the first tile of a workgroup; there is only one here
#endif
  PHASE_STAMP(0);
  const int m0 = (tidx % p.tiles_m) * CFG::BM;
  const int n0 = (tidx / p.tiles_m) * CFG::BN;
  const unsigned smem_base = __builtin_amdgcn_readfirstlane(lds_address(smem));

  // Heap bases: kernel arguments when the host knew them, else eight independent loads behind one
  // branch (slots past the world size repeat the last one, so that every load is in bounds).
  unsigned long long hb[kMaxCachedSlots];
  if (p.hb_in_args) {
#pragma unroll
    for (int r = 0; r < kMaxCachedSlots; ++r) hb[r] = (unsigned long long)p.hb_arg[r];
  } else {
#pragma unroll
    for (int r = 0; r < kMaxCachedSlots; ++r) hb[r] = (unsigned long long)p.heap_bases[min(r, p.world - 1)];
  }
#pragma unroll
  for (int r = 0; r < kMaxCachedSlots; ++r) hb[r] = uniform64(hb[r]);  // scalar registers, whichever branch ran
  unsigned long long hb_own = 0ull;
#pragma unroll
  for (int r = 0; r < kMaxCachedSlots; ++r) hb_own = (r == p.rank) ? hb[r] : hb_own;
  auto heap_base = [&](int r) -> unsigned long long {
    unsigned long long v = 0;
#pragma unroll
    for (int q = 0; q < kMaxCachedSlots; ++q) v = (r == q) ? hb[q] : v;
    return v;
  };
  auto in_slot = [&](unsigned long long own, int r) -> unsigned long long { return heap_base(r) + (own - hb_own); };
  // Slots of the peers in ascending rank order, own rank skipped.
  auto peer_slot = [&](int i) { return i < p.rank ? i : i + 1; };

  const bool flagged = epi_has_flags(p.epi);  // else: plain store, all-gather or atomic epilogue - no aux, no flags
  const bool solo = !flagged || !p.sum_peers || p.world == 1;
  const int npeers = solo ? 0 : p.world - 1;
  const int fbm = flagged ? p.flag_bm : CFG::BM, fbn = flagged ? p.flag_bn : CFG::BN;  // no flag tiles without flags
  const int ftn = cdiv(p.N, fbn);
  const int ftotal = cdiv(p.M, fbm) * ftn;
  const int m1 = min(m0 + CFG::BM, p.M), n1 = min(n0 + CFG::BN, p.N);
  const int fm_lo = m0 / fbm, fm_hi = (m1 - 1) / fbm;
  const int fn_lo = n0 / fbn, fn_hi = (n1 - 1) / fbn;
  const int nfn = fn_hi - fn_lo + 1;
  const int nft = (fm_hi - fm_lo + 1) * nfn;  // flag tiles under this output tile

  const bool helper = wave == CFG::NW;  // the wave that multiplies nothing
  const bool probing = helper && !solo && nft <= 64 && p.hb_in_args;

  // ---- helper wave: flag probe, then the peers' tiles -------------------------------------------------
  if (probing) {
    // Slot bases of the peers in ascending rank order (one select each).
    unsigned long long pbase[MAXP];
#pragma unroll
    for (int i = 0; i < MAXP; ++i) pbase[i] = i < p.rank ? hb[i] : hb[i + 1 < kMaxCachedSlots ? i + 1 : i];
    int t = 0;
    bool must_check = false;  // this lane's flag tile is one this rank reduces
    if (lane < nft) {
      t = (fm_lo + lane / nfn) * ftn + fn_lo + lane % nfn;
      must_check = p.all_owners || owner_of(p.epi, t, ftotal, p.world, p.rank) == p.rank;
    }
    const unsigned voff = must_check ? (unsigned)t * 4u : kInvalidOffset;
    const unsigned long long locks_off = (unsigned long long)p.locks - hb_own;
    for (int i = 0; i < npeers; ++i) dma4(make_rsrc_words(pbase[i] + locks_off), smem_base + CFG::PROBE_AREA + i * 256, voff);
    __builtin_amdgcn_s_barrier();  // the multiplying waves hold their operand loads back until the probes are out
    wait_vmcnt<0>();
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("" ::: "memory");
    bool ok = true;
    for (int i = 0; i < npeers; ++i) {
      const int v = *(const LDS_AS int*)(LDS_AS char*)(smem + CFG::PROBE_AREA + i * 256 + lane * 4);
      if (must_check && v != 1) ok = false;
    }
    const bool early = __builtin_amdgcn_readfirstlane(__all(ok) ? 1 : 0) != 0;
    if (early) {
      // System-scope loads, issued after the flags were seen up: they observe what the flags' writers
      // published, without an invalidation of this CU's and XCD's caches.
      const unsigned long long aux_off = (unsigned long long)p.aux - hb_own;
      unsigned pv_off[2];
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int q = lane + 64 * h, prow = q >> 2, pc = q & 3;
        pv_off[h] = (m0 + prow < p.M && n0 + 8 * pc < p.N) ? (unsigned)(((long long)(m0 + prow) * p.s_cm + n0 + 8 * pc) * 2) : kInvalidOffset;
      }
      for (int i = 0; i < npeers; ++i) {
        const i32x4_t rs = make_rsrc_words(pbase[i] + aux_off);
#pragma unroll
        for (int h = 0; h < 2; ++h)
          dma16_system(rs, smem_base + CFG::PEER_AREA + i * CFG::PEER_BYTES + h * kDmaBytes, pv_off[h]);
      }
    }
    if (lane == 0) *(LDS_AS int*)(LDS_AS char*)(smem + CFG::WORD_AREA) = early ? 1 : 0;
    // The helper has nothing else to do: it waits here for the peers' tiles, so that behind the barrier
    // that ends the K phase they are known to be in LDS.
    wait_vmcnt<0>();
  }

  // ---- operand loaders ---------------------------------------------------------------------------
  // Per lane and load: byte offset inside the operand and the k byte (A, K-contiguous B) or k row
  // (row-major B) it covers relative to the wave's first k of a chunk.
  // A gathered from the ranks' slots (iris/mem/triton/context.py:866-888): by rows, the tile's 32 rows
  // come from one slot (the host admits row gathering only for whole tiles per slot); by columns, the
  // slot changes along K and is looked up per chunk below.
  const unsigned long long a_own = (unsigned long long)p.A;
  unsigned long long a_base = a_own;
  int a_row0 = m0;
  if (p.gather == GATHER_M) {
    const int src = m0 / p.M_local;
    a_base = in_slot(a_own, src);
    a_row0 = m0 - src * p.M_local;
  }
  unsigned a_voff[LOADS / 2], b_voff[LOADS / 2];
  int a_kb[LOADS / 2], b_k[LOADS / 2];
#pragma unroll
  for (int i = 0; i < LOADS / 2; ++i) {
    int row, c;
    ATile::from_lds(i * kDmaBytes + lane * kChunkBytes, row, c);
    a_kb[i] = c * kChunkBytes;
    a_voff[i] = m0 + row < p.M ? (unsigned)((a_row0 + row) * p.s_am * ES + c * kChunkBytes) : kInvalidOffset;
    if constexpr (BKC) {
      b_k[i] = c * kChunkBytes;
      b_voff[i] = n0 + row < p.N ? (unsigned)(row * p.s_bn * ES + c * kChunkBytes) : kInvalidOffset;
    } else {
      const int off = i * kDmaBytes + lane * kChunkBytes;
      const int krow = off / CFG::RBB, cc = (off % CFG::RBB) / kChunkBytes;
      b_k[i] = krow;
      b_voff[i] = n0 + cc * CE < p.N ? (unsigned)(krow * p.s_bk * ES + cc * kChunkBytes) : kInvalidOffset;
    }
  }
  i32x4_t ra = make_rsrc_words(a_base);
  const int klb = p.K_local * ES;  // bytes of K one slot holds when A is gathered along K (a multiple of QB)
  const i32x4_t rb = make_rsrc_words((unsigned long long)p.B + (unsigned long long)n0 * (BKC ? p.s_bn : 1) * ES);
  const int kbytes = p.K * ES;
  const int nchunks = cdiv(kbytes, CFG::NW * CFG::QB);
  auto issue_chunk = [&](int ch) {  // this wave's loads of chunk ch
    const unsigned region = smem_base + CFG::OPERANDS + (ch & 1) * CFG::BUF_BYTES + wave * CFG::WAVE_BYTES;
    const int kb0 = (ch * CFG::NW + wave) * CFG::QB;  // first k byte of the wave in this chunk
    const int left = kbytes - kb0;                      // k bytes of this wave's share that exist
    unsigned a_soff = (unsigned)kb0;
    if (p.gather == GATHER_K) {  // the wave's bytes of K lie in one slot
      const int src = min(kb0 / klb, p.world - 1);
      ra = make_rsrc_words(in_slot(a_own, src));
      a_soff = (unsigned)(kb0 - src * klb);
    }
#pragma unroll
    for (int i = 0; i < LOADS / 2; ++i)
      dma16(ra, region + i * kDmaBytes, a_kb[i] < left ? a_voff[i] : kInvalidOffset, a_soff);
    const unsigned b_soff = __builtin_amdgcn_readfirstlane(BKC ? (unsigned)kb0 : (unsigned)((long long)(kb0 / ES) * p.s_bk * ES));
#pragma unroll
    for (int i = 0; i < LOADS / 2; ++i) {
      const bool live = BKC ? b_k[i] < left : b_k[i] * ES < left;
      dma16(rb, region + CFG::A_BYTES + i * kDmaBytes, live ? b_voff[i] : kInvalidOffset, b_soff);
    }
  };

  // ---- K phase of the four multiplying waves: no workgroup barrier -----------------------------------
  // A wave keeps at most two chunks in flight; its loads retire in issue order, so "chunk ch has landed"
  // is "at most the loads of the chunk after it are outstanding".  The operand loads go out before the
  // fragment addresses are worked out: every instruction ahead of them is latency of the whole launch.
  f32x16_t acc;
#pragma unroll
  for (int i = 0; i < 16; ++i) acc[i] = 0.f;
  int issued = 0;  // chunks whose loads have been issued
  const bool probes_first = !solo && nft <= 64 && p.hb_in_args;  // same condition in every wave
  if (!helper) {
    if (probes_first) __builtin_amdgcn_s_barrier();  // the helper's probes are the oldest loads of the CU
    issue_chunk(0);
    if (nchunks > 1) issue_chunk(1);
    issued = nchunks > 1 ? 2 : 1;
  }
  __builtin_amdgcn_sched_barrier(0);

  // ---- fragment addresses (inside a wave's region) --------------------------------------------------
  int fa_off[CFG::NSL][NFRAG], fb_off[CFG::NSL][BKC ? NFRAG : ((IN == IN_FP8) ? 4 : 2)];
#pragma unroll
  for (int kk = 0; kk < CFG::NSL; ++kk) {
#pragma unroll
    for (int h = 0; h < NFRAG; ++h) {
      const int c = (IN == IN_FP8) ? frag8_chunk(lane, kk, h) : frag16_chunk(lane, kk);
      fa_off[kk][h] = ATile::lds_offset(frag16_row(lane), c);
      if constexpr (BKC) fb_off[kk][h] = CFG::A_BYTES + ATile::lds_offset(frag16_row(lane), c);
    }
    if constexpr (!BKC) {
      // row-major B: the wave's region holds [k][32 columns] without swizzle; a half-wave of a
      // transpose read covers 256 contiguous bytes, one full sweep of the banks
      if constexpr (IN == IN_FP8) {
#pragma unroll
        for (int r = 0; r < 4; ++r)
          fb_off[kk][r] = CFG::A_BYTES + tr8_krow(lane, kk, r) * CFG::RBB + tr8_ncol(lane);
      } else {
#pragma unroll
        for (int j = 0; j < 2; ++j)
          fb_off[kk][j] = CFG::A_BYTES + tr16_krow(lane, kk, j) * CFG::RBB + tr16_ncol(lane) * 2;
      }
    }
  }

  for (int ch = 0; !helper && ch < nchunks; ++ch) {
    if (issued - ch - 1 > 0) wait_vmcnt<LOADS>(); else wait_vmcnt<0>();
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("" ::: "memory");
    if (ch == 0) PHASE_STAMP(1);
    const char* region = smem + CFG::OPERANDS + (ch & 1) * CFG::BUF_BYTES + wave * CFG::WAVE_BYTES;
#pragma unroll
    for (int kk = 0; kk < CFG::NSL; ++kk) {
      i32x4_t a[NFRAG], b[NFRAG];
#pragma unroll
      for (int h = 0; h < NFRAG; ++h) a[h] = *(const LDS_AS i32x4_t*)(LDS_AS char*)(region + fa_off[kk][h]);
      if constexpr (BKC) {
#pragma unroll
        for (int h = 0; h < NFRAG; ++h) b[h] = *(const LDS_AS i32x4_t*)(LDS_AS char*)(region + fb_off[kk][h]);
      } else if constexpr (IN == IN_FP8) {
        i32x2_t t[4];
#pragma unroll
        for (int r = 0; r < 4; ++r)
          t[r] = __builtin_amdgcn_ds_read_tr8_b64_v2i32((LDS_AS i32x2_t*)(LDS_AS char*)(region + fb_off[kk][r]));
        b[0] = (i32x4_t){t[0].x, t[0].y, t[1].x, t[1].y};
        b[NFRAG - 1] = (i32x4_t){t[2].x, t[2].y, t[3].x, t[3].y};
      } else {
        const i16x4_t t0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_AS i16x4_t*)(LDS_AS char*)(region + fb_off[kk][0]));
        const i16x4_t t1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_AS i16x4_t*)(LDS_AS char*)(region + fb_off[kk][1]));
        const i32x2_t u0 = __builtin_bit_cast(i32x2_t, t0), u1 = __builtin_bit_cast(i32x2_t, t1);
        b[0] = (i32x4_t){u0.x, u0.y, u1.x, u1.y};
      }
      acc = mfma_block<IN, NFRAG>(a, b, acc);
    }
    // Refill the buffer just read with the chunk after next (the wave's own reads have been consumed).
    if (issued < nchunks) {
      __builtin_amdgcn_s_waitcnt((0xF) | (0x3 << 14) | (0x7 << 4));  // lgkmcnt(0)
      __builtin_amdgcn_sched_barrier(0);
      issue_chunk(issued);
      ++issued;
    }
  }

  PHASE_STAMP(2);
  // ---- the four partial tiles meet in LDS ---------------------------------------------------------------
  // Each wave writes into its own operand region of buffer 0 (its reads there are long consumed).
  if (!helper) {
    float* part = (float*)(smem + CFG::OPERANDS + wave * CFG::WAVE_BYTES);
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int m = acc_col(lane), n = acc_row(lane, 4 * q);
      const f32x4_t v = {acc[4 * q], acc[4 * q + 1], acc[4 * q + 2], acc[4 * q + 3]};
      *(LDS_AS f32x4_t*)(LDS_AS char*)((char*)(part + m * CFG::RED_STRIDE + n)) = v;
    }
  }
  __syncthreads();
  PHASE_STAMP(3);

  // ---- epilogue: 256 threads, one 8-byte piece (4 values) of the tile each ----------------------------
  // (this part of the launch is bound by instruction issue: twice the threads, half the time)
  const bool worker = tid < 256;
  const int row = (tid >> 3) & 31, c = tid & 7;
  const int gm = m0 + row, gn = n0 + 4 * c;
  const bool valid = worker && gm < p.M && gn < p.N;
  const long long eoff = valid ? ((long long)gm * p.s_cm + gn) * 2 : 0;
  u32x2_t own = {0, 0};
  if (worker) {
    f32x4_t s4 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int w = 0; w < CFG::NW; ++w) {  // ascending k quarters
      const float* part = (const float*)(smem + CFG::OPERANDS + w * CFG::WAVE_BYTES) + row * CFG::RED_STRIDE + 4 * c;
      s4 += *(const LDS_AS f32x4_t*)(LDS_AS const char*)((const char*)part);
    }
    // per-row bias of the operators that have one (added in fp32, before the cast)
    const float badd = (p.bias && gm < p.M) ? load_scalar_as_float(p.bias, (long long)gm * p.s_bias, p.bias_dtype) : 0.f;
    own.x = Out::pack(s4.x * p.scale + badd, s4.y * p.scale + badd);
    own.y = Out::pack(s4.z * p.scale + badd, s4.w * p.scale + badd);
  }
  const unsigned long long c_own = (unsigned long long)p.C;
  if (!flagged) {
    // The operators without flags: the tile goes to C (plain GEMM), to every rank's gathered output at
    // this rank's row block (iris/mem/triton/context.py:841-864), or is added into every rank's C
    // (iris/mem/triton/context.py:689-702; two packed dwords per piece).
    if (valid) {
      const long long goff = ((long long)(gm + p.row_offset) * p.s_cm + gn) * 2;
      if (p.epi == EPI_ATOMIC) {
        for (int pr = 0; pr < p.world; ++pr) {
          char* dst = (char*)(in_slot(c_own, pr) + goff);
          atomic_add_packed<Out>(dst, own.x);
          atomic_add_packed<Out>(dst + 4, own.y);
        }
      } else if (p.epi == EPI_ALL_GATHER) {
        for (int pr = 0; pr < p.world; ++pr) __builtin_nontemporal_store(own, (u32x2_t*)(in_slot(c_own, pr) + goff));
      } else {
        __builtin_nontemporal_store(own, (u32x2_t*)(c_own + goff));
      }
    }
    PHASE_STAMP(4);
    return;
  }
  int owner = p.rank;
  if (p.epi != EPI_ONE_SHOT) owner = owner_of(p.epi, (gm / p.flag_bm) * ftn + gn / p.flag_bn, ftotal, p.world, p.rank);
  const bool reduces = valid && (p.all_owners || owner == p.rank);
  auto store_result = [&](const u32x2_t& v) {
    if (p.epi == EPI_TWO_SHOT) {
      for (int pr = 0; pr < p.world; ++pr) __builtin_nontemporal_store(v, (u32x2_t*)(in_slot(c_own, pr) + eoff));
    } else {
      const int dst = p.all_owners ? owner : p.rank;
      __builtin_nontemporal_store(v, (u32x2_t*)(in_slot(c_own, dst) + eoff));
    }
  };
  const bool ref_chain = (p.acc_mode == IRIS_HIP_ACC_REFERENCE) && !Out::kFp32SumInReference;
  const unsigned long long aux_own = (unsigned long long)p.aux;
  // Own tile + the peers' tiles in ascending rank order, cast once, stored where the operator says.
  auto reduce_and_store = [&](bool have_peers) {
    u32x2_t pv[MAXP];
#pragma unroll
    for (int i = 0; i < MAXP; ++i) {
      if (i < npeers) {
        if (have_peers) pv[i] = *(const LDS_AS u32x2_t*)(LDS_AS char*)(smem + CFG::PEER_AREA + i * CFG::PEER_BYTES + (tid & 255) * 8);
        else pv[i] = __builtin_nontemporal_load((const u32x2_t*)(in_slot(aux_own, peer_slot(i)) + eoff));
      }
    }
    float sum[4];
#pragma unroll
    for (int e = 0; e < 2; ++e) {
      sum[2 * e] = Out::to_float((unsigned short)(own[e] & 0xFFFF));
      sum[2 * e + 1] = Out::to_float((unsigned short)(own[e] >> 16));
    }
#pragma unroll
    for (int i = 0; i < MAXP; ++i) {
      if (i < npeers) {
#pragma unroll
        for (int e = 0; e < 2; ++e) {
          sum[2 * e] += Out::to_float((unsigned short)(pv[i][e] & 0xFFFF));
          sum[2 * e + 1] += Out::to_float((unsigned short)(pv[i][e] >> 16));
        }
        if (ref_chain) {
#pragma unroll
          for (int e = 0; e < 4; ++e) sum[e] = Out::to_float(Out::from_float(sum[e]));
        }
      }
    }
    u32x2_t res;
#pragma unroll
    for (int e = 0; e < 2; ++e)
      res[e] = Out::pack(sum[2 * e], sum[2 * e + 1]);
    store_result(res);
  };

  if (valid) store8_system(p.aux + eoff, own);  // read by the peers as soon as the flag is up
  if (solo && reduces) store_result(own);
  PHASE_STAMP(4);
  // When the helper found every flag up, the peers' tiles are in LDS by now (it waited for them before
  // the barrier above): the slot sum and the C stores go out right behind the aux stores, and one wait
  // covers both before the flags are raised - one memory round trip less in the chain.
  const bool have_peers = !solo && nft <= 64 && p.hb_in_args && *(const LDS_AS int*)(LDS_AS char*)(smem + CFG::WORD_AREA) != 0;
  if (have_peers && reduces) reduce_and_store(true);
  // Publish (as in the tiled kernel): stores acknowledged, workgroup barrier, flags.
  wait_vmcnt<0>();
  __syncthreads();
  PHASE_STAMP(5);
  raise_flags<CFG::BM, CFG::BN, CFG::NT, true>(p, m0, n0, tid);
  if (solo || have_peers) return;
  wait_peer_flags<CFG::BM, CFG::BN, CFG::NT>(p, m0, n0, tid);
  __syncthreads();
  PHASE_STAMP(6);
  if (reduces) reduce_and_store(false);
  PHASE_STAMP(7);
}

template <int IN, bool BKC, int QB>
int launch_decode(FusedParams& p, int device, hipStream_t stream, const char* name) {
  using CFG = DecodeCfg<IN, BKC, QB>;
  static std::atomic<bool> attr_set[64];
  if (device < 0 || device >= 64) return iris_host::fail("device index %d out of range", device);
  if (!attr_set[device].load(std::memory_order_acquire)) {
    hipError_t e = hipFuncSetAttribute((const void*)fused_decode_kernel<IN, BKC, QB>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, CFG::SMEM_BYTES);
    if (e != hipSuccess) return (int)e;
    attr_set[device].store(true, std::memory_order_release);
  }
  p.tiles_m = cdiv(p.M, CFG::BM);
  p.tiles_n = cdiv(p.N, CFG::BN);
  int grid = p.tiles_m * p.tiles_n;
  if (grid % p.num_xcd) grid += p.num_xcd - grid % p.num_xcd;  // the XCD mapping wants a multiple; surplus workgroups leave at once
  iris_host::set_last_kernel(name);
  hipLaunchKernelGGL((fused_decode_kernel<IN, BKC, QB>), dim3(grid), dim3(CFG::NT), CFG::SMEM_BYTES, stream, p);
  return (int)hipGetLastError();
}
