// 16-bit matmul / batch_matmul on 256 x BN x 64 tiles (BN = 256, 192 or 128), one workgroup per CU.
// Included by gemm.hip inside namespace llc::{anonymous} (uses GemmParams and the LDS-DMA helpers defined there).
//
// Why a second tile shape: a 128x128 tile needs 64 B/clk/CU of operands from L2 at the full MFMA rate and
// 192 B/clk of LDS traffic, both above what a CU gets; a 256x256 tile halves the first and, with 64x128 wave
// tiles, brings the second to 128 B/clk.
//
// Eight waves, two per SIMD, in two groups of four (waves w and w+4 share a SIMD).  A wave owns a
// 64 x BN/2 accumulator tile (group g = column half g, wave w of the group = row quarter w).  The groups
// run the same program half a step apart ("ping-pong"): per half k-tile (two MFMA k-steps) a wave first
// spends a MEMORY phase (issue its share of the next k-tile's direct-to-LDS loads, read the fragments
// of this half tile into registers, wait for them), then a COMPUTE phase (TM*TN*2 MFMAs at raised priority).
// Every phase ends at a workgroup barrier and group 1 enters the loop one barrier late, so in every barrier
// interval one wave of each SIMD issues MFMAs back to back while the other one issues the memory
// instructions.  Fragments need no double buffer (they are read in one phase and consumed in the next).
//
// LDS: NS stages of one k-tile each (A [256 m][128 B of k], then B as [BN n][128 B of k] or, row-major B,
// [64 k][2 BN B of n]), swizzled like the 128x128 kernels and filled by global_load_lds_dwordx4.  Stage of
// tile t-1 is reloaded with tile t+NS-1 in the first memory phase of tile t (every wave has read it by
// then: group 1's last read of tile t-1 ended one barrier earlier).  A wave waits for its own loads of tile
// t+1 before the barrier that ends the last phase of tile t (vmcnt counts in order, so the loads of later
// tiles may stay in flight).
//
// MFMA operands are swapped (C^T = B^T A^T per fragment pair): a lane then holds, per accumulator quad,
// four consecutive columns of ONE row, so the fused epilogue act(alpha acc + bias + residual) packs 8-byte
// groups, stages them in a wave-private LDS tile and stores row-major 16 bytes per lane.

template <int BN, int NS>
struct WideGeom {
  static constexpr int BM = 256;
  static constexpr int TM = 2, TN = BN / 64;          // 32x32 fragments per wave tile (64 x BN/2)
  static constexpr int WTN = BN / 2;
  static constexpr int kBOff = BM * 128;
  static constexpr int kStage = (BM + BN) * 128;
  static constexpr int kLoadsB = BN / 64;             // 1 KB slices per wave and tile: 4 of A, BN/64 of B
  static constexpr int kLoads = 4 + kLoadsB;
  static constexpr int kOutPitch = WTN * 2 + 16;      // bytes per row of a wave's 16-bit staging tile
  static constexpr int kOutWave = 64 * kOutPitch;
  static constexpr int kLds = NS * kStage > 8 * kOutWave ? NS * kStage : 8 * kOutWave;
};

#if defined(LLC_WIDE_ABL) && (LLC_WIDE_ABL & 4)
#define LLC_WAIT_VM_LOOP(VM)
#else
#define LLC_WAIT_VM_LOOP(VM) LLC_WAIT_VM(VM)
#endif
#define LLC_WAIT_VM(VM) __builtin_amdgcn_s_waitcnt(((VM) & 15) | (7 << 4) | (15 << 8) | (((VM) >> 4) << 14))
#define LLC_PHASE_END()                \
  __builtin_amdgcn_sched_barrier(0);   \
  __builtin_amdgcn_s_barrier();        \
  __builtin_amdgcn_sched_barrier(0)

#ifdef LLC_GEMM_TUNE
__device__ unsigned long long llc_dbg_clk[2];  // longest workgroup: shader clocks, 100 MHz ticks
#define LLC_DBG_T0() const long long dbg_c0 = clock64(), dbg_w0 = wall_clock64()
#define LLC_DBG_T1()                                                                   \
  if (threadIdx.x == 0) {                                                              \
    atomicMax(&llc_dbg_clk[0], (unsigned long long)(clock64() - dbg_c0));              \
    atomicMax(&llc_dbg_clk[1], (unsigned long long)(wall_clock64() - dbg_w0));         \
  }
#else
#define LLC_DBG_T0()
#define LLC_DBG_T1()
#endif

template <typename T, int BMODE, int BN, int NS>
__global__ __launch_bounds__(512) void gemm_wide_kernel(const GemmParams p) {
  static_assert(sizeof(T) == 2, "16-bit operands");
  static_assert(NS == 2 || NS == 3, "two or three LDS stages");
  static_assert(BMODE == kBKMajor || BN != 192, "row-major B: the chunk swizzle needs 16 or 32 chunks per row");
  using G = WideGeom<BN, NS>;
  constexpr int TM = G::TM, TN = G::TN;
  extern __shared__ __align__(16) char smem[];
  LLC_DBG_T0();
  int tile_m, tile_n;
  tile_of_block(p.tiles_m, p.tiles_n, tile_m, tile_n);
  const int m0 = tile_m * 256, n0 = tile_n * BN;
  const int z = blockIdx.z;
  const int z0 = z / p.bdiv, z1 = z - z0 * p.bdiv;
  const T* A = (const T*)p.A + (int64_t)z0 * p.a_sb + (int64_t)z1 * p.a_sb1;
  const T* B = (const T*)p.B + (int64_t)z0 * p.b_sb + (int64_t)z1 * p.b_sb1;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave), lane = threadIdx.x % kWave;
  const int grp = wave >> 2, wm = wave & 3, wn = grp;
  const int li = lane % 32, lh = lane / 32;
  const uint32_t lds0 = (uint32_t)(uintptr_t)smem;

  // ---- this wave's direct-to-LDS loads: slices wave + 8 j of the A tile (8 rows each), then of the B tile ----
  const char* ga[4];
  const char* gb[G::kLoadsB];
  int64_t b_step;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int row = (wave + 8 * j) * 8 + lane / 8;
    ga[j] = (const char*)(A + (int64_t)(m0 + row) * p.a_sm + (((lane % 8) ^ lds_swz(row)) << 3));
  }
#pragma unroll
  for (int j = 0; j < G::kLoadsB; ++j) {
    if constexpr (BMODE == kBKMajor) {
      const int row = (wave + 8 * j) * 8 + lane / 8;
      gb[j] = (const char*)(B + (int64_t)(n0 + row) * p.b_sn + (((lane % 8) ^ lds_swz(row)) << 3));
    } else {
      const int byte = (wave + 8 * j) * 1024 + lane * 16;
      const int krow = byte / (2 * BN), slot = (byte % (2 * BN)) / 16;
      gb[j] = (const char*)(B + (int64_t)krow * p.b_sk + n0 + ((slot ^ ((krow & 3) << 2)) << 3));
    }
  }
  if constexpr (BMODE == kBKMajor) b_step = 128;
  else b_step = 64 * p.b_sk * 2;
  auto issue = [&](int stage) {
    char* base = smem + stage * G::kStage;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      __builtin_amdgcn_global_load_lds(LLC_GPTR(ga[j]), LLC_LPTR(base + (wave + 8 * j) * 1024), 16, 0, 0);
      ga[j] += 128;
    }
#pragma unroll
    for (int j = 0; j < G::kLoadsB; ++j) {
      __builtin_amdgcn_global_load_lds(LLC_GPTR(gb[j]), LLC_LPTR(base + G::kBOff + (wave + 8 * j) * 1024), 16, 0, 0);
      gb[j] += b_step;
    }
  };

  // ---- fragment addresses.  k-major tiles: row r, 16-byte chunk c at r * 128 + ((c ^ swz(r)) << 4); lane half lh
  //      of k-step s takes chunk 2 s + lh: off = base + (x ^ (s << 5)) with x = (lh ^ swz) << 4. ----
  int a_base[TM], a_x[TM], b_base[TN], b_x[TN];
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int r = wm * 64 + i * 32 + li;
    a_base[i] = r * 128;
    a_x[i] = (lh ^ lds_swz(r)) << 4;
  }
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    if constexpr (BMODE == kBKMajor) {
      const int r = wn * G::WTN + j * 32 + li;
      b_base[j] = G::kBOff + r * 128;
      b_x[j] = (lh ^ lds_swz(r)) << 4;
    } else {
      // transposing read: lane = 16 g + 4 jj + q reads 8 bytes: k row 16 s + 8 (g >> 1) + 4 u + jj, n chunk
      // (16 (g & 1) + 4 q) / 8 of the fragment's 32 columns; slot = chunk ^ (jj << 2)
      const int g = lane / 16, jj = (lane / 4) % 4, q = lane % 4;
      const int nchunk = (wn * G::WTN + j * 32) / 8 + 2 * (g & 1) + (q >> 1);
      b_base[j] = G::kBOff + (8 * (g >> 1) + jj) * (2 * BN) + ((nchunk ^ (jj << 2)) << 4) + (q & 1) * 8;
      b_x[j] = 0;
    }
  }

  f32x16_t acc[TM][TN];  // register r of lane (li, lh): row li of A fragment i, column 8 (r / 4) + 4 lh + r % 4 of B fragment j
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;
  u32x4_t fa[2][TM], fb[2][TN];
  uint2 tb[2][TN][2];

  // fragments of half tile h of `stage` into registers
#define LLC_WIDE_READ(STAGE, H)                                                                                \
  {                                                                                                            \
    const int sb_ = (STAGE) * G::kStage;                                                                       \
    _Pragma("unroll") for (int s2 = 0; s2 < 2; ++s2) {                                                         \
      const int s_ = 2 * (H) + s2;                                                                             \
      _Pragma("unroll") for (int i = 0; i < TM; ++i)                                                           \
          fa[s2][i] = *(const u32x4_t*)(smem + sb_ + a_base[i] + (a_x[i] ^ (s_ << 5)));                        \
      _Pragma("unroll") for (int j = 0; j < TN; ++j) {                                                         \
        if constexpr (BMODE == kBKMajor) {                                                                     \
          fb[s2][j] = *(const u32x4_t*)(smem + sb_ + b_base[j] + (b_x[j] ^ (s_ << 5)));                        \
        } else {                                                                                               \
          _Pragma("unroll") for (int u = 0; u < 2; ++u)                                                        \
              tb[s2][j][u] = lds_read_tr16(lds0 + sb_ + b_base[j] + (16 * s_ + 4 * u) * (2 * BN));            \
        }                                                                                                      \
      }                                                                                                        \
    }                                                                                                          \
  }
  // after the wait: results of the (untracked) transposing reads become the B fragments
#define LLC_WIDE_TIE()                                                                                         \
  if constexpr (BMODE != kBKMajor) {                                                                           \
    _Pragma("unroll") for (int s2 = 0; s2 < 2; ++s2) _Pragma("unroll") for (int j = 0; j < TN; ++j) {          \
      asm volatile("" : "+v"(tb[s2][j][0]), "+v"(tb[s2][j][1]));                                               \
      fb[s2][j] = u32x4_t{tb[s2][j][0].x, tb[s2][j][0].y, tb[s2][j][1].x, tb[s2][j][1].y};                     \
    }                                                                                                          \
  }
#define LLC_WIDE_MMA()                                                                                         \
  _Pragma("unroll") for (int s2 = 0; s2 < 2; ++s2) _Pragma("unroll") for (int i = 0; i < TM; ++i)              \
      _Pragma("unroll") for (int j = 0; j < TN; ++j) mfma_step<T>(fb[s2][j], fa[s2][i], acc[i][j]);

  const int nk = p.K / 64;
#pragma unroll
  for (int x = 0; x < NS - 1; ++x)
    if (x < nk) issue(x);
  // tile 0 complete; with three stages tile 1 may still be in flight
  if (NS == 3 && nk >= 2) LLC_WAIT_VM(G::kLoads);
  else LLC_WAIT_VM(0);
  LLC_PHASE_END();
  if (grp == 1) { LLC_PHASE_END(); }  // group 1 runs one phase behind group 0

  auto main_loop = [&](auto grp_tag) {
    constexpr int GRP = decltype(grp_tag)::value;
    int st = 0;  // t % NS
    for (int t = 0; t < nk; ++t) {
      // ---- memory phase, first half of tile t ----
#if defined(LLC_WIDE_ABL) && (LLC_WIDE_ABL & 1)
      if (t + NS - 1 < nk && t < 0) {
#else
      if (t + NS - 1 < nk) {
#endif
        int dst = st + NS - 1;
        if (dst >= NS) dst -= NS;
        issue(dst);
      }
#if defined(LLC_WIDE_ABL) && (LLC_WIDE_ABL & 2)
      if (t < 1)
#endif
      LLC_WIDE_READ(st, 0)
      LLC_WAIT_LGKM0();
      LLC_WIDE_TIE()
      LLC_PHASE_END();
      // ---- compute phase ----
      __builtin_amdgcn_s_setprio(1);
      LLC_WIDE_MMA()
      __builtin_amdgcn_s_setprio(0);
      LLC_PHASE_END();
      // ---- memory phase, second half ----
#if defined(LLC_WIDE_ABL) && (LLC_WIDE_ABL & 2)
      if (t < 1)
#endif
      LLC_WIDE_READ(st, 1)
      LLC_WAIT_LGKM0();
      LLC_WIDE_TIE()
      if constexpr (GRP == 1) {
        // tile t+1 must be complete before the next barrier; the loads of tile t+2 (NS = 3) may still fly
        if (NS >= 3 && t + 2 < nk) { LLC_WAIT_VM_LOOP(G::kLoads); }
        else { LLC_WAIT_VM_LOOP(0); }
      }
      LLC_PHASE_END();
      // ---- compute phase ----
      __builtin_amdgcn_s_setprio(1);
      LLC_WIDE_MMA()
      __builtin_amdgcn_s_setprio(0);
      if constexpr (GRP == 0) {
        if (NS >= 3 && t + 2 < nk) { LLC_WAIT_VM_LOOP(G::kLoads); }
        else { LLC_WAIT_VM_LOOP(0); }
      }
      LLC_PHASE_END();
      st = st + 1 == NS ? 0 : st + 1;
    }
  };
  if (grp == 0) {
    main_loop(std::integral_constant<int, 0>{});
    LLC_PHASE_END();  // pairs with group 1's last compute phase
  } else {
    main_loop(std::integral_constant<int, 1>{});
  }
#undef LLC_WIDE_READ
#undef LLC_WIDE_TIE
#undef LLC_WIDE_MMA

  // ---- epilogue.  Every wave is past the last barrier: no fragment read and no load is outstanding, the
  //      stages are free.  Each wave stages its 64 x WTN tile in LDS of its own (no barrier needed). ----
  const int64_t c_off = (int64_t)z0 * p.c_sb + (int64_t)z1 * p.c_sb1;
  T* C = (T*)p.C + c_off;
  const T* res = p.residual ? (const T*)p.residual + c_off : nullptr;
  const T* bias = p.bias ? (const T*)p.bias + (int64_t)z0 * p.bias_sb : nullptr;
  char* wst = smem + wave * G::kOutWave;
  const int ncol0 = n0 + wn * G::WTN;
  // one instantiation per (activation, residual) so that the per-element code has no branches
  auto stage_out = [&](auto act_tag, auto res_tag) {
    constexpr int ACT = decltype(act_tag)::value;
    constexpr bool RES = decltype(res_tag)::value;
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int col = j * 32 + 8 * q + 4 * lh;  // first of 4 consecutive columns, inside the wave tile
        uint2 bq = {0, 0};
        if (bias) bq = *(const uint2*)(bias + ncol0 + col);
#pragma unroll
        for (int i = 0; i < TM; ++i) {
          const int row = i * 32 + li;
          uint2 rq = {0, 0};
          if constexpr (RES) rq = *(const uint2*)(res + (int64_t)(m0 + wm * 64 + row) * p.c_sm + ncol0 + col);
          uint32_t o[2];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const uint32_t bw = e < 2 ? bq.x : bq.y, rw = e < 2 ? rq.x : rq.y;
            const uint16_t bb = (uint16_t)(bw >> (16 * (e & 1))), rb = (uint16_t)(rw >> (16 * (e & 1)));
            float x = acc[i][j][4 * q + e] * p.alpha;
            if constexpr (Elem<T>::kDtype == LLC_BFLOAT16) x += bf16_bits_to_f32(bb);
            else x += f16_bits_to_f32(bb);
            if constexpr (RES) x += (Elem<T>::kDtype == LLC_BFLOAT16) ? bf16_bits_to_f32(rb) : f16_bits_to_f32(rb);
            if constexpr (ACT == LLC_ACT_RELU) x = x < 0.0f ? 0.0f : x;
            else if constexpr (ACT == LLC_ACT_GELU) x = gelu_exact(x);
            const uint32_t bits = (Elem<T>::kDtype == LLC_BFLOAT16) ? f32_to_bf16_bits(x) : f32_to_f16_bits(x);
            if (e & 1) o[e / 2] |= bits << 16;
            else o[e / 2] = bits;
          }
          *(uint2*)(wst + row * G::kOutPitch + col * 2) = uint2{o[0], o[1]};
        }
      }
  };
  auto with_res = [&](auto act_tag) {
    if (res) stage_out(act_tag, std::true_type{});
    else stage_out(act_tag, std::false_type{});
  };
  if (p.act == LLC_ACT_GELU) with_res(std::integral_constant<int, LLC_ACT_GELU>{});
  else if (p.act == LLC_ACT_RELU) with_res(std::integral_constant<int, LLC_ACT_RELU>{});
  else with_res(std::integral_constant<int, LLC_ACT_NONE>{});
  constexpr int kChunks = G::WTN / 8;  // 16-byte chunks per row of the wave tile
#pragma unroll
  for (int it = 0; it < kChunks; ++it) {
    const int idx = it * 64 + lane;
    const int row = idx / kChunks, ch = idx % kChunks;
    const u32x4_t v = *(const u32x4_t*)(wst + row * G::kOutPitch + ch * 16);
    *(u32x4_t*)(C + (int64_t)(m0 + wm * 64 + row) * p.c_sm + ncol0 + ch * 8) = v;
  }
  LLC_DBG_T1();
}

template <typename T, int BMODE, int BN>
int launch_wide(const GemmParams& p0, int batch, hipStream_t s) {
  constexpr int NS = BN == 128 ? 3 : 2;
  using G = WideGeom<BN, NS>;
  GemmParams p = p0;
  p.tiles_m = p.M / 256;
  p.tiles_n = p.N / BN;
  auto kern = gemm_wide_kernel<T, BMODE, BN, NS>;
  static std::atomic<uint32_t> lds_allowed{0};
  LLC_TRY(allow_dynamic_lds((const void*)kern, G::kLds, lds_allowed));
  hipLaunchKernelGGL(kern, dim3((unsigned)(p.tiles_m * p.tiles_n), 1, (unsigned)batch), dim3(512), G::kLds, s, p);
  return check_launch("gemm_wide_kernel");
}
