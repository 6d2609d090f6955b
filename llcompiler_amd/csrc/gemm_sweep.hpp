// matmul / batch_matmul with a reduction of exactly 64 (attention-style score products, the suite's
// [32,512,64] x [32,64,512]): the output is 8 .. 16 times the operands, so the kernel is a writer with a short
// burst of MFMAs per tile, and a one-tile-per-workgroup kernel runs its three phases (operands in, multiply,
// result out) one after the other on the whole chip.  Here a workgroup keeps a 64-row panel of A in registers
// for its whole life and sweeps the columns of B in tiles of 256 bytes (64 fp32 or 128 16-bit columns): the B tile
// two ahead is in flight (direct-to-LDS), the tile before is still draining to memory while the current one is
// multiplied; 50 KB of LDS, so three workgroups share a CU and one multiplies while another waits on its stores.
// Included by gemm.hip inside namespace llc::{anonymous}.
//
// 4 waves = 2 (32-row halves of the panel) x 2 (halves of the tile's columns).  MFMA operands are swapped
// (the B matrix feeds the row operand), which leaves a lane with 4 consecutive columns of one output row per
// accumulator quad: results pass through a wave-private LDS tile 16 (fp32) or 8 bytes at a time and leave as
// 16-byte stores of whole 128-byte rows (straight from the accumulators a store would touch 32 bytes of each of 32
// rows, four times the cache-line accesses).
//
// B tile in LDS: [64 k][256 B of n] as it lies in memory.
//   fp32: MFMA step s = 4 j + t of lane half lh multiplies k = 8 j + 4 lh + t (the same permutation on both
//         operands: A comes as 16-byte chunks 2 j + lh of its row).  The two lane halves read rows 4 apart, the
//         same banks; rows with k & 4 are stored with their 128-byte halves exchanged (chunk ^ 8, applied on the
//         global side of the load), so a read touches 64 different banks.
//   16-bit: chunks XOR-ed with 4 (k & 3), read with ds_read_b64_tr_b16 (the layout of the wide-tile kernel's
//         row-major B).

template <typename T>
struct SweepGeom {
  static constexpr int kES = sizeof(T);
  static constexpr int kTileN = kES == 4 ? 64 : 128;         // columns of a B tile: 256 bytes either way
  static constexpr int NB = kTileN / 64;                     // 32 x 32 accumulator blocks per wave
  static constexpr int kStage = 64 * 256;                    // one B tile
  static constexpr int kLoads = kStage / 4096;               // 1 KB slices per wave and tile
  static constexpr int kStores = 4;                          // global stores per wave and tile (32 rows x 128 bytes)
  static constexpr int kOutPitch = 128 + 16;                 // row pitch of a wave's staging tile
  static constexpr int kOutWave = 32 * kOutPitch;
  static constexpr int kLds = 2 * kStage + 4 * kOutWave;     // 50 KB: three workgroups per CU
};

// LDS reads as inline asm: the compiler orders every LDS read it knows about behind all direct-to-LDS loads in
// flight (s_waitcnt vmcnt(0)), which here would also wait for the previous tile's stores and the next tile's
// loads, once per tile.  Results may be used only behind an s_waitcnt lgkmcnt(0) followed by lds_tie().
template <int OFF>
__device__ __forceinline__ void lds_read_b32_asm(float& v, uint32_t addr) {
  asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF));
}
template <int OFF>
__device__ __forceinline__ void lds_read_b128_asm(u32x4_t& v, uint32_t addr) {
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF) : "memory");  // stays behind earlier LDS stores
}
template <int OFF>
__device__ __forceinline__ void lds_read_tr16_asm(uint2& v, uint32_t addr) {
  asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF));
}
template <int OFF>
__device__ __forceinline__ void lds_write_b64_asm(uint32_t addr, const uint2& v) {
  asm volatile("ds_write_b64 %0, %1 offset:%2" : : "v"(addr), "v"(v), "n"(OFF) : "memory");
}
template <int OFF>
__device__ __forceinline__ void lds_write_b128_asm(uint32_t addr, const u32x4_t& v) {
  asm volatile("ds_write_b128 %0, %1 offset:%2" : : "v"(addr), "v"(v), "n"(OFF) : "memory");
}
// The A panel the same way: a direct-to-LDS load in flight makes the compiler answer any dependency on a register
// loaded from memory with s_waitcnt vmcnt(0) (it takes such loads to complete out of order).
template <int OFF>
__device__ __forceinline__ void global_load_b128_asm(u32x4_t& v, const char* ptr) {
  asm volatile("global_load_dwordx4 %0, %1, off offset:%2" : "=v"(v) : "v"(ptr), "n"(OFF));
}
template <typename V>
__device__ __forceinline__ void lds_tie(V& v) {
  asm volatile("" : "+v"(v));
}

// NT: the result leaves in non-temporal stores.  These products are four fifths writes, and a result that no cache will hold
// until its reader runs streams out faster that way (32 x [512 x 64] x [64 x 512], operand sets rotating through 600 MB:
// bf16 8.8 -> 6.4 us, fp32 18.0 -> 14.7 us; 96 batches: 17.1 -> 13.3 and 41.7 -> 35.0); the launcher asks for them from
// 16 MiB of result on.
template <typename T, bool EPI, bool NT>
__global__ __launch_bounds__(256) void bmm_sweep_kernel(const GemmParams p, int tiles_per_wg) {
  using G = SweepGeom<T>;
  constexpr int ES = G::kES, NB = G::NB;
  extern __shared__ __align__(16) char smem[];
  int panel, range, z;
  tile_and_batch_of_block(p.tiles_m, p.tiles_n, panel, range, z);
  const int m0 = panel * 64;
  const int z0 = z / p.bdiv, z1 = z - z0 * p.bdiv;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave), lane = threadIdx.x % kWave;
  const int wm = wave >> 1, wn = wave & 1;
  const int li = lane % 32, lh = lane / 32;
  const int tile0 = range * tiles_per_wg;  // first column tile of this workgroup
  const int nt = tiles_per_wg;

  const char* A = (const char*)((const T*)p.A + (int64_t)z0 * p.a_sb + (int64_t)z1 * p.a_sb1 + (int64_t)(m0 + wm * 32 + li) * p.a_sm);
  const char* B = (const char*)((const T*)p.B + (int64_t)z0 * p.b_sb + (int64_t)z1 * p.b_sb1 + (int64_t)tile0 * G::kTileN);
  const int64_t b_row_bytes = p.b_sk * ES;

  // ---- direct-to-LDS loads of a B tile: slice d of a wave is LDS bytes [(wave + 4 d) KB, +1 KB) of the stage ----
  //      = four k rows of 256 bytes, 16 lanes each
  uint32_t lb_off;
  {
    const int krow0 = 4 * wave + lane / 16, slot = lane % 16;
    // fp32: the slice's rows all have k & 4 = 4 (wave & 1), whatever d is
    if constexpr (ES == 4) lb_off = (uint32_t)(krow0 * b_row_bytes) + ((slot ^ ((wave & 1) << 3)) << 4);
    else lb_off = (uint32_t)(krow0 * b_row_bytes) + ((slot ^ ((krow0 & 3) << 2)) << 4);
  }
  auto dma = [&](auto d_tag, int tile, int stage) {
    constexpr int D = decltype(d_tag)::value;
    uint32_t off = lb_off;
    const char* g = B + (int64_t)(16 * D) * b_row_bytes + (int64_t)tile * 256;
    asm volatile("" : "+v"(off));
    __builtin_amdgcn_global_load_lds(LLC_GPTR(g + off), LLC_LPTR(smem + stage * G::kStage + (wave + 4 * D) * 1024), 16, 0, 0);
  };
  auto dma_tile = [&](int tile, int stage) { static_for<G::kLoads>([&](auto d_tag) { dma(d_tag, tile, stage); }); };

  // ---- prologue: B tile 0 on its way, the A panel into registers (tile 1 follows below) ----
  dma_tile(0, 0);
  u32x4_t a[ES == 4 ? 8 : 4];
  static_for<(ES == 4 ? 8 : 4)>([&](auto c_tag) {
    constexpr int CC = decltype(c_tag)::value;
    u32x4_t& dst = a[CC];
    global_load_b128_asm<CC * 32>(dst, A + lh * 16);
  });

  // fragment addresses of the B tile (LDS byte addresses)
  const uint32_t lds0 = (uint32_t)(uintptr_t)smem;
  uint32_t ub[2];  // per 32-column block (fp32 has one)
  if constexpr (ES == 4) {
    ub[0] = ub[1] = lds0 + (uint32_t)((4 * lh) * 256 + ((((wn * 8 + (li >> 2)) ^ (lh << 3))) << 4) + (li & 3) * 4);
  } else {
    const int g = lane / 16, jj = (lane / 4) % 4, q = lane % 4;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int nchunk = (wn * 64 + j * 32) / 8 + 2 * (g & 1) + (q >> 1);
      ub[j] = lds0 + (uint32_t)((8 * (g >> 1) + jj) * 256 + ((nchunk ^ (jj << 2)) << 4) + (q & 1) * 8);
    }
  }

  const int64_t c_off = (int64_t)z0 * p.c_sb + (int64_t)z1 * p.c_sb1;
  T* C = (T*)p.C + c_off;
  const T* res = EPI && p.residual ? (const T*)p.residual + c_off : nullptr;
  const T* bias = EPI && p.bias ? (const T*)p.bias + (int64_t)z0 * p.bias_sb : nullptr;
  const int64_t row_off = (int64_t)(m0 + wm * 32 + li) * p.c_sm;
  using S0 = std::integral_constant<int, 0>;
  using S1 = std::integral_constant<int, 1>;

  // the A panel and tile 0 have landed once only tile 1's loads are outstanding
  // (immediates that say exactly what is waited for: the compiler reads them, and anything vaguer makes it wait
  // for the A panel again, with vmcnt(0), inside the loop)
  if (nt > 1) {
    dma_tile(1, 1);
    LLC_WAIT_VM(G::kLoads);
  } else {
    LLC_WAIT_VM(0);
  }
#pragma unroll
  for (int c = 0; c < (ES == 4 ? 8 : 4); ++c) lds_tie(a[c]);

  auto tile = [&](auto stage_tag, int it) {
    constexpr int ST = decltype(stage_tag)::value;
    // tile `it` has landed once at most the younger operations of this wave are outstanding: the next tile's loads
    // and the stores of the tile before (a smaller count than the true one only waits longer)
    if (it > 0) {
      if (it + 1 < nt) LLC_WAIT_VM(G::kLoads + G::kStores);
      else LLC_WAIT_VM(G::kStores);
    }
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);

    const int ncol0 = (tile0 + it) * G::kTileN + wn * 32 * NB;
    // bias and residual of the wave tile, requested before the multiply: [j][q] = columns 32 j + 8 q + 4 lh .. + 3
    u32x4_t bq4[NB][4], rq4[NB][4];  // fp32
    uint2 bq2[NB][4], rq2[NB][4];    // 16-bit
    if constexpr (EPI) {
#pragma unroll
      for (int j = 0; j < NB; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int col = ncol0 + j * 32 + 8 * q + 4 * lh;
          if constexpr (ES == 4) {
            bq4[j][q] = u32x4_t{0, 0, 0, 0};
            rq4[j][q] = u32x4_t{0, 0, 0, 0};
            if (bias) bq4[j][q] = *(const u32x4_t*)(bias + col);
            if (res) rq4[j][q] = *(const u32x4_t*)(res + row_off + col);
          } else {
            bq2[j][q] = uint2{0, 0};
            rq2[j][q] = uint2{0, 0};
            if (bias) bq2[j][q] = *(const uint2*)(bias + col);
            if (res) rq2[j][q] = *(const uint2*)(res + row_off + col);
          }
        }
    }

    f32x16_t acc[NB];
#pragma unroll
    for (int j = 0; j < NB; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[j][r] = 0.0f;
    if constexpr (ES == 4) {
      // groups of 4 reads (the 4 k of chunk j), two groups ahead of the MFMAs that use them
      float bv[3][4];
      auto read_group = [&](auto j_tag) {
        constexpr int J = decltype(j_tag)::value;
        static_for<4>([&](auto t_tag) {
          constexpr int TT = decltype(t_tag)::value;
          float& v0 = bv[J % 3][TT];
          lds_read_b32_asm<ST * G::kStage + (8 * J + TT) * 256>(v0, ub[0]);
        });
      };
      read_group(S0{});
      read_group(S1{});
      static_for<8>([&](auto j_tag) {
        constexpr int J = decltype(j_tag)::value;
        // group J is complete once only the 4 reads of group J + 1 are outstanding (LDS reads return in order)
        if constexpr (J + 1 < 8) __builtin_amdgcn_s_waitcnt(0xC07F | (4 << 8));
        else LLC_WAIT_LGKM0();
#pragma unroll
        for (int t = 0; t < 4; ++t) lds_tie(bv[J % 3][t]);
        if constexpr (J + 2 < 8) read_group(std::integral_constant<int, J + 2>{});
#pragma unroll
        for (int t = 0; t < 4; ++t)
          acc[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(bv[J % 3][t], __uint_as_float(a[J][t]), acc[0], 0, 0, 0);
      });
    } else {
      uint2 tb[4][2][2];
      static_for<4>([&](auto s_tag) {
        constexpr int S = decltype(s_tag)::value;
#pragma unroll
        for (int j = 0; j < NB; ++j) {
          uint2& t0 = tb[S][j][0];
          uint2& t1 = tb[S][j][1];
          lds_read_tr16_asm<ST * G::kStage + (16 * S) * 256>(t0, ub[j]);
          lds_read_tr16_asm<ST * G::kStage + (16 * S + 4) * 256>(t1, ub[j]);
        }
      });
      LLC_WAIT_LGKM0();
      static_for<4>([&](auto s_tag) {
        constexpr int S = decltype(s_tag)::value;
#pragma unroll
        for (int j = 0; j < NB; ++j) {
          lds_tie(tb[S][j][0]);
          lds_tie(tb[S][j][1]);
          mfma_step<T>(u32x4_t{tb[S][j][0].x, tb[S][j][0].y, tb[S][j][1].x, tb[S][j][1].y}, a[S], acc[j]);
        }
      });
    }
    if constexpr (EPI) {
      // bias and residual must be here before the next tile's loads go out behind them (they could then only be
      // waited for together with those loads)
#pragma unroll
      for (int j = 0; j < NB; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          if constexpr (ES == 4) {
            lds_tie(bq4[j][q]);
            lds_tie(rq4[j][q]);
          } else {
            lds_tie(bq2[j][q]);
            lds_tie(rq2[j][q]);
          }
        }
    }
    // every wave has read the stage: tile it + 2 may overwrite it
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    if (it + 2 < nt) dma_tile(it + 2, ST);

    // ---- act(alpha acc + bias + residual) out.  acc[j][4 q + e] = row li, column 32 j + 8 q + 4 lh + e of the wave tile ----
#pragma unroll
    for (int j = 0; j < NB; ++j)
#pragma unroll
      for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          float x = acc[j][4 * q + e] * p.alpha;
          if constexpr (EPI && ES == 4) x += __uint_as_float(bq4[j][q][e]) + __uint_as_float(rq4[j][q][e]);
          if constexpr (EPI && ES == 2) {
            const uint32_t bw = e < 2 ? bq2[j][q].x : bq2[j][q].y, rw = e < 2 ? rq2[j][q].x : rq2[j][q].y;
            const uint16_t bb = (uint16_t)(bw >> (16 * (e & 1))), rb = (uint16_t)(rw >> (16 * (e & 1)));
            if constexpr (Elem<T>::kDtype == LLC_BFLOAT16) x += bf16_bits_to_f32(bb) + bf16_bits_to_f32(rb);
            else x += f16_bits_to_f32(bb) + f16_bits_to_f32(rb);
          }
          acc[j][4 * q + e] = x;
        }
    if (p.act == LLC_ACT_RELU) {
#pragma unroll
      for (int j = 0; j < NB; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[j][r] = acc[j][r] < 0.0f ? 0.0f : acc[j][r];  // NaN passes through
    } else if (p.act == LLC_ACT_GELU) {
#pragma unroll
      for (int j = 0; j < NB; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[j][r] = gelu_for<T>(acc[j][r]);
    }
    // through the wave's own LDS tile, so that a store instruction writes whole 128-byte lines (straight from the
    // accumulators it would write 32 bytes of each of 32 rows: four times the line accesses, which is what the
    // store path counts)
    const uint32_t wst = lds0 + 2 * G::kStage + wave * G::kOutWave;
    const uint32_t wr = wst + li * G::kOutPitch + 4 * ES * lh;  // columns 32 j + 8 q + 4 lh .. + 3
    static_for<4 * NB>([&](auto g_tag) {
      constexpr int JQ = decltype(g_tag)::value, J = JQ / 4, Q = JQ % 4;
      if constexpr (ES == 4) {
        const u32x4_t ov = {__float_as_uint(acc[J][4 * Q]), __float_as_uint(acc[J][4 * Q + 1]), __float_as_uint(acc[J][4 * Q + 2]),
                            __float_as_uint(acc[J][4 * Q + 3])};
        lds_write_b128_asm<(32 * J + 8 * Q) * 4>(wr, ov);
      } else {
        uint32_t o[2];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float x = acc[J][4 * Q + e];
          const uint32_t bits = (Elem<T>::kDtype == LLC_BFLOAT16) ? f32_to_bf16_bits(x) : f32_to_f16_bits(x);
          if (e & 1) o[e / 2] |= bits << 16;
          else o[e / 2] = bits;
        }
        const uint2 ov = {o[0], o[1]};
        lds_write_b64_asm<(32 * J + 8 * Q) * 2>(wr, ov);
      }
    });
    // back as 16-byte pieces of whole rows (the wave's own LDS writes, in order)
    constexpr int LPR = 8, RPI = 8, NX = 4;  // lanes per 128-byte row, rows per instruction, instructions
    u32x4_t v[NX];
    const uint32_t rd = wst + (lane / LPR) * G::kOutPitch + (lane % LPR) * 16;
    static_for<NX>([&](auto x_tag) {
      constexpr int X = decltype(x_tag)::value;
      u32x4_t& dst = v[X];
      lds_read_b128_asm<X * RPI * G::kOutPitch>(dst, rd);
    });
    LLC_WAIT_LGKM0();
#pragma unroll
    for (int x = 0; x < NX; ++x) {
      lds_tie(v[x]);
      const int row = x * RPI + lane / LPR, ch = lane % LPR;
      u32x4_t* dst = (u32x4_t*)(C + (int64_t)(m0 + wm * 32 + row) * p.c_sm + ncol0 + ch * (16 / ES));
      if constexpr (NT) __builtin_nontemporal_store(v[x], dst);
      else *dst = v[x];
    }
  };
  int it = 0;
  for (; it + 1 < nt; it += 2) {
    tile(S0{}, it);
    tile(S1{}, it + 1);
  }
  if (it < nt) tile(S0{}, it);
}

// Whether the sweep kernel takes this product; the caller has checked operand alignment (a_kvec, b_rvec).
template <typename T>
bool sweep_ok(const GemmParams& p, int batch) {
  constexpr int ES = sizeof(T), EPV = 16 / ES;
  auto al16 = [](const void* q) { return ((uintptr_t)q % 16) == 0; };
  if (p.K != 64 || p.M % 64 != 0 || p.N % SweepGeom<T>::kTileN != 0 || p.c_f32) return false;
  if ((int64_t)(p.M / 64) * batch < 128) return false;  // too few panels to fill the chip: the tile kernels split finer
  if (!al16(p.C) || p.c_sm % EPV != 0 || p.c_sb % EPV != 0 || p.c_sb1 % EPV != 0) return false;
  if (p.bias && (!al16(p.bias) || p.bias_sb % EPV != 0)) return false;
  if (p.residual && !al16(p.residual)) return false;
  // lane offsets of the operand loads are 32-bit byte offsets inside one batch entry
  if (p.b_sk * 64 * ES >= ((int64_t)1 << 31) || p.b_sk < 0 || p.a_sm < 0) return false;
  return true;
}

template <typename T>
int launch_sweep(const GemmParams& p0, int batch, hipStream_t s) {
  using G = SweepGeom<T>;
  GemmParams p = p0;
  const int nt = p.N / G::kTileN;
  // column tiles per workgroup: all of them (A is fetched once), unless the workgroups would not fill the places the
  // chip has for them in one round (three workgroups per CU)
  const int64_t places = 256 * 3;
  int ranges = 1;
  while ((int64_t)(p.M / 64) * batch * ranges * 2 <= places && (nt / ranges) % 2 == 0) ranges *= 2;
  p.tiles_m = p.M / 64;
  p.tiles_n = ranges;
  const int64_t wgs = (int64_t)p.tiles_m * ranges;
  if (wgs > 0x7fffffff || batch > 65535) return set_error(LLC_ERR_TOO_LARGE, "matmul: grid too large");
  const bool epi = p.bias || p.residual;
  const bool nts = (int64_t)batch * p.M * p.N * G::kES >= ((int64_t)16 << 20);
  auto kern = nts ? (epi ? bmm_sweep_kernel<T, true, true> : bmm_sweep_kernel<T, false, true>)
                  : (epi ? bmm_sweep_kernel<T, true, false> : bmm_sweep_kernel<T, false, false>);
  static std::atomic<uint32_t> lds_allowed[4];
  LLC_TRY(allow_dynamic_lds((const void*)kern, G::kLds, lds_allowed[2 * nts + epi]));
  hipLaunchKernelGGL(kern, dim3((unsigned)wgs, 1, (unsigned)batch), dim3(256), G::kLds, s, p, nt / ranges);
  return check_launch("bmm_sweep_kernel");
}
