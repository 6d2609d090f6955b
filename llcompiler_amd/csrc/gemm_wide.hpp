// 16-bit matmul / batch_matmul on 256 x BN x 64 tiles (BN = 256, 192 or 128), one workgroup per CU.
// Included by gemm.hip inside namespace llc::{anonymous} (uses GemmParams and the LDS-DMA helpers defined there).
//
// Why a second tile shape: a 128x128 tile needs 64 B/clk/CU of operands from L2 at the full MFMA rate and
// 192 B/clk of LDS traffic, both above what a CU gets; a 256x256 tile halves the first and, with 128x128 wave
// tiles, brings the second to 96 B/clk.

#define LLC_WAIT_VM(VM) __builtin_amdgcn_s_waitcnt(((VM) & 15) | (7 << 4) | (15 << 8) | (((VM) >> 4) << 14))


// ---------------------------------------------------------------------------------------------
// FOUR waves, one per SIMD, each owning a 128 x BN/2 accumulator tile (up to 256 accumulator registers per
// lane, which the compiler keeps in the accumulation half of the register file).  With one wave per SIMD
// nothing else can issue while that wave waits, so the instruction stream is ordered by hand: a k-step
// (TM x TN MFMAs) is cut into slots of one MFMA, each followed by at most one fragment read of the NEXT k-step
// and at most one direct-to-LDS load of a later k-tile, and slots are fenced (sched_barrier) so that the
// compiler keeps that order; in-order issue then hides the memory instructions behind the 32 clocks an MFMA
// occupies the matrix pipe.  (A variant with eight waves in two groups that alternate between a memory phase
// and an MFMA phase, one barrier per phase, was measured at 0.43 of peak on 8192^3 against 0.49 here: its
// 64 x 128 wave tiles read half as much again from LDS per MFMA and every phase pays a barrier.)
//
// LDS: two stages; A tiles at [0, 64 KB), B tiles behind them, so that the stage and the fragment row block
// are immediate offsets of the LDS reads and a lane needs four address registers per operand (its row's
// swizzled chunk for each k-step).  Stage of tile t is free once every wave has read its last fragments:
// the barrier sits in front of the last k-step's MFMAs, the loads of tile t+2 go out behind it (first in that
// k-step, the rest in the first k-steps of tile t+1) and have a whole k-tile of MFMAs to land.
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (N > 0) {
    static_for<N - 1>(f);
    f(std::integral_constant<int, N - 1>{});
  }
}

template <int TM, int TN>
struct MmaOrder {
  int i[TM * TN], j[TM * TN];
  // growing squares: (0,0); (0,1) (1,0) (1,1); ... so that fragments are needed in the order A0 B0 A1 B1 ...
  constexpr MmaOrder() : i{}, j{} {
    int n = 0;
    for (int d = 0; d < (TM > TN ? TM : TN); ++d) {
      if (d < TN)
        for (int a = 0; a < d && a < TM; ++a) { i[n] = a; j[n] = d; ++n; }
      if (d < TM)
        for (int b = 0; b <= d && b < TN; ++b) { i[n] = d; j[n] = b; ++n; }
    }
  }
};

template <int TM, int TN>
constexpr MmaOrder<TM, TN> kMmaOrder{};

template <int BN>
struct WideGeom {
  static constexpr int TM = 4, TN = BN / 64, WTN = BN / 2;
  static constexpr int kAStage = 256 * 128, kBStage = BN * 128, kB0 = 2 * kAStage;
  static constexpr int kLoadsA = 8, kLoadsB = BN / 32, kLoads = kLoadsA + kLoadsB;  // 1 KB slices per wave and k-tile
  static constexpr int NG = TM * TN / 2;  // MFMA slots of a k-step that may carry a direct-to-LDS load (every other one)
  static constexpr int NR = TM + TN;      // fragment reads per k-step
  // direct-to-LDS loads of a tile by the k-step they are issued in: the last k-step of the tile two ahead of it,
  // then k-steps 0 and 1 of the tile before it
  static constexpr int kD3 = NG < 6 ? NG : 6, kD0 = (kLoads - kD3 + 1) / 2, kD1 = kLoads - kD3 - kD0;
  static_assert(kD1 >= 0 && kD1 <= NG && kD0 <= NG, "load schedule");
  static constexpr int kOutPitch = WTN * 2 + 16, kOutWave = 128 * kOutPitch;
  static constexpr int kLds = 2 * (kAStage + kBStage) > 4 * kOutWave ? 2 * (kAStage + kBStage) : 4 * kOutWave;
};

// Rows of zeros for the taps of a convolution window that fall outside the image (CONV: a lane whose tap is outside
// loads from here instead).
static __device__ __align__(256) unsigned char llc_zero_row[256];

// CONV: A is a channels-last image [n, H, W, C] and row m of the product is output pixel m; k runs over (tap, channel)
// in 64-channel k-tiles that lie inside one tap, so a k-tile of a row is 128 contiguous bytes of the image (or of
// zeros).  Each lane keeps, for its 8 rows, the element offset of the window origin and one validity bit per tap,
// computed once; a k-tile adds one scalar offset.  B is the weight [F, taps * C].
template <typename T, int BMODE, int BN, bool CONV = false>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void gemm_wide_kernel(const GemmParams p) {
  static_assert(sizeof(T) == 2, "16-bit operands");
  static_assert(!CONV || BMODE == kBKMajor, "convolution weights are k-contiguous");
  static_assert(BMODE == kBKMajor || BN != 192, "row-major B: the chunk swizzle needs 16 or 32 chunks per row");
  using G = WideGeom<BN>;
  constexpr int TM = G::TM, TN = G::TN;
  extern __shared__ __align__(16) char smem[];
  int tile_m, tile_n;
  int z;
  tile_and_batch_of_block(p.tiles_m, p.tiles_n, tile_m, tile_n, z);
  const int m0 = tile_m * 256, n0 = tile_n * BN;
  const int z0 = z / p.bdiv, z1 = z - z0 * p.bdiv;
  const char* A = CONV ? p.A : (const char*)((const T*)p.A + (int64_t)z0 * p.a_sb + (int64_t)z1 * p.a_sb1 + (int64_t)m0 * p.a_sm);
  const char* B = (const char*)((const T*)p.B + (int64_t)z0 * p.b_sb + (int64_t)z1 * p.b_sb1 +
                                (BMODE == kBKMajor ? (int64_t)n0 * p.b_sn : (int64_t)n0));
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave), lane = threadIdx.x % kWave;
  const int wm = wave >> 1, wn = wave & 1;
  const int li = lane % 32, lh = lane / 32;

  // ---- direct-to-LDS loads.  Load d < 8 of a tile is A slice wave + 4 d (rows 8 wave + lane / 8 + 32 d), the others
  //      B slices the same way: a uniform base per load plus one of two lane offsets (the row swizzle alternates
  //      with d).  Offsets are bytes. ----
  const int64_t a_row_bytes = p.a_sm * 2, b_row_bytes = (BMODE == kBKMajor ? p.b_sn : p.b_sk) * 2;
  uint32_t la_off[2], lb_off[2];
  {
    const int row0 = wave * 8 + lane / 8;
#pragma unroll
    for (int par = 0; par < 2; ++par) {
      la_off[par] = (uint32_t)(row0 * a_row_bytes) + ((((lane % 8) ^ lds_swz(row0) ^ (4 * par)) & 7) << 4);
      if constexpr (BMODE == kBKMajor) lb_off[par] = (uint32_t)(row0 * b_row_bytes) + ((((lane % 8) ^ lds_swz(row0) ^ (4 * par)) & 7) << 4);
    }
    if constexpr (BMODE != kBKMajor) {
      constexpr int RPS = 1024 / (2 * BN);  // k rows per slice
      const int krow0 = RPS * wave + lane / (64 / RPS), slot = lane % (64 / RPS);
      lb_off[0] = lb_off[1] = (uint32_t)(krow0 * b_row_bytes) + ((slot ^ ((krow0 & 3) << 2)) << 4);
    }
  }
  // CONV: window origin (element offset into the image, may be negative) and valid taps of this lane's row in each of
  // its 8 A loads (rows wave * 8 + lane / 8 + 32 d of the tile)
  int pix_off[CONV ? 8 : 1];
  uint32_t pix_taps[CONV ? 8 : 1];
  if constexpr (CONV) {
    const ConvWideGeom& cg = p.cg;
    const int ohw = cg.OH * cg.OW;
#pragma unroll
    for (int d = 0; d < 8; ++d) {
      const int m = m0 + wave * 8 + lane / 8 + 32 * d;
      pix_off[d] = 0;
      pix_taps[d] = 0;
      if (m < cg.ncols) {
        const int n = m / ohw, rem = m - n * ohw;
        const int oh = rem / cg.OW, ow = rem - oh * cg.OW;
        const int ih0 = oh * cg.sh - cg.ph, iw0 = ow * cg.sw - cg.pw;
        pix_off[d] = ((n * cg.H + ih0) * cg.W + iw0) * cg.C;
        uint32_t bits = 0;
        for (int kh = 0; kh < cg.KH; ++kh)
          for (int kw = 0; kw < cg.KW; ++kw) {
            const int ih = ih0 + kh * cg.dh, iw = iw0 + kw * cg.dw;
            if (ih >= 0 && ih < cg.H && iw >= 0 && iw < cg.W) bits |= 1u << (kh * cg.KW + kw);
          }
        pix_taps[d] = bits;
      }
    }
  }
  // load d of k-tile kt into `stage`: a uniform 64-bit base (scalar registers) plus the lane's 32-bit offset.  The
  // empty asm keeps the compiler from folding base and offset into sixteen loop-invariant 64-bit lane pointers.
  auto dma = [&](auto d_tag, int kt, int stage) {
    constexpr int D = decltype(d_tag)::value;
    if constexpr (CONV && D < G::kLoadsA) {
      const ConvWideGeom& cg = p.cg;
      // uniform: tap and channel block of the k-tile, the tap's offset from the window origin
      // (n / d as (n * magic) >> 32 with magic = floor(2^32 / d) + 1; magic 0 stands for d = 1)
      const uint32_t tap = cg.cblocks_magic ? (uint32_t)(((uint64_t)(uint32_t)kt * cg.cblocks_magic) >> 32) : (uint32_t)kt;
      const int c0 = (kt - (int)tap * cg.cblocks) * 64;
      const uint32_t kh = cg.kw_magic ? (uint32_t)(((uint64_t)tap * cg.kw_magic) >> 32) : tap, kw = tap - kh * cg.KW;
      const int64_t toff = (int64_t)(((int)kh * cg.dh * cg.W + (int)kw * cg.dw) * cg.C + c0) * 2;
      const uint32_t chunk = ((((lane % 8) ^ lds_swz(wave * 8 + lane / 8) ^ (4 * (D & 1))) & 7) << 4);
      const bool inside = (pix_taps[D] >> tap) & 1u;
      const char* g = inside ? A + (int64_t)pix_off[D] * 2 + toff + chunk : (const char*)llc_zero_row + chunk;
      __builtin_amdgcn_global_load_lds(LLC_GPTR(g), LLC_LPTR(smem + stage * G::kAStage + (wave + 4 * D) * 1024), 16, 0, 0);
    } else if constexpr (D < G::kLoadsA) {
      uint32_t off = la_off[D & 1];
      asm volatile("" : "+v"(off));
      const char* g = A + (int64_t)(32 * D) * a_row_bytes + (int64_t)kt * 128;
      __builtin_amdgcn_global_load_lds(LLC_GPTR(g + off), LLC_LPTR(smem + stage * G::kAStage + (wave + 4 * D) * 1024), 16, 0, 0);
    } else {
      constexpr int DB = D - G::kLoadsA;
      uint32_t off = lb_off[BMODE == kBKMajor ? (DB & 1) : 0];
      asm volatile("" : "+v"(off));
      const char* g;
      if constexpr (BMODE == kBKMajor) g = B + (int64_t)(32 * DB) * b_row_bytes + (int64_t)kt * 128;
      else g = B + ((int64_t)(4 * DB * (1024 / (2 * BN))) + (int64_t)kt * 64) * b_row_bytes;
      __builtin_amdgcn_global_load_lds(LLC_GPTR(g + off), LLC_LPTR(smem + G::kB0 + stage * G::kBStage + (wave + 4 * DB) * 1024), 16, 0, 0);
    }
  };

  // ---- fragment addresses: ua[c] / ub[c] = this lane's row with k chunk pair c; fragment (k-step s, row block i) reads
  //      ua[s ^ 2 (i & 1)] + 4096 i + stage (the row swizzle of block i differs from block 0's by 4 (i & 1)) ----
  uint32_t ua[4], ub[4];
  {
    const int ra = wm * 128 + li, va = lh ^ lds_swz(ra);
#pragma unroll
    for (int c = 0; c < 4; ++c) ua[c] = ra * 128 + (((va ^ (2 * c)) & 7) << 4);
    if constexpr (BMODE == kBKMajor) {
      const int rb = wn * G::WTN + li, vb = lh ^ lds_swz(rb);
#pragma unroll
      for (int c = 0; c < 4; ++c) ub[c] = G::kB0 + rb * 128 + (((vb ^ (2 * c)) & 7) << 4);
    } else {
      // transposing read of fragment j: lane = 16 g + 4 jj + q reads 8 bytes of k row 16 s + 8 (g >> 1) + 4 u + jj at
      // n chunk (16 (g & 1) + 4 q) / 8 of the fragment's 32 columns, stored at slot chunk ^ (jj << 2)
      const int g = lane / 16, jj = (lane / 4) % 4, q = lane % 4;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int nchunk = (wn * G::WTN + j * 32) / 8 + 2 * (g & 1) + (q >> 1);
        ub[j] = G::kB0 + (8 * (g >> 1) + jj) * (2 * BN) + ((nchunk ^ (jj << 2)) << 4) + (q & 1) * 8;
      }
    }
  }

  f32x16_t acc[TM][TN];  // register r of lane (li, lh): row li of A block i, column 8 (r / 4) + 4 lh + r % 4 of B block j
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;
  u32x4_t fa[2][TM], fb[2][TN];
  uint2 tb[2][TN][2];  // row-major B: the two transposing reads of each B fragment
  const uint32_t lds0 = (uint32_t)(uintptr_t)smem;

  // read item R (A0 B0 A1 B1 ... in the order the MFMAs need them) of k-step S of `STAGE` into fragment set SET
  auto read_item = [&](auto r_tag, auto s_tag, auto stage_tag, auto set_tag) {
    constexpr int R = decltype(r_tag)::value, S = decltype(s_tag)::value, ST = decltype(stage_tag)::value, SET = decltype(set_tag)::value;
    // item R: blocks alternate A, B while both remain
    constexpr int both = 2 * (TM < TN ? TM : TN);
    constexpr bool is_a = R < both ? (R % 2 == 0) : (TM > TN);
    constexpr int blk = R < both ? R / 2 : (R - both) + (TM < TN ? TM : TN);
    if constexpr (is_a) {
      fa[SET][blk] = *(const u32x4_t*)(smem + (ua[S ^ (2 * (blk & 1))] + blk * 4096 + ST * G::kAStage));
    } else if constexpr (BMODE == kBKMajor) {
      fb[SET][blk] = *(const u32x4_t*)(smem + (ub[S ^ (2 * (blk & 1))] + blk * 4096 + ST * G::kBStage));
    } else {
      // inline asm: the compiler would order a transposing read it knows about behind every direct-to-LDS load in
      // flight (vmcnt(0)).  Its result is used only behind the s_waitcnt at the top of the k-step that consumes it.
      uint2& t0 = tb[SET][blk][0];  // asm operands inside a generic lambda must be locals
      uint2& t1 = tb[SET][blk][1];
      const uint32_t addr = lds0 + ub[blk];
      asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(t0) : "v"(addr), "n"((16 * S) * (2 * BN) + ST * G::kBStage));
      asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(t1) : "v"(addr), "n"((16 * S + 4) * (2 * BN) + ST * G::kBStage));
    }
  };

  const int nk = p.K / 64;
  // One k-step: S of tile t (stage ST).  The fragments of the next k-step are read here (behind the last tile that is
  // the other stage's stale data, read and never used).  The loads scheduled in this k-step belong to tile t+1 (S < 3) or
  // t+2 (S == 3); CHECK: that tile may not exist, look before loading.
  auto step = [&](auto stage_tag, auto s_tag, auto check_tag, int t) {
    constexpr int ST = decltype(stage_tag)::value, S = decltype(s_tag)::value;
    constexpr bool CHECK = decltype(check_tag)::value;
    constexpr int CUR = S & 1, NXT = CUR ^ 1;
    constexpr int RST = S == 3 ? (ST ^ 1) : ST, RS = (S + 1) & 3;
    if constexpr (S == 3) {
      // every fragment of this tile is in registers (this wave's), tile t+1 has landed (this wave's loads)
      __builtin_amdgcn_s_waitcnt(0 | (7 << 4) | (0 << 8) | (0 << 14));
      __builtin_amdgcn_sched_barrier(0);
      __builtin_amdgcn_s_barrier();
      __builtin_amdgcn_sched_barrier(0);
    }
    if constexpr (BMODE != kBKMajor) {
      // the transposing reads of this k-step's B fragments were issued at least four MFMAs ago
      LLC_WAIT_LGKM0();
      static_for<TN>([&](auto j_tag) {
        constexpr int J = decltype(j_tag)::value;
        uint2& t0 = tb[CUR][J][0];
        uint2& t1 = tb[CUR][J][1];
        asm volatile("" : "+v"(t0), "+v"(t1));
        fb[CUR][J] = u32x4_t{t0.x, t0.y, t1.x, t1.y};
      });
    }
    constexpr int dlo = S == 3 ? 0 : (S == 0 ? G::kD3 : G::kD3 + G::kD0);
    constexpr int dcnt = S == 3 ? G::kD3 : (S == 0 ? G::kD0 : (S == 1 ? G::kD1 : 0));
    const int kt = S == 3 ? t + 2 : t + 1;
    const bool load = !CHECK || kt < nk;
    // one MFMA per slot; behind it at most one memory instruction of either kind: fragment reads of the next k-step in
    // the odd slots, direct-to-LDS loads in the even ones (what does not fit that pattern shares a slot)
    constexpr int NS1 = TM * TN;                                       // MFMA slots
    constexpr int NRS = BMODE == kBKMajor ? NS1 : NS1 - 4;             // slots that may carry reads (asm reads: not the last four)
    static_for<NS1>([&](auto q_tag) {
      constexpr int Q = decltype(q_tag)::value;
      constexpr int i0 = kMmaOrder<TM, TN>.i[Q], j0 = kMmaOrder<TM, TN>.j[Q];
      mfma_step<T>(fb[CUR][j0], fa[CUR][i0], acc[i0][j0]);
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (Q < NRS) {
        constexpr int lo = Q * G::NR / NRS, hi = (Q + 1) * G::NR / NRS;
        static_for<hi - lo>([&](auto r_tag) {
          read_item(std::integral_constant<int, lo + decltype(r_tag)::value>{}, std::integral_constant<int, RS>{},
                    std::integral_constant<int, RST>{}, std::integral_constant<int, NXT>{});
        });
      }
      if constexpr (!(Q & 1) && (Q / 2) < dcnt) {
        if (load) dma(std::integral_constant<int, dlo + Q / 2>{}, kt, S == 3 ? ST : (ST ^ 1));
      }
      __builtin_amdgcn_sched_barrier(0);
    });
  };
  auto tile = [&](auto stage_tag, auto check_tag, int t) {
    step(stage_tag, std::integral_constant<int, 0>{}, check_tag, t);
    step(stage_tag, std::integral_constant<int, 1>{}, check_tag, t);
    step(stage_tag, std::integral_constant<int, 2>{}, check_tag, t);
    step(stage_tag, std::integral_constant<int, 3>{}, check_tag, t);
  };
  using S0 = std::integral_constant<int, 0>;
  using S1 = std::integral_constant<int, 1>;

  // ---- prologue: tile 0 whole, the first loads of tile 1; fragments of the first k-step ----
  static_for<G::kLoads>([&](auto d_tag) { dma(d_tag, 0, 0); });
  static_for<G::kD3>([&](auto d_tag) { dma(d_tag, 1, 1); });
  LLC_WAIT_VM(G::kD3);
  __builtin_amdgcn_sched_barrier(0);
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_sched_barrier(0);
  static_for<G::NR>([&](auto r_tag) { read_item(r_tag, S0{}, S0{}, S0{}); });

  // tiles in pairs (the stage is a compile-time constant) while the loads they schedule all exist, then one by one
  int t = 0;
  for (; t + 3 < nk; t += 2) {
    tile(S0{}, std::false_type{}, t);
    tile(S1{}, std::false_type{}, t + 1);
  }
  // two or three tiles are left, the first of them at stage 0
  tile(S0{}, std::true_type{}, t);
  tile(S1{}, std::true_type{}, t + 1);
  if (t + 2 < nk) tile(S0{}, std::true_type{}, t + 2);

  // ---- epilogue.  The last barrier (in front of the last k-step) has seen every wave's last fragment read and
  //      last load complete: the stages are free.  Each wave stages its 128 x WTN tile in LDS of its own. ----
  const int64_t c_off = (int64_t)z0 * p.c_sb + (int64_t)z1 * p.c_sb1;
  T* C = (T*)p.C + c_off;
  const T* res = p.residual ? (const T*)p.residual + c_off : nullptr;
  const T* bias = p.bias ? (const T*)p.bias + (int64_t)z0 * p.bias_sb : nullptr;
  char* wst = smem + wave * G::kOutWave;
  const int ncol0 = n0 + wn * G::WTN, mrow0 = m0 + wm * 128;
  // Row block by row block: for one block of 32 rows a lane's sixteen residual loads (8 bytes each) cover, together
  // with the other lanes', 32 rows x 512 contiguous bytes, so every 128-byte line that is fetched is used whole
  // while it is still in the CU's cache (walking the row blocks inside each column group instead cycles through
  // 128 rows x 16 bytes and fetches every line eight times); the next block's loads are requested before this
  // block's arithmetic.
  auto stage_out = [&](auto act_tag, auto res_tag) {
    constexpr int ACT = decltype(act_tag)::value;
    constexpr bool RES = decltype(res_tag)::value;
    uint2 bq[TN][4];
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        bq[j][q] = uint2{0, 0};
        if (bias) bq[j][q] = *(const uint2*)(bias + ncol0 + j * 32 + 8 * q + 4 * lh);
      }
    uint2 rq[2][TN][4];
    auto load_res = [&](int i, int buf) {
      if constexpr (RES) {
        // rows past the last pixel of a convolution are computed and dropped: read their residual from the last row
        const int row = i * 32 + li;
        const int rrow = (CONV && mrow0 + row >= p.M) ? p.M - 1 : mrow0 + row;
        const T* rp = res + (int64_t)rrow * p.c_sm + ncol0 + 4 * lh;
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
          for (int q = 0; q < 4; ++q) rq[buf][j][q] = *(const uint2*)(rp + j * 32 + 8 * q);
      }
    };
    load_res(0, 0);
    // left alone, the scheduler sinks these sixteen loads to their uses, one wait each (16384 x 768 x 768 + bias +
    // residual 28.8 -> 27.9 us)
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      if (i + 1 < TM) load_res(i + 1, (i + 1) & 1);
      const int row = i * 32 + li;
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int col = j * 32 + 8 * q + 4 * lh;  // first of 4 consecutive columns, inside the wave tile
          const uint2 bw2 = bq[j][q];
          uint2 rw2 = {0, 0};
          if constexpr (RES) rw2 = rq[i & 1][j][q];
          float xv[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const uint32_t bw = e < 2 ? bw2.x : bw2.y, rw = e < 2 ? rw2.x : rw2.y;
            const uint16_t bb = (uint16_t)(bw >> (16 * (e & 1))), rb = (uint16_t)(rw >> (16 * (e & 1)));
            float x = acc[i][j][4 * q + e] * p.alpha;
            if constexpr (Elem<T>::kDtype == LLC_BFLOAT16) x += bf16_bits_to_f32(bb);
            else x += f16_bits_to_f32(bb);
            if constexpr (RES) x += (Elem<T>::kDtype == LLC_BFLOAT16) ? bf16_bits_to_f32(rb) : f16_bits_to_f32(rb);
            if constexpr (ACT == LLC_ACT_RELU) x = x < 0.0f ? 0.0f : x;
            else if constexpr (ACT == LLC_ACT_GELU) x = gelu_for<T>(x);
            xv[e] = x;
          }
          *(uint2*)(wst + row * G::kOutPitch + col * 2) =
              uint2{pack_pair<Elem<T>::kDtype>(xv[0], xv[1]), pack_pair<Elem<T>::kDtype>(xv[2], xv[3])};
        }
      // this block of 32 rows goes out now, as 16-byte pieces of whole rows: its stores drain while the next block's
      // arithmetic runs (the stores of a whole tile issued together at the end cost 10 us of a 93 us product)
      constexpr int kChunks = G::WTN / 8;   // 16-byte chunks per row of the wave tile
      constexpr int kIts = kChunks / 2;     // 64 lanes cover 64 / kChunks rows: kIts steps per 32 rows
#pragma unroll
      for (int it = 0; it < kIts; ++it) {
        const int idx = (i * kIts + it) * 64 + lane;
        const int orow = idx / kChunks, ch = idx % kChunks;
        const u32x4_t v = *(const u32x4_t*)(wst + orow * G::kOutPitch + ch * 16);
        if (!CONV || mrow0 + orow < p.M) *(u32x4_t*)(C + (int64_t)(mrow0 + orow) * p.c_sm + ncol0 + ch * 8) = v;
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
}

template <typename T, int BMODE, int BN, bool CONV = false>
int launch_wide(const GemmParams& p0, int batch, hipStream_t s) {
  using G = WideGeom<BN>;
  GemmParams p = p0;
  p.tiles_m = (p.M + 255) / 256;  // whole tiles, except the last rows of a convolution
  p.tiles_n = p.N / BN;
  auto kern = gemm_wide_kernel<T, BMODE, BN, CONV>;
  static std::atomic<uint32_t> lds_allowed{0};
  LLC_TRY(allow_dynamic_lds((const void*)kern, G::kLds, lds_allowed));
  hipLaunchKernelGGL(kern, dim3((unsigned)(p.tiles_m * p.tiles_n), 1, (unsigned)batch), dim3(256), G::kLds, s, p);
  return check_launch("gemm_wide_kernel");
}
