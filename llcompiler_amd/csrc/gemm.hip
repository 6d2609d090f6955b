// llh.matmul / llh.batch_matmul on the CDNA4 matrix cores.
//
//   C[z][m][n] = act(alpha * sum_k A[z][m][k] * B[z][k][n] + bias[n] + residual[z][m][n])
//
// bf16 / f16 operands use v_mfma_f32_32x32x16_{bf16,f16}; fp32 operands use
// v_mfma_f32_32x32x2_f32 (fp32 products, fp32 accumulate) so that fp32 graphs keep fp32 accuracy.
// Accumulation is always fp32.
//
// Three kernels share the tile geometry of gemm_core.hpp.  gemm_kernel (any type, any strides, ragged shapes)
// is described here; gemm_dma_kernel and gemm_dma2_kernel (16-bit operands, complete tiles, operands moved
// straight into LDS) are described where they are defined.  A fourth, gemm_skinny_kernel, takes products of
// at most 16 rows without the matrix cores (one pass over the weight, bound by its latency).
//
// Data path of gemm_kernel per workgroup (4 waves in a 2x2 grid, or 8 waves 4x2 on 128x128 tiles with a deep
// reduction; macro tile BM x BN):
//   HBM/L2 --16-byte global loads--> registers --> LDS tile [row][128 bytes of k] whose 16-byte
//   chunks are XOR-swizzled by the row (no padding; fragment reads, row copies and transposing
//   stores all spread over the banks) --> ds_read_b128 fragments --> MFMA.  Two LDS buffers and two
//   register stages: global loads for k-tile t+2 are issued before the MFMAs of tile t, tile t+1 is
//   written to the other buffer after them, one barrier per tile.
// A fragment is "8 consecutive k of one row" for both operands.  Operands whose unit-stride dim is
// k (row-major A; B given as [N,K], i.e. a transposed weight view) are copied as they are; a
// row-major B (unit stride along n) is transposed in registers on its way to LDS.  Anything else
// (odd strides, extents that break 16-byte alignment) takes an element-wise loader.
//
// Workgroup -> tile mapping is XCD aware: consecutive workgroup ids are dealt round-robin to the 8
// XCDs by the hardware, so ids are first regrouped per XCD and then walked in column-grouped order,
// which gives each XCD's L2 a compact patch of the output (few distinct A row-panels / B
// column-panels).

#include <cstdlib>
#include <mutex>
#include <type_traits>

#include "gemm_core.hpp"

namespace llc {
using namespace gemm;
namespace {

struct GemmParams {
  const char* A;
  const char* B;
  char* C;
  const char* bias;      // [N] (or [outer batches, N], row pitch bias_sb) or null, same type as C
  int64_t bias_sb;       // elements between the bias rows of consecutive outer batches (0: one row for all)
  const char* residual;  // [batch, M, N] contiguous or null, same type as C
  int32_t M, N, K;
  int64_t a_sm, a_sk, a_sb;  // element strides of A along m, k, batch
  int64_t b_sk, b_sn, b_sb;  // element strides of B along k, n, batch
  int64_t c_sb;              // batch stride of C (outer batch stride when bdiv > 1)
  int64_t c_sb1, c_sm;       // inner batch stride and row pitch of C (c_sm = N, c_sb1 = M N for a contiguous output)
  // Two-level batches ([B0, B1, M, K] operands: attention heads taken as a strided view of [B, S, H*D]):
  // batch z = z0 * bdiv + z1 reads A + z0 * a_sb + z1 * a_sb1.  One-level batches have bdiv = 1.
  int64_t a_sb1, b_sb1;
  int32_t bdiv;
  float alpha;
  int32_t act;
  int32_t tiles_m, tiles_n;
  int32_t c_f32;  // gemm_kernel only: C holds raw fp32 sums whatever T is (the chunks of a split reduction)
  ConvWideGeom cg;  // gemm_wide_kernel<.., CONV = true> only: A is an image, its rows are gathered windows
};

template <typename T, int BM, int BN, int WM, int WN, int LA, int LB, bool FULL>
__global__ __launch_bounds__(64 * WM * WN) void gemm_kernel(const GemmParams p) {
  constexpr int NT = 64 * WM * WN;
  constexpr int BK = kRowBytes / sizeof(T);
  constexpr int WTM = BM / WM, WTN = BN / WN;  // wave tile
  constexpr int TM = WTM / 32, TN = WTN / 32;
  constexpr int kABytes = BM * kRowStride, kBBytes = BN * kRowStride;
  constexpr int kBufBytes = kABytes + kBBytes;  // buffer b: A tile at b*kBufBytes, B tile right after it
  extern __shared__ __align__(16) char smem[];

  int tile_m, tile_n;
  int z;
  tile_and_batch_of_block(p.tiles_m, p.tiles_n, tile_m, tile_n, z);
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  const int z0 = z / p.bdiv, z1 = z - z0 * p.bdiv;
  const T* A = (const T*)p.A + (int64_t)z0 * p.a_sb + (int64_t)z1 * p.a_sb1;
  const T* B = (const T*)p.B + (int64_t)z0 * p.b_sb + (int64_t)z1 * p.b_sb1;

  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int wm = wave / WN, wn = wave % WN;
  const int li = lane % 32, lh = lane / 32;

  f32x16_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  // Two register stages: the global loads of k-tile t+2 are issued before the MFMAs of tile t, tile t+1
  // (issued one iteration earlier) is written to the other LDS buffer after them.  The loop is unrolled
  // by two so that the stage index is a compile-time constant (register arrays, not scratch).
  TileLoader<T, BM, LA, NT> la0, la1;
  TileLoader<T, BN, LB, NT> lb0, lb1;
  const int nk = (p.K + BK - 1) / BK;
  la0.template load<FULL>(A, m0, p.M, 0, p.K, p.a_sm, p.a_sk);
  lb0.template load<FULL>(B, n0, p.N, 0, p.K, p.b_sn, p.b_sk);
  if (nk > 1) {
    la1.template load<FULL>(A, m0, p.M, BK, p.K, p.a_sm, p.a_sk);
    lb1.template load<FULL>(B, n0, p.N, BK, p.K, p.b_sn, p.b_sk);
  }
  la0.store(smem);
  lb0.store(smem + kABytes);
  __syncthreads();

#define LLC_GEMM_STEP(KT, CUR, LA2, LB2, LA1, LB1, GUARDED)                                                     \
  {                                                                                                             \
    /* LA2/LB2: stage that held tile KT (now in LDS) and receives tile KT+2; LA1/LB1 hold tile KT+1 */          \
    if (!(GUARDED) || (KT) + 2 < nk) {                                                        \
      LA2.template load<FULL>(A, m0, p.M, ((KT) + 2) * BK, p.K, p.a_sm, p.a_sk);                                \
      LB2.template load<FULL>(B, n0, p.N, ((KT) + 2) * BK, p.K, p.b_sn, p.b_sk);                                \
    }                                                                                                           \
    /* keep the loads up here: they must be in flight for two tiles, the scheduler would sink them */         \
    \
    mma_tile<T, TM, TN>(smem + (CUR) * kBufBytes, wm * WTM + li, smem + (CUR) * kBufBytes + kABytes,          \
                          wn * WTN + li, lh, acc);                                                              \
    \
    if (!(GUARDED) || (KT) + 1 < nk) {                                                       \
      LA1.store(smem + ((CUR) ^ 1) * kBufBytes);                                                                \
      LB1.store(smem + ((CUR) ^ 1) * kBufBytes + kABytes);                                                      \
    }                                                                                                           \
    __syncthreads();                                                                                            \
  }
  // steady state: no control flow inside the body (every load and store is known to be needed), so the
  // accumulators stay where the MFMAs leave them; the last up to three tiles run the guarded form
  int kt = 0;
  for (; kt + 3 < nk; kt += 2) {
    LLC_GEMM_STEP(kt, 0, la0, lb0, la1, lb1, false)
    LLC_GEMM_STEP(kt + 1, 1, la1, lb1, la0, lb0, false)
  }
  for (; kt < nk; kt += 2) {
    LLC_GEMM_STEP(kt, 0, la0, lb0, la1, lb1, true)
    if (kt + 1 < nk) LLC_GEMM_STEP(kt + 1, 1, la1, lb1, la0, lb0, true)
  }
#undef LLC_GEMM_STEP

  // ---- epilogue.  32x32 accumulator layout: register r of lane (li, lh) is row 8*(r/4) + 4*lh + r%4,
  //      column li: for fixed r, 32 lanes store 32 consecutive columns of one row. ----
  const int64_t c_off = (int64_t)z0 * p.c_sb + (int64_t)z1 * p.c_sb1;
  T* C = (T*)p.C + c_off;
  const char* res = p.residual ? p.residual + c_off * (int64_t)sizeof(T) : nullptr;
  // the bias of every column block is requested before the first block stores (behind a store, which may alias it, the
  // next block's bias would wait for that store)
  float bvs[TN];
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int col = n0 + wn * WTN + j * 32 + li;
    bvs[j] = p.bias ? load_as_f32(p.bias, Elem<T>::kDtype, (int64_t)z0 * p.bias_sb + (FULL || col < p.N ? col : p.N - 1)) : 0.0f;
  }
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int col = n0 + wn * WTN + j * 32 + li;
    if (!FULL && col >= p.N) continue;
    const float bv = bvs[j];
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const int row0 = m0 + wm * WTM + i * 32 + lh * 4;  // the lane's first row of this block
      const int rows_left = p.M - row0;
      const int64_t base = (int64_t)(FULL || rows_left > 0 ? row0 : p.M - 1) * p.c_sm + col;
      if (sizeof(T) != 4 && p.c_f32) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int ro = (r / 4) * 8 + (r % 4);
          if (FULL || ro < rows_left) ((float*)p.C)[c_off + base + (int64_t)ro * p.c_sm] = acc[i][j][r];
        }
      } else {
        epilogue_block16<T, !FULL>(C, res, base, p.c_sm, rows_left, acc[i][j], p.alpha, [&](int) { return bv; }, p.act);
      }
    }
  }
}

// ---------------------------------------------------------------------------------------------
// 16-bit operands, complete 128x128x64 tiles, 16-byte aligned rows: operands go HBM/L2 -> LDS
// directly (global_load_lds_dwordx4, no staging registers and no ds_write), NS LDS stages deep.
//
// 8 waves = 2 (m) x 2 (n) x 2 (k halves): each wave owns a 64x64 accumulator tile over one half of
// every k-tile, which halves the LDS fragment traffic per MFMA against a 32x64 wave tile while
// keeping two waves per SIMD (an LDS instruction stream is rate-limited per wave).  The two k halves
// are summed through LDS in the epilogue, which also turns the accumulator layout into row-major
// 16-byte stores.
//
// LDS stage: A tile [128 m][128 B of k] with the row-XOR chunk swizzle of lds_off(); B tile either
// the same [128 n][128 B of k] (B unit-stride along k) or, for a row-major B, the tile as it lies in
// memory, [64 k][256 B of n], read back with ds_read_b64_tr_b16 (each 16-lane group reads a 4(k) x
// 16(n) patch and receives, per lane, the four k of one n).  The swizzle is applied on the global
// side: lane L of a load lands at LDS byte 16 L of its 1 KB slice, so it fetches the chunk that
// belongs there.
//
// Frag registers are double-buffered across k-tiles: the ds_reads of tile t+1 are issued before the
// MFMAs of tile t, one barrier per tile.  Load completion is tracked by hand (s_waitcnt vmcnt): every
// wave issues exactly four loads per tile and nothing else in the loop uses that counter.
enum { kBKMajor = 0, kBNMajor = 1 };
typedef float f32x4_t __attribute__((ext_vector_type(4)));

// ds_read_b64_tr_b16: the 16 lanes of a group each address 8 bytes (four 16-bit values); lane i of the group
// receives value i % 4 of lanes i / 4, 4 + i / 4, 8 + i / 4, 12 + i / 4.
__device__ __forceinline__ uint2 lds_read_tr16(uint32_t addr) {
  uint2 v;
  asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(v) : "v"(addr));
  return v;
}
#define LLC_GPTR(p) ((const __attribute__((address_space(1))) void*)(p))
#define LLC_LPTR(p) ((__attribute__((address_space(3))) void*)(p))
// s_waitcnt immediate (gfx9 encoding): vmcnt <= VM and lgkmcnt <= 0, expcnt untouched
#define LLC_WAIT_VM_LGKM0(VM) __builtin_amdgcn_s_waitcnt(((VM) & 15) | (7 << 4) | (0 << 8) | (((VM) >> 4) << 14))

constexpr int kDmaStage = 32768;       // bytes of one LDS stage: A tile, then B tile
constexpr int kDmaBOff = 16384;
constexpr int kStagePitch = 136;       // floats per row of the epilogue staging tile (bank spread)
constexpr int kStageHalf = 128 * kStagePitch * 4;

// Addresses of one wave's share of the direct-to-LDS loads and of its fragment reads (see the layout notes
// above).  Wave = ks * 4 + wm * 2 + wn.
template <typename T, int BMODE>
struct DmaOperands {
  const char* ga[2];
  const char* gb[2];
  int la[2], lb[2];
  int64_t b_step;
  int oa[2][2], ob[2][2][BMODE == kBKMajor ? 1 : 2];  // [k step][fragment]([transposing read])

  __device__ __forceinline__ void init(const GemmParams& p, const T* A, const T* B, int m0, int n0, int wave, int lane) {
    const int ks = wave >> 2, wm = (wave >> 1) & 1, wn = wave & 1;
    const int li = lane % 32, lh = lane / 32;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int r0 = (wave * 2 + j) * 8, row = r0 + lane / 8;
      ga[j] = (const char*)(A + (int64_t)(m0 + row) * p.a_sm + (((lane % 8) ^ lds_swz(row)) << 3));
      la[j] = r0 * kRowStride;
      if constexpr (BMODE == kBKMajor) {
        gb[j] = (const char*)(B + (int64_t)(n0 + row) * p.b_sn + (((lane % 8) ^ lds_swz(row)) << 3));
        lb[j] = kDmaBOff + r0 * kRowStride;
      } else {
        const int k0 = (wave * 2 + j) * 4, krow = k0 + lane / 16;
        gb[j] = (const char*)(B + (int64_t)krow * p.b_sk + n0 + (((lane % 16) ^ ((krow & 3) << 2)) << 3));
        lb[j] = kDmaBOff + k0 * 256;
      }
    }
    if constexpr (BMODE == kBKMajor) b_step = 128;
    else b_step = 64 * p.b_sk * 2;
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      const int chunk = ks * 4 + s * 2 + lh;
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int ra = wm * 64 + i * 32 + li;
        oa[s][i] = ra * kRowStride + ((chunk ^ lds_swz(ra)) << 4);
        if constexpr (BMODE == kBKMajor) {
          const int rb = wn * 64 + i * 32 + li;
          ob[s][i][0] = kDmaBOff + rb * kRowStride + ((chunk ^ lds_swz(rb)) << 4);
        } else {
          // lane = 16 g + 4 jj + q reads 8 bytes: k row jj of the patch, n = 16 (g & 1) + 4 q .. + 3
          const int g = lane / 16, jj = (lane / 4) % 4, q = lane % 4;
          const int nchunk = (wn * 64 + i * 32) / 8 + 2 * (g & 1) + (q >> 1);
#pragma unroll
          for (int u = 0; u < 2; ++u) {
            const int krow = ks * 32 + s * 16 + 8 * (g >> 1) + 4 * u + jj;
            ob[s][i][u] = kDmaBOff + krow * 256 + ((nchunk ^ (jj << 2)) << 4) + (q & 1) * 8;
          }
        }
      }
    }
  }

  // next k-tile of both operands into `stage`
  __device__ __forceinline__ void issue(char* smem, int stage) {
    char* base = smem + stage * kDmaStage;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      __builtin_amdgcn_global_load_lds(LLC_GPTR(ga[j]), LLC_LPTR(base + la[j]), 16, 0, 0);
      ga[j] += 128;
    }
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      __builtin_amdgcn_global_load_lds(LLC_GPTR(gb[j]), LLC_LPTR(base + lb[j]), 16, 0, 0);
      gb[j] += b_step;
    }
  }
};

template <typename T, int BMODE, int NS>
__global__ __launch_bounds__(512) void gemm_dma_kernel(const GemmParams p) {
  static_assert(sizeof(T) == 2, "16-bit operands");
  extern __shared__ __align__(16) char smem[];
  int tile_m, tile_n;
  int z;
  tile_and_batch_of_block(p.tiles_m, p.tiles_n, tile_m, tile_n, z);
  const int m0 = tile_m * 128, n0 = tile_n * 128;
  const int z0 = z / p.bdiv, z1 = z - z0 * p.bdiv;
  const T* A = (const T*)p.A + (int64_t)z0 * p.a_sb + (int64_t)z1 * p.a_sb1;
  const T* B = (const T*)p.B + (int64_t)z0 * p.b_sb + (int64_t)z1 * p.b_sb1;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave), lane = threadIdx.x % kWave;
  const int ks = wave >> 2, wm = (wave >> 1) & 1, wn = wave & 1;
  const int li = lane % 32, lh = lane / 32;

  DmaOperands<T, BMODE> op;
  op.init(p, A, B, m0, n0, wave, lane);

  f32x16_t acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;
  u32x4_t fa[2][2][2], fb[2][2][2];  // [set][k step][fragment]
  uint2 tb[2][2][2][2];              // row-major B: the two transposing reads of each B fragment
  const uint32_t lds0 = (uint32_t)(uintptr_t)smem;  // LDS byte address of the first stage

  auto issue = [&](int stage) { op.issue(smem, stage); };
#define LLC_DMA_READ(SET, STAGE)                                                                              \
  {                                                                                                           \
    const char* base = smem + (STAGE) * kDmaStage;                                                            \
    _Pragma("unroll") for (int s = 0; s < 2; ++s) _Pragma("unroll") for (int i = 0; i < 2; ++i) {             \
      fa[SET][s][i] = *(const u32x4_t*)(base + op.oa[s][i]);                                                     \
      if constexpr (BMODE == kBKMajor) {                                                                      \
        fb[SET][s][i] = *(const u32x4_t*)(base + op.ob[s][i][0]);                                                \
      } else {                                                                                                \
        _Pragma("unroll") for (int u = 0; u < 2; ++u)                                                         \
            tb[SET][s][i][u] = lds_read_tr16(lds0 + (STAGE) * kDmaStage + op.ob[s][i][BMODE == kBKMajor ? 0 : u]); \
      }                                                                                                       \
    }                                                                                                         \
  }
// The transposing reads are issued from inline asm, which the compiler does not track: their results may be
// used only after an s_waitcnt lgkmcnt(0).  LLC_DMA_TIE, placed right after that wait, makes every use
// depend on it.
#define LLC_DMA_TIE(SET)                                                                                      \
  if constexpr (BMODE != kBKMajor) {                                                                          \
    asm volatile("" : "+v"(tb[SET][0][0][0]), "+v"(tb[SET][0][0][1]), "+v"(tb[SET][0][1][0]), "+v"(tb[SET][0][1][1]), \
                      "+v"(tb[SET][1][0][0]), "+v"(tb[SET][1][0][1]), "+v"(tb[SET][1][1][0]), "+v"(tb[SET][1][1][1])); \
    _Pragma("unroll") for (int s = 0; s < 2; ++s) _Pragma("unroll") for (int i = 0; i < 2; ++i)               \
        fb[SET][s][i] = u32x4_t{tb[SET][s][i][0].x, tb[SET][s][i][0].y, tb[SET][s][i][1].x, tb[SET][s][i][1].y}; \
  }
#define LLC_DMA_MMA(SET)                                                                                      \
  _Pragma("unroll") for (int s = 0; s < 2; ++s) _Pragma("unroll") for (int i = 0; i < 2; ++i)                 \
      _Pragma("unroll") for (int j = 0; j < 2; ++j) mfma_step<T>(fa[SET][s][i], fb[SET][s][j], acc[i][j]);

  const int nk = p.K / 64;
#pragma unroll
  for (int x = 0; x < NS; ++x)
    if (x < nk) issue(x);
  if (nk >= NS) LLC_WAIT_VM_LGKM0(4 * (NS - 1));
  else LLC_WAIT_VM_LGKM0(0);
  __builtin_amdgcn_s_barrier();
  LLC_DMA_READ(0, 0)

  // Iteration t: tile t's fragments are in registers (set t & 1).  After the barrier tile t+1 is complete
  // in LDS and stage t % NS is free again: it receives tile t + NS.
  int t = 0, st = 0;  // st = t % NS
#define LLC_DMA_NEXT(ST) ((ST) + 1 == NS ? 0 : (ST) + 1)
#define LLC_DMA_STEADY(SET)                                                                                   \
  {                                                                                                           \
    LLC_WAIT_VM_LGKM0(4 * (NS - 2));                                                                          \
    LLC_DMA_TIE(SET)                                                                                          \
    __builtin_amdgcn_s_barrier();                                                                             \
    issue(st);                                                                                                \
    st = LLC_DMA_NEXT(st);                                                                                    \
    LLC_DMA_READ((SET) ^ 1, st)                                                                               \
    LLC_DMA_MMA(SET)                                                                                          \
  }
  for (; t + 1 + NS < nk; t += 2) {
    LLC_DMA_STEADY(0)
    LLC_DMA_STEADY(1)
  }
  // tail: whatever is still to be loaded is loaded, every wait is a full one
#define LLC_DMA_TAIL(TT, SET)                                                                                 \
  {                                                                                                           \
    LLC_WAIT_VM_LGKM0(0);                                                                                     \
    LLC_DMA_TIE(SET)                                                                                          \
    __builtin_amdgcn_s_barrier();                                                                             \
    if ((TT) + NS < nk) issue(st);                                                                            \
    st = LLC_DMA_NEXT(st);                                                                                    \
    if ((TT) + 1 < nk) LLC_DMA_READ((SET) ^ 1, st)                                                            \
    LLC_DMA_MMA(SET)                                                                                          \
  }
  for (; t < nk; t += 2) {
    LLC_DMA_TAIL(t, 0)
    if (t + 1 < nk) LLC_DMA_TAIL(t + 1, 1)
  }
#undef LLC_DMA_READ
#undef LLC_DMA_TIE
#undef LLC_DMA_MMA
#undef LLC_DMA_STEADY
#undef LLC_DMA_TAIL
#undef LLC_DMA_NEXT

  // ---- epilogue: both k halves to LDS as fp32 [half][128][kStagePitch], then row-major 16-byte stores.
  //      No wave reads operand tiles any more (the last fragments were in registers before the last
  //      barrier) and no load is in flight. ----
  float* stage = (float*)(smem + ks * kStageHalf);
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = wm * 64 + i * 32 + (r / 4) * 8 + lh * 4 + (r % 4);
        stage[row * kStagePitch + wn * 64 + j * 32 + li] = acc[i][j][r];
      }
  __syncthreads();
  const int64_t c_off = (int64_t)z0 * p.c_sb + (int64_t)z1 * p.c_sb1;
  T* C = (T*)p.C + c_off;
  const T* res = p.residual ? (const T*)p.residual + c_off : nullptr;
  // bias and residual of all four passes are requested before the first pass stores: inside the loop each pass's loads
  // waited behind the stores of the pass before, which may alias them (a lane's eight columns are the same in every pass)
  u32x4_t bq_all = {0, 0, 0, 0}, rq_all[4] = {{0, 0, 0, 0}, {0, 0, 0, 0}, {0, 0, 0, 0}, {0, 0, 0, 0}};
  if (p.bias) bq_all = *(const u32x4_t*)((const T*)p.bias + (int64_t)z0 * p.bias_sb + n0 + (threadIdx.x % 16) * 8);
  if (res) {
#pragma unroll
    for (int it = 0; it < 4; ++it)
      rq_all[it] = *(const u32x4_t*)(res + (int64_t)(m0 + it * 32 + threadIdx.x / 16) * p.c_sm + n0 + (threadIdx.x % 16) * 8);
  }
#pragma unroll
  for (int it = 0; it < 4; ++it) {
    const int vid = it * 512 + threadIdx.x;
    const int row = vid / 16, c0 = (vid % 16) * 8;
    const float* s0 = (const float*)smem + row * kStagePitch + c0;
    const float* s1 = (const float*)(smem + kStageHalf) + row * kStagePitch + c0;
    float v[8];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const float4 x = *(const float4*)(s0 + 4 * h), y = *(const float4*)(s1 + 4 * h);
      v[4 * h + 0] = x.x + y.x;
      v[4 * h + 1] = x.y + y.y;
      v[4 * h + 2] = x.z + y.z;
      v[4 * h + 3] = x.w + y.w;
    }
    const int64_t o = (int64_t)(m0 + row) * p.c_sm + n0 + c0;
    const u32x4_t bq = bq_all, rq = rq_all[it];
    float xs[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const uint16_t bb = (uint16_t)(bq[e / 2] >> (16 * (e & 1))), rb = (uint16_t)(rq[e / 2] >> (16 * (e & 1)));
      float x = v[e] * p.alpha;
      if constexpr (Elem<T>::kDtype == LLC_BFLOAT16) x += bf16_bits_to_f32(bb);
      else x += f16_bits_to_f32(bb);
      if (res) x += (Elem<T>::kDtype == LLC_BFLOAT16) ? bf16_bits_to_f32(rb) : f16_bits_to_f32(rb);
      if (p.act == LLC_ACT_RELU) x = x < 0.0f ? 0.0f : x;
      else if (p.act == LLC_ACT_GELU) x = gelu_for<T>(x);
      xs[e] = x;
    }
    *(u32x4_t*)(C + o) = u32x4_t{pack_pair<Elem<T>::kDtype>(xs[0], xs[1]), pack_pair<Elem<T>::kDtype>(xs[2], xs[3]),
                                pack_pair<Elem<T>::kDtype>(xs[4], xs[5]), pack_pair<Elem<T>::kDtype>(xs[6], xs[7])};
  }
}

template <typename T, int BMODE>
int launch_dma(const GemmParams& p0, int batch, hipStream_t s) {
#ifndef LLC_DMA_NS
#define LLC_DMA_NS 4
#endif
  constexpr int NS = LLC_DMA_NS;
  GemmParams p = p0;
  p.tiles_m = p.M / 128;
  p.tiles_n = p.N / 128;
  const size_t lds = NS * kDmaStage > 2 * kStageHalf ? NS * kDmaStage : 2 * kStageHalf;
  auto kern = gemm_dma_kernel<T, BMODE, NS>;
  static std::atomic<uint32_t> lds_allowed{0};
  LLC_TRY(allow_dynamic_lds((const void*)kern, (int)lds, lds_allowed));
  hipLaunchKernelGGL(kern, dim3((unsigned)(p.tiles_m * p.tiles_n), 1, (unsigned)batch), dim3(512), lds, s, p);
  return check_launch("gemm_dma_kernel");
}

// ---------------------------------------------------------------------------------------------
// The same tile and wave layout for short reductions (few k-tiles per output tile), where the pipeline
// fill and the epilogue of a workgroup weigh as much as its main loop: two workgroups per CU, so that one
// computes while the other fills or stores.  That halves what a workgroup may hold: two LDS stages (64 KB;
// the epilogue staging fits in the same space), at most 128 registers per lane, hence fragments of one
// k-tile at a time (the other workgroup's waves cover the LDS latency).  The load of tile t+1 is issued at
// the start of iteration t, into the stage all waves left at the barrier.
//
// MFMA operands are swapped (C^T = B^T A^T per fragment pair), which leaves every lane with four
// consecutive columns of one row per accumulator quad: all epilogue LDS traffic is 16-byte accesses.
// The k halves meet through a lane-private layout (same lane, same register in both waves of a pair),
// the sums go to a row-major fp32 tile, and all eight waves apply the epilogue and store 16 bytes per lane.
constexpr int kStage2Pitch = 132;  // floats per row of the fp32 staging tile
constexpr int kDma2Lds = 128 * kStage2Pitch * 4 > 2 * kDmaStage ? 128 * kStage2Pitch * 4 : 2 * kDmaStage;
// s_waitcnt immediate: lgkmcnt <= 0, vmcnt and expcnt untouched
#define LLC_WAIT_LGKM0() __builtin_amdgcn_s_waitcnt(0xC07F)

template <typename T, int BMODE>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(4, 4))) void gemm_dma2_kernel(const GemmParams p) {
  static_assert(sizeof(T) == 2, "16-bit operands");
  extern __shared__ __align__(16) char smem[];
  int tile_m, tile_n;
  int z;
  tile_and_batch_of_block(p.tiles_m, p.tiles_n, tile_m, tile_n, z);
  const int m0 = tile_m * 128, n0 = tile_n * 128;
  const int z0 = z / p.bdiv, z1 = z - z0 * p.bdiv;
  const T* A = (const T*)p.A + (int64_t)z0 * p.a_sb + (int64_t)z1 * p.a_sb1;
  const T* B = (const T*)p.B + (int64_t)z0 * p.b_sb + (int64_t)z1 * p.b_sb1;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave), lane = threadIdx.x % kWave;
  const int ks = wave >> 2, wm = (wave >> 1) & 1, wn = wave & 1;
  const int li = lane % 32, lh = lane / 32;
  DmaOperands<T, BMODE> op;
  op.init(p, A, B, m0, n0, wave, lane);
  const uint32_t lds0 = (uint32_t)(uintptr_t)smem;

  f32x16_t acc[2][2];  // [A fragment][B fragment]; register r: row li of the A fragment, column 8 (r/4) + 4 lh + r%4
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  const int nk = p.K / 64;
  op.issue(smem, 0);
  if (nk > 1) op.issue(smem, 1);
  for (int t = 0; t < nk; ++t) {
    const int st = t & 1;
    // tile t has landed (at t = 0 tile 1 may still be in flight); after the barrier nobody reads the other stage
    if (t == 0 && nk > 1) LLC_WAIT_VM_LGKM0(4);
    else LLC_WAIT_VM_LGKM0(0);
    __builtin_amdgcn_s_barrier();
    if (t >= 1 && t + 1 < nk) op.issue(smem, st ^ 1);
    const char* base = smem + st * kDmaStage;
    u32x4_t fa[2][2], fb[2][2];
    if constexpr (BMODE == kBKMajor) {
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2)
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          fa[s2][i] = *(const u32x4_t*)(base + op.oa[s2][i]);
          fb[s2][i] = *(const u32x4_t*)(base + op.ob[s2][i][0]);
        }
    } else {
      uint2 tb[2][2][2];
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2)
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          fa[s2][i] = *(const u32x4_t*)(base + op.oa[s2][i]);
#pragma unroll
          for (int u = 0; u < 2; ++u) tb[s2][i][u] = lds_read_tr16(lds0 + st * kDmaStage + op.ob[s2][i][BMODE == kBKMajor ? 0 : u]);
        }
      // the transposing reads are inline asm: wait for them by hand and make every use depend on the wait
      LLC_WAIT_LGKM0();
      asm volatile("" : "+v"(tb[0][0][0]), "+v"(tb[0][0][1]), "+v"(tb[0][1][0]), "+v"(tb[0][1][1]), "+v"(tb[1][0][0]),
                        "+v"(tb[1][0][1]), "+v"(tb[1][1][0]), "+v"(tb[1][1][1]));
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2)
#pragma unroll
        for (int i = 0; i < 2; ++i) fb[s2][i] = u32x4_t{tb[s2][i][0].x, tb[s2][i][0].y, tb[s2][i][1].x, tb[s2][i][1].y};
    }
#pragma unroll
    for (int s2 = 0; s2 < 2; ++s2)
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) mfma_step<T>(fb[s2][j], fa[s2][i], acc[i][j]);  // swapped: lane = row, quad = 4 columns
  }

  // ---- epilogue ----
  LLC_WAIT_LGKM0();
  __builtin_amdgcn_s_barrier();  // every wave has read its last fragments: the stages are free
  {
    // k halves: same lane, same register in both waves of a pair
    char* priv = smem + ((((wave & 3) * 16) * 64 + lane) << 4);
    if (ks == 1) {
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
          for (int q = 0; q < 4; ++q)
            *(f32x4_t*)(priv + (((i * 2 + j) * 4 + q) << 10)) = f32x4_t{acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]};
    }
    __syncthreads();
    if (ks == 0) {
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const f32x4_t o = *(const f32x4_t*)(priv + (((i * 2 + j) * 4 + q) << 10));
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[i][j][4 * q + e] += o[e];
          }
    }
    __syncthreads();
    if (ks == 0) {
      float* tile = (float*)smem;
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
          for (int q = 0; q < 4; ++q)
            *(f32x4_t*)(tile + (wm * 64 + i * 32 + li) * kStage2Pitch + wn * 64 + j * 32 + 8 * q + 4 * lh) =
                f32x4_t{acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]};
    }
    __syncthreads();
  }
  const int64_t c_off = (int64_t)z0 * p.c_sb + (int64_t)z1 * p.c_sb1;
  T* C = (T*)p.C + c_off;
  const T* res = p.residual ? (const T*)p.residual + c_off : nullptr;
  // bias and residual of all four passes are requested before the first pass stores: inside the loop each pass's loads
  // waited behind the stores of the pass before, which may alias them (a lane's eight columns are the same in every pass)
  u32x4_t bq_all = {0, 0, 0, 0}, rq_all[4] = {{0, 0, 0, 0}, {0, 0, 0, 0}, {0, 0, 0, 0}, {0, 0, 0, 0}};
  if (p.bias) bq_all = *(const u32x4_t*)((const T*)p.bias + (int64_t)z0 * p.bias_sb + n0 + (threadIdx.x % 16) * 8);
  if (res) {
#pragma unroll
    for (int it = 0; it < 4; ++it)
      rq_all[it] = *(const u32x4_t*)(res + (int64_t)(m0 + it * 32 + threadIdx.x / 16) * p.c_sm + n0 + (threadIdx.x % 16) * 8);
  }
#pragma unroll
  for (int it = 0; it < 4; ++it) {
    const int vid = it * 512 + threadIdx.x;
    const int row = vid / 16, c0 = (vid % 16) * 8;
    const float* s0 = (const float*)smem + row * kStage2Pitch + c0;
    float v[8];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const f32x4_t x = *(const f32x4_t*)(s0 + 4 * h);
      v[4 * h + 0] = x[0];
      v[4 * h + 1] = x[1];
      v[4 * h + 2] = x[2];
      v[4 * h + 3] = x[3];
    }
    const int64_t o = (int64_t)(m0 + row) * p.c_sm + n0 + c0;
    const u32x4_t bq = bq_all, rq = rq_all[it];
    float xs[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const uint16_t bb = (uint16_t)(bq[e / 2] >> (16 * (e & 1))), rb = (uint16_t)(rq[e / 2] >> (16 * (e & 1)));
      float x = v[e] * p.alpha;
      if constexpr (Elem<T>::kDtype == LLC_BFLOAT16) x += bf16_bits_to_f32(bb);
      else x += f16_bits_to_f32(bb);
      if (res) x += (Elem<T>::kDtype == LLC_BFLOAT16) ? bf16_bits_to_f32(rb) : f16_bits_to_f32(rb);
      if (p.act == LLC_ACT_RELU) x = x < 0.0f ? 0.0f : x;
      else if (p.act == LLC_ACT_GELU) x = gelu_for<T>(x);
      xs[e] = x;
    }
    *(u32x4_t*)(C + o) = u32x4_t{pack_pair<Elem<T>::kDtype>(xs[0], xs[1]), pack_pair<Elem<T>::kDtype>(xs[2], xs[3]),
                                pack_pair<Elem<T>::kDtype>(xs[4], xs[5]), pack_pair<Elem<T>::kDtype>(xs[6], xs[7])};
  }
}

template <typename T, int BMODE>
int launch_dma2(const GemmParams& p0, int batch, hipStream_t s) {
  GemmParams p = p0;
  p.tiles_m = p.M / 128;
  p.tiles_n = p.N / 128;
  auto kern = gemm_dma2_kernel<T, BMODE>;
  static std::atomic<uint32_t> lds_allowed{0};
  LLC_TRY(allow_dynamic_lds((const void*)kern, (int)kDma2Lds, lds_allowed));
  hipLaunchKernelGGL(kern, dim3((unsigned)(p.tiles_m * p.tiles_n), 1, (unsigned)batch), dim3(512), kDma2Lds, s, p);
  return check_launch("gemm_dma2_kernel");
}

#include "gemm_wide.hpp"
#include "gemm_sweep.hpp"
#include "gemm_deep.hpp"

template <typename T, int BM, int BN, int WM, int WN, int LA, int LB>
int launch_cfg(const GemmParams& p0, int batch, hipStream_t s) {
  GemmParams p = p0;
  p.tiles_m = (p.M + BM - 1) / BM;
  p.tiles_n = (p.N + BN - 1) / BN;
  const size_t lds = 2 * (size_t)(BM + BN) * kRowStride;
  // every tile complete: the unguarded instantiation (no per-access branches in the main loop)
  const bool full = p.M % BM == 0 && p.N % BN == 0 && p.K % (kRowBytes / (int)sizeof(T)) == 0;
  auto kern = full ? gemm_kernel<T, BM, BN, WM, WN, LA, LB, true> : gemm_kernel<T, BM, BN, WM, WN, LA, LB, false>;
  static std::atomic<uint32_t> lds_allowed[2];  // one per instantiation
  LLC_TRY(allow_dynamic_lds((const void*)kern, (int)lds, lds_allowed[full]));
  const int64_t tiles = (int64_t)p.tiles_m * p.tiles_n;
  if (tiles > 0x7fffffff || batch > 65535) return set_error(LLC_ERR_TOO_LARGE, "matmul: grid too large");
  hipLaunchKernelGGL(kern, dim3((unsigned)tiles, 1, (unsigned)batch), dim3(64 * WM * WN), lds, s, p);
  return check_launch("gemm_kernel");
}

template <typename T, int LA, int LB>
int launch_tiles(const GemmParams& p, int batch, hipStream_t s) {
  // LDS instructions are rate-limited per wave (a wave gets one ds_read_b128 through every ~37 cycles
  // whatever the other waves do), so the deep-K shapes run 8 waves on a 128x128 tile (two per SIMD,
  // wave tile 32x64) to keep the LDS pipe and the matrix cores busy at once.  Short-K or skinny
  // shapes keep 4 waves and rely on several workgroups per CU.
  const int64_t t128 = (int64_t)((p.M + 127) / 128) * ((p.N + 127) / 128) * batch;
  const bool deep = p.K >= 512;
  if constexpr (sizeof(T) == 4) {
    // fp32 is bound by the (slow) fp32 MFMA, not by LDS or L2: what counts is how evenly the tiles fill the
    // 256 CUs.  A last round that is mostly empty costs more than the ~7% a 64x64 tile loses to a 128x128 one.
    auto fill = [](int64_t blocks) { return (double)blocks / (double)(((blocks + 255) / 256) * 256); };
    const int64_t t64 = (int64_t)((p.M + 63) / 64) * ((p.N + 63) / 64) * batch;
    if (p.N > 64 && p.M > 64 && fill(t128) < 0.8 && fill(t64) > fill(t128) + 0.1)
      return launch_cfg<T, 64, 64, 2, 2, LA, LB>(p, batch, s);
  }
  if (p.N > 64 && p.M > 64 && t128 >= 128) {
    if constexpr (LA != kLoadGeneric) {  // the element-wise loader needs too many registers for 8 waves
      if (deep) return launch_cfg<T, 128, 128, 4, 2, LA, LB>(p, batch, s);
    }
    return launch_cfg<T, 128, 128, 2, 2, LA, LB>(p, batch, s);
  }
  if (p.N <= 64 && p.M > 64) return launch_cfg<T, 128, 64, 2, 2, LA, LB>(p, batch, s);
  return launch_cfg<T, 64, 64, 2, 2, LA, LB>(p, batch, s);
}

// ---- skinny products: at most 16 rows, both operands contiguous along k (x [M,K] times a linear layer's
// weight [N,K] read as its transpose).  A tile kernel would leave all but a few CUs idle and walk k in ~30
// dependent steps; this one is a single pass: one workgroup per NW output columns, its four waves split k in
// 64-lane vector chunks, every lane keeps MR x NW partial sums that are then added across the wave and
// across the waves (LDS).  The sums are taken in a fixed order, so results do not vary from run to run.
template <typename T>
__device__ __forceinline__ void unpack_vec(const u32x4_t& v, float* f) {
  if constexpr (sizeof(T) == 4) {
#pragma unroll
    for (int e = 0; e < 4; ++e) f[e] = __uint_as_float(v[e]);
  } else if constexpr (Elem<T>::kDtype == LLC_BFLOAT16) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      f[2 * e] = __uint_as_float(v[e] << 16);
      f[2 * e + 1] = __uint_as_float(v[e] & 0xffff0000u);
    }
  } else {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      f[2 * e] = f16_bits_to_f32((uint16_t)(v[e] & 0xffffu));
      f[2 * e + 1] = f16_bits_to_f32((uint16_t)(v[e] >> 16));
    }
  }
}

template <typename T, int MR, int NW>
__global__ __launch_bounds__(256) void gemm_skinny_kernel(const GemmParams p) {
  constexpr int VEC = 16 / sizeof(T);
  __shared__ float red[4][MR * NW];
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int n0 = blockIdx.x * NW;
  const T* A = (const T*)p.A;
  const T* B = (const T*)p.B;
  float acc[MR][NW];
#pragma unroll
  for (int m = 0; m < MR; ++m)
#pragma unroll
    for (int j = 0; j < NW; ++j) acc[m][j] = 0.0f;
  for (int k = (int)threadIdx.x * VEC; k < p.K; k += 256 * VEC) {
    u32x4_t av[MR], bv[NW];
    // rows and columns past the end re-read the last one; their sums are never stored
#pragma unroll
    for (int m = 0; m < MR; ++m) av[m] = *(const u32x4_t*)(A + (int64_t)(m < p.M ? m : p.M - 1) * p.a_sm + k);
#pragma unroll
    for (int j = 0; j < NW; ++j) bv[j] = *(const u32x4_t*)(B + (int64_t)(n0 + j < p.N ? n0 + j : p.N - 1) * p.b_sn + k);
    float bf[NW][VEC];
#pragma unroll
    for (int j = 0; j < NW; ++j) unpack_vec<T>(bv[j], bf[j]);
#pragma unroll
    for (int m = 0; m < MR; ++m) {
      float af[VEC];
      unpack_vec<T>(av[m], af);
#pragma unroll
      for (int j = 0; j < NW; ++j)
#pragma unroll
        for (int e = 0; e < VEC; ++e) acc[m][j] = fmaf(af[e], bf[j][e], acc[m][j]);
    }
  }
#pragma unroll
  for (int m = 0; m < MR; ++m)
#pragma unroll
    for (int j = 0; j < NW; ++j) {
      const float v = wave_sum(acc[m][j]);
      if (lane == 0) red[wave][m * NW + j] = v;
    }
  __syncthreads();
  if (threadIdx.x < MR * NW) {
    const int m = threadIdx.x / NW, n = n0 + threadIdx.x % NW;
    if (m < p.M && n < p.N) {
      const float v = (red[0][threadIdx.x] + red[1][threadIdx.x]) + (red[2][threadIdx.x] + red[3][threadIdx.x]);
      const float bias = p.bias ? load_as_f32(p.bias, Elem<T>::kDtype, n) : 0.0f;
      epilogue_store<T>((T*)p.C, (int64_t)m * p.c_sm + n, v, p.alpha, bias, p.residual, p.act);
    }
  }
}

template <typename T>
int launch_skinny(const GemmParams& p, hipStream_t s) {
  if (p.M <= 4) {
    hipLaunchKernelGGL((gemm_skinny_kernel<T, 4, 2>), dim3((unsigned)((p.N + 1) / 2)), dim3(256), 0, s, p);
  } else {
    hipLaunchKernelGGL((gemm_skinny_kernel<T, 16, 1>), dim3((unsigned)p.N), dim3(256), 0, s, p);
  }
  return check_launch("gemm_skinny_kernel");
}

// ---- products with a long reduction and too few output tiles to fill the chip (a transformer's second
// feed-forward layer at a short sequence: 1024 x 768 x 3072 is 192 tiles of 64x64), any storage type.  The reduction is cut into
// `splits` equal chunks that run as the batches of one batched product into fp32 partial results
// [splits][M][N] in the workspace; a second kernel sums them in chunk order (the same order on every run)
// and applies the epilogue.
template <typename T>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float* __restrict__ part, int splits, int64_t mn,
                                                            int n, float alpha, const char* __restrict__ bias,
                                                            const char* __restrict__ residual, int act, T* __restrict__ out) {
  const int64_t i4 = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
  if (i4 >= mn) return;
  const int col = (int)(i4 % n);  // n is a multiple of 4: the four values share a row
  split_epilogue4<T>(part, splits, mn, i4, col, alpha, bias, residual, act, out);
}

// Number of reduction chunks, 1 = no split; bk = elements of a k-tile (32 for fp32, 64 for the 16-bit types).  A
// split pays when the 64x64 tiles cover less than two rounds of the 256 CUs and the reduction is long (measured,
// fp32: 1024 x 768 x 3072 goes from 64 to 50 us in four chunks, 2048 x 768 x 3072 from 110 to 94 us in two; bf16:
// 512 x 768 x 3072 from 22 to 15 us, 1024 x 768 x 3072 from 23 to 18.5 us; at K = 768 every split loses to the plain
// kernel).  The smallest chunk count that gives three (fp32) or two (16-bit, whose tiles are done sooner)
// workgroups per CU is taken, chunks of at least 256.
inline int splitk_chunks(const GemmParams& p, int bk) {
  const int64_t t64 = (int64_t)((p.M + 63) / 64) * ((p.N + 63) / 64);
  if (p.K < 1536 || t64 >= 512 || p.M <= 64 || p.N <= 64 || p.N % 4 != 0 || p.c_sm != p.N) return 1;
  const int64_t enough = bk == 32 ? 768 : 512;
  int best = 1;
  for (int sp = 2; sp <= 8; ++sp) {
    if (p.K % (sp * bk) != 0 || p.K / sp < 256) continue;
    if (t64 * sp > 1024) break;
    best = sp;
    if (t64 * sp >= enough) break;
  }
  return best;
}

template <typename T, int LB>
int launch_splitk(const GemmParams& p, int splits, hipStream_t s) {
  const int64_t mn = (int64_t)p.M * p.N;
  void* ws = nullptr;
  LLC_TRY(get_workspace((size_t)splits * mn * sizeof(float), &ws, s));
  GemmParams q = p;
  q.K = p.K / splits;
  q.a_sb = (int64_t)q.K * p.a_sk;
  q.b_sb = (int64_t)q.K * p.b_sk;
  q.a_sb1 = q.b_sb1 = 0;
  q.bdiv = 1;
  q.C = (char*)ws;
  q.c_sb = mn;
  q.c_sb1 = 0;
  q.c_sm = p.N;
  q.c_f32 = 1;
  q.bias = nullptr;
  q.bias_sb = 0;
  q.residual = nullptr;
  q.alpha = 1.0f;
  q.act = LLC_ACT_NONE;
  LLC_TRY((launch_tiles<T, kLoadKVec, LB>(q, splits, s)));
  const int64_t blocks = (mn / 4 + 255) / 256;
  hipLaunchKernelGGL(splitk_reduce_kernel<T>, dim3((unsigned)blocks), dim3(256), 0, s, (const float*)ws, splits, mn, p.N,
                     p.alpha, p.bias, p.residual, p.act, (T*)p.C);
  return check_launch("splitk_reduce_kernel");
}

// Column extent of the 256 x BN tile for a 16-bit product with complete tiles, 0 = keep the 128 x 128 kernels.
// One workgroup per CU: the cost of a candidate is its number of rounds over the 256 CUs times the tile's work,
// weighted by how well that tile shape runs (narrower tiles read more LDS and L2 bytes per MFMA).
inline int wide_tile_n(const GemmParams& p, int batch, bool b_kvec) {
  int best = 0;
  double best_cost = 0.0;
  const int cand[3] = {256, 192, 128};
  const double weight[3] = {1.0, 1.05, 1.2};
  for (int c = 0; c < 3; ++c) {
    const int bn = cand[c];
    if (p.N % bn != 0 || (bn == 192 && !b_kvec)) continue;
    const int64_t tiles = (int64_t)(p.M / 256) * (p.N / bn) * batch;
    if (tiles > 0x7fffffff || batch > 65535) continue;
    const double cost = (double)((tiles + 255) / 256) * bn * weight[c];
    if (best == 0 || cost < best_cost) {
      best = bn;
      best_cost = cost;
    }
  }
  if (best == 0) return 0;
  // fewer workgroups than 3/4 of the CUs: the 128 x 128 kernels fill the chip better
  const int64_t tiles = (int64_t)(p.M / 256) * (p.N / best) * batch;
  if (tiles < 192) return 0;
  return best;
}

template <typename T>
int launch_loaders(const GemmParams& p, int batch, hipStream_t s) {
  constexpr int EPV = 16 / sizeof(T);
  auto al16 = [](const void* q) { return ((uintptr_t)q % 16) == 0; };
  const bool a_kvec = p.a_sk == 1 && p.a_sm % EPV == 0 && p.a_sb % EPV == 0 && p.a_sb1 % EPV == 0 && p.K % EPV == 0 && al16(p.A);
  const bool b_kvec = p.b_sk == 1 && p.b_sn % EPV == 0 && p.b_sb % EPV == 0 && p.b_sb1 % EPV == 0 && p.K % EPV == 0 && al16(p.B);
  const bool b_rvec = p.b_sn == 1 && p.b_sk % EPV == 0 && p.b_sb % EPV == 0 && p.b_sb1 % EPV == 0 && p.N % EPV == 0 && al16(p.B);
  if (batch == 1 && p.M <= 16 && a_kvec && b_kvec) return launch_skinny<T>(p, s);
  if (batch == 1 && a_kvec && (b_kvec || b_rvec) && al16(p.C) && (!p.residual || al16(p.residual))) {
    const int splits = splitk_chunks(p, kRowBytes / (int)sizeof(T));
    if (splits > 1) return b_kvec ? launch_splitk<T, kLoadKVec>(p, splits, s) : launch_splitk<T, kLoadRVec>(p, splits, s);
  }
  if (p.K == 64 && a_kvec && b_rvec && sweep_ok<T>(p, batch)) return launch_sweep<T>(p, batch, s);
  if constexpr (sizeof(T) == 2) {
    const bool dma_ok = a_kvec && (b_kvec || b_rvec) && p.K % 64 == 0 && al16(p.C) && p.c_sb % EPV == 0 && p.c_sb1 % EPV == 0 &&
                        p.c_sm % EPV == 0 && (!p.bias || (al16(p.bias) && p.bias_sb % EPV == 0)) && (!p.residual || al16(p.residual));
    if (dma_ok && p.M % 256 == 0 && p.K >= 128) {
      const int bn = wide_tile_n(p, batch, b_kvec);
      if (bn == 256) return b_kvec ? launch_wide<T, kBKMajor, 256>(p, batch, s) : launch_wide<T, kBNMajor, 256>(p, batch, s);
      if (bn == 192) return launch_wide<T, kBKMajor, 192>(p, batch, s);
      if (bn == 128) return b_kvec ? launch_wide<T, kBKMajor, 128>(p, batch, s) : launch_wide<T, kBNMajor, 128>(p, batch, s);
    }
    const int64_t tiles = (int64_t)(p.M / 128) * (p.N / 128) * batch;
    if (a_kvec && (b_kvec || b_rvec) && p.M % 128 == 0 && p.N % 128 == 0 && p.K % 64 == 0 && (p.K >= 256 || tiles >= 512) &&
        tiles >= 128 && tiles <= 0x7fffffff && al16(p.C) && p.c_sb % EPV == 0 && p.c_sb1 % EPV == 0 && p.c_sm % EPV == 0 && (!p.bias || (al16(p.bias) && p.bias_sb % EPV == 0)) &&
        (!p.residual || al16(p.residual)))
    {
      // short reductions, or more tiles than one round of workgroups: two workgroups per CU
      const bool two = p.K <= 1536 && tiles >= 512;
      if (two) return b_kvec ? launch_dma2<T, kBKMajor>(p, batch, s) : launch_dma2<T, kBNMajor>(p, batch, s);
      return b_kvec ? launch_dma<T, kBKMajor>(p, batch, s) : launch_dma<T, kBNMajor>(p, batch, s);
    }
    if (dma_ok && b_kvec && deep_ok(p, batch)) return launch_deep<T>(p, batch, s);
  }
  if (a_kvec && b_kvec) return launch_tiles<T, kLoadKVec, kLoadKVec>(p, batch, s);
  if (a_kvec && b_rvec) return launch_tiles<T, kLoadKVec, kLoadRVec>(p, batch, s);
  return launch_tiles<T, kLoadGeneric, kLoadGeneric>(p, batch, s);
}

}  // namespace

int conv_wide_16bit(int dtype, const char* x, const char* w, char* y, const char* bias, const char* residual, int F,
                    const ConvWideGeom& g, float alpha, int act, hipStream_t s) {
  const int64_t K = (int64_t)g.KH * g.KW * g.C;
  // (reductions shorter than 2048 are too few k-tiles per tile for one workgroup per CU: a tile's fill and drain weigh
  // as much as its loop, and the kernels that keep two workgroups on a CU are faster; measured at batch 32:
  // 128 -> 128 channels 3x3 on 56x56 68 us here against 61, 256 -> 256 159 against 197, 512 -> 512 on 28x28 127 against 177)
  if ((dtype != LLC_BFLOAT16 && dtype != LLC_FLOAT16) || g.C % 64 != 0 || g.KH * g.KW > 32 || K < 2048 || F % 128 != 0) return 1;
  // one workgroup per CU and tile: worth it only when the tiles fill at least three quarters of the chip
  const int64_t tiles_m = (g.ncols + 255) / 256;
  int bn = 0;
  if (F % 256 == 0 && tiles_m * (F / 256) >= 192) bn = 256;
  else if (tiles_m * (F / 128) >= 192) bn = 128;
  if (bn == 0 || tiles_m * (F / bn) > 0x7fffffff) return 1;
  GemmParams p{};
  p.A = x;
  p.B = w;
  p.C = y;
  p.bias = bias;
  p.residual = residual;
  p.M = g.ncols;
  p.N = F;
  p.K = (int32_t)K;
  p.a_sk = 1;
  p.b_sk = 1;
  p.b_sn = K;
  p.c_sm = F;
  p.bdiv = 1;
  p.alpha = alpha;
  p.act = act;
  p.cg = g;
  if (dtype == LLC_BFLOAT16) return bn == 256 ? launch_wide<__bf16, kBKMajor, 256, true>(p, 1, s) : launch_wide<__bf16, kBKMajor, 128, true>(p, 1, s);
  return bn == 256 ? launch_wide<_Float16, kBKMajor, 256, true>(p, 1, s) : launch_wide<_Float16, kBKMajor, 128, true>(p, 1, s);
}

namespace {
int gemm_dispatch(int dtype, const GemmParams& p, int batch, hipStream_t s) {
  if (p.M == 0 || p.N == 0 || batch == 0) return LLC_OK;
  switch (dtype) {
    case LLC_FLOAT32: return launch_loaders<float>(p, batch, s);
    case LLC_BFLOAT16: return launch_loaders<__bf16>(p, batch, s);
    case LLC_FLOAT16: return launch_loaders<_Float16>(p, batch, s);
  }
  return set_error(LLC_ERR_DTYPE, "matmul: element type %d (f32, bf16 or f16 expected)", dtype);
}

// n_outer: number of outer batches (1 for matmul); a bias of n_outer rows gives every outer batch its own
int fill_epilogue(const llc_epilogue* epi, const View& o, int64_t n_cols, GemmParams* p, int64_t n_outer = 1) {
  p->alpha = 1.0f;
  p->act = LLC_ACT_NONE;
  p->bias = nullptr;
  p->bias_sb = 0;
  p->residual = nullptr;
  if (!epi) return LLC_OK;
  p->alpha = epi->alpha;
  if (epi->act < LLC_ACT_NONE || epi->act > LLC_ACT_GELU) return set_error(LLC_ERR_BAD_ARG, "epilogue: activation %d", epi->act);
  p->act = epi->act;
  if (epi->bias) {
    View b;
    LLC_TRY(make_view(epi->bias, "epilogue bias", &b));
    if (b.dtype != o.dtype) return set_error(LLC_ERR_DTYPE, "epilogue: bias type differs from output");
    const bool rows = n_outer > 1 && b.rank == 2 && b.size[0] == n_outer && b.size[1] == n_cols;
    if ((b.numel() != n_cols && !rows) || !b.contiguous())
      return set_error(LLC_ERR_SHAPE, "epilogue: bias must hold %lld contiguous values (or one such row per outer batch)", (long long)n_cols);
    p->bias = b.ptr;
    p->bias_sb = rows ? n_cols : 0;
  }
  if (epi->residual) {
    View r;
    LLC_TRY(make_view(epi->residual, "epilogue residual", &r));
    if (r.dtype != o.dtype) return set_error(LLC_ERR_DTYPE, "epilogue: residual type differs from output");
    if (r.numel() != o.numel() || !r.contiguous()) return set_error(LLC_ERR_SHAPE, "epilogue: residual must match the output and be contiguous");
    p->residual = r.ptr;
  }
  return LLC_OK;
}

}  // namespace
}  // namespace llc

using namespace llc;

int llc_impl_matmul(const llc_tensor* lhs, const llc_tensor* rhs, const llc_epilogue* epi, llc_tensor* out,
                              void* stream) {
  View a, b, o;
  LLC_TRY(make_view(lhs, "matmul lhs", &a));
  LLC_TRY(make_view(rhs, "matmul rhs", &b));
  LLC_TRY(make_view(out, "matmul out", &o));
  if (a.rank != 2 || b.rank != 2 || o.rank != 2) return set_error(LLC_ERR_SHAPE, "matmul: rank-2 tensors expected (LLH_2DTensor)");
  if (a.dtype != b.dtype || a.dtype != o.dtype) return set_error(LLC_ERR_DTYPE, "matmul: operand types differ");
  if (a.size[1] != b.size[0] || o.size[0] != a.size[0] || o.size[1] != b.size[1])
    return set_error(LLC_ERR_SHAPE, "matmul: [%lld,%lld] x [%lld,%lld] -> [%lld,%lld]", (long long)a.size[0], (long long)a.size[1],
                     (long long)b.size[0], (long long)b.size[1], (long long)o.size[0], (long long)o.size[1]);
  if (!o.contiguous()) return set_error(LLC_ERR_LAYOUT, "matmul: output must be contiguous");
  if (a.size[0] > 0x7fffffff || a.size[1] > 0x7fffffff || b.size[1] > 0x7fffffff) return set_error(LLC_ERR_TOO_LARGE, "matmul: extent too large");
  GemmParams p{};
  p.A = a.ptr;
  p.B = b.ptr;
  p.C = o.ptr;
  p.M = (int)a.size[0];
  p.K = (int)a.size[1];
  p.N = (int)b.size[1];
  p.a_sm = a.stride[0];
  p.a_sk = a.stride[1];
  p.b_sk = b.stride[0];
  p.b_sn = b.stride[1];
  p.bdiv = 1;
  p.c_sm = p.N;
  LLC_TRY(fill_epilogue(epi, o, p.N, &p));
  return gemm_dispatch(a.dtype, p, 1, as_stream(stream));
}

int llc_impl_batch_matmul(const llc_tensor* lhs, const llc_tensor* rhs, const llc_epilogue* epi,
                                    llc_tensor* out, void* stream) {
  View a, b, o;
  LLC_TRY(make_view(lhs, "batch_matmul lhs", &a));
  LLC_TRY(make_view(rhs, "batch_matmul rhs", &b));
  LLC_TRY(make_view(out, "batch_matmul out", &o));
  // LLH_3DTensor operands; as an extension an operand may be rank 4, [B0, B1, M, K]: the head split of an
  // attention layer is then a strided view of the [B, S, H*D] activation instead of a copy.
  if ((a.rank != 3 && a.rank != 4) || (b.rank != 3 && b.rank != 4) || (o.rank != 3 && o.rank != 4))
    return set_error(LLC_ERR_SHAPE, "batch_matmul: rank-3 tensors expected (LLH_3DTensor), or rank 4 with two batch dims");
  if (a.dtype != b.dtype || a.dtype != o.dtype) return set_error(LLC_ERR_DTYPE, "batch_matmul: operand types differ");
  const int ra = a.rank - 2, rb = b.rank - 2, ro = o.rank - 2;  // number of batch dims
  const int64_t nba = ra == 2 ? a.size[0] * a.size[1] : a.size[0], nbb = rb == 2 ? b.size[0] * b.size[1] : b.size[0];
  const int64_t nbo = ro == 2 ? o.size[0] * o.size[1] : o.size[0];
  int64_t bdiv = 1;
  if (ra == 2) bdiv = a.size[1];
  if (rb == 2) {
    if (ra == 2 && b.size[1] != bdiv) return set_error(LLC_ERR_SHAPE, "batch_matmul: inner batch extents differ");
    bdiv = b.size[1];
  }
  if (ro == 2) {
    if ((ra == 2 || rb == 2) && o.size[1] != bdiv) return set_error(LLC_ERR_SHAPE, "batch_matmul: inner batch extents differ");
    bdiv = o.size[1];
  }
  if (nba != nbb || nbo != nba || a.size[ra + 1] != b.size[rb] || o.size[ro] != a.size[ra] || o.size[ro + 1] != b.size[rb + 1] ||
      (bdiv > 0 && nba % (bdiv ? bdiv : 1) != 0))
    return set_error(LLC_ERR_SHAPE, "batch_matmul: [%lld x %lld,%lld] x [%lld x %lld,%lld] -> [%lld x %lld,%lld]", (long long)nba,
                     (long long)a.size[ra], (long long)a.size[ra + 1], (long long)nbb, (long long)b.size[rb], (long long)b.size[rb + 1],
                     (long long)nbo, (long long)o.size[ro], (long long)o.size[ro + 1]);
  // the output is contiguous, or (rank 4) has unit-stride columns and any strides on rows and batches: the
  // head merge [B, H, S, D] -> [B, S, H*D] is then written in place
  const bool o_strided = !o.contiguous();
  if (o_strided && (ro != 2 || o.stride[3] != 1 || o.size[1] != bdiv))
    return set_error(LLC_ERR_LAYOUT, "batch_matmul: output must be contiguous, or rank 4 with unit-stride columns");
  if (o_strided && epi && epi->residual) return set_error(LLC_ERR_UNSUPPORTED, "batch_matmul: residual with a strided output");
  if (a.size[ra] > 0x7fffffff || a.size[ra + 1] > 0x7fffffff || b.size[rb + 1] > 0x7fffffff || bdiv > 0x7fffffff)
    return set_error(LLC_ERR_TOO_LARGE, "batch_matmul: extent too large");
  GemmParams p{};
  p.A = a.ptr;
  p.B = b.ptr;
  p.C = o.ptr;
  p.M = (int)a.size[ra];
  p.K = (int)a.size[ra + 1];
  p.N = (int)b.size[rb + 1];
  p.bdiv = (int)(bdiv > 0 ? bdiv : 1);
  // batch z = z0 * bdiv + z1; a one-level operand with batch stride s is (bdiv * s, s)
  if (ra == 2) { p.a_sb = a.stride[0]; p.a_sb1 = a.stride[1]; }
  else { p.a_sb = a.stride[0] * p.bdiv; p.a_sb1 = a.stride[0]; }
  p.a_sm = a.stride[ra];
  p.a_sk = a.stride[ra + 1];
  if (rb == 2) { p.b_sb = b.stride[0]; p.b_sb1 = b.stride[1]; }
  else { p.b_sb = b.stride[0] * p.bdiv; p.b_sb1 = b.stride[0]; }
  p.b_sk = b.stride[rb];
  p.b_sn = b.stride[rb + 1];
  if (o_strided) {
    p.c_sb = o.stride[0];
    p.c_sb1 = o.stride[1];
    p.c_sm = o.stride[2];
  } else {
    p.c_sb1 = (int64_t)p.M * p.N;
    p.c_sb = p.c_sb1 * p.bdiv;
    p.c_sm = p.N;
  }
  LLC_TRY(fill_epilogue(epi, o, p.N, &p, nba / p.bdiv));
  // blockIdx.z carries the batch; larger batches are issued in slices
  hipStream_t s = as_stream(stream);
  const int64_t nb = nba;
  // slices of whole outer batches, at most 65535 batches each
  const int64_t per = p.bdiv > 65535 ? 0 : (65535 / p.bdiv) * p.bdiv;
  if (per == 0) return set_error(LLC_ERR_TOO_LARGE, "batch_matmul: inner batch extent %d", p.bdiv);
  for (int64_t z0 = 0; z0 < nb; z0 += per) {
    GemmParams q = p;
    const int cnt = (int)((nb - z0) < per ? (nb - z0) : per);
    q.A = p.A + (z0 / p.bdiv) * p.a_sb * (int64_t)a.esize();
    q.B = p.B + (z0 / p.bdiv) * p.b_sb * (int64_t)a.esize();
    q.C = p.C + (z0 / p.bdiv) * p.c_sb * (int64_t)a.esize();
    if (p.residual) q.residual = p.residual + (z0 / p.bdiv) * p.c_sb * (int64_t)a.esize();
    if (p.bias) q.bias = p.bias + (z0 / p.bdiv) * p.bias_sb * (int64_t)a.esize();
    LLC_TRY(gemm_dispatch(a.dtype, q, cnt, s));
  }
  return LLC_OK;
}

// ---- llc_hip_matmul for callers that may not allocate -------------------------------------------------------
// The split reductions keep their partial sums in `scratch`, device memory that is part of the library's
// code object (every GPU the library runs on holds its own copy from load to process end), instead of the
// per-device buffer that llc_hip_matmul grows with hipMalloc.
constexpr size_t kStaticScratchBytes = (size_t)32 << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace {
constexpr int kScratchDevices = 64;
std::mutex g_scratch_mu;
void* g_scratch_ptr[kScratchDevices];  // device address of `scratch` on each device, null until asked for

// `scratch` names a host-side stand-in, not a device address: the address on the current device comes from
// hipGetSymbolAddress, once per device, and is what every kernel and copy is given afterwards.
int static_scratch(void** out) {
  int dev = -1;
  LLC_HIP_TRY(hipGetDevice(&dev));
  if (dev < 0 || dev >= kScratchDevices) return set_error(LLC_ERR_BAD_ARG, "matmul_static: device %d", dev);
  std::lock_guard<std::mutex> lock(g_scratch_mu);
  if (!g_scratch_ptr[dev]) {
    void* ptr = nullptr;
    LLC_HIP_TRY(hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch)));
    if (!ptr) return set_error(LLC_ERR_HIP, "matmul_static: the scratch array has no address on device %d", dev);
    g_scratch_ptr[dev] = ptr;
  }
  *out = g_scratch_ptr[dev];
  return LLC_OK;
}
}  // namespace

// called by llc_hip_init with the device current
int llc_impl_static_scratch_setup(void) {
  void* ptr = nullptr;
  return static_scratch(&ptr);
}

extern "C" int llc_hip_matmul_static(const llc_tensor* lhs, const llc_tensor* rhs, const llc_epilogue* epi, llc_tensor* out,
                                     void* stream) {
  void* ptr = nullptr;
  LLC_TRY(static_scratch(&ptr));
  // while this scope lives, get_workspace hands out `ptr` and refuses what does not fit; nothing allocates
  WorkspaceScope scope(ptr, kStaticScratchBytes);
  return llc_impl_matmul(lhs, rhs, epi, out, stream);
}

