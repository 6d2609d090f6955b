// llh.conv / llh.conv_bias as implicit GEMM on the matrix cores (NCHW x FCHW -> NCHW).
//
//   Y[n, f, oh, ow] = act(alpha * sum_{c,kh,kw} W[f, c, kh, kw] * X[n, c, ih, iw] + bias[f] + residual)
//   ih = oh*stride_h - pad_h + kh*dil_h,  iw = ow*stride_w - pad_w + kw*dil_w   (zero outside)
//
// GEMM view per group: rows = filters (FCHW weights are already [F, K] with k = (c,kh,kw)
// contiguous), columns = output pixels of the whole batch (n, oh, ow), K = C/g*KH*KW.  Pixels are
// the column dim because they are the contiguous dim of the NCHW output: for a fixed accumulator
// register 32 lanes store 32 consecutive pixels of one filter plane.
//
// The im2col matrix is never materialised.  Each lane owns one pixel column of the tile and a run
// of consecutive k; it walks (c, kh, kw) incrementally, gathers X with bounds checks (lanes of a
// wave read consecutive pixels, so loads coalesce for stride 1) and writes its run k-contiguous
// into the same swizzled LDS tile layout the matmul kernel uses.  Weights go through the shared
// vector loader.  fp32 tensors use the fp32 MFMA, bf16/f16 the 16-bit MFMA; accumulation is fp32.

#include "gemm_core.hpp"

namespace llc {
using namespace gemm;
namespace {

struct ConvParams {
  const char* X;
  const char* W;
  char* Y;
  const char* bias;      // [F] or null
  const char* residual;  // same layout as Y or null
  int32_t N, C, H, Wd, F, KH, KW, OH, OW;
  int32_t ph, pw, sh, sw, dh, dw;
  int32_t Cg, Fg;   // channels / filters per group
  int32_t Kdim;     // Cg*KH*KW
  int32_t ncols;    // N*OH*OW
  float alpha;
  int32_t act;
  int32_t tiles_m, tiles_n;
  int32_t OWp;     // fp32 kernel: output row length padded to a multiple of 4 (ncols counts padded pixels)
  int32_t splits;  // split-k factor (fp32 kernel)
  char* partial;   // [splits][F][ncols] fp32 partial sums when splits > 1
  int32_t y_nhwc;  // NCHW operands with a channels-last result (the first-layer kernels only)
};

// Gathers this lane's run of k for one pixel column of the im2col matrix.
template <typename T, int BN>
struct Im2colLoader {
  static constexpr int BK = kRowBytes / sizeof(T);
  static constexpr int KPT = BK * BN / 256;   // consecutive k per lane
  static constexpr int kParts = 256 / BN;     // lanes sharing one column
  static_assert(KPT * sizeof(T) % 16 == 0, "a lane's run must be whole 16-byte vectors");
  static_assert(KPT <= 32, "one mask word");
  T v[KPT];
  uint32_t okm;
  const T* plane0;  // X + (n*C + g*Cg)*H*W for this lane's pixel
  int ih0, iw0;
  bool valid;

  __device__ __forceinline__ void init(const ConvParams& p, int g, int col0) {
    const int j = threadIdx.x % BN;
    const int col = col0 + j;
    valid = col < p.ncols;
    const int ohw = p.OH * p.OW;
    const int n = valid ? col / ohw : 0;
    const int pix = valid ? col % ohw : 0;
    const int oh = pix / p.OW, ow = pix % p.OW;
    ih0 = oh * p.sh - p.ph;
    iw0 = ow * p.sw - p.pw;
    plane0 = (const T*)p.X + ((int64_t)n * p.C + (int64_t)g * p.Cg) * p.H * p.Wd;
  }

  // Every element is loaded unconditionally from an index clamped into the image; which ones lie outside
  // (padding, k tail, columns past the batch) is kept as a bit mask and applied when the run is written to
  // LDS.  Guarded loads would compile to a branch with a wait each: one memory round trip after the other.
  __device__ __forceinline__ void load(const ConvParams& p, int k0) {
    const int kpart = threadIdx.x / BN;
    int k = k0 + kpart * KPT;
    const int khw = p.KH * p.KW;
    int c = k / khw;
    int r = k - c * khw;
    int kh = r / p.KW;
    int kw = r - kh * p.KW;
    okm = 0;
#pragma unroll
    for (int i = 0; i < KPT; ++i) {
      const int ih = ih0 + kh * p.dh, iw = iw0 + kw * p.dw;
      const bool ok = valid && k < p.Kdim && ih >= 0 && ih < p.H && iw >= 0 && iw < p.Wd;
      const int cc = k < p.Kdim ? c : 0;
      const int ch = ih < 0 ? 0 : (ih >= p.H ? p.H - 1 : ih), cw = iw < 0 ? 0 : (iw >= p.Wd ? p.Wd - 1 : iw);
      v[i] = plane0[((int64_t)cc * p.H + ch) * p.Wd + cw];
      okm |= ok ? (1u << i) : 0u;
      ++k;
      if (++kw == p.KW) {
        kw = 0;
        if (++kh == p.KH) {
          kh = 0;
          ++c;
        }
      }
    }
  }

  __device__ __forceinline__ void store(char* lds) const {
    const int j = threadIdx.x % BN, kpart = threadIdx.x / BN;
    constexpr int EPV = 16 / sizeof(T);
#pragma unroll
    for (int q = 0; q < KPT / EPV; ++q) {
      struct alignas(16) Pack { T e[EPV]; } pk;
#pragma unroll
      for (int e = 0; e < EPV; ++e) pk.e[e] = (okm >> (q * EPV + e)) & 1u ? v[q * EPV + e] : static_cast<T>(0.0f);
      *(Pack*)(lds + lds_off(j, kpart * KPT * (int)sizeof(T) + q * 16)) = pk;
    }
  }
};

template <typename T, int BM, int BN, int LA>
__global__ __launch_bounds__(256) void conv_kernel(const ConvParams p) {
  constexpr int BK = kRowBytes / sizeof(T);
  constexpr int WTM = BM / 2, WTN = BN / 2;
  constexpr int TM = WTM / 32, TN = WTN / 32;
  constexpr int kABytes = BM * kRowStride, kBBytes = BN * kRowStride;
  constexpr int kBufBytes = kABytes + kBBytes;
  extern __shared__ __align__(16) char smem[];

  int tile_m, tile_n;
  tile_of_block(p.tiles_m, p.tiles_n, tile_m, tile_n);
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  const int g = blockIdx.z;
  const T* Wg = (const T*)p.W + (int64_t)g * p.Fg * p.Kdim;

  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int wm = wave / 2, wn = wave % 2;
  const int li = lane % 32, lh = lane / 32;

  f32x16_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  TileLoader<T, BM, LA, 256> la;
  Im2colLoader<T, BN> lb;
  lb.init(p, g, n0);
  const int nk = (p.Kdim + BK - 1) / BK;
  la.load(Wg, m0, p.Fg, 0, p.Kdim, p.Kdim, 1);
  lb.load(p, 0);
  la.store(smem);
  lb.store(smem + kABytes);
  __syncthreads();

  for (int kt = 0; kt < nk; ++kt) {
    const int cur = kt & 1;
    if (kt + 1 < nk) {
      la.load(Wg, m0, p.Fg, (kt + 1) * BK, p.Kdim, p.Kdim, 1);
      lb.load(p, (kt + 1) * BK);
    }
    mma_tile<T, TM, TN>(smem + cur * kBufBytes, wm * WTM + li, smem + cur * kBufBytes + kABytes, wn * WTN + li, lh, acc);
    if (kt + 1 < nk) {
      la.store(smem + (cur ^ 1) * kBufBytes);
      lb.store(smem + (cur ^ 1) * kBufBytes + kABytes);
    }
    __syncthreads();
  }

  // ---- epilogue: column = pixel (n, oh*OW+ow), row = filter of this group ----
  T* Y = (T*)p.Y;
  const int ohw = p.OH * p.OW;
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int col = n0 + wn * WTN + j * 32 + li;
    if (col >= p.ncols) continue;
    const int n = col / ohw, pix = col - n * ohw;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const int row0 = m0 + wm * WTM + i * 32 + lh * 4;  // the lane's first filter (inside the group) of this block
      const int rows_left = p.Fg - row0;
      const int f0 = g * p.Fg + (rows_left > 0 ? row0 : p.Fg - 1);
      float b16[16];
#pragma unroll
      for (int r = 0; r < 16; ++r) b16[r] = 0.0f;
      if (p.bias) {  // one test around the sixteen loads: they travel together
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int ro = (r / 4) * 8 + (r % 4);
          b16[r] = load_as_f32(p.bias, Elem<T>::kDtype, f0 + (ro < rows_left ? ro : 0));
        }
      }
      epilogue_block16<T, true>(Y, p.residual, ((int64_t)n * p.F + f0) * ohw + pix, ohw, rows_left, acc[i][j], p.alpha,
                                [&](int r) { return b16[r]; }, p.act);
    }
  }
}

// ---------------------------------------------------------------------------------------------
// fp32 convolutions with Kdim % 4 == 0 (every layer but an RGB stem).
//
// The pixel operand is staged the way it lies in memory: LDS tile [32 k][BN pixels], pixels
// contiguous.  For a fixed (c, kh, kw) consecutive output pixels of a stride-1 convolution read
// consecutive input elements, so a lane gathers four pixels with one (4-byte aligned) 16-byte load;
// window borders, image-row ends and strided convolutions take the element path.  The fp32 MFMA
// (32x32x2) takes one k per lane and instruction, which fits that layout: lane (li, lh) reads NJ
// consecutive pixels of row k = k0 + 4 lh + s with one ds_read and uses them as the B operands of NJ
// interleaved column sets (column set j of a wave holds pixels NJ li + j), while one 16-byte read of
// the k-contiguous weight tile gives the A operands of four k.  One A read and four B reads feed
// 4 NJ MFMAs, and because a lane's NJ accumulators are consecutive pixels of one filter plane the
// epilogue stores 4 NJ bytes per lane straight into NCHW, with no staging.
//
// Layers with few output pixels (late ResNet stages) do not have enough tiles for 256 CUs: their
// reduction is split over blockIdx.y, partial sums go to the scratch buffer in a fixed layout
// [split][F][pixels], and a second kernel adds them in split order (deterministic) and applies the
// epilogue.
typedef float f32x4u_t __attribute__((ext_vector_type(4), aligned(4)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));

template <int WM, int WN, int NJ, bool AFULL>
__global__ __launch_bounds__(256) void conv_f32_kernel(const ConvParams p) {
  constexpr int BM = 32 * WM, BN = 32 * NJ * WN, BK = 32;
  constexpr int kABytes = BM * kRowStride;
  constexpr int kBPitch = BN * 4;
  constexpr int kBuf = kABytes + BK * kBPitch;
  constexpr int VC = BN / 4;    // 4-pixel columns of the tile
  constexpr int KG = 256 / VC;  // lanes sharing one of them
  constexpr int KPT = BK / KG;  // consecutive k per lane
  static_assert(WM * WN == 4 && KPT >= 1, "4 waves");
  extern __shared__ __align__(16) char smem[];

  int tile_m, tile_n;
  tile_of_block(p.tiles_m, p.tiles_n, tile_m, tile_n);
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  const int g = blockIdx.z, split = blockIdx.y;
  const float* X = (const float*)p.X;
  const float* Wg = (const float*)p.W + (int64_t)g * p.Fg * p.Kdim;
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int wm = wave / WN, wn = wave % WN;
  const int li = lane % 32, lh = lane / 32;
  const int khw = p.KH * p.KW;

  // ---- this lane's four pixels: consecutive in one output row (rows are padded to OWp) ----
  const int vc = threadIdx.x % VC, kg = threadIdx.x / VC;
  int pbase, pih, piw0;
  {
    const int col0 = n0 + 4 * vc;
    const int in_range = col0 < p.ncols;
    const int rowi = in_range ? col0 / p.OWp : 0;  // n * OH + oh
    const int ow = in_range ? col0 - rowi * p.OWp : 0;
    const int nn = rowi / p.OH, oh = rowi - nn * p.OH;
    pbase = (nn * p.C + g * p.Cg) * p.H * p.Wd;
    pih = oh * p.sh - p.ph;
    piw0 = ow * p.sw - p.pw;
  }
  const bool wide = p.sw == 1 && p.Wd >= 4;  // four pixels read four consecutive elements

  // The gather is split in two: `gather_issue` computes addresses and issues every load of the next tile
  // (before the MFMAs of the current one), `gather_finish` zeroes what lies outside the image and writes
  // the tile to LDS (after them).  The loads are inline asm so that they stay where they are written and
  // stay unconditional: written as guarded C++ loads they compile to a branch and a wait per element,
  // which puts every memory round trip on the critical path.  Addresses are clamped into the tensor.
  TileLoader<float, BM, kLoadKVec, 256> la;
  f32x4_t raw[KPT];
  int gd[KPT];     // wide: 3 + offset of the wanted run inside the loaded window, 7 = all zero; else: valid bits
  // (c, kh, kw) of this lane's first k in the tile being gathered, kept across tiles: a tile advances k by 32,
  // added in the mixed radix (c, kh, kw) with one carry per digit (two integer divisions per tile otherwise)
  const int kstart = (int)((int64_t)blockIdx.y * ((p.Kdim + BK - 1) / BK) / p.splits) * BK + kg * KPT;
  int gk = kstart;
  int gc = kstart / khw;
  int gkh = (kstart - gc * khw) / p.KW;
  int gkw = kstart - gc * khw - gkh * p.KW;
  const int step_c = BK / khw, step_kh = (BK - step_c * khw) / p.KW, step_kw = BK - step_c * khw - step_kh * p.KW;
  const int hw = p.H * p.Wd;
  // offset of the wanted run inside the clamped window: -pw .. OWp - W - pw + (KW-1) dw over all taps and
  // pixel groups; within -1..1 for 3x3 pad 1 on rows that are a multiple of 4 wide
  const bool small_shift = p.pw <= 1 && p.OWp - p.Wd - p.pw + (p.KW - 1) * p.dw <= 1;
  auto gather_issue = [&]() {
    int k = gk, c = gc, kh = gkh, kw = gkw;
#pragma unroll
    for (int i = 0; i < KPT; ++i) {
      const bool kin = k < p.Kdim;
      const int ihr = pih + kh * p.dh, iw = piw0 + kw * p.dw;
      const bool hok = kin && ihr >= 0 && ihr < p.H;
      const int ih = ihr < 0 ? 0 : (ihr >= p.H ? p.H - 1 : ihr);
      const int rowoff = pbase + (kin ? c : 0) * hw + ih * p.Wd;  // floats from X
      if (wide) {
        // window of four elements clamped into the row
        const int st = iw < 0 ? 0 : (iw > p.Wd - 4 ? p.Wd - 4 : iw);
        const uint32_t boff = (uint32_t)(rowoff + st) * 4u;
        asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(raw[i]) : "v"(boff), "s"(X));
        gd[i] = hok ? iw - st + 3 : 7;
      } else {
        int mask = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int x = iw + j * p.sw;
          const uint32_t boff = (uint32_t)(rowoff + (x < 0 ? 0 : (x >= p.Wd ? p.Wd - 1 : x))) * 4u;
          float t;
          asm volatile("global_load_dword %0, %1, %2" : "=v"(t) : "v"(boff), "s"(X));
          raw[i][j] = t;
          mask |= (hok && x >= 0 && x < p.Wd) ? (1 << j) : 0;
        }
        gd[i] = mask;
      }
      ++k;
      if (++kw == p.KW) {
        kw = 0;
        if (++kh == p.KH) {
          kh = 0;
          ++c;
        }
      }
    }
    // next tile
    gk += BK;
    gkw += step_kw;
    if (gkw >= p.KW) {
      gkw -= p.KW;
      ++gkh;
    }
    gkh += step_kh;
    if (gkh >= p.KH) {
      gkh -= p.KH;
      ++gc;
    }
    gc += step_c;
  };
  auto gather_finish = [&](char* tb) {
    static_assert(KPT == 4, "the wait below names four registers");
    asm volatile("s_waitcnt vmcnt(0)" : "+v"(raw[0]), "+v"(raw[1]), "+v"(raw[2]), "+v"(raw[3]));
#pragma unroll
    for (int i = 0; i < KPT; ++i) {
      u32x4_t v;
      const u32x4_t e = __builtin_bit_cast(u32x4_t, raw[i]);
      const uint32_t sh = (uint32_t)gd[i];
      if (wide && small_shift) {
        // sh = 3: the window is the run; 4: the run starts one element later; 2: one earlier; 7: all zero
        const uint32_t m0 = sh == 3u ? 0xffffffffu : 0u, ml = sh == 2u ? 0xffffffffu : 0u, mr = sh == 4u ? 0xffffffffu : 0u;
        v[0] = (e[0] & m0) | (e[1] & mr);
        v[1] = (e[1] & m0) | (e[2] & mr) | (e[0] & ml);
        v[2] = (e[2] & m0) | (e[3] & mr) | (e[1] & ml);
        v[3] = (e[3] & m0) | (e[2] & ml);
      } else if (wide) {
        // out[j] = window[j + d], zero outside: a funnel shift by sh = d + 3 (0..6, 7 = all zero) over
        // {0,0,0,e0,e1,e2,e3,0,0,0}, one bit of the shift per stage, each select a bit-field insert
        const uint32_t m4 = 0u - ((sh >> 2) & 1u), m2 = 0u - ((sh >> 1) & 1u), m1 = 0u - (sh & 1u);
        const uint32_t x0 = e[1] & m4, x1 = e[2] & m4, x2 = e[3] & m4;
        const uint32_t x3 = e[0] & ~m4, x4 = e[1] & ~m4, x5 = e[2] & ~m4, x6 = e[3] & ~m4;
        const uint32_t y0 = (x2 & m2) | (x0 & ~m2), y1 = (x3 & m2) | (x1 & ~m2), y2 = (x4 & m2) | (x2 & ~m2);
        const uint32_t y3 = (x5 & m2) | (x3 & ~m2), y4 = (x6 & m2) | (x4 & ~m2);
        v[0] = (y1 & m1) | (y0 & ~m1);
        v[1] = (y2 & m1) | (y1 & ~m1);
        v[2] = (y3 & m1) | (y2 & ~m1);
        v[3] = (y4 & m1) | (y3 & ~m1);
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] = e[j] & (0u - ((sh >> j) & 1u));
      }
      *(u32x4_t*)(tb + (kg * KPT + i) * kBPitch + vc * 16) = v;
    }
  };

  f32x16_t acc[NJ];
#pragma unroll
  for (int j = 0; j < NJ; ++j)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[j][r] = 0.0f;
  const int arow = wm * 32 + li;
  const int abase = arow * kRowStride, aswz = lds_swz(arow);
  auto mma = [&](const char* ta, const char* tb) {
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      const u32x4_t a = *(const u32x4_t*)(ta + abase + (((2 * ks + lh) ^ aswz) << 4));
#pragma unroll
      for (int s2 = 0; s2 < 4; ++s2) {
        const float* bp = (const float*)(tb + (ks * 8 + 4 * lh + s2) * kBPitch) + wn * 32 * NJ + NJ * li;
        float b[NJ];
        if constexpr (NJ == 4) {
          const f32x4_t q = *(const f32x4_t*)bp;
          b[0] = q[0]; b[1] = q[1]; b[2] = q[2]; b[3] = q[3];
        } else {
          const f32x2_t q = *(const f32x2_t*)bp;
          b[0] = q[0]; b[1] = q[1];
        }
#pragma unroll
        for (int j = 0; j < NJ; ++j)
          acc[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a[s2]), b[j], acc[j], 0, 0, 0);
      }
    }
  };

  // k-tiles of this split
  const int nk = (p.Kdim + BK - 1) / BK;
  const int kt0 = (int)((int64_t)split * nk / p.splits), kt1 = (int)((int64_t)(split + 1) * nk / p.splits);
  la.template load<AFULL>(Wg, m0, p.Fg, kt0 * BK, p.Kdim, p.Kdim, 1);
  gather_issue();
  la.store(smem);
  gather_finish(smem + kABytes);
  __syncthreads();
  int cur = 0;
  for (int kt = kt0; kt + 1 < kt1; ++kt) {
    la.template load<AFULL>(Wg, m0, p.Fg, (kt + 1) * BK, p.Kdim, p.Kdim, 1);
    gather_issue();
    mma(smem + cur * kBuf, smem + cur * kBuf + kABytes);
    la.store(smem + (cur ^ 1) * kBuf);
    gather_finish(smem + (cur ^ 1) * kBuf + kABytes);
    __syncthreads();
    cur ^= 1;
  }
  mma(smem + cur * kBuf, smem + cur * kBuf + kABytes);

  // ---- epilogue: lane holds NJ consecutive pixels (columns) of 16 filter rows ----
  const int col = n0 + wn * 32 * NJ + NJ * li;
  if (col >= p.ncols) return;
  if (p.splits > 1) {
    float* part = (float*)p.partial;  // [split][F][padded pixels]: NJ divides the padded row length
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int row = m0 + wm * 32 + (r / 4) * 8 + lh * 4 + (r % 4);
      if (row >= p.Fg) continue;
      float* dst = part + ((int64_t)split * p.F + g * p.Fg + row) * p.ncols + col;
      if constexpr (NJ == 4) *(f32x4_t*)dst = f32x4_t{acc[0][r], acc[1][r], acc[2][r], acc[3][r]};
      else *(f32x2_t*)dst = f32x2_t{acc[0][r], acc[1][r]};
    }
    return;
  }
  float* Y = (float*)p.Y;
  const float* res = (const float*)p.residual;
  const int rowi = col / p.OWp, ow = col - rowi * p.OWp;  // rowi = n * OH + oh
  const int nn = rowi / p.OH, oh = rowi - nn * p.OH;
  const int nv = p.OW - ow < NJ ? (p.OW - ow < 0 ? 0 : p.OW - ow) : NJ;  // pixels of this lane that exist
  if (nv == 0) return;              // padding pixels
  const bool vec = p.OW % NJ == 0;  // then all NJ exist and their address is NJ * 4 byte aligned
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int row = m0 + wm * 32 + (r / 4) * 8 + lh * 4 + (r % 4);
    if (row >= p.Fg) continue;
    const int f = g * p.Fg + row;
    const float bvv = p.bias ? ((const float*)p.bias)[f] : 0.0f;
    const int64_t o0 = (((int64_t)nn * p.F + f) * p.OH + oh) * p.OW + ow;
    float rr[NJ], o[NJ];
#pragma unroll
    for (int j = 0; j < NJ; ++j) rr[j] = 0.0f;
    if (res) {
      if (vec) {
        if constexpr (NJ == 4) { const f32x4_t q = *(const f32x4_t*)(res + o0); rr[0] = q[0]; rr[1] = q[1]; rr[2] = q[2]; rr[3] = q[3]; }
        else { const f32x2_t q = *(const f32x2_t*)(res + o0); rr[0] = q[0]; rr[1] = q[1]; }
      } else {
#pragma unroll
        for (int j = 0; j < NJ; ++j)
          if (j < nv) rr[j] = res[o0 + j];
      }
    }
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      float v = acc[j][r] * p.alpha + bvv;
      if (res) v += rr[j];
      if (p.act == LLC_ACT_RELU) v = v < 0.0f ? 0.0f : v;
      else if (p.act == LLC_ACT_GELU) v = gelu_exact(v);
      o[j] = v;
    }
    if (vec) {
      if constexpr (NJ == 4) *(f32x4_t*)(Y + o0) = f32x4_t{o[0], o[1], o[2], o[3]};
      else *(f32x2_t*)(Y + o0) = f32x2_t{o[0], o[1]};
    } else {
#pragma unroll
      for (int j = 0; j < NJ; ++j)
        if (j < nv) Y[o0 + j] = o[j];
    }
  }
}

// Sums the split partials [splits][F][ncols] in split order and applies the epilogue.
__global__ __launch_bounds__(256) void conv_split_reduce_kernel(const ConvParams p) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;  // index into Y
  const int ohw = p.OH * p.OW;
  const int64_t total = (int64_t)p.N * p.F * ohw;
  if (i >= total) return;
  const int ow = (int)(i % p.OW);
  const int64_t t = i / p.OW;
  const int oh = (int)(t % p.OH);
  const int64_t t2 = t / p.OH;
  const int f = (int)(t2 % p.F), nn = (int)(t2 / p.F);
  const int col = (nn * p.OH + oh) * p.OWp + ow;
  const float* part = (const float*)p.partial + (int64_t)f * p.ncols + col;
  const int64_t stride = (int64_t)p.F * p.ncols;
  float s = 0.0f;
  for (int k = 0; k < p.splits; ++k) s += part[k * stride];
  float v = s * p.alpha + (p.bias ? ((const float*)p.bias)[f] : 0.0f);
  if (p.residual) v += ((const float*)p.residual)[i];
  if (p.act == LLC_ACT_RELU) v = v < 0.0f ? 0.0f : v;
  else if (p.act == LLC_ACT_GELU) v = gelu_exact(v);
  ((float*)p.Y)[i] = v;
}

int launch_f32(const ConvParams& p0, int groups, hipStream_t s) {
  constexpr int BM = 64, BN = 128;
  ConvParams p = p0;
  // pixel columns: output rows padded to a multiple of 4, so that a lane's four pixels share a row
  p.OWp = (p.OW + 3) / 4 * 4;
  const int64_t ncols = (int64_t)p.N * p.OH * p.OWp;
  if (ncols >= (int64_t)1 << 31) return set_error(LLC_ERR_TOO_LARGE, "conv: too many output pixels");
  p.ncols = (int)ncols;
  p.tiles_m = (p.Fg + BM - 1) / BM;
  p.tiles_n = (p.ncols + BN - 1) / BN;
  const int64_t tiles = (int64_t)p.tiles_m * p.tiles_n;
  if (tiles > 0x7fffffff || groups > 65535) return set_error(LLC_ERR_TOO_LARGE, "conv: grid too large");
  const int nk = (p.Kdim + 31) / 32;
  // enough workgroups for two per CU, at least eight k-tiles per split
  int splits = 1;
  if (tiles * groups < 384) {
    splits = (int)((512 + tiles * groups - 1) / (tiles * groups));
    if (splits > nk / 8) splits = nk / 8;
    if (splits < 1) splits = 1;
  }
  p.splits = splits;
  if (splits > 1) {
    void* ws = nullptr;
    LLC_TRY(get_workspace((size_t)splits * p.F * p.ncols * sizeof(float), &ws, s));
    p.partial = (char*)ws;
  }
  const size_t lds = 2 * (size_t)(BM * kRowStride + 32 * BN * 4);
  // weight tiles complete in both dims: unguarded weight loads
  const bool afull = p.Fg % BM == 0 && p.Kdim % 32 == 0;
  auto kern = afull ? conv_f32_kernel<2, 2, 2, true> : conv_f32_kernel<2, 2, 2, false>;
  hipLaunchKernelGGL(kern, dim3((unsigned)tiles, (unsigned)splits, (unsigned)groups), dim3(256), lds, s, p);
  LLC_TRY(check_launch("conv_f32_kernel"));
  if (splits > 1) {
    const int64_t total = (int64_t)p.N * p.F * p.OH * p.OW;
    hipLaunchKernelGGL(conv_split_reduce_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, p);
    LLC_TRY(check_launch("conv_split_reduce_kernel"));
  }
  return LLC_OK;
}

// ---------------------------------------------------------------------------------------------
// Channels-last (NHWC) convolution, fp32 and the 16-bit types: x [N,C,H,W] with strides (HWC, 1, WC, C), weight
// [F,C,KH,KW] with strides (KH KW C, 1, KW C, C), output and residual channels-last too.
//
// In this layout the im2col matrix needs no gather arithmetic: with k ordered (kh, kw, c) a row of it is, per
// filter tap, a run of C contiguous values of the input, and a k-tile of 128 bytes (32 floats, 64 16-bit values;
// C a multiple of that) lies inside one tap.  So the convolution is the GEMM  out[pixel, f] = sum_k im2col[pixel, k] * weight[f, k]  with both
// operands contiguous along k and the output row-major [pixels, F], i.e. channels-last again, and it runs on
// the tile machinery of gemm_kernel (LDS layout, fragment reads, MFMA loop, two register stages).  What is
// specific is the loader of the pixel operand: every lane keeps, for each of its rows, the offset of the
// window origin and one validity bit per tap, computed once; a k-tile adds one scalar offset (tap, channel
// block) to them.  A lane spends a handful of integer instructions per 16-byte vector where the NCHW kernel
// spends about forty on (c, kh, kw) bookkeeping, window clamping and border shifts.
template <typename T, int BM, int NT>
struct NhwcLoader {
  static constexpr int EPV = 16 / (int)sizeof(T);
  static constexpr int kIters = BM * 8 / NT;
  static_assert(BM * 8 % NT == 0 && kIters >= 1 && kIters <= 32, "whole vectors per lane");
  u32x4_t v[kIters];
  uint32_t okm = 0;
  int base[kIters];       // element offset of (n, oh*sh - ph, ow*sw - pw, channel 0) from X; may be negative
  uint64_t taps[kIters];  // bit kh*KW + kw: that tap of the row's window lies inside the image

  __device__ __forceinline__ void init(const ConvParams& p, int m0) {
    const int ohw = p.OH * p.OW;
#pragma unroll
    for (int i = 0; i < kIters; ++i) {
      const int m = m0 + ((i * NT + (int)threadIdx.x) >> 3);
      base[i] = 0;
      taps[i] = 0;
      if (m < p.ncols) {
        const int n = m / ohw, rem = m - n * ohw;
        const int oh = rem / p.OW, ow = rem - oh * p.OW;
        const int ih0 = oh * p.sh - p.ph, iw0 = ow * p.sw - p.pw;
        base[i] = ((n * p.H + ih0) * p.Wd + iw0) * p.C;
        uint64_t bits = 0;
        for (int kh = 0; kh < p.KH; ++kh)
          for (int kw = 0; kw < p.KW; ++kw) {
            const int ih = ih0 + kh * p.dh, iw = iw0 + kw * p.dw;
            if (ih >= 0 && ih < p.H && iw >= 0 && iw < p.Wd) bits |= (uint64_t)1 << (kh * p.KW + kw);
          }
        taps[i] = bits;
      }
    }
  }
  // all loads are issued, from offset 0 where the tap falls outside; what was outside is zeroed in store()
  __device__ __forceinline__ void load(const T* X, const ConvParams& p, int k0) {
    const int tap = k0 / p.C, c0 = k0 - tap * p.C;
    const int kh = tap / p.KW, kw = tap - kh * p.KW;
    const int toff = (kh * p.dh * p.Wd + kw * p.dw) * p.C + c0;
    okm = 0;
#pragma unroll
    for (int i = 0; i < kIters; ++i) {
      const int kv = (i * NT + (int)threadIdx.x) & 7;
      const uint32_t ok = (uint32_t)(taps[i] >> tap) & 1u;
      const int off = ok ? base[i] + toff + kv * EPV : 0;
      v[i] = *(const u32x4_t*)(X + off);
      okm |= ok << i;
    }
  }
  __device__ __forceinline__ void store(char* lds) const {
#pragma unroll
    for (int i = 0; i < kIters; ++i) {
      const int vid = i * NT + (int)threadIdx.x;
      const uint32_t m = 0u - ((okm >> i) & 1u);
      *(u32x4_t*)(lds + lds_off(vid >> 3, (vid & 7) * 16)) = u32x4_t{v[i][0] & m, v[i][1] & m, v[i][2] & m, v[i][3] & m};
    }
  }
};

template <typename T, int BM, int BN, int WM, int WN, bool BFULL>
__global__ __launch_bounds__(64 * WM * WN) void conv_nhwc_kernel(const ConvParams p) {
  constexpr int NT = 64 * WM * WN;
  constexpr int BK = kRowBytes / (int)sizeof(T);
  constexpr int WTM = BM / WM, WTN = BN / WN;
  constexpr int TM = WTM / 32, TN = WTN / 32;
  constexpr int kABytes = BM * kRowStride, kBBytes = BN * kRowStride;
  constexpr int kBufBytes = kABytes + kBBytes;
  extern __shared__ __align__(16) char smem[];
  int tile_m, tile_n;
  tile_of_block(p.tiles_m, p.tiles_n, tile_m, tile_n);
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  const T* X = (const T*)p.X;
  const T* Wt = (const T*)p.W;
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

  // k-tiles of this split
  const int nk_all = p.Kdim / BK;
  const int split = blockIdx.y;
  const int kt0 = (int)((int64_t)split * nk_all / p.splits), nk = (int)((int64_t)(split + 1) * nk_all / p.splits) - kt0;
  NhwcLoader<T, BM, NT> la0, la1;
  TileLoader<T, BN, kLoadKVec, NT> lb0, lb1;
  la0.init(p, m0);
#pragma unroll
  for (int i = 0; i < NhwcLoader<T, BM, NT>::kIters; ++i) {
    la1.base[i] = la0.base[i];
    la1.taps[i] = la0.taps[i];
  }
  la0.load(X, p, kt0 * BK);
  lb0.template load<BFULL>(Wt, n0, p.F, kt0 * BK, p.Kdim, p.Kdim, 1);
  if (nk > 1) {
    la1.load(X, p, (kt0 + 1) * BK);
    lb1.template load<BFULL>(Wt, n0, p.F, (kt0 + 1) * BK, p.Kdim, p.Kdim, 1);
  }
  la0.store(smem);
  lb0.store(smem + kABytes);
  __syncthreads();
#define LLC_NHWC_STEP(KT, CUR, LA2, LB2, LA1, LB1, GUARDED)                                                     \
  {                                                                                                             \
    if (!(GUARDED) || (KT) + 2 < nk) {                                                                          \
      LA2.load(X, p, (kt0 + (KT) + 2) * BK);                                                                    \
      LB2.template load<BFULL>(Wt, n0, p.F, (kt0 + (KT) + 2) * BK, p.Kdim, p.Kdim, 1);                          \
    }                                                                                                           \
    /* nothing moves across: left alone, the scheduler sinks the loads into the MFMAs and lifts the masking of  \
       the previous tile's vectors (and with it the wait for them) above the MFMAs */                           \
    __builtin_amdgcn_sched_barrier(0);                                                                          \
    mma_tile<T, TM, TN>(smem + (CUR) * kBufBytes, wm * WTM + li, smem + (CUR) * kBufBytes + kABytes,            \
                        wn * WTN + li, lh, acc);                                                                \
    __builtin_amdgcn_sched_barrier(0);                                                                          \
    if (!(GUARDED) || (KT) + 1 < nk) {                                                                          \
      LA1.store(smem + ((CUR) ^ 1) * kBufBytes);                                                                \
      LB1.store(smem + ((CUR) ^ 1) * kBufBytes + kABytes);                                                      \
    }                                                                                                           \
    __syncthreads();                                                                                            \
  }
  // steady state without control flow in the body: with the guards inside, the compiler must assume at the top of
  // an iteration that the loads of either register stage may still be in flight and waits for all of them before
  // it issues the next ones, which puts the memory latency of every k-tile in front of its MFMAs
  int kt = 0;
  for (; kt + 3 < nk; kt += 2) {
    LLC_NHWC_STEP(kt, 0, la0, lb0, la1, lb1, false)
    LLC_NHWC_STEP(kt + 1, 1, la1, lb1, la0, lb0, false)
  }
  for (; kt < nk; kt += 2) {
    LLC_NHWC_STEP(kt, 0, la0, lb0, la1, lb1, true)
    if (kt + 1 < nk) LLC_NHWC_STEP(kt + 1, 1, la1, lb1, la0, lb0, true)
  }
#undef LLC_NHWC_STEP

  // ---- epilogue: register r of lane (li, lh) is row 8 (r/4) + 4 lh + r%4, column li: 32 lanes store 32 consecutive
  //      filters of one pixel ----
  float* part = (float*)p.partial + (int64_t)split * p.ncols * p.F;
  const char* res = p.splits > 1 ? nullptr : p.residual;
  // the bias of every column block is requested before the first block stores (behind a store, which may alias it, the
  // next block's bias would wait for that store)
  float bvs[TN];
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int col = n0 + wn * WTN + j * 32 + li;
    bvs[j] = (p.bias && p.splits == 1) ? load_as_f32(p.bias, Elem<T>::kDtype, BFULL || col < p.F ? col : p.F - 1) : 0.0f;
  }
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int col = n0 + wn * WTN + j * 32 + li;
    if (!BFULL && col >= p.F) continue;
    const float bv = bvs[j];
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const int row0 = m0 + wm * WTM + i * 32 + lh * 4;  // the lane's first pixel of this block
      const int rows_left = p.ncols - row0;
      const int64_t base = (int64_t)(rows_left > 0 ? row0 : p.ncols - 1) * p.F + col;
      if (p.splits > 1) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int ro = (r / 4) * 8 + (r % 4);
          if (ro < rows_left) part[base + (int64_t)ro * p.F] = acc[i][j][r];
        }
      } else {
        epilogue_block16<T, true>((T*)p.Y, res, base, p.F, rows_left, acc[i][j], p.alpha, [&](int) { return bv; }, p.act);
      }
    }
  }
}

// Sums the split partials [splits][pixels][F] in split order and applies the epilogue (channels-last output).
template <typename T>
__global__ __launch_bounds__(256) void nhwc_split_reduce_kernel(const ConvParams p) {
  const int64_t i4 = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
  const int64_t total = (int64_t)p.ncols * p.F;
  if (i4 >= total) return;  // F % 4 == 0: a vector never straddles the end
  const int f = (int)(i4 % p.F);
  gemm::split_epilogue4<T>((const float*)p.partial, p.splits, total, i4, f, p.alpha, p.bias, p.residual, p.act, (T*)p.Y);
}

template <typename T, int BM, int BN, int WM, int WN>
int launch_nhwc_cfg(const ConvParams& p0, hipStream_t s) {
  ConvParams p = p0;
  p.tiles_m = (p.ncols + BM - 1) / BM;
  p.tiles_n = (p.F + BN - 1) / BN;
  const int64_t tiles = (int64_t)p.tiles_m * p.tiles_n;
  if (tiles > 0x7fffffff) return set_error(LLC_ERR_TOO_LARGE, "conv: grid too large");
  const int nk = p.Kdim / (kRowBytes / (int)sizeof(T));
  // too few tiles for 256 CUs: split the reduction (at least eight k-tiles per split)
  int splits = 1;
  if (tiles < 256 || (BM == 128 && tiles < 384)) {
    splits = (int)((512 + tiles - 1) / tiles);
    if (splits > nk / 8) splits = nk / 8;
    if (splits < 1) splits = 1;
  }
  p.splits = splits;
  if (splits > 1) {
    void* ws = nullptr;
    LLC_TRY(get_workspace((size_t)splits * p.ncols * p.F * sizeof(float), &ws, s));
    p.partial = (char*)ws;
  }
  const size_t lds = 2 * (size_t)(BM + BN) * kRowStride;
  const bool bfull = p.F % BN == 0;
  auto kern = bfull ? conv_nhwc_kernel<T, BM, BN, WM, WN, true> : conv_nhwc_kernel<T, BM, BN, WM, WN, false>;
  static std::atomic<uint32_t> lds_allowed[2];  // one per instantiation
  LLC_TRY(allow_dynamic_lds((const void*)kern, (int)lds, lds_allowed[bfull]));
  hipLaunchKernelGGL(kern, dim3((unsigned)tiles, (unsigned)splits, 1), dim3(64 * WM * WN), lds, s, p);
  LLC_TRY(check_launch("conv_nhwc_kernel"));
  if (splits > 1) {
    const int64_t total4 = (int64_t)p.ncols * p.F / 4;
    hipLaunchKernelGGL(nhwc_split_reduce_kernel<T>, dim3((unsigned)((total4 + 255) / 256)), dim3(256), 0, s, p);
    LLC_TRY(check_launch("nhwc_split_reduce_kernel"));
  }
  return LLC_OK;
}

#include "conv_rows.hpp"
#include "conv_patch.hpp"

template <typename T>
int launch_nhwc(const ConvParams& p, hipStream_t s) {
  if constexpr (sizeof(T) == 2) {
    // layers with work for the whole chip: the wide-tile matmul kernel with the image as its row operand
    auto magic = [](uint32_t d) { return d == 1 ? 0u : (uint32_t)(((uint64_t)1 << 32) / d) + 1u; };
    ConvWideGeom g{};
    g.C = p.C, g.H = p.H, g.W = p.Wd, g.OH = p.OH, g.OW = p.OW, g.KH = p.KH, g.KW = p.KW;
    g.sh = p.sh, g.sw = p.sw, g.ph = p.ph, g.pw = p.pw, g.dh = p.dh, g.dw = p.dw;
    g.ncols = p.ncols;
    g.cblocks = p.C / 64;
    g.cblocks_magic = magic((uint32_t)(p.C / 64));
    g.kw_magic = magic((uint32_t)p.KW);
    const int st = conv_wide_16bit(Elem<T>::kDtype, p.X, p.W, p.Y, p.bias, p.residual, p.F, g, p.alpha, p.act, s);
    if (st != 1) return st;
  }
  // stride-1 windows over images small enough for an LDS patch: the input is read once, not once per tap
  if (conv_patch_ok<T>(p)) return launch_conv_patch<T>(p, s);
  // 128-pixel tiles when they fill the chip by themselves; else 64 x 64 tiles if those are numerous enough to need
  // no split of the reduction (a split costs a pass over the partial sums: the middle layers of a ResNet); the
  // last layers split either way and do better on the large tiles, unless their reduction is too short to split
  // (1x1 downsampling convolutions: 3136 x 256 x 128 is 50 large tiles and 18 us, 196 small ones and 9 us)
  const int64_t bn = p.F <= 64 ? 64 : 128;
  const int64_t t128 = (int64_t)((p.ncols + 127) / 128) * ((p.F + bn - 1) / bn);
  const int64_t t64 = (int64_t)((p.ncols + 63) / 64) * ((p.F + 63) / 64);
  if (t128 < 384 && t64 >= 256) return launch_nhwc_cfg<T, 64, 64, 2, 2>(p, s);
  const int64_t max_splits = std::max<int64_t>(1, (p.Kdim / (kRowBytes / (int)sizeof(T))) / 8);
  if (t128 * max_splits < 192 && t64 > t128 * max_splits) return launch_nhwc_cfg<T, 64, 64, 2, 2>(p, s);
  return p.F <= 64 ? launch_nhwc_cfg<T, 128, 64, 4, 2>(p, s) : launch_nhwc_cfg<T, 128, 128, 4, 2>(p, s);
}

template <typename T, int BM, int BN, int LA>
int launch_cfg(const ConvParams& p0, int groups, hipStream_t s) {
  ConvParams p = p0;
  p.tiles_m = (p.Fg + BM - 1) / BM;
  p.tiles_n = (p.ncols + BN - 1) / BN;
  const size_t lds = 2 * (size_t)(BM + BN) * kRowStride;
  auto kern = conv_kernel<T, BM, BN, LA>;
  static std::atomic<uint32_t> lds_allowed{0};
  LLC_TRY(allow_dynamic_lds((const void*)kern, (int)lds, lds_allowed));
  const int64_t tiles = (int64_t)p.tiles_m * p.tiles_n;
  if (tiles > 0x7fffffff || groups > 65535) return set_error(LLC_ERR_TOO_LARGE, "conv: grid too large");
  hipLaunchKernelGGL(kern, dim3((unsigned)tiles, 1, (unsigned)groups), dim3(256), lds, s, p);
  return check_launch("conv_kernel");
}

template <typename T, int LA>
int launch_tiles(const ConvParams& p, int groups, hipStream_t s) {
  const int64_t t128 = (int64_t)((p.Fg + 127) / 128) * ((p.ncols + 127) / 128) * groups;
  if (p.Fg > 64 && t128 >= 128) return launch_cfg<T, 128, 128, LA>(p, groups, s);
  if (p.Fg > 64) return launch_cfg<T, 128, 64, LA>(p, groups, s);
  if ((int64_t)((p.ncols + 127) / 128) * groups >= 128) return launch_cfg<T, 64, 128, LA>(p, groups, s);
  return launch_cfg<T, 64, 64, LA>(p, groups, s);
}

template <typename T>
int launch_loaders(const ConvParams& p, int groups, hipStream_t s) {
  constexpr int EPV = 16 / sizeof(T);
  const bool w_vec = p.Kdim % EPV == 0 && ((uintptr_t)p.W % 16) == 0;
  if constexpr (sizeof(T) == 4) {
    if (conv_rows_ok(p, groups)) return launch_conv_rows<float>(p, s);
    if (p.y_nhwc) return set_error(LLC_ERR_UNSUPPORTED, "conv: no kernel for NCHW operands with a channels-last result of this shape");
    if (w_vec && ((uintptr_t)p.Y % 16) == 0 && (!p.residual || ((uintptr_t)p.residual % 16) == 0) &&
        ((uintptr_t)p.X % 4) == 0 && (int64_t)p.N * p.C * p.H * p.Wd < ((int64_t)1 << 30))  // 32-bit byte offsets
      return launch_f32(p, groups, s);
  }
  if constexpr (sizeof(T) == 2) {
    // an image network's first layer in 16-bit storage: the 16-bit row kernel, or the fp32 one on widened copies
    if (conv_rows_16bit_ok(p, groups)) return launch_conv_rows_16bit_mfma<T>(p, s);
    if (conv_rows_ok(p, groups) && ((uintptr_t)p.W % 16) == 0 && (int64_t)p.N * p.C * p.H * p.Wd % 8 == 0 &&
        (!p.bias || ((uintptr_t)p.bias % 2) == 0))
      return launch_conv_rows_16bit<T>(p, s);
    if (p.y_nhwc) return set_error(LLC_ERR_UNSUPPORTED, "conv: no kernel for NCHW operands with a channels-last result of this shape");
  }
  if (w_vec) return launch_tiles<T, kLoadKVec>(p, groups, s);
  return launch_tiles<T, kLoadGeneric>(p, groups, s);
}

}  // namespace
}  // namespace llc

using namespace llc;

int llc_impl_conv2d(const llc_tensor* x, const llc_tensor* w, const llc_conv_attrs* at, const llc_epilogue* epi,
                              llc_tensor* out, void* stream) {
  View a, k, o;
  LLC_TRY(make_view(x, "conv input", &a));
  LLC_TRY(make_view(w, "conv weight", &k));
  LLC_TRY(make_view(out, "conv output", &o));
  if (!at) return set_error(LLC_ERR_BAD_ARG, "conv: null attributes");
  if (a.dtype != k.dtype || a.dtype != o.dtype) return set_error(LLC_ERR_DTYPE, "conv: operand types differ");
  if (a.dtype != LLC_FLOAT32 && a.dtype != LLC_BFLOAT16 && a.dtype != LLC_FLOAT16)
    return set_error(LLC_ERR_DTYPE, "conv: element type %d (LLH_FloatTensor expected)", a.dtype);
  if (a.rank != 4 || k.rank != 4 || o.rank != 4) return set_error(LLC_ERR_SHAPE, "conv: NCHW x FCHW -> NCHW expected");
  // Layout travels in the strides, as in torch: all tensors NCHW-contiguous, or all channels-last (NHWC in memory).
  auto channels_last = [](const View& v) {
    const int64_t C = v.size[1], H = v.size[2], W = v.size[3];
    return (C == 1 || v.stride[1] == 1) && (W == 1 || v.stride[3] == C) && (H == 1 || v.stride[2] == W * C) &&
           (v.size[0] == 1 || v.stride[0] == H * W * C);
  };
  const bool nhwc = !(a.contiguous() && k.contiguous() && o.contiguous()) && channels_last(a) && channels_last(k) && channels_last(o);
  // a first layer that hands its result to channels-last layers: NCHW operands, channels-last result
  const bool y_nhwc = !nhwc && a.contiguous() && k.contiguous() && !o.contiguous() && channels_last(o);
  if (!nhwc && !y_nhwc && (!a.contiguous() || !k.contiguous() || !o.contiguous()))
    return set_error(LLC_ERR_LAYOUT, "conv: tensors must all be contiguous (NCHW) or all channels-last");
  const int64_t group = at->group;
  for (int i = 0; i < 2; ++i)
    if (at->stride[i] <= 0 || at->dilation[i] <= 0 || at->pad[i] < 0 || at->pad[i + 2] < 0)
      return set_error(LLC_ERR_BAD_ARG, "conv: bad window attributes");
  if (group <= 0 || a.size[1] % group || k.size[0] % group || k.size[1] * group != a.size[1])
    return set_error(LLC_ERR_SHAPE, "conv: C=%lld, weight [%lld,%lld,..], group=%lld do not agree", (long long)a.size[1],
                     (long long)k.size[0], (long long)k.size[1], (long long)group);
  if (at->kernel_shape[0] != k.size[2] || at->kernel_shape[1] != k.size[3])
    return set_error(LLC_ERR_SHAPE, "conv: kernel_shape attribute does not match the weight");
  // LLHinfersymbolShape.cpp:257-268
  const int64_t OH = (a.size[2] + at->pad[0] + at->pad[2] - at->dilation[0] * (k.size[2] - 1) - 1) / at->stride[0] + 1;
  const int64_t OW = (a.size[3] + at->pad[1] + at->pad[3] - at->dilation[1] * (k.size[3] - 1) - 1) / at->stride[1] + 1;
  if (o.size[0] != a.size[0] || o.size[1] != k.size[0] || o.size[2] != OH || o.size[3] != OW)
    return set_error(LLC_ERR_SHAPE, "conv: output is %lldx%lldx%lldx%lld, expected %lldx%lldx%lldx%lld", (long long)o.size[0],
                     (long long)o.size[1], (long long)o.size[2], (long long)o.size[3], (long long)a.size[0],
                     (long long)k.size[0], (long long)OH, (long long)OW);
  if (o.numel() == 0) return LLC_OK;
  if (a.numel() >= (int64_t)1 << 31 || o.numel() >= (int64_t)1 << 31 || k.numel() >= (int64_t)1 << 31)
    return set_error(LLC_ERR_TOO_LARGE, "conv: tensors of 2^31 elements or more");
  ConvParams p{};
  p.X = a.ptr;
  p.W = k.ptr;
  p.Y = o.ptr;
  p.N = (int)a.size[0];
  p.C = (int)a.size[1];
  p.H = (int)a.size[2];
  p.Wd = (int)a.size[3];
  p.F = (int)k.size[0];
  p.KH = (int)k.size[2];
  p.KW = (int)k.size[3];
  p.OH = (int)OH;
  p.OW = (int)OW;
  p.ph = (int)at->pad[0];
  p.pw = (int)at->pad[1];
  p.sh = (int)at->stride[0];
  p.sw = (int)at->stride[1];
  p.dh = (int)at->dilation[0];
  p.dw = (int)at->dilation[1];
  p.Cg = (int)(a.size[1] / group);
  p.Fg = (int)(k.size[0] / group);
  p.Kdim = p.Cg * p.KH * p.KW;
  p.ncols = (int)(a.size[0] * OH * OW);
  p.alpha = 1.0f;
  p.act = LLC_ACT_NONE;
  p.y_nhwc = y_nhwc ? 1 : 0;
  if (epi) {
    p.alpha = epi->alpha;
    if (epi->act < LLC_ACT_NONE || epi->act > LLC_ACT_GELU) return set_error(LLC_ERR_BAD_ARG, "conv: activation %d", epi->act);
    p.act = epi->act;
    if (epi->bias) {
      View b;
      LLC_TRY(make_view(epi->bias, "conv bias", &b));
      if (b.dtype != o.dtype) return set_error(LLC_ERR_DTYPE, "conv: bias type differs from output");
      if (b.numel() != p.F || !b.contiguous()) return set_error(LLC_ERR_SHAPE, "conv: bias must hold %d contiguous values", p.F);
      p.bias = b.ptr;
    }
    if (epi->residual) {
      View r;
      LLC_TRY(make_view(epi->residual, "conv residual", &r));
      if (r.dtype != o.dtype) return set_error(LLC_ERR_DTYPE, "conv: residual type differs from output");
      bool same = r.rank == 4 && r.numel() == o.numel();
      for (int d = 0; same && d < 4; ++d) same = r.size[d] == o.size[d];
      if (!(nhwc ? same && channels_last(r) : r.numel() == o.numel() && r.contiguous()))
        return set_error(LLC_ERR_SHAPE, "conv: residual must match the output in shape and layout");
      p.residual = r.ptr;
    }
  }
  hipStream_t s = as_stream(stream);
  if (nhwc) {
    const int ktile = 128 / (int)a.esize();  // values in the 128 bytes of a k-tile: they must share a tap
    if (group != 1 || p.C % ktile != 0 || p.KH * p.KW > 64 || p.F % 4 != 0 ||
        ((uintptr_t)p.X | (uintptr_t)p.W | (uintptr_t)p.Y | (uintptr_t)p.residual | (uintptr_t)p.bias) % 16 != 0)
      return set_error(LLC_ERR_UNSUPPORTED, "conv: channels-last tensors need group 1, C %% %d == 0, F %% 4 == 0, at most 64 taps and 16-byte alignment", ktile);
    switch (a.dtype) {
      case LLC_FLOAT32: return launch_nhwc<float>(p, s);
      case LLC_BFLOAT16: return launch_nhwc<__bf16>(p, s);
      default: return launch_nhwc<_Float16>(p, s);
    }
  }
  switch (a.dtype) {
    case LLC_FLOAT32: return launch_loaders<float>(p, (int)group, s);
    case LLC_BFLOAT16: return launch_loaders<__bf16>(p, (int)group, s);
    default: return launch_loaders<_Float16>(p, (int)group, s);
  }
}
