// Fused attention: out = softmax(scale * Q K^T + mask) V in one pass over the keys.
//
// The unfused group (llh.batch_matmul, the mask add folded into its epilogue, the softmax chain,
// llh.batch_matmul) writes and re-reads the [B, H, Sq, Skv] score tensor four times; it is the largest
// stream of bytes of an attention layer.  Here a workgroup keeps 128 queries of one head in registers and walks
// the keys in blocks of 64 with a running maximum and a running sum (the scores never leave the CU):
//
//   per wave: 32 queries.  S^T[key, query] = K Q^T on the matrix cores with the K block as the row operand
//   (read from LDS) and the wave's Q fragments as the column operand (registers, loaded once).  In the
//   accumulator layout a lane then owns ONE query (lane % 32) and 32 of the 64 keys, so the row maximum and row
//   sum are in-lane loops plus one exchange with lane ^ 32.  exp2 of the shifted scores, rounded to the storage
//   type, is already laid out as the column operand of O^T[d, query] += V^T P^T when the key order inside a
//   16-key step is taken as the accumulator's (keys 4h..4h+3 and 8+4h..8+4h+3 for lane half h); the V block is
//   read from LDS with the transposing read, which hands a lane four consecutive keys of one d.
//   O^T keeps the query on the lane, so the rescaling by exp2(m_old - m_new) is one multiplier per lane.
//
// LDS per stage: K block [64 keys][128 B] with the row-XOR chunk swizzle of the GEMM tiles, V block
// [64 keys][128 B] with chunk c stored at c ^ 2 (key & 3) (the four key rows a transposing read touches fall
// in different banks), and the additive row (mask, -inf past the last key) as fp32.  Two stages: the global
// loads of block i+1 are issued before the arithmetic of block i and written to the other stage after it; one
// barrier per block.
#include "gemm_core.hpp"

namespace llc {
namespace {
using namespace gemm;

struct AttnParams {
  const char* Q;
  const char* K;
  const char* V;
  const char* mask;  // [B, Skv] additive, storage type, or null
  char* O;
  int32_t B, H, Sq, Skv;
  int64_t q_sb, q_sh, q_ss;  // element strides of the [B, H, S, 64] views; the last dim is contiguous
  int64_t k_sb, k_sh, k_ss;
  int64_t v_sb, v_sh, v_ss;
  int64_t o_sb, o_sh, o_ss;
  int64_t m_sb;
  float scale_log2e;
};

typedef float f32x4_t __attribute__((ext_vector_type(4)));
constexpr float kLog2e = 1.4426950408889634f;

// An additive mask value in log2 units.  A finite value that overflows in the conversion (the most negative number
// of the storage type, a common "minus infinity") stays finite: a row whose every key carries it then softmaxes to
// the uniform row an unscaled evaluation gives, instead of 0 * inf.  A true -inf stays -inf (and such a row NaN).
__device__ __forceinline__ float mask_log2(float m) {
  const float r = m * kLog2e;
  return (r == -INFINITY && m != -INFINITY) ? -3.4028234663852886e38f : r;
}
constexpr int kD = 64;
constexpr int kBlockQ = 128, kBlockKV = 64;
constexpr int kTileBytes = kBlockKV * 128;

template <typename T>
__device__ __forceinline__ uint32_t pack2(float a, float b) {
  if constexpr (Elem<T>::kDtype == LLC_BFLOAT16) {
    typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
    typedef float f2 __attribute__((ext_vector_type(2)));
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f2{a, b}, bf2));
  } else {
    return (uint32_t)f32_to_f16_bits(a) | ((uint32_t)f32_to_f16_bits(b) << 16);
  }
}

typedef short s16x4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint2 lds_tr16(const char* p) {
  const s16x4_t v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4_t*)p);
  return __builtin_bit_cast(uint2, v);
}

// ADD: scores get the additive LDS row (a mask, and -inf for keys past Skv).  Without it Skv is a multiple of 64.
// D: head dim, 32, 64 or 128.  A K or V block is [64 keys][D values]: 128-byte rows as described above for D = 64; for
// D = 128 two such tiles side by side (d 0..63, then d 64..127: a k-step of S^T or a d tile of O^T lies in one of
// them); for D = 32 the same tile with half of every row used (four chunks, swizzled among themselves).
template <int D>
struct AttnGeom {
  static_assert(D == 32 || D == 64 || D == 128, "head dims 32, 64 and 128");
  static constexpr int KS = D / 16;                    // 16-d steps of S^T
  static constexpr int DT = D / 32;                    // 32-d tiles of O^T
  static constexpr int NH = D == 128 ? 2 : 1;          // 64-d tiles side by side
  static constexpr int CH = D == 32 ? 4 : 8;           // 16-byte chunks in use per 128-byte row
  static constexpr int kStage = NH * kTileBytes;       // one K (or V) block
  static constexpr int kLoads = 64 * (D / 8) / 256;    // 16-byte chunks per lane, tensor and block
  static constexpr int kLds = 4 * kStage + 2 * kBlockKV * 4;
};

template <typename T, bool ADD, int D>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(D == 128 ? 2 : 3, D == 128 ? 2 : 3))) void attention_kernel(const AttnParams p) {
  using G = AttnGeom<D>;
  constexpr int KS = G::KS, DT = G::DT, CH = G::CH;
  extern __shared__ __align__(16) char smem[];
  char* kt0 = smem;                                        // [2][G::kStage]
  char* vt0 = smem + 2 * G::kStage;                        // [2][G::kStage]
  float* addrow = (float*)(smem + 4 * G::kStage);          // [2][kBlockKV]
  const int tid = threadIdx.x, wave = tid / kWave, lane = tid % kWave;
  const int li = lane % 32, lh = lane / 32;
  const int bh = blockIdx.y, b = bh / p.H, h = bh - b * p.H;
  const int q0 = blockIdx.x * kBlockQ + wave * 32;
  const T* Q = (const T*)p.Q + (int64_t)b * p.q_sb + (int64_t)h * p.q_sh;
  const T* K = (const T*)p.K + (int64_t)b * p.k_sb + (int64_t)h * p.k_sh;
  const T* V = (const T*)p.V + (int64_t)b * p.v_sb + (int64_t)h * p.v_sh;
  const T* M = p.mask ? (const T*)p.mask + (int64_t)b * p.m_sb : nullptr;

  // this lane's query row as the column operand of S^T: 8 consecutive d per 16-d step
  u32x4_t qf[KS];
  {
    const int qrow = q0 + li < p.Sq ? q0 + li : p.Sq - 1;
    const T* qp = Q + (int64_t)qrow * p.q_ss + lh * 8;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qf[ks] = *(const u32x4_t*)(qp + ks * 16);
  }

  // block loader: 64 D / 8 16-byte chunks of K and of V by 256 lanes
  int lrow[G::kLoads], lcol[G::kLoads], koff[G::kLoads], voff[G::kLoads];
#pragma unroll
  for (int j = 0; j < G::kLoads; ++j) {
    const int id = tid + 256 * j;
    lrow[j] = id / (D / 8);
    lcol[j] = id % (D / 8);
    const int half = lcol[j] / 8, lc = lcol[j] % 8;
    koff[j] = half * kTileBytes + lrow[j] * 128 + ((lc ^ (lds_swz(lrow[j]) & (CH - 1))) << 4);
    voff[j] = half * kTileBytes + lrow[j] * 128 + ((lc ^ (((lrow[j] & 3) << 1) & (CH - 1))) << 4);
  }
  u32x4_t kr[G::kLoads], vr[G::kLoads];
  float ar = 0.0f;
  auto gload = [&](int blk) {
#pragma unroll
    for (int j = 0; j < G::kLoads; ++j) {
      int row = blk * kBlockKV + lrow[j];
      row = row < p.Skv ? row : p.Skv - 1;
      kr[j] = *(const u32x4_t*)(K + (int64_t)row * p.k_ss + lcol[j] * 8);
      vr[j] = *(const u32x4_t*)(V + (int64_t)row * p.v_ss + lcol[j] * 8);
    }
    if constexpr (ADD) {
      if (tid < kBlockKV) {
        const int key = blk * kBlockKV + tid;
        const int kc = key < p.Skv ? key : p.Skv - 1;
        float mv = 0.0f;
        if (M) mv = mask_log2(load_as_f32((const char*)M, Elem<T>::kDtype, kc));
        ar = key < p.Skv ? mv : -INFINITY;
      }
    }
  };
  auto lstore = [&](int s) {
#pragma unroll
    for (int j = 0; j < G::kLoads; ++j) {
      *(u32x4_t*)(kt0 + s * G::kStage + koff[j]) = kr[j];
      *(u32x4_t*)(vt0 + s * G::kStage + voff[j]) = vr[j];
    }
    if constexpr (ADD) {
      if (tid < kBlockKV) addrow[s * kBlockKV + tid] = ar;
    }
  };

  // fragment addresses inside a stage
  int ka[2][KS];  // K rows 32 T + li, chunk 2 ks + lh of the 64-d tile the k-step lies in
#pragma unroll
  for (int t2 = 0; t2 < 2; ++t2)
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int row = 32 * t2 + li;
      ka[t2][ks] = (ks / 4) * kTileBytes + row * 128 + (((2 * (ks % 4) + lh) ^ (lds_swz(row) & (CH - 1))) << 4);
    }
  // V: a 16-lane group reads a 4 (keys) x 16 (d) patch; lane = 16 g + 4 jj + q addresses key row jj, d chunk q
  int va[DT][2];  // [d tile][which run of four keys]
  {
    const int g = lane / 16, jj = (lane / 4) % 4, q = lane % 4;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const int row = 8 * u + 4 * (g >> 1) + jj;
        const int c = 4 * (dt % 2) + 2 * (g & 1) + (q >> 1);
        va[dt][u] = (dt / 2) * kTileBytes + row * 128 + ((c ^ ((jj << 1) & (CH - 1))) << 4) + (q & 1) * 8;
      }
  }

  f32x16_t oacc[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int r = 0; r < 16; ++r) oacc[dt][r] = 0.0f;
  float m_run = -INFINITY, l_run = 0.0f;

  const int nblk = (p.Skv + kBlockKV - 1) / kBlockKV;
  gload(0);
  lstore(0);
  __syncthreads();
  for (int blk = 0; blk < nblk; ++blk) {
    const int s = blk & 1;
    // Without a mask row the next block's loads are unconditional (the last iteration fetches its own block again and drops
    // it): under `if (blk + 1 < nblk)` the registers they define must be valid where the branch ends, so the wave waited
    // for them there, in front of this block's arithmetic instead of behind it (batch 8, 12 heads, 512 x 512 x 64:
    // 18.7 -> 17.6 us; 4 x 16 heads, 2048 x 2048: 105.8 -> 94.5).  The variant with a mask row measured the other way
    // round (512 x 500 keys: 17.9 us with the branch, 18.6 without) and keeps the branch.
    if constexpr (ADD) {
      if (blk + 1 < nblk) gload(blk + 1);
    } else {
      gload(blk + 1 < nblk ? blk + 1 : blk);
    }
    const char* kb = kt0 + s * G::kStage;
    const char* vb = vt0 + s * G::kStage;

    // S^T = K Q^T for 64 keys x 32 queries
    f32x16_t sacc[2];
#pragma unroll
    for (int t2 = 0; t2 < 2; ++t2) {
#pragma unroll
      for (int r = 0; r < 16; ++r) sacc[t2][r] = 0.0f;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) mfma_step<T>(*(const u32x4_t*)(kb + ka[t2][ks]), qf[ks], sacc[t2]);
    }
    // x = scores in log2 units; accumulator register 4 i + j of tile T is key 32 T + 8 i + 4 lh + j
    float mx = -INFINITY;
#pragma unroll
    for (int t2 = 0; t2 < 2; ++t2)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if constexpr (ADD) {
          const f32x4_t av = *(const f32x4_t*)&addrow[s * kBlockKV + 32 * t2 + 8 * i + 4 * lh];
#pragma unroll
          for (int j = 0; j < 4; ++j) sacc[t2][4 * i + j] = fmaf(sacc[t2][4 * i + j], p.scale_log2e, av[j]);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) mx = fmaxf(mx, sacc[t2][4 * i + j]);
      }
    if constexpr (!ADD) mx *= p.scale_log2e;  // scale > 0: the maximum commutes with it
    mx = fmaxf(mx, __shfl_xor(mx, 32, kWave));
    // The shift m only has to keep exp2(x - m) in range, it need not be the exact maximum: it is raised (and
    // the sums rescaled) only when some row of the wave has grown by more than 2^8 over its shift; until
    // then the probabilities are at most 256 and the final division by the row sum takes the factor out.
    // (A row whose keys so far are all masked with -inf keeps m = -inf and shifts by 0: no inf - inf forms.)
    float m_use = m_run == -INFINITY ? 0.0f : m_run;
    if (__any(mx > m_run + 8.0f)) {
      const float m_max = fmaxf(m_run, mx);
      m_use = m_max == -INFINITY ? 0.0f : m_max;
      const float corr = __builtin_amdgcn_exp2f(m_run - m_use);
      m_run = m_max;
      l_run *= corr;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[dt][r] *= corr;
    }
    const float m_new = m_use;
    float psum = 0.0f;
    u32x4_t pb[2][2];
#pragma unroll
    for (int t2 = 0; t2 < 2; ++t2)
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          float pv[2];
#pragma unroll
          for (int w = 0; w < 2; ++w) {
            const float x = sacc[t2][8 * t + 2 * e + w];
            pv[w] = ADD ? __builtin_amdgcn_exp2f(x - m_new) : __builtin_amdgcn_exp2f(fmaf(x, p.scale_log2e, -m_new));
            psum += pv[w];
          }
          pb[t2][t][e] = pack2<T>(pv[0], pv[1]);
        }
    l_run += psum;
    // O^T += V^T P^T, 16 keys per step
#pragma unroll
    for (int t2 = 0; t2 < 2; ++t2)
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        const char* vrow = vb + (32 * t2 + 16 * t) * 128;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
          const uint2 lo = lds_tr16(vrow + va[dt][0]), hi = lds_tr16(vrow + va[dt][1]);
          mfma_step<T>(u32x4_t{lo.x, lo.y, hi.x, hi.y}, pb[t2][t], oacc[dt]);
        }
      }
    if (blk + 1 < nblk) lstore(s ^ 1);
    __syncthreads();
  }

  const float l_tot = l_run + __shfl_xor(l_run, 32, kWave);
  const float inv = 1.0f / l_tot;
  if (q0 + li < p.Sq) {
    T* op = (T*)p.O + (int64_t)b * p.o_sb + (int64_t)h * p.o_sh + (int64_t)(q0 + li) * p.o_ss;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        uint2 w;
        w.x = pack2<T>(oacc[dt][4 * i] * inv, oacc[dt][4 * i + 1] * inv);
        w.y = pack2<T>(oacc[dt][4 * i + 2] * inv, oacc[dt][4 * i + 3] * inv);
        *(uint2*)(op + 32 * dt + 8 * i + 4 * lh) = w;
      }
  }
}

// ---- few workgroups (one sequence, a dozen heads): the keys split over the waves ----
// With 128 queries per workgroup a batch of one leaves most CUs idle and every wave walks all the keys of its 32
// queries, one block after the other.  Here a workgroup has 32 queries and its four waves take every fourth key block
// each (a K / V stage of its own per wave: no barrier inside the walk), so the chain is a quarter as long and there
// are four times the workgroups; the four partial results (running shift, row sum, O^T) meet in LDS at the end and
// are combined like the blocks of one wave are: scaled by exp2(shift - largest shift), summed, divided by the sum.
constexpr int kSplitLds = 8 * kTileBytes + 4 * kBlockKV * 4;
template <typename T, bool ADD>
__global__ __launch_bounds__(256) void attention_split_kernel(const AttnParams p) {
  extern __shared__ __align__(16) char smem[];
  const int tid = threadIdx.x, wave = tid / kWave, lane = tid % kWave;
  char* kt = smem + wave * kTileBytes;
  char* vt = smem + (4 + wave) * kTileBytes;
  float* addrow = (float*)(smem + 8 * kTileBytes) + wave * kBlockKV;
  const int li = lane % 32, lh = lane / 32;
  const int bh = blockIdx.y, b = bh / p.H, h = bh - b * p.H;
  const int q0 = blockIdx.x * 32;
  const T* Q = (const T*)p.Q + (int64_t)b * p.q_sb + (int64_t)h * p.q_sh;
  const T* K = (const T*)p.K + (int64_t)b * p.k_sb + (int64_t)h * p.k_sh;
  const T* V = (const T*)p.V + (int64_t)b * p.v_sb + (int64_t)h * p.v_sh;
  const T* M = p.mask ? (const T*)p.mask + (int64_t)b * p.m_sb : nullptr;

  u32x4_t qf[4];
  {
    const int qrow = q0 + li < p.Sq ? q0 + li : p.Sq - 1;
    const T* qp = Q + (int64_t)qrow * p.q_ss + lh * 8;
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) qf[ks] = *(const u32x4_t*)(qp + ks * 16);
  }
  // block loader: 512 16-byte chunks of K and of V by the 64 lanes of this wave
  const int lc = lane % 8;
  int koff[8], voff[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const int row = lane / 8 + 8 * j;
    koff[j] = row * 128 + ((lc ^ lds_swz(row)) << 4);
    voff[j] = row * 128 + ((lc ^ ((row & 3) << 1)) << 4);
  }
  u32x4_t kr[8], vr[8];
  float ar = 0.0f;
  auto gload = [&](int blk) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      int row = blk * kBlockKV + lane / 8 + 8 * j;
      row = row < p.Skv ? row : p.Skv - 1;
      kr[j] = *(const u32x4_t*)(K + (int64_t)row * p.k_ss + lc * 8);
      vr[j] = *(const u32x4_t*)(V + (int64_t)row * p.v_ss + lc * 8);
    }
    if constexpr (ADD) {
      const int key = blk * kBlockKV + lane;
      const int kc = key < p.Skv ? key : p.Skv - 1;
      float mv = 0.0f;
      if (M) mv = mask_log2(load_as_f32((const char*)M, Elem<T>::kDtype, kc));
      ar = key < p.Skv ? mv : -INFINITY;
    }
  };
  auto lstore = [&]() {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      *(u32x4_t*)(kt + koff[j]) = kr[j];
      *(u32x4_t*)(vt + voff[j]) = vr[j];
    }
    if constexpr (ADD) addrow[lane] = ar;
  };
  int ka[2][4];
#pragma unroll
  for (int t2 = 0; t2 < 2; ++t2)
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      const int row = 32 * t2 + li;
      ka[t2][ks] = row * 128 + (((2 * ks + lh) ^ lds_swz(row)) << 4);
    }
  int va[2][2];
  {
    const int g = lane / 16, jj = (lane / 4) % 4, q = lane % 4;
#pragma unroll
    for (int dt = 0; dt < 2; ++dt)
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const int row = 8 * u + 4 * (g >> 1) + jj;
        const int c = 4 * dt + 2 * (g & 1) + (q >> 1);
        va[dt][u] = row * 128 + ((c ^ (jj << 1)) << 4) + (q & 1) * 8;
      }
  }

  f32x16_t oacc[2];
#pragma unroll
  for (int dt = 0; dt < 2; ++dt)
#pragma unroll
    for (int r = 0; r < 16; ++r) oacc[dt][r] = 0.0f;
  float m_run = -INFINITY, l_run = 0.0f;

  const int nblk = (p.Skv + kBlockKV - 1) / kBlockKV;
  if (wave < nblk) gload(wave);
  for (int blk = wave; blk < nblk; blk += 4) {
    // the stage is this wave's own: its previous reads are done when these writes are issued (LDS works in order)
    lstore();
    if constexpr (ADD) {
      if (blk + 4 < nblk) gload(blk + 4);
    } else {
      gload(blk + 4 < nblk ? blk + 4 : blk);  // unconditional, as in attention_kernel
    }
    f32x16_t sacc[2];
#pragma unroll
    for (int t2 = 0; t2 < 2; ++t2) {
#pragma unroll
      for (int r = 0; r < 16; ++r) sacc[t2][r] = 0.0f;
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) mfma_step<T>(*(const u32x4_t*)(kt + ka[t2][ks]), qf[ks], sacc[t2]);
    }
    float mx = -INFINITY;
#pragma unroll
    for (int t2 = 0; t2 < 2; ++t2)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if constexpr (ADD) {
          const f32x4_t av = *(const f32x4_t*)&addrow[32 * t2 + 8 * i + 4 * lh];
#pragma unroll
          for (int j = 0; j < 4; ++j) sacc[t2][4 * i + j] = fmaf(sacc[t2][4 * i + j], p.scale_log2e, av[j]);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) mx = fmaxf(mx, sacc[t2][4 * i + j]);
      }
    if constexpr (!ADD) mx *= p.scale_log2e;
    mx = fmaxf(mx, __shfl_xor(mx, 32, kWave));
    float m_use = m_run == -INFINITY ? 0.0f : m_run;
    if (__any(mx > m_run + 8.0f)) {
      const float m_max = fmaxf(m_run, mx);
      m_use = m_max == -INFINITY ? 0.0f : m_max;
      const float corr = __builtin_amdgcn_exp2f(m_run - m_use);
      m_run = m_max;
      l_run *= corr;
#pragma unroll
      for (int dt = 0; dt < 2; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[dt][r] *= corr;
    }
    const float m_new = m_use;
    float psum = 0.0f;
    u32x4_t pb[2][2];
#pragma unroll
    for (int t2 = 0; t2 < 2; ++t2)
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          float pv[2];
#pragma unroll
          for (int w = 0; w < 2; ++w) {
            const float x = sacc[t2][8 * t + 2 * e + w];
            pv[w] = ADD ? __builtin_amdgcn_exp2f(x - m_new) : __builtin_amdgcn_exp2f(fmaf(x, p.scale_log2e, -m_new));
            psum += pv[w];
          }
          pb[t2][t][e] = pack2<T>(pv[0], pv[1]);
        }
    l_run += psum;
#pragma unroll
    for (int t2 = 0; t2 < 2; ++t2)
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        const char* vrow = vt + (32 * t2 + 16 * t) * 128;
#pragma unroll
        for (int dt = 0; dt < 2; ++dt) {
          const uint2 lo = lds_tr16(vrow + va[dt][0]), hi = lds_tr16(vrow + va[dt][1]);
          mfma_step<T>(u32x4_t{lo.x, lo.y, hi.x, hi.y}, pb[t2][t], oacc[dt]);
        }
      }
  }

  // ---- the four partial results meet: xo[wave][register][lane] over the K / V stages, shift and row sum beside ----
  const float l_part = l_run + __shfl_xor(l_run, 32, kWave);
  __syncthreads();  // every wave has left its stages
  float* xo = (float*)smem;                            // [4][32][64]
  float* xm = (float*)(smem + 8 * kTileBytes);         // [4][32] shifts, then [4][32] sums
#pragma unroll
  for (int dt = 0; dt < 2; ++dt)
#pragma unroll
    for (int r = 0; r < 16; ++r) xo[((wave * 32) + dt * 16 + r) * 64 + lane] = oacc[dt][r];
  if (lh == 0) {
    xm[wave * 32 + li] = m_run;
    xm[128 + wave * 32 + li] = l_part;
  }
  __syncthreads();
  float mw[4], sc[4];
  float m_ref = -INFINITY;
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    mw[w] = xm[w * 32 + li];
    m_ref = fmaxf(m_ref, mw[w]);
  }
  float l_tot = 0.0f;
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    // a wave that saw no key, or only keys masked with -inf, holds zeros against a shift of 0: it adds nothing
    sc[w] = mw[w] == -INFINITY ? 0.0f : __builtin_amdgcn_exp2f(mw[w] - m_ref);
    l_tot += xm[128 + w * 32 + li] * sc[w];
  }
  const float inv = 1.0f / l_tot;
  if (q0 + li < p.Sq) {
    // this wave writes registers 8 wave .. 8 wave + 7 of the O^T layout: d tile wave / 2, i = 2 (wave % 2) + {0, 1}
    T* op = (T*)p.O + (int64_t)b * p.o_sb + (int64_t)h * p.o_sh + (int64_t)(q0 + li) * p.o_ss;
    const int dt = wave >> 1;
#pragma unroll
    for (int ii = 0; ii < 2; ++ii) {
      const int i = 2 * (wave & 1) + ii;
      float o[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        float acc = 0.0f;
#pragma unroll
        for (int w = 0; w < 4; ++w) acc += xo[((w * 32) + dt * 16 + 4 * i + j) * 64 + lane] * sc[w];
        o[j] = acc * inv;
      }
      uint2 wv;
      wv.x = pack2<T>(o[0], o[1]);
      wv.y = pack2<T>(o[2], o[3]);
      *(uint2*)(op + 32 * dt + 8 * i + 4 * lh) = wv;
    }
  }
}

// ---- fp32 operands: v_mfma_f32_32x32x2_f32 takes one k per lane and instruction ----
// Same plan as above with these differences.  K block [64 keys][256 B] and V block [64 keys][256 B] come straight
// into LDS (global_load_lds: no staging registers; lane L of a wave load lands at byte 16 L of its 1 KB, so it
// fetches the chunk that belongs there: K chunk c of row r sits at c ^ (r & 15), V elements of rows with bit 2
// set sit 32 floats further, which spreads the fragment reads over the banks).  S^T: one 16-byte read of a K row
// feeds four MFMAs (lane half h owns d = 8c + 4h + s, the same permutation of k on both operands).  The
// probabilities stay fp32 in the accumulator registers and ARE the column operand of O^T += V^T P^T: in register
// 4i + j lane half 0 holds key 8i + j and half 1 key 8i + 4 + j, which is one k pair.  V is read 4 bytes per lane
// and MFMA.  64 or 128 queries per workgroup (2 or 4 waves), whichever gives the CUs more to share.
constexpr int kF32Tile = kBlockKV * 256;

template <int NW, bool MASK>
__global__ __launch_bounds__(64 * NW) void attention_f32_kernel(const AttnParams p) {
  extern __shared__ __align__(16) char smem[];
  char* kt = smem;                                        // [2][kF32Tile]
  char* vt = smem + 2 * kF32Tile;                         // [2][kF32Tile]
  float* addrow = (float*)(smem + 4 * kF32Tile);          // [2][64] raw mask values
  constexpr int LPW = 16 / NW;  // wave loads of K (and of V) per wave and block
  const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid / kWave), lane = tid % kWave;
  const int li = lane % 32, lh = lane / 32;
  const int bh = blockIdx.y, b = bh / p.H, h = bh - b * p.H;
  const int q0 = blockIdx.x * (32 * NW) + wave * 32;
  const float* Q = (const float*)p.Q + (int64_t)b * p.q_sb + (int64_t)h * p.q_sh;
  const float* K = (const float*)p.K + (int64_t)b * p.k_sb + (int64_t)h * p.k_sh;
  const float* V = (const float*)p.V + (int64_t)b * p.v_sb + (int64_t)h * p.v_sh;
  const float* M = MASK ? (const float*)p.mask + (int64_t)b * p.m_sb : nullptr;

  f32x4_t qf[8];
  {
    const int qrow = q0 + li < p.Sq ? q0 + li : p.Sq - 1;
    const float* qp = Q + (int64_t)qrow * p.q_ss + 4 * lh;
#pragma unroll
    for (int c = 0; c < 8; ++c) qf[c] = *(const f32x4_t*)(qp + 8 * c);
  }

  auto issue = [&](int blk, int s) {
#pragma unroll
    for (int j = 0; j < LPW; ++j) {
      const int x = wave * LPW + j;            // rows 4x .. 4x + 3 of the block
      const int r = 4 * x + lane / 16, pos = lane % 16;
      int row = blk * kBlockKV + r;
      row = row < p.Skv ? row : p.Skv - 1;
      const float* ks = K + (int64_t)row * p.k_ss + ((pos ^ (r & 15)) << 2);
      const float* vs = V + (int64_t)row * p.v_ss + ((pos ^ (((r >> 2) & 1) << 3)) << 2);
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)ks,
                                       (__attribute__((address_space(3))) void*)(kt + s * kF32Tile + x * 1024), 16, 0, 0);
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)vs,
                                       (__attribute__((address_space(3))) void*)(vt + s * kF32Tile + x * 1024), 16, 0, 0);
    }
    if constexpr (MASK) {
      // every wave brings the same 64 values (identical bytes to the same place): no wave is special
      int key = blk * kBlockKV + lane;
      key = key < p.Skv ? key : p.Skv - 1;
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(M + key),
                                       (__attribute__((address_space(3))) void*)(addrow + s * kBlockKV), 4, 0, 0);
    }
  };

  int ka[2];  // K rows 32 T + li: row offset; the chunk swizzle is applied per read
#pragma unroll
  for (int t2 = 0; t2 < 2; ++t2) ka[t2] = (32 * t2 + li) * 256;
  const int kswz = li & 15;
  // V element (key, d) sits at key * 256 + 4 * (d ^ 32 * ((key >> 2) & 1)); this lane's keys have (key >> 2) & 1 = lh
  const int va0 = 4 * lh * 256 + 4 * li + 128 * lh, va1 = 4 * lh * 256 + 4 * li + 128 * (1 - lh);

  f32x16_t oacc[2];
#pragma unroll
  for (int dt = 0; dt < 2; ++dt)
#pragma unroll
    for (int r = 0; r < 16; ++r) oacc[dt][r] = 0.0f;
  float m_run = -INFINITY, l_run = 0.0f;
  const int nblk = (p.Skv + kBlockKV - 1) / kBlockKV;
  issue(0, 0);
  for (int blk = 0; blk < nblk; ++blk) {
    const int s = blk & 1;
    // this wave's share of block blk has landed; after the barrier everybody's has, and nobody reads the other stage
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (blk + 1 < nblk) issue(blk + 1, s ^ 1);
    const char* kb = kt + s * kF32Tile;
    const char* vb = vt + s * kF32Tile;
    f32x16_t sacc[2];
#pragma unroll
    for (int t2 = 0; t2 < 2; ++t2) {
#pragma unroll
      for (int r = 0; r < 16; ++r) sacc[t2][r] = 0.0f;
#pragma unroll
      for (int c = 0; c < 8; ++c) {
        const f32x4_t a = *(const f32x4_t*)(kb + ka[t2] + (((2 * c + lh) ^ kswz) << 4));
#pragma unroll
        for (int e = 0; e < 4; ++e) sacc[t2] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[e], qf[c][e], sacc[t2], 0, 0, 0);
      }
    }
    // scores in log2 units; register 4 i + j of tile T is key 32 T + 8 i + 4 lh + j
    const bool tail = blk == nblk - 1 && (p.Skv % kBlockKV) != 0;
    float mx = -INFINITY;
#pragma unroll
    for (int t2 = 0; t2 < 2; ++t2)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        f32x4_t av = {0.0f, 0.0f, 0.0f, 0.0f};
        if constexpr (MASK) av = *(const f32x4_t*)&addrow[s * kBlockKV + 32 * t2 + 8 * i + 4 * lh];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          float x = MASK ? fmaf(sacc[t2][4 * i + j], p.scale_log2e, mask_log2(av[j])) : sacc[t2][4 * i + j] * p.scale_log2e;
          if (tail && blk * kBlockKV + 32 * t2 + 8 * i + 4 * lh + j >= p.Skv) x = -INFINITY;
          sacc[t2][4 * i + j] = x;
          mx = fmaxf(mx, x);
        }
      }
    mx = fmaxf(mx, __shfl_xor(mx, 32, kWave));
    float m_use = m_run == -INFINITY ? 0.0f : m_run;
    if (__any(mx > m_run + 8.0f)) {  // see attention_kernel: the shift follows the maximum lazily
      const float m_max = fmaxf(m_run, mx);
      m_use = m_max == -INFINITY ? 0.0f : m_max;
      const float corr = __builtin_amdgcn_exp2f(m_run - m_use);
      m_run = m_max;
      l_run *= corr;
#pragma unroll
      for (int dt = 0; dt < 2; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[dt][r] *= corr;
    }
    float psum = 0.0f;
#pragma unroll
    for (int t2 = 0; t2 < 2; ++t2)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float pv = __builtin_amdgcn_exp2f(sacc[t2][r] - m_use);
        sacc[t2][r] = pv;
        psum += pv;
      }
    l_run += psum;
    // O^T += V^T P^T, one k pair (keys 8 i + j and 8 i + 4 + j of tile T) per MFMA
#pragma unroll
    for (int t2 = 0; t2 < 2; ++t2)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int koff = (32 * t2 + 8 * (r / 4) + (r % 4)) * 256;
        const float a0 = *(const float*)(vb + va0 + koff), a1 = *(const float*)(vb + va1 + koff);
        oacc[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, sacc[t2][r], oacc[0], 0, 0, 0);
        oacc[1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, sacc[t2][r], oacc[1], 0, 0, 0);
      }
  }

  const float l_tot = l_run + __shfl_xor(l_run, 32, kWave);
  const float inv = 1.0f / l_tot;
  if (q0 + li < p.Sq) {
    float* op = (float*)p.O + (int64_t)b * p.o_sb + (int64_t)h * p.o_sh + (int64_t)(q0 + li) * p.o_ss;
#pragma unroll
    for (int dt = 0; dt < 2; ++dt)
#pragma unroll
      for (int i = 0; i < 4; ++i)
        *(f32x4_t*)(op + 32 * dt + 8 * i + 4 * lh) =
            f32x4_t{oacc[dt][4 * i] * inv, oacc[dt][4 * i + 1] * inv, oacc[dt][4 * i + 2] * inv, oacc[dt][4 * i + 3] * inv};
  }
}

template <int NW, bool MASK>
int launch_f32(const AttnParams& p, hipStream_t s) {
  constexpr int lds = 4 * kF32Tile + 2 * kBlockKV * 4;
  auto kern = attention_f32_kernel<NW, MASK>;
  static std::atomic<uint32_t> lds_allowed{0};
  LLC_TRY(allow_dynamic_lds((const void*)kern, (int)lds, lds_allowed));
  const dim3 grid((unsigned)((p.Sq + 32 * NW - 1) / (32 * NW)), (unsigned)(p.B * p.H));
  hipLaunchKernelGGL(kern, grid, dim3(64 * NW), lds, s, p);
  return check_launch("attention_f32_kernel");
}

int view4(const llc_tensor* t, const char* what, View* v) {
  LLC_TRY(make_view(t, what, v));
  if (v->rank != 4) return set_error(LLC_ERR_SHAPE, "%s: rank 4 expected, [B, H, S, D]", what);
  const bool wide = v->dtype == LLC_BFLOAT16 || v->dtype == LLC_FLOAT16;
  if (v->size[3] != kD && !(wide && (v->size[3] == 32 || v->size[3] == 128)))
    return set_error(LLC_ERR_UNSUPPORTED, "%s: head dim %lld (64, and 32 or 128 in the 16-bit types, are implemented)", what,
                     (long long)v->size[3]);
  if (v->stride[3] != 1 || v->stride[0] % 8 || v->stride[1] % 8 || v->stride[2] % 8 || ((uintptr_t)v->ptr % 16))
    return set_error(LLC_ERR_LAYOUT, "%s: the head dim must be contiguous and every row 16-byte aligned", what);
  return LLC_OK;
}

}  // namespace
}  // namespace llc

using namespace llc;

int llc_impl_attention(const llc_tensor* q, const llc_tensor* k, const llc_tensor* v, const llc_tensor* mask, float scale,
                       llc_tensor* out, void* stream) {
  View a, b, c, o, m;
  LLC_TRY(view4(q, "attention q", &a));
  LLC_TRY(view4(k, "attention k", &b));
  LLC_TRY(view4(v, "attention v", &c));
  LLC_TRY(view4(out, "attention out", &o));
  if (a.dtype != b.dtype || a.dtype != c.dtype || a.dtype != o.dtype) return set_error(LLC_ERR_DTYPE, "attention: operand types differ");
  if (a.size[3] != b.size[3] || a.size[3] != c.size[3] || a.size[3] != o.size[3]) return set_error(LLC_ERR_SHAPE, "attention: head dims differ");
  const int hd = (int)a.size[3];
  if (a.dtype != LLC_BFLOAT16 && a.dtype != LLC_FLOAT16 && a.dtype != LLC_FLOAT32)
    return set_error(LLC_ERR_DTYPE, "attention: f32, bf16 or f16 operands (type %d given)", a.dtype);
  for (int d = 0; d < 2; ++d)
    if (a.size[d] != b.size[d] || a.size[d] != c.size[d] || a.size[d] != o.size[d])
      return set_error(LLC_ERR_SHAPE, "attention: batch dims differ");
  if (b.size[2] != c.size[2] || o.size[2] != a.size[2]) return set_error(LLC_ERR_SHAPE, "attention: sequence lengths differ");
  if (!(scale > 0.0f)) return set_error(LLC_ERR_UNSUPPORTED, "attention: scale must be positive");
  AttnParams p{};
  p.B = (int)a.size[0];
  p.H = (int)a.size[1];
  p.Sq = (int)a.size[2];
  p.Skv = (int)b.size[2];
  if (a.size[0] * a.size[1] > 65535 || a.size[2] > 0x7fffff00 || b.size[2] > 0x7fffff00)
    return set_error(LLC_ERR_TOO_LARGE, "attention: more than 65535 heads in all, or a sequence too long");
  if (mask) {
    LLC_TRY(make_view(mask, "attention mask", &m));
    if (m.dtype != a.dtype) return set_error(LLC_ERR_DTYPE, "attention: mask type differs");
    if (m.rank != 2 || m.size[0] != a.size[0] || m.size[1] != b.size[2] || (m.size[1] != 1 && m.stride[1] != 1))
      return set_error(LLC_ERR_SHAPE, "attention: mask must be [B, Skv] with contiguous rows");
    p.mask = m.ptr;
    p.m_sb = m.stride[0];
  }
  if (o.numel() == 0) return LLC_OK;
  if (p.Skv == 0) return set_error(LLC_ERR_SHAPE, "attention: no keys");
  p.Q = a.ptr, p.K = b.ptr, p.V = c.ptr, p.O = o.ptr;
  p.q_sb = a.stride[0], p.q_sh = a.stride[1], p.q_ss = a.stride[2];
  p.k_sb = b.stride[0], p.k_sh = b.stride[1], p.k_ss = b.stride[2];
  p.v_sb = c.stride[0], p.v_sh = c.stride[1], p.v_ss = c.stride[2];
  p.o_sb = o.stride[0], p.o_sh = o.stride[1], p.o_ss = o.stride[2];
  p.scale_log2e = scale * kLog2e;
  hipStream_t s = as_stream(stream);
  if (a.dtype == LLC_FLOAT32) {
    // 128 queries per workgroup (K and V blocks are then shared by four waves) unless that leaves half the CUs
    // without work; LDS holds two workgroups per CU either way
    const bool four = (int64_t)((p.Sq + 127) / 128) * p.B * p.H >= 128;
    if (four) return p.mask ? launch_f32<4, true>(p, s) : launch_f32<4, false>(p, s);
    return p.mask ? launch_f32<2, true>(p, s) : launch_f32<2, false>(p, s);
  }
  const bool add = p.mask || p.Skv % kBlockKV != 0;
  if (hd == kD && (int64_t)((p.Sq + kBlockQ - 1) / kBlockQ) * p.B * p.H < 128 && p.Skv > 3 * kBlockKV) {
    // fewer workgroups of 128 queries than half the CUs, and keys enough for every wave: 32 queries per workgroup,
    // the key blocks dealt to its four waves (12 heads, 512 x 512: one sequence 10.7 -> 6.6 us, two 10.9 -> 9.4 us;
    // four sequences, 192 workgroups of 128 queries, are faster as they were: 11.4 against 16.6 us)
    const dim3 g32((unsigned)((p.Sq + 31) / 32), (unsigned)(p.B * p.H));
    auto go = [&](auto kern) {
      static std::atomic<uint32_t> lds_allowed{0};
      LLC_TRY(allow_dynamic_lds((const void*)kern, kSplitLds, lds_allowed));
      hipLaunchKernelGGL(kern, g32, dim3(256), kSplitLds, s, p);
      return check_launch("attention_split_kernel");
    };
    if (a.dtype == LLC_BFLOAT16) return add ? go(attention_split_kernel<__bf16, true>) : go(attention_split_kernel<__bf16, false>);
    return add ? go(attention_split_kernel<_Float16, true>) : go(attention_split_kernel<_Float16, false>);
  }
  const dim3 grid((unsigned)((p.Sq + kBlockQ - 1) / kBlockQ), (unsigned)(p.B * p.H));
  auto run = [&](auto kern, int lds, std::atomic<uint32_t>& allowed) {
    LLC_TRY(allow_dynamic_lds((const void*)kern, lds, allowed));
    hipLaunchKernelGGL(kern, grid, dim3(256), lds, s, p);
    return (int)LLC_OK;
  };
#define LLC_ATTN_LAUNCH(TT, DD)                                                                          \
  {                                                                                                      \
    static std::atomic<uint32_t> allowed[2];                                                             \
    LLC_TRY(add ? run(attention_kernel<TT, true, DD>, AttnGeom<DD>::kLds, allowed[1])                    \
                : run(attention_kernel<TT, false, DD>, AttnGeom<DD>::kLds, allowed[0]));                 \
  }
  if (a.dtype == LLC_BFLOAT16) {
    if (hd == 32) LLC_ATTN_LAUNCH(__bf16, 32)
    else if (hd == 64) LLC_ATTN_LAUNCH(__bf16, 64)
    else LLC_ATTN_LAUNCH(__bf16, 128)
  } else {
    if (hd == 32) LLC_ATTN_LAUNCH(_Float16, 32)
    else if (hd == 64) LLC_ATTN_LAUNCH(_Float16, 64)
    else LLC_ATTN_LAUNCH(_Float16, 128)
  }
#undef LLC_ATTN_LAUNCH
  return check_launch("attention_kernel");
}
