// Building blocks shared by the matrix-core kernels (matmul / batch_matmul / conv2d): LDS tile
// geometry, global->LDS operand staging, the MFMA step and the fused epilogue.
#pragma once
#include "common.hpp"

namespace llc {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(8 * sizeof(_Float16)))) _Float16 f16x8_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16_t;
typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4_t;

namespace gemm {

constexpr int kRowBytes = 128;   // bytes of k per LDS tile row
constexpr int kRowStride = 128;  // row pitch in LDS: unpadded, 16-byte chunks XOR-swizzled by the row
constexpr int kXcds = 8;

enum Loader { kLoadKVec = 0, kLoadRVec = 1, kLoadGeneric = 2 };

// LDS tile layout: row r holds 128 bytes of k; its eight 16-byte chunks are stored at chunk index
// c ^ swz(r), swz(r) = (r ^ (r >> 3)) & 7.  Fragment reads (lanes = consecutive rows, one chunk each),
// the k-contiguous copy (8 lanes = one row) and the transposing store (lanes = rows 8 apart) all
// spread over the banks, with no padding bytes.
__device__ __forceinline__ int lds_swz(int r) { return (r ^ (r >> 3)) & 7; }
__device__ __forceinline__ int lds_off(int r, int kbyte) {
  return r * kRowStride + ((((kbyte >> 4) ^ lds_swz(r)) & 7) << 4) + (kbyte & 15);
}

template <typename T> struct Elem;
template <> struct Elem<float> { static constexpr int kDtype = LLC_FLOAT32; };
template <> struct Elem<__bf16> { static constexpr int kDtype = LLC_BFLOAT16; };
template <> struct Elem<_Float16> { static constexpr int kDtype = LLC_FLOAT16; };

// ---- one MFMA step on a 16-byte A fragment and a 16-byte B fragment ----
template <typename T>
__device__ __forceinline__ void mfma_step(const u32x4_t& a, const u32x4_t& b, f32x16_t& acc) {
  if constexpr (sizeof(T) == 4) {
    // k slots inside an 8-k chunk are permuted identically for A and B (lane half h owns k = 4h..4h+3)
#pragma unroll
    for (int s = 0; s < 4; ++s)
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a[s]), __uint_as_float(b[s]), acc, 0, 0, 0);
  } else if constexpr (Elem<T>::kDtype == LLC_BFLOAT16) {
    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), acc,
                                                  0, 0, 0);
  } else {
    acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), acc, 0,
                                                 0, 0);
  }
}

// ---- global -> register staging of one operand tile: ROWS rows x 128 bytes of k, by NT lanes ----
// kLoadKVec : unit stride along k.  Each lane moves 16-byte vectors (one row, 8 or 4 consecutive k).
// kLoadRVec : unit stride along the row index.  Each lane owns a KB(k) x EPV(rows) block (KB = 4, or 2
//             when that is what it takes to give every lane a block), transposed in registers before
//             it is written to LDS.
// kLoadGeneric : element-wise with arbitrary strides.
template <typename T, int ROWS, int MODE, int NT>
struct TileLoader {
  static constexpr int EPV = 16 / sizeof(T);       // elements per 16 bytes
  static constexpr int BK = kRowBytes / sizeof(T);  // k extent of a tile
  static constexpr int kVecs = ROWS * 8;            // 16-byte vectors per tile
  static constexpr int kIters = (kVecs + NT - 1) / NT;
  static constexpr int kRBlocksPerK = ROWS / EPV;
  static constexpr int KB = ((BK / 4) * kRBlocksPerK >= NT) ? 4 : 2;
  static constexpr int kRBlocks = (BK / KB) * kRBlocksPerK;
  static constexpr int kRIters = (kRBlocks + NT - 1) / NT;
  static constexpr int kGenElems = (ROWS * BK + NT - 1) / NT;

  u32x4_t v[MODE == kLoadKVec ? kIters : (MODE == kLoadRVec ? kRIters * KB : 1)];
  T g[MODE == kLoadGeneric ? kGenElems : 1];
  uint32_t okm = 0xffffffffu;  // bit per vector of v: inside the operand (partial tiles)
  static_assert((MODE == kLoadKVec ? kIters : (MODE == kLoadRVec ? kRIters * KB : 1)) <= 32, "one mask word");

  // rows: valid row count of the operand; row0/k0: tile origin; s_r / s_k: element strides.
  // FULL: the tile lies entirely inside the operand, so no access is guarded.
  template <bool FULL = false>
  __device__ __forceinline__ void load(const T* base, int row0, int rows, int k0, int K, int64_t s_r, int64_t s_k) {
    const int tid = threadIdx.x;
    // Partial tiles: every load is issued unconditionally from an index clamped into the operand; which
    // vectors lie outside is kept as a bit mask and applied when the tile is written to LDS (a guarded load
    // compiles to a branch with a wait inside: one memory round trip after the other, none of them in
    // flight across the MFMAs).
    if constexpr (MODE == kLoadKVec) {
#pragma unroll
      for (int i = 0; i < kIters; ++i) {
        const int vid = i * NT + tid;
        const int r = vid >> 3, kv = vid & 7;
        const int gr = row0 + r, gk = k0 + kv * EPV;
        if constexpr (FULL) {
          if (kVecs % NT == 0 || vid < kVecs) v[i] = *(const u32x4_t*)(base + (int64_t)gr * s_r + gk);
        } else {
          const int cr = gr < rows ? gr : rows - 1, ck = gk < K ? gk : K - EPV;
          v[i] = *(const u32x4_t*)(base + (int64_t)cr * s_r + ck);
        }
      }
      if constexpr (!FULL) {
        okm = 0;
#pragma unroll
        for (int i = 0; i < kIters; ++i) {
          const int vid = i * NT + tid;
          const bool ok = (kVecs % NT == 0 || vid < kVecs) && row0 + (vid >> 3) < rows && k0 + (vid & 7) * EPV < K;
          okm |= ok ? (1u << i) : 0u;
        }
      }
    } else if constexpr (MODE == kLoadRVec) {
#pragma unroll
      for (int i = 0; i < kRIters; ++i) {
        const int bid = i * NT + tid;
        const int rb = bid % kRBlocksPerK, kb = bid / kRBlocksPerK;
        const int gr = row0 + rb * EPV;
#pragma unroll
        for (int kk = 0; kk < KB; ++kk) {
          const int gk = k0 + kb * KB + kk;
          if constexpr (FULL) {
            if (kRBlocks % NT == 0 || bid < kRBlocks) v[i * KB + kk] = *(const u32x4_t*)(base + (int64_t)gk * s_k + gr);
          } else {
            const int cr = gr < rows ? gr : rows - EPV, ck = gk < K ? gk : K - 1;
            v[i * KB + kk] = *(const u32x4_t*)(base + (int64_t)ck * s_k + cr);
          }
        }
      }
      if constexpr (!FULL) {
        okm = 0;
#pragma unroll
        for (int i = 0; i < kRIters; ++i) {
          const int bid = i * NT + tid;
          const int rb = bid % kRBlocksPerK, kb = bid / kRBlocksPerK;
#pragma unroll
          for (int kk = 0; kk < KB; ++kk) {
            const bool ok = (kRBlocks % NT == 0 || bid < kRBlocks) && row0 + rb * EPV < rows && k0 + kb * KB + kk < K;
            okm |= ok ? (1u << (i * KB + kk)) : 0u;
          }
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < kGenElems; ++i) {
        const int e = i * NT + tid;
        const int r = e / BK, k = e % BK;
        const int gr = row0 + r, gk = k0 + k;
        if constexpr (FULL) {
          if (e < ROWS * BK) g[i] = base[(int64_t)gr * s_r + (int64_t)gk * s_k];
        } else {
          const bool ok = e < ROWS * BK && gr < rows && gk < K;
          const int cr = gr < rows ? gr : rows - 1, ck = gk < K ? gk : K - 1;
          const T z = base[(int64_t)cr * s_r + (int64_t)ck * s_k];
          g[i] = ok ? z : static_cast<T>(0.0f);
        }
      }
    }
  }

  __device__ __forceinline__ u32x4_t masked(int i) const {
    const uint32_t m = 0u - ((okm >> i) & 1u);
    return u32x4_t{v[i][0] & m, v[i][1] & m, v[i][2] & m, v[i][3] & m};
  }

  __device__ __forceinline__ void store(char* lds) const {
    const int tid = threadIdx.x;
    if constexpr (MODE == kLoadKVec) {
#pragma unroll
      for (int i = 0; i < kIters; ++i) {
        const int vid = i * NT + tid;
        if (kVecs % NT == 0 || vid < kVecs) *(u32x4_t*)(lds + lds_off(vid >> 3, (vid & 7) * 16)) = masked(i);
      }
    } else if constexpr (MODE == kLoadRVec) {
#pragma unroll
      for (int i = 0; i < kRIters; ++i) {
        const int bid = i * NT + tid;
        if (!(kRBlocks % NT == 0 || bid < kRBlocks)) continue;
        const int rb = bid % kRBlocksPerK, kb = bid / kRBlocksPerK;
        const int row0 = rb * EPV, kbyte = kb * KB * (int)sizeof(T);
        const u32x4_t r0 = masked(i * KB + 0), r1 = masked(i * KB + 1);
        if constexpr (sizeof(T) == 4 && KB == 4) {
          const u32x4_t r2 = masked(i * KB + 2), r3 = masked(i * KB + 3);
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            u32x4_t o = {r0[j], r1[j], r2[j], r3[j]};
            *(u32x4_t*)(lds + lds_off(row0 + j, kbyte)) = o;
          }
        } else if constexpr (sizeof(T) == 4) {
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            uint2 o;
            o.x = r0[j];
            o.y = r1[j];
            *(uint2*)(lds + lds_off(row0 + j, kbyte)) = o;
          }
        } else if constexpr (KB == 4) {
          const u32x4_t r2 = masked(i * KB + 2), r3 = masked(i * KB + 3);
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            // 16-bit element j of each k-row: low halves for even j, high halves for odd j
            const uint32_t sel = (j & 1) ? 0x07060302u : 0x05040100u;
            uint2 o;
            o.x = __builtin_amdgcn_perm(r1[j >> 1], r0[j >> 1], sel);
            o.y = __builtin_amdgcn_perm(r3[j >> 1], r2[j >> 1], sel);
            *(uint2*)(lds + lds_off(row0 + j, kbyte)) = o;
          }
        } else {
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            const uint32_t sel = (j & 1) ? 0x07060302u : 0x05040100u;
            *(uint32_t*)(lds + lds_off(row0 + j, kbyte)) = __builtin_amdgcn_perm(r1[j >> 1], r0[j >> 1], sel);
          }
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < kGenElems; ++i) {
        const int e = i * NT + tid;
        if (e < ROWS * BK) *(T*)(lds + lds_off(e / BK, (e % BK) * (int)sizeof(T))) = g[i];
      }
    }
  }
};

__device__ __forceinline__ float load_as_f32(const char* p, int dtype, int64_t i) {
  if (dtype == LLC_FLOAT32) return ((const float*)p)[i];
  if (dtype == LLC_BFLOAT16) return bf16_bits_to_f32(((const uint16_t*)p)[i]);
  return f16_bits_to_f32(((const uint16_t*)p)[i]);
}


// XCD-aware workgroup -> tile mapping.  Consecutive workgroup ids are dealt round-robin to the 8
// XCDs by the hardware, so ids are first regrouped per XCD, then walked in column-grouped order
// (8 tile rows per group): each XCD's L2 sees a compact patch of the output.
__device__ __forceinline__ void tile_of_id(int id, int tiles_m, int tiles_n, int& tm, int& tn) {
  const int G = 8;
  const int per_group = G * tiles_n;
  const int group = id / per_group;
  const int first_m = group * G;
  const int gsize = (tiles_m - first_m) < G ? (tiles_m - first_m) : G;
  const int in_group = id % per_group;
  tm = first_m + in_group % gsize;
  tn = in_group / gsize;
}
__device__ __forceinline__ void tile_of_block(int tiles_m, int tiles_n, int& tm, int& tn) {
  const int total = tiles_m * tiles_n;
  int id = blockIdx.x;
  if (total % kXcds == 0) id = (id % kXcds) * (total / kXcds) + id / kXcds;
  tile_of_id(id, tiles_m, tiles_n, tm, tn);
}
// The same for a grid (tiles, 1, batch): the hardware deals workgroups to the XCDs in x-then-z order, so with a
// tile count that is a multiple of 8 every XCD would get an eighth of EVERY batch entry and each operand panel
// would be fetched into all eight L2s.  The (tile, batch) pairs are regrouped so that an XCD walks whole batch
// entries, one after the other.
__device__ __forceinline__ void tile_and_batch_of_block(int tiles_m, int tiles_n, int& tm, int& tn, int& z) {
  if (gridDim.z == 1) {
    z = 0;
    tile_of_block(tiles_m, tiles_n, tm, tn);
    return;
  }
  const unsigned tiles = (unsigned)(tiles_m * tiles_n);
  const unsigned long long total = (unsigned long long)tiles * gridDim.z;
  unsigned long long w = blockIdx.x + (unsigned long long)tiles * blockIdx.z;
  if (total % kXcds == 0) w = (w % kXcds) * (total / kXcds) + w / kXcds;
  z = (int)(w / tiles);
  tile_of_id((int)(w % tiles), tiles_m, tiles_n, tm, tn);
}

// MFMAs of one LDS tile pair for one wave: TM x TN fragments of 32x32, four steps of two 16-byte
// k-chunks (lane half lh takes chunk 2s+lh).  ta / tb are the A / B tiles; arow / brow are this lane's
// first fragment row in each (fragment i covers rows arow + 32 i).
template <typename T, int TM, int TN, int S0 = 0, int S1 = 4>
__device__ __forceinline__ void mma_tile(const char* ta, int arow, const char* tb, int brow, int lh,
                                         f32x16_t (&acc)[TM][TN]) {
  int abase[TM], aswz[TM], bbase[TN], bswz[TN];
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    abase[i] = (arow + i * 32) * kRowStride;
    aswz[i] = lds_swz(arow + i * 32);
  }
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    bbase[j] = (brow + j * 32) * kRowStride;
    bswz[j] = lds_swz(brow + j * 32);
  }
#pragma unroll
  for (int s = S0; s < S1; ++s) {
    u32x4_t fa[TM], fb[TN];
#pragma unroll
    for (int i = 0; i < TM; ++i) fa[i] = *(const u32x4_t*)(ta + abase[i] + (((2 * s + lh) ^ aswz[i]) << 4));
#pragma unroll
    for (int j = 0; j < TN; ++j) fb[j] = *(const u32x4_t*)(tb + bbase[j] + (((2 * s + lh) ^ bswz[j]) << 4));
    if constexpr (sizeof(T) == 4) {
      // four fp32 MFMAs per fragment pair (one per k slot of the 16-byte chunk): walk the k slots outermost so
      // that consecutive MFMAs write different accumulators instead of forming a dependent chain of four
#pragma unroll
      for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(fa[i][q]), __uint_as_float(fb[j][q]), acc[i][j], 0, 0, 0);
    } else {
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) mfma_step<T>(fa[i], fb[j], acc[i][j]);
    }
  }
}

// act(alpha * acc + bias + residual) -> storage type, one element
template <typename T>
__device__ __forceinline__ void epilogue_store(T* C, int64_t o, float acc, float alpha, float bias, const char* res,
                                               int act) {
  constexpr int dt = Elem<T>::kDtype;
  float v = acc * alpha + bias;
  if (res) v += load_as_f32(res, dt, o);
  if (act == LLC_ACT_RELU) v = v < 0.0f ? 0.0f : v;  // NaN passes through, like torch.relu
  else if (act == LLC_ACT_GELU) v = gelu_for<T>(v);
  if constexpr (dt == LLC_FLOAT32) C[o] = v;
  else if constexpr (dt == LLC_BFLOAT16) ((uint16_t*)C)[o] = f32_to_bf16_bits(v);
  else ((uint16_t*)C)[o] = f32_to_f16_bits(v);
}

// A lane's sixteen values of one 32x32 accumulator block through the epilogue.  Value r belongs to row 8 (r / 4) + r % 4 of
// the lane's sixteen (its first row and its column are in `base`, an element offset into C and the residual; rows are `ld`
// elements apart): C[..] = act(alpha * acc[r] + bias_of(r) + residual[..]).  GUARD: only the first `rows_left` of those
// row numbers exist (base then points at an existing row; rows_left may be <= 0); what does not exist is computed from
// the lane's first row and not stored.  All sixteen residual values are requested before the first result is stored:
// written element by element (load, add, store), every load waits for the store before it, which may alias it, and
// every store for its load: thirty-two trips to memory in a row on each lane.  A residual that is the output tensor
// itself (an in-place add) stays correct: a lane reads exactly the elements it writes.  The row offsets are multiples
// of `ld` known when compiling, so they live in scalar registers: sixteen 64-bit offsets per lane had cost the
// 128 x 128 four-wave configuration half its waves (272 registers against 240).
template <typename T, bool GUARD, typename BiasFn>
__device__ __forceinline__ void epilogue_block16(T* C, const char* res, int64_t base, int64_t ld, int rows_left,
                                                 const f32x16_t& acc, float alpha, BiasFn bias_of, int act) {
  constexpr int dt = Elem<T>::kDtype;
  float rv[16];
  if (res) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int ro = (r / 4) * 8 + (r % 4);
      rv[r] = load_as_f32(res, dt, base + (int64_t)((!GUARD || ro < rows_left) ? ro : 0) * ld);
    }
  }
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int ro = (r / 4) * 8 + (r % 4);
    if (!GUARD || ro < rows_left) {  // nothing is computed for rows that do not exist (grouped convolutions: most of a block)
      float v = acc[r] * alpha + bias_of(r);
      if (res) v += rv[r];
      if (act == LLC_ACT_RELU) v = v < 0.0f ? 0.0f : v;  // NaN passes through, like torch.relu
      else if (act == LLC_ACT_GELU) v = gelu_for<T>(v);
      const int64_t o = base + (int64_t)ro * ld;
      if constexpr (dt == LLC_FLOAT32) C[o] = v;
      else if constexpr (dt == LLC_BFLOAT16) ((uint16_t*)C)[o] = f32_to_bf16_bits(v);
      else ((uint16_t*)C)[o] = f32_to_f16_bits(v);
    }
  }
}

// The pass over the partial sums of a split reduction, four consecutive outputs of one row per lane:
// out[i4 .. i4 + 3] = act(alpha * (part[0] + part[1] + ...) + bias[col ..] + residual[i4 ..]), the partial sums `stride`
// floats apart and added in split order (the same order on every run).  Written as a loop of load-and-add, each load waits
// for the one before it, nine to eighteen trips to memory in a row on every lane, and bias and residual follow after the
// last; here bias and residual are requested first (unconditionally: an absent operand reads the first partial sum's
// memory and is ignored) and the partial sums eight at a time.
template <typename T>
__device__ __forceinline__ void split_epilogue4(const float* part, int splits, int64_t stride, int64_t i4, int col, float alpha,
                                                const char* bias, const char* residual, int act, T* out) {
  typedef float v4f __attribute__((ext_vector_type(4)));
  constexpr int dt = Elem<T>::kDtype;
  const char* bsrc = bias ? bias + (int64_t)col * sizeof(T) : (const char*)part;
  const char* rsrc = residual ? residual + i4 * (int64_t)sizeof(T) : (const char*)part;
  float b[4], r[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) b[j] = load_as_f32(bsrc, dt, j);
#pragma unroll
  for (int j = 0; j < 4; ++j) r[j] = load_as_f32(rsrc, dt, j);
  const float* src = part + i4;
  v4f acc = {0.0f, 0.0f, 0.0f, 0.0f};
  for (int k0 = 0; k0 < splits; k0 += 8) {
    v4f v[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = *(const v4f*)(src + (int64_t)(k0 + j < splits ? k0 + j : splits - 1) * stride);
#pragma unroll
    for (int j = 0; j < 8; ++j)
      if (k0 + j < splits) acc = k0 + j == 0 ? v[j] : acc + v[j];
  }
  float o[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    float v = acc[j] * alpha + (bias ? b[j] : 0.0f);
    if (residual) v += r[j];
    if (act == LLC_ACT_RELU) v = v < 0.0f ? 0.0f : v;  // NaN passes through, like torch.relu
    else if (act == LLC_ACT_GELU) v = gelu_for<T>(v);
    o[j] = v;
  }
  if constexpr (dt == LLC_FLOAT32) {
    *(v4f*)((float*)out + i4) = v4f{o[0], o[1], o[2], o[3]};
  } else {
    *(uint2*)((uint16_t*)out + i4) = uint2{pack_pair<dt>(o[0], o[1]), pack_pair<dt>(o[2], o[3])};
  }
}

}  // namespace gemm
}  // namespace llc
