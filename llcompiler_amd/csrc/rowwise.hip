// Row-wise kernels over the last (contiguous) dim: softmax, layer_norm and reduce_sum/max/min.
//
// A row is read from HBM exactly once: TPR lanes share a row, each lane keeps ITEMS vectors of VEC
// elements in registers, statistics are reduced with wave64 cross-lane shuffles (and one LDS hop
// when a row spans several waves), and the result is written once.  Statistics are always fp32.
// Algorithmic traffic is therefore read + write of the tensor, which is what these kernels are
// measured against.

#include "common.hpp"

namespace llc {
namespace {

enum RowOp { kSoftmax = 0, kLayerNorm = 1, kReduce = 2 };

struct RowParams {
  const char* x;
  char* y;
  const char* gamma;  // layer_norm scale (may be null)
  const char* beta;   // layer_norm bias (may be null)
  int32_t dtype;      // storage type of x / y / gamma / beta
  int32_t kind;       // llc_reduce_kind for kReduce
  int64_t rows;
  int32_t cols;
  float eps;
  float scale;  // kReduce: result multiplied by this (1/HW for average pooling)
  int32_t streaming;  // non-temporal accesses: the tensor is far larger than the caches and touched once
};

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// VEC elements of the storage type as raw bytes (16 bytes when VEC > 1), optionally non-temporal
template <int VEC, int ES>
struct RowPack {
  alignas(VEC * ES) unsigned char b[VEC * ES];
};
template <int VEC, int ES>
__device__ __forceinline__ RowPack<VEC, ES> ld_pack(const char* p, bool nt) {
  RowPack<VEC, ES> r;
  if constexpr (VEC * ES == 16) {
    u32x4 v = nt ? __builtin_nontemporal_load((const u32x4*)p) : *(const u32x4*)p;
    __builtin_memcpy(r.b, &v, 16);
  } else if constexpr (VEC * ES == 4) {
    uint32_t v = *(const uint32_t*)p;
    __builtin_memcpy(r.b, &v, 4);
  } else {
    uint16_t v = *(const uint16_t*)p;
    __builtin_memcpy(r.b, &v, 2);
  }
  return r;
}
template <int VEC, int ES>
__device__ __forceinline__ void st_pack(char* p, const RowPack<VEC, ES>& r, bool nt) {
  if constexpr (VEC * ES == 16) {
    u32x4 v;
    __builtin_memcpy(&v, r.b, 16);
    if (nt) __builtin_nontemporal_store(v, (u32x4*)p);
    else *(u32x4*)p = v;
  } else if constexpr (VEC * ES == 4) {
    uint32_t v;
    __builtin_memcpy(&v, r.b, 4);
    *(uint32_t*)p = v;
  } else {
    uint16_t v;
    __builtin_memcpy(&v, r.b, 2);
    *(uint16_t*)p = v;
  }
}

template <int VEC>
__device__ __forceinline__ void load_row_vec(const char* base, int dtype, int64_t off, float* dst, bool nt = false) {
  if (dtype == LLC_FLOAT32) {
    // rows are read 4 wide (fp32) or 8 wide (16-bit types), i.e. 16 bytes, or element-wise; the width
    // that does not belong to a storage type is never launched for it and is only remapped so that the
    // run-time dtype switch compiles
    constexpr int V = VEC == 8 ? 4 : VEC;
    RowPack<V, 4> p = ld_pack<V, 4>(base + off * 4, nt);
    float t[V];
    __builtin_memcpy(t, p.b, sizeof(t));
#pragma unroll
    for (int j = 0; j < V; ++j) dst[j] = t[j];
  } else {
    constexpr int V = VEC == 4 ? 8 : VEC;  // 16-bit rows are never read 4 wide
    RowPack<V, 2> p = ld_pack<V, 2>(base + off * 2, nt);
    uint16_t t[V];
    __builtin_memcpy(t, p.b, sizeof(t));
    if (dtype == LLC_BFLOAT16) {
#pragma unroll
      for (int j = 0; j < (V < VEC ? V : VEC); ++j) dst[j] = bf16_bits_to_f32(t[j]);
    } else {
#pragma unroll
      for (int j = 0; j < (V < VEC ? V : VEC); ++j) dst[j] = f16_bits_to_f32(t[j]);
    }
  }
}
template <int VEC>
__device__ __forceinline__ void store_row_vec(char* base, int dtype, int64_t off, const float* src, bool nt = false) {
  if (dtype == LLC_FLOAT32) {
    constexpr int V = VEC == 8 ? 4 : VEC;
    float t[V];
#pragma unroll
    for (int j = 0; j < V; ++j) t[j] = src[j];
    RowPack<V, 4> p;
    __builtin_memcpy(p.b, t, sizeof(t));
    st_pack<V, 4>(base + off * 4, p, nt);
  } else {
    constexpr int V = VEC == 4 ? 8 : VEC;
    uint16_t t[V];
    if (dtype == LLC_BFLOAT16) {
#pragma unroll
      for (int j = 0; j < V; ++j) t[j] = f32_to_bf16_bits(src[j < VEC ? j : 0]);
    } else {
#pragma unroll
      for (int j = 0; j < V; ++j) t[j] = f32_to_f16_bits(src[j < VEC ? j : 0]);
    }
    RowPack<V, 2> p;
    __builtin_memcpy(p.b, t, sizeof(t));
    st_pack<V, 2>(base + off * 2, p, nt);
  }
}

__device__ __forceinline__ float nmax(float a, float b) { return (a > b || a != a) ? a : b; }
__device__ __forceinline__ float nmin(float a, float b) { return (a < b || a != a) ? a : b; }

enum Combine { kAdd = 0, kMax = 1, kMin = 2 };
template <int C> __device__ __forceinline__ float combine(float a, float b) {
  if constexpr (C == kAdd) return a + b;
  else if constexpr (C == kMax) return nmax(a, b);
  else return nmin(a, b);
}

// Reduction over the TPR lanes that share a row.  TPR <= 64: xor-shuffles inside the wave.
// TPR == 256: the whole block is one row; wave results meet in LDS.
template <int TPR, int C>
__device__ __forceinline__ float row_reduce(float v, float* smem) {
  constexpr int W = TPR < kWave ? TPR : kWave;
#pragma unroll
  for (int o = W / 2; o > 0; o >>= 1) v = combine<C>(v, __shfl_xor(v, o, kWave));
  if constexpr (TPR > kWave) {
    constexpr int NW = TPR / kWave;
    const int wave = threadIdx.x / kWave;
    __syncthreads();  // smem reuse across successive reductions
    if ((threadIdx.x & (kWave - 1)) == 0) smem[wave] = v;
    __syncthreads();
    v = smem[0];
#pragma unroll
    for (int w = 1; w < NW; ++w) v = combine<C>(v, smem[w]);
  }
  return v;
}

// 16 bytes of a row as VEC floats (VEC = 4: fp32; VEC = 8: bf16 / f16).  The load itself does not depend on
// the storage type; the conversion branches on it, uniformly, after every load of the lane has been issued.
template <int VEC>
__device__ __forceinline__ void unpack_row_vec(const u32x4& raw, int dtype, float* dst) {
  if constexpr (VEC == 4) {
#pragma unroll
    for (int j = 0; j < 4; ++j) dst[j] = __uint_as_float(raw[j]);
  } else {
    if (dtype == LLC_BFLOAT16) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        dst[2 * j] = __uint_as_float(raw[j] << 16);
        dst[2 * j + 1] = __uint_as_float(raw[j] & 0xffff0000u);
      }
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        dst[2 * j] = f16_bits_to_f32((uint16_t)(raw[j] & 0xffffu));
        dst[2 * j + 1] = f16_bits_to_f32((uint16_t)(raw[j] >> 16));
      }
    }
  }
}

template <int OP, int VEC, int TPR, int ITEMS>
__global__ __launch_bounds__(256) void row_kernel(const RowParams p) {
  __shared__ float smem[4];
  constexpr int RPB = 256 / TPR;  // rows per block
  const int lane = threadIdx.x % TPR;
  const int64_t row = (int64_t)blockIdx.x * RPB + threadIdx.x / TPR;
  const bool row_ok = row < p.rows;
  const int64_t base = row * p.cols;
  // full: every lane of the launch owns ITEMS complete vectors, nothing to mask
  const bool full = p.cols == TPR * ITEMS * VEC && p.rows % RPB == 0;

  float v[ITEMS][VEC];
  bool ok[ITEMS];
  u32x4 graw[OP == kLayerNorm && VEC > 1 ? ITEMS : 1], braw[OP == kLayerNorm && VEC > 1 ? ITEMS : 1];  // scale / bias
  const float fill = (OP == kSoftmax) ? -INFINITY
                     : (OP == kReduce) ? (p.kind == LLC_REDUCE_SUM ? 0.0f : (p.kind == LLC_REDUCE_MAX ? -INFINITY : INFINITY))
                                       : 0.0f;
  if constexpr (VEC > 1) {
    // Every load is issued before anything waits: unconditional, from an address clamped into the tensor
    // (a guarded load compiles to a branch with a wait inside, which serialises the round trips).
    const int es = p.dtype == LLC_FLOAT32 ? 4 : 2;
    const int64_t crow = row_ok ? row : p.rows - 1;
    u32x4 raw[ITEMS];
    const u32x4* src[ITEMS];
    int ccol[ITEMS];
#pragma unroll
    for (int it = 0; it < ITEMS; ++it) {
      const int col = (it * TPR + lane) * VEC;
      ok[it] = row_ok && col < p.cols;
      ccol[it] = col < p.cols ? col : p.cols - VEC;
      src[it] = (const u32x4*)(p.x + (crow * p.cols + ccol[it]) * es);
    }
    if (p.streaming) {
#pragma unroll
      for (int it = 0; it < ITEMS; ++it) raw[it] = __builtin_nontemporal_load(src[it]);
    } else {
#pragma unroll
      for (int it = 0; it < ITEMS; ++it) raw[it] = *src[it];
    }
    if constexpr (OP == kLayerNorm) {
      // scale and bias do not depend on the statistics: their loads travel while the row is reduced
      if (p.gamma) {
#pragma unroll
        for (int it = 0; it < ITEMS; ++it) graw[it] = *(const u32x4*)(p.gamma + (int64_t)ccol[it] * es);
      }
      if (p.beta) {
#pragma unroll
        for (int it = 0; it < ITEMS; ++it) braw[it] = *(const u32x4*)(p.beta + (int64_t)ccol[it] * es);
      }
    }
#pragma unroll
    for (int it = 0; it < ITEMS; ++it) unpack_row_vec<VEC>(raw[it], p.dtype, v[it]);
    if (!full) {
#pragma unroll
      for (int it = 0; it < ITEMS; ++it)
#pragma unroll
        for (int j = 0; j < VEC; ++j) v[it][j] = ok[it] ? v[it][j] : fill;
    }
  } else {
#pragma unroll
    for (int it = 0; it < ITEMS; ++it) {
      const int col = (it * TPR + lane) * VEC;
      ok[it] = row_ok && col < p.cols;
      if (ok[it]) load_row_vec<VEC>(p.x, p.dtype, base + col, v[it], p.streaming != 0);
      else {
#pragma unroll
        for (int j = 0; j < VEC; ++j) v[it][j] = fill;
      }
    }
  }

  if constexpr (OP == kSoftmax) {
    float m = -INFINITY;
#pragma unroll
    for (int it = 0; it < ITEMS; ++it)
#pragma unroll
      for (int j = 0; j < VEC; ++j) m = nmax(m, v[it][j]);
    m = row_reduce<TPR, kMax>(m, smem);
    float s = 0.0f;
#pragma unroll
    for (int it = 0; it < ITEMS; ++it)
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        // exp through the hardware exp2 (relative error below 1e-5 for arguments down to -88).  Masked
        // lanes hold -inf: exp(-inf - m) = 0 for finite m; they are kept out when m is -inf too
        float e = __builtin_amdgcn_exp2f((v[it][j] - m) * 1.4426950408889634f);
        if (!full) e = ok[it] ? e : 0.0f;
        v[it][j] = e;
        s += e;
      }
    s = row_reduce<TPR, kAdd>(s, smem);
    const float inv = 1.0f / s;
#pragma unroll
    for (int it = 0; it < ITEMS; ++it) {
      if (ok[it]) {
#pragma unroll
        for (int j = 0; j < VEC; ++j) v[it][j] *= inv;
        store_row_vec<VEC>(p.y, p.dtype, base + (it * TPR + lane) * VEC, v[it], p.streaming != 0);
      }
    }
  } else if constexpr (OP == kLayerNorm) {
    float s = 0.0f;
#pragma unroll
    for (int it = 0; it < ITEMS; ++it)
#pragma unroll
      for (int j = 0; j < VEC; ++j) s += v[it][j];
    s = row_reduce<TPR, kAdd>(s, smem);
    const float mean = s / (float)p.cols;
    float q = 0.0f;
#pragma unroll
    for (int it = 0; it < ITEMS; ++it)
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        float d = v[it][j] - mean;
        if (!full) d = ok[it] ? d : 0.0f;
        v[it][j] = d;
        q += d * d;
      }
    q = row_reduce<TPR, kAdd>(q, smem);
    const float rstd = 1.0f / sqrtf(q / (float)p.cols + p.eps);
#pragma unroll
    for (int it = 0; it < ITEMS; ++it) {
      if (ok[it]) {
        const int col = (it * TPR + lane) * VEC;
        float g[VEC], b[VEC];
        if constexpr (VEC > 1) {
          if (p.gamma) unpack_row_vec<VEC>(graw[it], p.dtype, g);
          if (p.beta) unpack_row_vec<VEC>(braw[it], p.dtype, b);
        } else {
          if (p.gamma) load_row_vec<VEC>(p.gamma, p.dtype, col, g);
          if (p.beta) load_row_vec<VEC>(p.beta, p.dtype, col, b);
        }
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
          float t = v[it][j] * rstd;
          if (p.gamma) t *= g[j];
          if (p.beta) t += b[j];
          v[it][j] = t;
        }
        store_row_vec<VEC>(p.y, p.dtype, base + col, v[it], p.streaming != 0);
      }
    }
  } else {
    float r;
    if (p.kind == LLC_REDUCE_SUM) {
      r = 0.0f;
#pragma unroll
      for (int it = 0; it < ITEMS; ++it)
#pragma unroll
        for (int j = 0; j < VEC; ++j) r += v[it][j];
      r = row_reduce<TPR, kAdd>(r, smem) * p.scale;
    } else if (p.kind == LLC_REDUCE_MAX) {
      r = -INFINITY;
#pragma unroll
      for (int it = 0; it < ITEMS; ++it)
#pragma unroll
        for (int j = 0; j < VEC; ++j) r = nmax(r, v[it][j]);
      r = row_reduce<TPR, kMax>(r, smem);
    } else {
      r = INFINITY;
#pragma unroll
      for (int it = 0; it < ITEMS; ++it)
#pragma unroll
        for (int j = 0; j < VEC; ++j) r = nmin(r, v[it][j]);
      r = row_reduce<TPR, kMin>(r, smem);
    }
    if (row_ok && lane == 0) {
      float one[1] = {r};
      store_row_vec<1>(p.y, p.dtype, row, one);
    }
  }
}

template <int DT, bool NT>
__device__ __forceinline__ void store_typed(char* dst, const float* src) {
  if constexpr (NT) __builtin_nontemporal_store(pack_typed<DT>(src), (u32x4*)dst);
  else *(u32x4*)dst = pack_typed<DT>(src);
}

// Softmax, and layer norm with both a scale and a bias (what nn.LayerNorm is), for rows read 16 bytes wide, with the
// storage type DT known when compiling.  In row_kernel the storage type and the optional operands sit behind uniform
// branches, and every value a branch defines must have arrived where the branch ends: the layer norm's bias loads left
// only after the row and the scale had come back, one more trip to memory on every wave's path, and each vector's
// conversion is a branch of its own.  Here every load is unconditional and issued before anything waits, and the rest is
// straight-line code (8192 x 1024 bf16 layer norm: 10.1 -> 8.1 us; 16384 x 768: 15.2 -> 12.2 us).
//
// NT: the row is read and the result written with non-temporal accesses.  Measured on tensors no cache holds (operand sets
// rotating through 400 MB), typed kernel without | with: softmax 8192 x 1024 bf16 8.7 | 6.6 us, 16384 x 768 bf16 12.2 | 9.3,
// 4096 x 4096 f32 24.2 | 23.4; layer norm 8192 x 1024 bf16 8.1 | 7.4, 262144 x 768 bf16 132 | 128.  Inside a network, where
// the next kernel finds a small result in the caches, they cost instead (encoder block, batch 8, 6 MB rows tensors:
// 0.124 | 0.129 ms; batch 32, 25 MB: 0.344 | 0.344), so the launcher asks for them from 16 MiB on.
template <int OP, int DT, int TPR, int ITEMS, bool NT>
__global__ __launch_bounds__(256) void row_typed_kernel(const RowParams p) {
  __shared__ float smem[4];
  constexpr int VEC = DT == LLC_FLOAT32 ? 4 : 8;
  constexpr int ES = DT == LLC_FLOAT32 ? 4 : 2;
  constexpr int RPB = 256 / TPR;
  const int lane = threadIdx.x % TPR;
  const int64_t row = (int64_t)blockIdx.x * RPB + threadIdx.x / TPR;
  const bool full = p.cols == TPR * ITEMS * VEC;

  bool cok[ITEMS];
  int ccol[ITEMS];
#pragma unroll
  for (int it = 0; it < ITEMS; ++it) {
    const int col = (it * TPR + lane) * VEC;
    cok[it] = col < p.cols;
    ccol[it] = cok[it] ? col : p.cols - VEC;  // addresses clamped into the tensor; what they bring is masked below
  }
  const char* xrow = p.x + (row < p.rows ? row : p.rows - 1) * p.cols * ES;
  u32x4 raw[ITEMS], graw[OP == kLayerNorm ? ITEMS : 1], braw[OP == kLayerNorm ? ITEMS : 1];
#pragma unroll
  for (int it = 0; it < ITEMS; ++it) {
    const u32x4* src = (const u32x4*)(xrow + ccol[it] * ES);
    if constexpr (NT) raw[it] = __builtin_nontemporal_load(src);
    else raw[it] = *src;
  }
  if constexpr (OP == kLayerNorm) {
#pragma unroll
    for (int it = 0; it < ITEMS; ++it) graw[it] = *(const u32x4*)(p.gamma + ccol[it] * ES);
#pragma unroll
    for (int it = 0; it < ITEMS; ++it) braw[it] = *(const u32x4*)(p.beta + ccol[it] * ES);
    // left alone, the instruction scheduler moves the scale and bias loads down to their use behind the reductions
    __builtin_amdgcn_sched_barrier(0);
  }

  float v[ITEMS][VEC];
#pragma unroll
  for (int it = 0; it < ITEMS; ++it) unpack_typed<DT>(raw[it], v[it]);
  if constexpr (OP == kSoftmax) {
    float m = -INFINITY;
#pragma unroll
    for (int it = 0; it < ITEMS; ++it)
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        if (!full) v[it][j] = cok[it] ? v[it][j] : -INFINITY;
        m = nmax(m, v[it][j]);
      }
    m = row_reduce<TPR, kMax>(m, smem);
    float s = 0.0f;
#pragma unroll
    for (int it = 0; it < ITEMS; ++it)
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        // exp through the hardware exp2, as in row_kernel; masked lanes hold -inf and stay out when m is -inf too
        float e = __builtin_amdgcn_exp2f((v[it][j] - m) * 1.4426950408889634f);
        if (!full) e = cok[it] ? e : 0.0f;
        v[it][j] = e;
        s += e;
      }
    s = row_reduce<TPR, kAdd>(s, smem);
    const float inv = 1.0f / s;
#pragma unroll
    for (int it = 0; it < ITEMS; ++it) {
      float t[VEC];
#pragma unroll
      for (int j = 0; j < VEC; ++j) t[j] = v[it][j] * inv;
      if (row < p.rows && cok[it]) store_typed<DT, NT>(p.y + (row * p.cols + (it * TPR + lane) * VEC) * ES, t);
    }
  } else {
    float s = 0.0f;
#pragma unroll
    for (int it = 0; it < ITEMS; ++it)
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        if (!full) v[it][j] = cok[it] ? v[it][j] : 0.0f;
        s += v[it][j];
      }
    s = row_reduce<TPR, kAdd>(s, smem);
    const float mean = s / (float)p.cols;
    float q = 0.0f;
#pragma unroll
    for (int it = 0; it < ITEMS; ++it)
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        float d = v[it][j] - mean;
        if (!full) d = cok[it] ? d : 0.0f;
        v[it][j] = d;
        q += d * d;
      }
    q = row_reduce<TPR, kAdd>(q, smem);
    const float rstd = 1.0f / sqrtf(q / (float)p.cols + p.eps);
#pragma unroll
    for (int it = 0; it < ITEMS; ++it) {
      float g[VEC], b[VEC], t[VEC];
      unpack_typed<DT>(graw[it], g);
      unpack_typed<DT>(braw[it], b);
#pragma unroll
      for (int j = 0; j < VEC; ++j) t[j] = v[it][j] * rstd * g[j] + b[j];
      if (row < p.rows && cok[it]) store_typed<DT, NT>(p.y + (row * p.cols + (it * TPR + lane) * VEC) * ES, t);
    }
  }
}

// Rows too long for registers: one block per row, three strided sweeps over the row (the second
// and third hit L2).  Correctness path for rare shapes, not a tuned one.
template <int OP>
__global__ __launch_bounds__(256) void row_loop_kernel(const RowParams p) {
  __shared__ float smem[4];
  const int64_t row = blockIdx.x;
  const int64_t base = row * p.cols;
  float one[1];
  if constexpr (OP == kSoftmax) {
    float m = -INFINITY;
    for (int c = threadIdx.x; c < p.cols; c += 256) {
      load_row_vec<1>(p.x, p.dtype, base + c, one);
      m = nmax(m, one[0]);
    }
    m = row_reduce<256, kMax>(m, smem);
    float s = 0.0f;
    for (int c = threadIdx.x; c < p.cols; c += 256) {
      load_row_vec<1>(p.x, p.dtype, base + c, one);
      s += expf(one[0] - m);
    }
    s = row_reduce<256, kAdd>(s, smem);
    const float inv = 1.0f / s;
    for (int c = threadIdx.x; c < p.cols; c += 256) {
      load_row_vec<1>(p.x, p.dtype, base + c, one);
      one[0] = expf(one[0] - m) * inv;
      store_row_vec<1>(p.y, p.dtype, base + c, one);
    }
  } else if constexpr (OP == kLayerNorm) {
    float s = 0.0f;
    for (int c = threadIdx.x; c < p.cols; c += 256) {
      load_row_vec<1>(p.x, p.dtype, base + c, one);
      s += one[0];
    }
    s = row_reduce<256, kAdd>(s, smem);
    const float mean = s / (float)p.cols;
    float q = 0.0f;
    for (int c = threadIdx.x; c < p.cols; c += 256) {
      load_row_vec<1>(p.x, p.dtype, base + c, one);
      float d = one[0] - mean;
      q += d * d;
    }
    q = row_reduce<256, kAdd>(q, smem);
    const float rstd = 1.0f / sqrtf(q / (float)p.cols + p.eps);
    for (int c = threadIdx.x; c < p.cols; c += 256) {
      load_row_vec<1>(p.x, p.dtype, base + c, one);
      float t = (one[0] - mean) * rstd;
      float g[1], b[1];
      if (p.gamma) { load_row_vec<1>(p.gamma, p.dtype, c, g); t *= g[0]; }
      if (p.beta) { load_row_vec<1>(p.beta, p.dtype, c, b); t += b[0]; }
      one[0] = t;
      store_row_vec<1>(p.y, p.dtype, base + c, one);
    }
  } else {
    float r = p.kind == LLC_REDUCE_SUM ? 0.0f : (p.kind == LLC_REDUCE_MAX ? -INFINITY : INFINITY);
    for (int c = threadIdx.x; c < p.cols; c += 256) {
      load_row_vec<1>(p.x, p.dtype, base + c, one);
      r = p.kind == LLC_REDUCE_SUM ? r + one[0] : (p.kind == LLC_REDUCE_MAX ? nmax(r, one[0]) : nmin(r, one[0]));
    }
    if (p.kind == LLC_REDUCE_SUM) r = row_reduce<256, kAdd>(r, smem) * p.scale;
    else if (p.kind == LLC_REDUCE_MAX) r = row_reduce<256, kMax>(r, smem);
    else r = row_reduce<256, kMin>(r, smem);
    if (threadIdx.x == 0) {
      one[0] = r;
      store_row_vec<1>(p.y, p.dtype, row, one);
    }
  }
}

// Reduction over a middle dim: x viewed as [outer, R, inner], inner > 1.  One lane per output
// element, lanes consecutive along `inner` so every load is coalesced; R is walked sequentially.
__global__ __launch_bounds__(256) void mid_reduce_kernel(const RowParams p, int64_t outer, int64_t R, int64_t inner) {
  const int64_t o = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (o >= outer * inner) return;
  const int64_t i = o % inner, b = o / inner;
  float r = p.kind == LLC_REDUCE_SUM ? 0.0f : (p.kind == LLC_REDUCE_MAX ? -INFINITY : INFINITY);
  float one[1];
  for (int64_t k = 0; k < R; ++k) {
    load_row_vec<1>(p.x, p.dtype, (b * R + k) * inner + i, one);
    r = p.kind == LLC_REDUCE_SUM ? r + one[0] : (p.kind == LLC_REDUCE_MAX ? nmax(r, one[0]) : nmin(r, one[0]));
  }
  if (p.kind == LLC_REDUCE_SUM) r *= p.scale;
  one[0] = r;
  store_row_vec<1>(p.y, p.dtype, o, one);
}

// The same reduction when the outputs are too few to fill the chip with one lane each (a global average pool over a
// channels-last tensor: 16 x 512 outputs of 49 values): 64 consecutive outputs per workgroup, the reduced range dealt
// to its four waves (wave w takes k = w, w + 4, ...), four loads in flight per lane, the four partial results combined
// in wave order.
__global__ __launch_bounds__(256) void mid_reduce_split_kernel(const RowParams p, int64_t outer, int64_t R, int64_t inner) {
  __shared__ float part[4][64];
  const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
  const int64_t chunks = (inner + 63) / 64;
  const int64_t b = blockIdx.x / chunks, i = (blockIdx.x % chunks) * 64 + lane;
  const float init = p.kind == LLC_REDUCE_SUM ? 0.0f : (p.kind == LLC_REDUCE_MAX ? -INFINITY : INFINITY);
  auto combine = [&](float a, float v) {
    return p.kind == LLC_REDUCE_SUM ? a + v : (p.kind == LLC_REDUCE_MAX ? nmax(a, v) : nmin(a, v));
  };
  float r = init;
  if (i < inner) {
    const int64_t base = b * R * inner + i;
    int64_t k = wave;
    for (; k + 12 < R; k += 16) {
      float v[4][1];
#pragma unroll
      for (int u = 0; u < 4; ++u) load_row_vec<1>(p.x, p.dtype, base + (k + 4 * u) * inner, v[u]);
#pragma unroll
      for (int u = 0; u < 4; ++u) r = combine(r, v[u][0]);
    }
    for (; k < R; k += 4) {
      float v[1];
      load_row_vec<1>(p.x, p.dtype, base + k * inner, v);
      r = combine(r, v[0]);
    }
  }
  part[wave][lane] = r;
  __syncthreads();
  if (wave == 0 && i < inner) {
    r = combine(combine(part[0][lane], part[1][lane]), combine(part[2][lane], part[3][lane]));
    if (p.kind == LLC_REDUCE_SUM) r *= p.scale;
    float one[1] = {r};
    store_row_vec<1>(p.y, p.dtype, b * inner + i, one);
  }
}

template <int OP, int VEC, int TPR>
void launch_items(const RowParams& p, int items, hipStream_t s) {
  const int rpb = 256 / TPR;
  const unsigned blocks = (unsigned)((p.rows + rpb - 1) / rpb);
  switch (items) {
    case 1: hipLaunchKernelGGL((row_kernel<OP, VEC, TPR, 1>), dim3(blocks), dim3(256), 0, s, p); break;
    case 2: hipLaunchKernelGGL((row_kernel<OP, VEC, TPR, 2>), dim3(blocks), dim3(256), 0, s, p); break;
    case 3: hipLaunchKernelGGL((row_kernel<OP, VEC, TPR, 3>), dim3(blocks), dim3(256), 0, s, p); break;
    case 4: hipLaunchKernelGGL((row_kernel<OP, VEC, TPR, 4>), dim3(blocks), dim3(256), 0, s, p); break;
    case 6: hipLaunchKernelGGL((row_kernel<OP, VEC, TPR, 6>), dim3(blocks), dim3(256), 0, s, p); break;
    case 8: hipLaunchKernelGGL((row_kernel<OP, VEC, TPR, 8>), dim3(blocks), dim3(256), 0, s, p); break;
    default: hipLaunchKernelGGL((row_kernel<OP, VEC, TPR, 16>), dim3(blocks), dim3(256), 0, s, p); break;
  }
}

// The register tile for rows of p.cols elements read VEC wide: lanes per row and vectors per lane; false if no tile
// holds a row.
template <int VEC>
bool pick_tile(const RowParams& p, int* tpr, int* vectors) {
  // smallest register tile that holds a row; among equal capacities prefer 4 then 2 vectors per
  // lane (enough loads in flight per lane, rows spread over many lanes), then 3 and 6 (rows of 3 x 2^n
  // elements, a transformer's 768, fit them exactly: no masked lanes), then 8, then 1
  const int tprs[4] = {16, 32, 64, 256};
  const int items[6] = {4, 2, 3, 6, 8, 1};
  int best_t = 0, best_i = 0;
  int64_t best_cap = -1;
  for (int i : items)
    for (int t : tprs) {
      // six vectors on each of 16 lanes: few lanes per row, worth it only with rows enough to fill the chip anyway
      // (768 bf16 elements: 16384 rows 14.6 -> 13.3 us, 4096 rows 5.3 -> 5.6 us, 512 rows 3.8 -> 4.9 us)
      if (i == 6 && t == 16 && p.rows < 8192) continue;
      if (t == 32 && i != 3 && i != 4) continue;  // 32 lanes: measured with three and four vectors only
      int64_t cap = (int64_t)t * i * VEC;
      if (cap >= p.cols && (best_cap < 0 || cap < best_cap)) {
        best_cap = cap;
        best_t = t;
        best_i = i;
      }
    }
  *tpr = best_t;
  *vectors = best_i;
  return best_cap >= 0;
}

template <int OP, int VEC>
bool launch_tpr(const RowParams& p, hipStream_t s) {
  int best_t, best_i;
  if (!pick_tile<VEC>(p, &best_t, &best_i)) return false;
  if (best_t == 16) launch_items<OP, VEC, 16>(p, best_i, s);
  else if (best_t == 32) launch_items<OP, VEC, 32>(p, best_i, s);
  else if (best_t == 64) launch_items<OP, VEC, 64>(p, best_i, s);
  else launch_items<OP, VEC, 256>(p, best_i, s);
  return true;
}

template <int OP, int DT, int TPR, bool NT>
void launch_typed_items(const RowParams& p, int items, hipStream_t s) {
  const int64_t rpb = 256 / TPR;
  const dim3 grid((unsigned)((p.rows + rpb - 1) / rpb));
  switch (items) {
    case 1: hipLaunchKernelGGL((row_typed_kernel<OP, DT, TPR, 1, NT>), grid, dim3(256), 0, s, p); break;
    case 2: hipLaunchKernelGGL((row_typed_kernel<OP, DT, TPR, 2, NT>), grid, dim3(256), 0, s, p); break;
    case 3: hipLaunchKernelGGL((row_typed_kernel<OP, DT, TPR, 3, NT>), grid, dim3(256), 0, s, p); break;
    case 4: hipLaunchKernelGGL((row_typed_kernel<OP, DT, TPR, 4, NT>), grid, dim3(256), 0, s, p); break;
    case 6: hipLaunchKernelGGL((row_typed_kernel<OP, DT, TPR, 6, NT>), grid, dim3(256), 0, s, p); break;
    default: hipLaunchKernelGGL((row_typed_kernel<OP, DT, TPR, 8, NT>), grid, dim3(256), 0, s, p); break;
  }
}
template <int OP, int DT, int TPR>
void launch_typed_nt(const RowParams& p, int items, hipStream_t s) {
  if (p.streaming) launch_typed_items<OP, DT, TPR, true>(p, items, s);
  else launch_typed_items<OP, DT, TPR, false>(p, items, s);
}

// Rows read 16 bytes wide on the kernel compiled for their storage type; false: no tile of up to eight vectors per lane
// holds a row.
template <int OP, int DT>
bool launch_typed(const RowParams& p, hipStream_t s) {
  int t, i;
  const bool ok = DT == LLC_FLOAT32 ? pick_tile<4>(p, &t, &i) : pick_tile<8>(p, &t, &i);
  if (!ok || i > 8) return false;
  if (t == 16) launch_typed_nt<OP, DT, 16>(p, i, s);
  else if (t == 32) launch_typed_nt<OP, DT, 32>(p, i, s);
  else if (t == 64) launch_typed_nt<OP, DT, 64>(p, i, s);
  else launch_typed_nt<OP, DT, 256>(p, i, s);
  return true;
}

template <int OP>
int launch_rows(const RowParams& p0, hipStream_t s) {
  RowParams p = p0;
  if (p.rows == 0 || p.cols == 0) return LLC_OK;
  p.streaming = p.rows * (int64_t)p.cols * (p.dtype == LLC_FLOAT32 ? 4 : 2) >= ((int64_t)16 << 20) ? 1 : 0;
  if (p.rows > 0x7fffffff) return set_error(LLC_ERR_TOO_LARGE, "row kernel: %lld rows", (long long)p.rows);
  const int es = p.dtype == LLC_FLOAT32 ? 4 : 2;
  const int wide = 16 / es;
  auto al = [&](const void* q) { return q == nullptr || ((uintptr_t)q % 16) == 0; };
  bool vec_ok = (p.cols % wide) == 0 && al(p.x) && (OP == kReduce || al(p.y)) && al(p.gamma) && al(p.beta);
  bool done = false;
  if constexpr (OP == kSoftmax || OP == kLayerNorm) {
    if (vec_ok && (OP == kSoftmax || (p.gamma && p.beta)))
      done = p.dtype == LLC_FLOAT32    ? launch_typed<OP, LLC_FLOAT32>(p, s)
             : p.dtype == LLC_BFLOAT16 ? launch_typed<OP, LLC_BFLOAT16>(p, s)
                                       : launch_typed<OP, LLC_FLOAT16>(p, s);
  }
  if (vec_ok && !done) done = es == 4 ? launch_tpr<OP, 4>(p, s) : launch_tpr<OP, 8>(p, s);
  if (!done && p.cols <= 2048) done = launch_tpr<OP, 1>(p, s);
  if (!done) hipLaunchKernelGGL((row_loop_kernel<OP>), dim3((unsigned)p.rows), dim3(256), 0, s, p);
  return check_launch("row_kernel");
}

int row_dtype_ok(const View& v, const char* what) {
  if (v.dtype != LLC_FLOAT32 && v.dtype != LLC_BFLOAT16 && v.dtype != LLC_FLOAT16)
    return set_error(LLC_ERR_DTYPE, "%s: element type %d (f32, bf16 or f16 expected)", what, v.dtype);
  return LLC_OK;
}

}  // namespace
}  // namespace llc

using namespace llc;

int llc_impl_softmax(const llc_tensor* x, llc_tensor* out, void* stream) {
  View a, o;
  LLC_TRY(make_view(x, "softmax input", &a));
  LLC_TRY(make_view(out, "softmax output", &o));
  LLC_TRY(row_dtype_ok(a, "softmax"));
  if (a.dtype != o.dtype) return set_error(LLC_ERR_DTYPE, "softmax: input and output types differ");
  if (a.rank < 1 || a.rank != o.rank) return set_error(LLC_ERR_SHAPE, "softmax: rank mismatch");
  for (int d = 0; d < a.rank; ++d)
    if (a.size[d] != o.size[d]) return set_error(LLC_ERR_SHAPE, "softmax: extent mismatch at dim %d", d);
  if (!a.contiguous() || !o.contiguous()) return set_error(LLC_ERR_LAYOUT, "softmax: contiguous tensors expected");
  RowParams p{};
  p.x = a.ptr;
  p.y = o.ptr;
  p.dtype = a.dtype;
  p.cols = (int32_t)a.size[a.rank - 1];
  if (a.size[a.rank - 1] >= (int64_t)1 << 31) return set_error(LLC_ERR_TOO_LARGE, "softmax: row too long");
  p.rows = p.cols ? a.numel() / p.cols : 0;
  return launch_rows<kSoftmax>(p, as_stream(stream));
}

int llc_impl_layer_norm(const llc_tensor* x, const llc_tensor* scale, const llc_tensor* bias, double epsilon,
                                  llc_tensor* out, void* stream) {
  View a, o, g, b;
  LLC_TRY(make_view(x, "layer_norm input", &a));
  LLC_TRY(make_view(out, "layer_norm output", &o));
  LLC_TRY(row_dtype_ok(a, "layer_norm"));
  if (a.dtype != o.dtype) return set_error(LLC_ERR_DTYPE, "layer_norm: input and output types differ");
  if (a.rank < 1 || a.rank != o.rank) return set_error(LLC_ERR_SHAPE, "layer_norm: rank mismatch");
  for (int d = 0; d < a.rank; ++d)
    if (a.size[d] != o.size[d]) return set_error(LLC_ERR_SHAPE, "layer_norm: extent mismatch at dim %d", d);
  if (!a.contiguous() || !o.contiguous()) return set_error(LLC_ERR_LAYOUT, "layer_norm: contiguous tensors expected");
  RowParams p{};
  const int64_t cols = a.size[a.rank - 1];
  if (cols >= (int64_t)1 << 31) return set_error(LLC_ERR_TOO_LARGE, "layer_norm: row too long");
  if (scale) {
    LLC_TRY(make_view(scale, "layer_norm scale", &g));
    if (g.dtype != a.dtype) return set_error(LLC_ERR_DTYPE, "layer_norm: scale type differs from input");
    if (g.numel() != cols || !g.contiguous()) return set_error(LLC_ERR_SHAPE, "layer_norm: scale must hold %lld contiguous values", (long long)cols);
    p.gamma = g.ptr;
  }
  if (bias) {
    LLC_TRY(make_view(bias, "layer_norm bias", &b));
    if (b.dtype != a.dtype) return set_error(LLC_ERR_DTYPE, "layer_norm: bias type differs from input");
    if (b.numel() != cols || !b.contiguous()) return set_error(LLC_ERR_SHAPE, "layer_norm: bias must hold %lld contiguous values", (long long)cols);
    p.beta = b.ptr;
  }
  p.x = a.ptr;
  p.y = o.ptr;
  p.dtype = a.dtype;
  p.cols = (int32_t)cols;
  p.rows = cols ? a.numel() / cols : 0;
  p.eps = (float)epsilon;
  return launch_rows<kLayerNorm>(p, as_stream(stream));
}

namespace llc {
// [outer, R, inner] reduction used by llc_hip_reduce and the global average pool.
int reduce_3d(const View& a, const View& o, int kind, int64_t outer, int64_t R, int64_t inner, float scale,
              hipStream_t s) {
  RowParams p{};
  p.x = a.ptr;
  p.y = o.ptr;
  p.dtype = a.dtype;
  p.kind = kind;
  p.scale = scale;
  if (outer * inner == 0) return LLC_OK;
  if (R >= (int64_t)1 << 31) return set_error(LLC_ERR_TOO_LARGE, "reduce: %lld reduced elements", (long long)R);
  if (!p.y || (R > 0 && !p.x)) return set_error(LLC_ERR_BAD_ARG, "reduce: null operand with %lld outputs", (long long)(outer * inner));
  // an empty reduction stores the init value: mid_reduce_kernel does that without reading anything (the row
  // kernels return early on empty rows and would leave the output unwritten)
  if (inner == 1 && R > 0) {
    p.rows = outer;
    p.cols = (int32_t)R;
    return launch_rows<kReduce>(p, s);
  }
  const int64_t n = outer * inner;
  if ((n + 255) / 256 > 0x7fffffff) return set_error(LLC_ERR_TOO_LARGE, "reduce: too many outputs");
  if (R >= 8 && n < 512 * 256) {  // under two workgroups per CU at one lane per output
    const int64_t blocks = outer * ((inner + 63) / 64);
    hipLaunchKernelGGL(mid_reduce_split_kernel, dim3((unsigned)blocks), dim3(256), 0, s, p, outer, R, inner);
    return check_launch("mid_reduce_split_kernel");
  }
  hipLaunchKernelGGL(mid_reduce_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, p, outer, R, inner);
  return check_launch("mid_reduce_kernel");
}
}  // namespace llc

int llc_impl_reduce(int kind, const llc_tensor* x, const int64_t* axes, size_t n_axes, llc_tensor* out,
                              void* stream) {
  View a, o;
  LLC_TRY(make_view(x, "reduce input", &a));
  LLC_TRY(make_view(out, "reduce output", &o));
  LLC_TRY(row_dtype_ok(a, "reduce"));
  if (a.dtype != o.dtype) return set_error(LLC_ERR_DTYPE, "reduce: input and output types differ");
  if (kind < LLC_REDUCE_SUM || kind > LLC_REDUCE_MIN) return set_error(LLC_ERR_BAD_ARG, "reduce: kind %d", kind);
  if (n_axes == 0 || !axes) return set_error(LLC_ERR_BAD_ARG, "reduce: no axes");
  if (!a.contiguous() || !o.contiguous()) return set_error(LLC_ERR_LAYOUT, "reduce: contiguous tensors expected");
  bool red[LLC_MAX_RANK] = {false};
  for (size_t i = 0; i < n_axes; ++i) {
    int64_t ax = axes[i] < 0 ? axes[i] + a.rank : axes[i];
    if (ax < 0 || ax >= a.rank) return set_error(LLC_ERR_BAD_ARG, "reduce: axis %lld out of range", (long long)axes[i]);
    red[ax] = true;
  }
  // Runs of adjacent dims with the same role (dims of extent 1 belong to whatever surrounds them): sizes alternate
  // between kept and reduced.
  int64_t run_size[LLC_MAX_RANK + 1];
  bool run_red[LLC_MAX_RANK + 1];
  int runs = 0;
  int64_t kept = 1;
  for (int d = 0; d < a.rank; ++d) {
    if (!red[d]) kept *= a.size[d];
    if (a.size[d] == 1) continue;
    if (runs > 0 && run_red[runs - 1] == red[d]) run_size[runs - 1] *= a.size[d];
    else {
      run_size[runs] = a.size[d];
      run_red[runs] = red[d];
      ++runs;
    }
  }
  if (o.numel() != kept) return set_error(LLC_ERR_SHAPE, "reduce: output holds %lld elements, expected %lld", (long long)o.numel(), (long long)kept);
  int n_red = 0;
  for (int r = 0; r < runs; ++r) n_red += run_red[r] ? 1 : 0;
  hipStream_t s = as_stream(stream);
  if (a.numel() == 0) {
    // some extent is 0: nothing to write when it is a kept one, else every output is the init value
    // (one launch that reads nothing; no partial results, no scratch memory)
    if (kept == 0) return LLC_OK;
    return reduce_3d(a, o, kind, kept, 0, 1, 1.0f, s);
  }
  if (n_red == 0) {
    // every reduced dim has extent 1 (or an extent is 0 and there is nothing to write): the values themselves
    if (kept == 0) return LLC_OK;
    return reduce_3d(a, o, kind, kept, 1, 1, 1.0f, s);
  }
  // One kernel per reduced run, innermost first; partial results of all but the last alternate between the two
  // halves of the scratch buffer.  (Sums are then grouped by run, maxima and minima do not care.)
  const int es = a.dtype == LLC_FLOAT32 ? 4 : 2;
  char* scratch = nullptr;
  size_t half = 0;
  if (n_red > 1) {
    // the largest partial result is what the innermost reduced run leaves: the product of all other runs
    int innermost = -1;
    for (int r = runs - 1; r >= 0 && innermost < 0; --r)
      if (run_red[r]) innermost = r;
    int64_t partial = 1;
    for (int r = 0; r < runs; ++r)
      if (r != innermost) partial *= run_size[r];
    half = ((size_t)partial * es + 255) & ~(size_t)255;
    void* ws = nullptr;
    LLC_TRY(get_workspace(2 * half, &ws, s));
    scratch = (char*)ws;
    if (!scratch) return set_error(LLC_ERR_HIP, "reduce: no scratch memory for %lld partial results", (long long)partial);
  }
  View cur = a;
  int left = n_red, flip = 0;
  for (int r = runs - 1; r >= 0; --r) {
    if (!run_red[r]) continue;
    int64_t outer = 1, inner = 1;
    for (int q = 0; q < r; ++q) outer *= run_size[q];
    for (int q = r + 1; q < runs; ++q) inner *= run_size[q];
    View dst = o;
    if (--left > 0) {
      dst.ptr = scratch + flip * half;
      flip ^= 1;
    }
    LLC_TRY(reduce_3d(cur, dst, kind, outer, run_size[r], inner, 1.0f, s));
    run_size[r] = 1;
    cur = dst;
  }
  return LLC_OK;
}

int llc_impl_global_avg_pool(const llc_tensor* x, llc_tensor* out, void* stream) {
  View a, o;
  LLC_TRY(make_view(x, "global_avg_pool input", &a));
  LLC_TRY(make_view(out, "global_avg_pool output", &o));
  LLC_TRY(row_dtype_ok(a, "global_avg_pool"));
  if (a.dtype != o.dtype) return set_error(LLC_ERR_DTYPE, "global_avg_pool: input and output types differ");
  if (a.rank != 4) return set_error(LLC_ERR_SHAPE, "global_avg_pool: NCHW input expected");
  // a channels-last input ([N][H W][C] in memory) is a reduction over the middle of three runs
  const int64_t C = a.size[1], H = a.size[2], W = a.size[3];
  const bool nhwc = !a.contiguous() && (C == 1 || a.stride[1] == 1) && (W == 1 || a.stride[3] == C) &&
                    (H == 1 || a.stride[2] == W * C) && (a.size[0] == 1 || a.stride[0] == H * W * C);
  if ((!a.contiguous() && !nhwc) || !o.contiguous())
    return set_error(LLC_ERR_LAYOUT, "global_avg_pool: a contiguous or channels-last input and a contiguous output expected");
  const int64_t nc = a.size[0] * a.size[1], hw = a.size[2] * a.size[3];
  if (o.numel() != nc) return set_error(LLC_ERR_SHAPE, "global_avg_pool: output holds %lld elements, expected %lld", (long long)o.numel(), (long long)nc);
  if (hw == 0) return set_error(LLC_ERR_SHAPE, "global_avg_pool: empty window");
  if (nhwc) return reduce_3d(a, o, LLC_REDUCE_SUM, a.size[0], hw, C, 1.0f / (float)hw, as_stream(stream));
  return reduce_3d(a, o, LLC_REDUCE_SUM, nc, hw, 1, 1.0f / (float)hw, as_stream(stream));
}
