// Fused elementwise chains: one launch evaluates a whole chain of LLH elementwise ops.
//
// The chain arrives as a tiny register program (llc_ew_program).  Every lane owns ONE vector of VEC
// consecutive output elements (16 bytes of the output type), loads that vector of every chain input
// first, runs the program on registers and stores once.  The grid covers the output exactly (one
// vector per lane, no grid-stride loop): on this part many small waves keep more memory requests
// in flight than few looping ones.  Large streams use non-temporal loads and stores, which is worth
// ~10% of HBM bandwidth for data that is touched once.  Program control flow is uniform across the
// wave, so instruction decode runs on the scalar unit; the kernel is bound by HBM traffic: bytes
// moved = each distinct input once + the output once.
//
// Broadcast operands (llh.broadcast_to folded into the consumer) are read with stride 0; the host
// collapses the iteration space to at most four dims so that the common cases (same shape, bias
// over the last dim, per-channel NCHW, attention mask) need at most three integer divisions per
// vector.

#include "common.hpp"

namespace llc {
namespace {

constexpr int kMaxDims = 4;

// Everything a wave needs before it can issue its first global load sits in one contiguous block,
// so that it arrives with one wide scalar load instead of a chain of dependent ones.
struct EwHot {
  uint32_t n_vec;           // number of VEC-wide vectors in the output
  int32_t flat;             // 1: every input is either same-shape contiguous or a scalar
  int32_t streaming;        // 1: non-temporal accesses for the full-size operands
  int32_t n_inputs;
  int32_t out_dtype;
  int32_t n_insts;
  int32_t result;
  int32_t integer;
  uint32_t dims[kMaxDims];  // collapsed output extents, dims[3] innermost
  int32_t in_dtype[LLC_EW_MAX_INPUTS];
  int32_t in_inner[LLC_EW_MAX_INPUTS];  // innermost stride: 0 or 1 when VEC > 1
};

struct EwKernelParams {
  EwHot hot;
  char* out;
  const char* in[LLC_EW_MAX_INPUTS];
  int32_t in_stride[LLC_EW_MAX_INPUTS][kMaxDims];  // elements
  llc_ew_inst insts[LLC_EW_MAX_INSTS];
};

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// N bytes, naturally aligned, optionally with the non-temporal hint.  The hint is a template argument: with a run-time
// choice between the two forms of an access the compiler folds them into one plain instruction and the hint is lost.
template <int N>
struct Bytes {
  alignas(N >= 16 ? 16 : N) unsigned char b[N];
};
template <int N, bool NT>
__device__ __forceinline__ Bytes<N> ld_bytes(const char* p) {
  Bytes<N> r;
  if constexpr (N >= 16) {
#pragma unroll
    for (int i = 0; i < N / 16; ++i) {
      u32x4 v;
      if constexpr (NT) v = __builtin_nontemporal_load((const u32x4*)p + i);
      else v = ((const u32x4*)p)[i];
      __builtin_memcpy(r.b + 16 * i, &v, 16);
    }
  } else if constexpr (N == 8) {
    u32x2 v;
    if constexpr (NT) v = __builtin_nontemporal_load((const u32x2*)p);
    else v = *(const u32x2*)p;
    __builtin_memcpy(r.b, &v, 8);
  } else if constexpr (N == 4) {
    uint32_t v;
    if constexpr (NT) v = __builtin_nontemporal_load((const uint32_t*)p);
    else v = *(const uint32_t*)p;
    __builtin_memcpy(r.b, &v, 4);
  } else if constexpr (N == 2) {
    uint16_t v = *(const uint16_t*)p;
    __builtin_memcpy(r.b, &v, 2);
  } else {
    r.b[0] = *(const unsigned char*)p;
  }
  return r;
}
template <int N, bool NT>
__device__ __forceinline__ void st_bytes(char* p, const Bytes<N>& r) {
  if constexpr (N >= 16) {
#pragma unroll
    for (int i = 0; i < N / 16; ++i) {
      u32x4 v;
      __builtin_memcpy(&v, r.b + 16 * i, 16);
      if constexpr (NT) __builtin_nontemporal_store(v, (u32x4*)p + i);
      else ((u32x4*)p)[i] = v;
    }
  } else if constexpr (N == 8) {
    u32x2 v;
    __builtin_memcpy(&v, r.b, 8);
    if constexpr (NT) __builtin_nontemporal_store(v, (u32x2*)p);
    else *(u32x2*)p = v;
  } else if constexpr (N == 4) {
    uint32_t v;
    __builtin_memcpy(&v, r.b, 4);
    if constexpr (NT) __builtin_nontemporal_store(v, (uint32_t*)p);
    else *(uint32_t*)p = v;
  } else if constexpr (N == 2) {
    uint16_t v;
    __builtin_memcpy(&v, r.b, 2);
    *(uint16_t*)p = v;
  } else {
    *(unsigned char*)p = r.b[0];
  }
}

template <typename S, int VEC, bool NT>
__device__ __forceinline__ void ld_elems(const char* base, uint32_t off, S* dst) {
  Bytes<(int)sizeof(S) * VEC> r = ld_bytes<(int)sizeof(S) * VEC, NT>(base + (size_t)off * sizeof(S));
  __builtin_memcpy(dst, r.b, sizeof(S) * VEC);
}
template <typename S, int VEC, bool NT>
__device__ __forceinline__ void st_elems(char* base, uint32_t off, const S* src) {
  Bytes<(int)sizeof(S) * VEC> r;
  __builtin_memcpy(r.b, src, sizeof(S) * VEC);
  st_bytes<(int)sizeof(S) * VEC, NT>(base + (size_t)off * sizeof(S), r);
}

// ---- typed loads: VEC consecutive elements (inner stride 1) or one element repeated (stride 0) ----
template <int VEC, typename CT, bool NT>
__device__ __forceinline__ void load_vec(const char* base, int dtype, uint32_t off, int inner_stride, CT* dst) {
  if (inner_stride == 0) {
    CT v;
    switch (dtype) {
      case LLC_FLOAT32: v = (CT) * (const float*)(base + (size_t)off * 4); break;
      case LLC_BFLOAT16: v = (CT)bf16_bits_to_f32(*(const uint16_t*)(base + (size_t)off * 2)); break;
      case LLC_FLOAT16: v = (CT)f16_bits_to_f32(*(const uint16_t*)(base + (size_t)off * 2)); break;
      case LLC_INT64: v = (CT) * (const int64_t*)(base + (size_t)off * 8); break;
      case LLC_INT32: v = (CT) * (const int32_t*)(base + (size_t)off * 4); break;
      default: v = (CT) * (const uint8_t*)(base + (size_t)off); break;
    }
#pragma unroll
    for (int j = 0; j < VEC; ++j) dst[j] = v;
    return;
  }
  switch (dtype) {
    case LLC_FLOAT32: {
      float t[VEC];
      ld_elems<float, VEC, NT>(base, off, t);
#pragma unroll
      for (int j = 0; j < VEC; ++j) dst[j] = (CT)t[j];
    } break;
    case LLC_BFLOAT16: {
      uint16_t t[VEC];
      ld_elems<uint16_t, VEC, NT>(base, off, t);
#pragma unroll
      for (int j = 0; j < VEC; ++j) dst[j] = (CT)bf16_bits_to_f32(t[j]);
    } break;
    case LLC_FLOAT16: {
      uint16_t t[VEC];
      ld_elems<uint16_t, VEC, NT>(base, off, t);
#pragma unroll
      for (int j = 0; j < VEC; ++j) dst[j] = (CT)f16_bits_to_f32(t[j]);
    } break;
    case LLC_INT64: {
      int64_t t[VEC];
      ld_elems<int64_t, VEC, NT>(base, off, t);
#pragma unroll
      for (int j = 0; j < VEC; ++j) dst[j] = (CT)t[j];
    } break;
    case LLC_INT32: {
      int32_t t[VEC];
      ld_elems<int32_t, VEC, NT>(base, off, t);
#pragma unroll
      for (int j = 0; j < VEC; ++j) dst[j] = (CT)t[j];
    } break;
    default: {
      uint8_t t[VEC];
      ld_elems<uint8_t, VEC, NT>(base, off, t);
#pragma unroll
      for (int j = 0; j < VEC; ++j) dst[j] = (CT)t[j];
    } break;
  }
}

template <int VEC, typename CT, bool NT>
__device__ __forceinline__ void store_vec(char* base, int dtype, uint32_t off, const CT* src) {
  switch (dtype) {
    case LLC_FLOAT32: {
      float t[VEC];
#pragma unroll
      for (int j = 0; j < VEC; ++j) t[j] = (float)src[j];
      st_elems<float, VEC, NT>(base, off, t);
    } break;
    case LLC_BFLOAT16: {
      uint16_t t[VEC];
#pragma unroll
      for (int j = 0; j < VEC; ++j) t[j] = f32_to_bf16_bits((float)src[j]);
      st_elems<uint16_t, VEC, NT>(base, off, t);
    } break;
    case LLC_FLOAT16: {
      uint16_t t[VEC];
#pragma unroll
      for (int j = 0; j < VEC; ++j) t[j] = f32_to_f16_bits((float)src[j]);
      st_elems<uint16_t, VEC, NT>(base, off, t);
    } break;
    case LLC_INT64: {
      int64_t t[VEC];
#pragma unroll
      for (int j = 0; j < VEC; ++j) t[j] = (int64_t)src[j];
      st_elems<int64_t, VEC, NT>(base, off, t);
    } break;
    case LLC_INT32: {
      int32_t t[VEC];
#pragma unroll
      for (int j = 0; j < VEC; ++j) t[j] = (int32_t)src[j];
      st_elems<int32_t, VEC, NT>(base, off, t);
    } break;
    case LLC_INT1: {
      uint8_t t[VEC];
#pragma unroll
      for (int j = 0; j < VEC; ++j) t[j] = src[j] != (CT)0 ? 1 : 0;
      st_elems<uint8_t, VEC, NT>(base, off, t);
    } break;
    default: {
      uint8_t t[VEC];
#pragma unroll
      for (int j = 0; j < VEC; ++j) t[j] = (uint8_t)(int8_t)src[j];
      st_elems<uint8_t, VEC, NT>(base, off, t);
    } break;
  }
}

// NaN-propagating max/min, like stablehlo.maximum and torch.maximum
__device__ __forceinline__ float nanmax(float a, float b) { return (a > b || a != a) ? a : b; }
__device__ __forceinline__ float nanmin(float a, float b) { return (a < b || a != a) ? a : b; }
__device__ __forceinline__ int64_t nanmax(int64_t a, int64_t b) { return a > b ? a : b; }
__device__ __forceinline__ int64_t nanmin(int64_t a, int64_t b) { return a < b ? a : b; }

#define LLC_EW_CASE(OP, EXPR)          \
  case OP:                             \
    _Pragma("unroll") for (int j = 0; j < E; ++j) { \
      const CT a = av[j], b = bv[j], c = cv[j];     \
      (void)a; (void)b; (void)c;                    \
      dv[j] = (EXPR);                               \
    }                                               \
    break;

// The opcode is wave-uniform: one scalar branch selects a fully unrolled loop over the lane's elements.
template <int E>
__device__ __forceinline__ void apply_all(int op, const float* av, const float* bv, const float* cv, float* dv) {
  using CT = float;
  switch (op) {
    LLC_EW_CASE(LLC_EW_ABS, fabsf(a))
    LLC_EW_CASE(LLC_EW_SQRT, sqrtf(a))
    LLC_EW_CASE(LLC_EW_EXP, expf(a))
    LLC_EW_CASE(LLC_EW_RELU, a < 0.0f ? 0.0f : a)  // NaN passes through, like torch.relu
    LLC_EW_CASE(LLC_EW_RSQRT, 1.0f / sqrtf(a))
    LLC_EW_CASE(LLC_EW_NEG, -a)
    LLC_EW_CASE(LLC_EW_GELU, gelu_exact(a))
    LLC_EW_CASE(LLC_EW_TANH, tanhf(a))
    LLC_EW_CASE(LLC_EW_ERF, erff(a))
    LLC_EW_CASE(LLC_EW_SIGMOID, 1.0f / (1.0f + expf(-a)))
    LLC_EW_CASE(LLC_EW_LOG, logf(a))
    LLC_EW_CASE(LLC_EW_RECIP, 1.0f / a)
    LLC_EW_CASE(LLC_EW_MOV, a)
    LLC_EW_CASE(LLC_EW_ADD, a + b)
    LLC_EW_CASE(LLC_EW_SUB, a - b)
    LLC_EW_CASE(LLC_EW_MUL, a * b)
    LLC_EW_CASE(LLC_EW_DIV, a / b)
    LLC_EW_CASE(LLC_EW_MAX, nanmax(a, b))
    LLC_EW_CASE(LLC_EW_MIN, nanmin(a, b))
    LLC_EW_CASE(LLC_EW_POW, powf(a, b))
    LLC_EW_CASE(LLC_EW_CMP_EQ, a == b ? 1.0f : 0.0f)
    LLC_EW_CASE(LLC_EW_CMP_NE, a != b ? 1.0f : 0.0f)
    LLC_EW_CASE(LLC_EW_CMP_GE, a >= b ? 1.0f : 0.0f)
    LLC_EW_CASE(LLC_EW_CMP_GT, a > b ? 1.0f : 0.0f)
    LLC_EW_CASE(LLC_EW_CMP_LE, a <= b ? 1.0f : 0.0f)
    LLC_EW_CASE(LLC_EW_CMP_LT, a < b ? 1.0f : 0.0f)
    LLC_EW_CASE(LLC_EW_WHERE, a != 0.0f ? b : c)
    default: break;
  }
}
// floor division, matching torch for integer tensors
__device__ __forceinline__ int64_t floordiv(int64_t a, int64_t b) {
  if (b == 0) return 0;
  int64_t q = a / b;
  if ((a % b != 0) && ((a < 0) != (b < 0))) --q;
  return q;
}
template <int E>
__device__ __forceinline__ void apply_all(int op, const int64_t* av, const int64_t* bv, const int64_t* cv, int64_t* dv) {
  using CT = int64_t;
  switch (op) {
    LLC_EW_CASE(LLC_EW_ABS, a < 0 ? -a : a)
    LLC_EW_CASE(LLC_EW_RELU, a > 0 ? a : 0)
    LLC_EW_CASE(LLC_EW_NEG, -a)
    LLC_EW_CASE(LLC_EW_MOV, a)
    LLC_EW_CASE(LLC_EW_ADD, a + b)
    LLC_EW_CASE(LLC_EW_SUB, a - b)
    LLC_EW_CASE(LLC_EW_MUL, a * b)
    LLC_EW_CASE(LLC_EW_DIV, floordiv(a, b))
    LLC_EW_CASE(LLC_EW_MAX, nanmax(a, b))
    LLC_EW_CASE(LLC_EW_MIN, nanmin(a, b))
    LLC_EW_CASE(LLC_EW_CMP_EQ, (int64_t)(a == b))
    LLC_EW_CASE(LLC_EW_CMP_NE, (int64_t)(a != b))
    LLC_EW_CASE(LLC_EW_CMP_GE, (int64_t)(a >= b))
    LLC_EW_CASE(LLC_EW_CMP_GT, (int64_t)(a > b))
    LLC_EW_CASE(LLC_EW_CMP_LE, (int64_t)(a <= b))
    LLC_EW_CASE(LLC_EW_CMP_LT, (int64_t)(a < b))
    LLC_EW_CASE(LLC_EW_WHERE, a != 0 ? b : c)
    default: break;
  }
}
#undef LLC_EW_CASE

template <int E, typename CT>
struct RegFile {
  CT r0[E], r1[E], r2[E], r3[E];
  CT i0[E], i1[E], i2[E], i3[E], i4[E], i5[E];
};

#define LLC_COPY(DST, SRC) \
  _Pragma("unroll") for (int j = 0; j < E; ++j) (DST)[j] = (SRC)[j]

// Selector decode is wave-uniform: the switch compiles to scalar branches around register copies.
// Every array is named explicitly (no pointer to a run-time chosen array), so the register file
// stays in VGPRs.
template <int E, int MAXIN, typename CT>
__device__ __forceinline__ void fetch(const RegFile<E, CT>& f, int sel, CT imm, CT* dst) {
  if constexpr (MAXIN > 2) {
    switch (sel) {
      case LLC_EW_IN0 + 2: LLC_COPY(dst, f.i2); return;
      case LLC_EW_IN0 + 3: LLC_COPY(dst, f.i3); return;
      case LLC_EW_IN0 + 4: LLC_COPY(dst, f.i4); return;
      case LLC_EW_IN0 + 5: LLC_COPY(dst, f.i5); return;
      default: break;
    }
  }
  switch (sel) {
    case 0: LLC_COPY(dst, f.r0); break;
    case 1: LLC_COPY(dst, f.r1); break;
    case 2: LLC_COPY(dst, f.r2); break;
    case 3: LLC_COPY(dst, f.r3); break;
    case LLC_EW_IN0 + 0: LLC_COPY(dst, f.i0); break;
    case LLC_EW_IN0 + 1: LLC_COPY(dst, f.i1); break;
    default:
#pragma unroll
      for (int j = 0; j < E; ++j) dst[j] = imm;
      break;
  }
}

template <int VEC, int U, int MAXIN, typename CT, bool NT>
__global__ __launch_bounds__(256) void ew_kernel(const EwKernelParams p) {
  constexpr int E = VEC * U;
  const EwHot h = p.hot;
  // block b owns vectors [b*256*U, (b+1)*256*U); slot u of a lane is vector b*256*U + u*256 + lane
  const uint32_t v0 = blockIdx.x * (256u * U) + threadIdx.x;
  if (v0 >= h.n_vec) return;
  RegFile<E, CT> f;
  // ---- phase 1: issue every load ----
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const uint32_t v = v0 + u * 256u;
    if (U > 1 && v >= h.n_vec) break;
    const uint32_t e = v * VEC;
    uint32_t idx0 = 0, idx1 = 0, idx2 = 0, idx3 = e;
    if (!h.flat) {
      uint32_t t = e;
      idx3 = t % h.dims[3];
      t /= h.dims[3];
      idx2 = t % h.dims[2];
      t /= h.dims[2];
      idx1 = t % h.dims[1];
      idx0 = t / h.dims[1];
    }
#define LLC_LOAD_INPUT(K, ARR)                                                                          \
  if (K < MAXIN && K < h.n_inputs) {                                                                    \
    uint32_t off = idx3 * (uint32_t)h.in_inner[K];                                                      \
    if (!h.flat)                                                                                        \
      off += idx0 * (uint32_t)p.in_stride[K][0] + idx1 * (uint32_t)p.in_stride[K][1] +                  \
             idx2 * (uint32_t)p.in_stride[K][2];                                                        \
    load_vec<VEC, CT, NT>(p.in[K], h.in_dtype[K], off, h.in_inner[K], &ARR[u * VEC]);                   \
  }
    LLC_LOAD_INPUT(0, f.i0)
    LLC_LOAD_INPUT(1, f.i1)
    LLC_LOAD_INPUT(2, f.i2)
    LLC_LOAD_INPUT(3, f.i3)
    LLC_LOAD_INPUT(4, f.i4)
    LLC_LOAD_INPUT(5, f.i5)
#undef LLC_LOAD_INPUT
  }
  // ---- phase 2: run the chain on registers ----
  for (int i = 0; i < h.n_insts; ++i) {
    const llc_ew_inst inst = p.insts[i];
    CT a[E], b[E], c[E], d[E];
    const CT imm = (CT)inst.imm;
    fetch<E, MAXIN, CT>(f, inst.a, imm, a);
    if (inst.op >= LLC_EW_ADD) fetch<E, MAXIN, CT>(f, inst.b, imm, b);
    if (inst.op == LLC_EW_WHERE) fetch<E, MAXIN, CT>(f, inst.c, imm, c);
    apply_all<E>(inst.op, a, b, c, d);
    switch (inst.dst) {
      case 0: LLC_COPY(f.r0, d); break;
      case 1: LLC_COPY(f.r1, d); break;
      case 2: LLC_COPY(f.r2, d); break;
      default: LLC_COPY(f.r3, d); break;
    }
  }
  // ---- phase 3: store ----
  CT res[E];
  fetch<E, MAXIN, CT>(f, h.result, (CT)0, res);
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const uint32_t v = v0 + u * 256u;
    if (v < h.n_vec) store_vec<VEC, CT, NT>(p.out, h.out_dtype, v * VEC, res + u * VEC);
  }
}
#undef LLC_COPY

// ---------------------------------------------------------------------------------------------
// Linear chains.  Most fused groups are a straight line: a running value that each op combines with
// an input, an immediate or itself (add+relu, bias+gelu, scale+mask, ...).  For those the host
// rewrites the program into accumulator form, "acc = op(acc, x)", with the input that seeds acc moved
// to slot 0, and this kernel runs it without a register file: acc and up to three other inputs live
// in named registers, an immediate is used as a scalar operand, and no operand is copied.  That
// cuts the vector instructions per element severalfold, which is what bounds a 16-bit stream.
enum { kKindNone = 0, kKindImm = 1, kKindAcc = 2, kKindIn1 = 3 };  // kKindIn1 + k: input slot 1 + k
enum { kOpRSub = 23, kOpRDiv = 24, kOpRPow = 25 };                 // operand order swapped: x op acc

#define LLC_CH_CASE(OP, EXPR)                         \
  case OP:                                            \
    _Pragma("unroll") for (int j = 0; j < E; ++j) {   \
      const float a = acc[j], b = LLC_CH_B;           \
      (void)b;                                        \
      acc[j] = (EXPR);                                \
    }                                                 \
    break;
template <int E>
__device__ __forceinline__ void chain_unary(int op, float* acc) {
#define LLC_CH_B 0.0f
  switch (op) {
    LLC_CH_CASE(LLC_EW_ABS, fabsf(a))
    LLC_CH_CASE(LLC_EW_SQRT, sqrtf(a))
    LLC_CH_CASE(LLC_EW_EXP, expf(a))
    LLC_CH_CASE(LLC_EW_RELU, a < 0.0f ? 0.0f : a)
    LLC_CH_CASE(LLC_EW_RSQRT, 1.0f / sqrtf(a))
    LLC_CH_CASE(LLC_EW_NEG, -a)
    LLC_CH_CASE(LLC_EW_GELU, gelu_exact(a))
    LLC_CH_CASE(LLC_EW_TANH, tanhf(a))
    LLC_CH_CASE(LLC_EW_ERF, erff(a))
    LLC_CH_CASE(LLC_EW_SIGMOID, 1.0f / (1.0f + expf(-a)))
    LLC_CH_CASE(LLC_EW_LOG, logf(a))
    LLC_CH_CASE(LLC_EW_RECIP, 1.0f / a)
    default: break;  // LLC_EW_MOV
  }
#undef LLC_CH_B
}
#define LLC_CH_BINARY_CASES                                   \
    LLC_CH_CASE(LLC_EW_ADD, a + b)                            \
    LLC_CH_CASE(LLC_EW_SUB, a - b)                            \
    LLC_CH_CASE(kOpRSub, b - a)                               \
    LLC_CH_CASE(LLC_EW_MUL, a * b)                            \
    LLC_CH_CASE(LLC_EW_DIV, a / b)                            \
    LLC_CH_CASE(kOpRDiv, b / a)                               \
    LLC_CH_CASE(LLC_EW_MAX, nanmax(a, b))                     \
    LLC_CH_CASE(LLC_EW_MIN, nanmin(a, b))                     \
    LLC_CH_CASE(LLC_EW_POW, powf(a, b))                       \
    LLC_CH_CASE(kOpRPow, powf(b, a))                          \
    LLC_CH_CASE(LLC_EW_CMP_EQ, a == b ? 1.0f : 0.0f)          \
    LLC_CH_CASE(LLC_EW_CMP_NE, a != b ? 1.0f : 0.0f)          \
    LLC_CH_CASE(LLC_EW_CMP_GE, a >= b ? 1.0f : 0.0f)          \
    LLC_CH_CASE(LLC_EW_CMP_GT, a > b ? 1.0f : 0.0f)           \
    LLC_CH_CASE(LLC_EW_CMP_LE, a <= b ? 1.0f : 0.0f)          \
    LLC_CH_CASE(LLC_EW_CMP_LT, a < b ? 1.0f : 0.0f)
template <int E>
__device__ __forceinline__ void chain_binary(int op, float* acc, const float* x) {
#define LLC_CH_B x[j]
  switch (op) {
    LLC_CH_BINARY_CASES
    default: break;
  }
#undef LLC_CH_B
}
template <int E>
__device__ __forceinline__ void chain_binary_imm(int op, float* acc, float imm) {
#define LLC_CH_B imm
  switch (op) {
    LLC_CH_BINARY_CASES
    default: break;
  }
#undef LLC_CH_B
}
#undef LLC_CH_CASE
#undef LLC_CH_BINARY_CASES

// insts[i]: op (with the swapped forms above), b = operand kind, imm
template <int VEC, int NIN, bool NT>
__global__ __launch_bounds__(256) void ew_chain_kernel(const EwKernelParams p) {
  constexpr int E = VEC;
  const EwHot h = p.hot;
  const uint32_t v = blockIdx.x * 256u + threadIdx.x;
  if (v >= h.n_vec) return;
  const uint32_t e = v * VEC;
  uint32_t idx0 = 0, idx1 = 0, idx2 = 0, idx3 = e;
  if (!h.flat) {
    uint32_t t = e;
    idx3 = t % h.dims[3];
    t /= h.dims[3];
    idx2 = t % h.dims[2];
    t /= h.dims[2];
    idx1 = t % h.dims[1];
    idx0 = t / h.dims[1];
  }
  float acc[E], x1[E], x2[E], x3[E];
#define LLC_LOAD_INPUT(K, ARR)                                                                          \
  if (K < NIN && K < h.n_inputs) {                                                                      \
    uint32_t off = idx3 * (uint32_t)h.in_inner[K];                                                      \
    if (!h.flat)                                                                                        \
      off += idx0 * (uint32_t)p.in_stride[K][0] + idx1 * (uint32_t)p.in_stride[K][1] +                  \
             idx2 * (uint32_t)p.in_stride[K][2];                                                        \
    load_vec<VEC, float, NT>(p.in[K], h.in_dtype[K], off, h.in_inner[K], ARR);                          \
  }
  LLC_LOAD_INPUT(0, acc)
  LLC_LOAD_INPUT(1, x1)
  LLC_LOAD_INPUT(2, x2)
  LLC_LOAD_INPUT(3, x3)
#undef LLC_LOAD_INPUT
  for (int i = 0; i < h.n_insts; ++i) {
    const int op = p.insts[i].op, kind = p.insts[i].b;
    switch (kind) {
      case kKindNone: chain_unary<E>(op, acc); break;
      case kKindImm: chain_binary_imm<E>(op, acc, p.insts[i].imm); break;
      case kKindAcc: chain_binary<E>(op, acc, acc); break;
      case kKindIn1: if constexpr (NIN > 1) chain_binary<E>(op, acc, x1); break;
      case kKindIn1 + 1: if constexpr (NIN > 2) chain_binary<E>(op, acc, x2); break;
      default: if constexpr (NIN > 2) chain_binary<E>(op, acc, x3); break;
    }
  }
  store_vec<VEC, float, NT>(p.out, h.out_dtype, e, acc);
}

// The chain kernel for the plain case: every operand and the result are contiguous tensors of one floating storage type DT
// and move 16 bytes per lane.  ew_chain_kernel picks the storage type of each operand in a switch, and a value a switch
// defines must have arrived where the switch ends: its operands travel one after the other.  Here the NIN loads leave
// back to back (operands beyond the program's own repeat operand 0 and are ignored), then the chain runs.
template <int DT, int NIN, bool NT>
__global__ __launch_bounds__(256) void ew_chain_typed_kernel(const EwKernelParams p) {
  // one vector per lane: two and four per lane were slower at every size (64 Mi fp32 elements 124 | 130 | 127 us)
  constexpr int E = DT == LLC_FLOAT32 ? 4 : 8;
  const EwHot h = p.hot;
  const uint32_t v = blockIdx.x * 256u + threadIdx.x;
  if (v >= h.n_vec) return;
  u32x4 raw[NIN];
#pragma unroll
  for (int k = 0; k < NIN; ++k) {
    const u32x4* src = (const u32x4*)p.in[k < h.n_inputs ? k : 0] + v;
    if constexpr (NT) raw[k] = __builtin_nontemporal_load(src);
    else raw[k] = *src;
  }
  float acc[E], x[NIN > 1 ? NIN - 1 : 1][E];
  unpack_typed<DT>(raw[0], acc);
#pragma unroll
  for (int k = 1; k < NIN; ++k) unpack_typed<DT>(raw[k], x[k - 1]);
  for (int i = 0; i < h.n_insts; ++i) {
    const int op = p.insts[i].op, kind = p.insts[i].b;
    switch (kind) {
      case kKindNone: chain_unary<E>(op, acc); break;
      case kKindImm: chain_binary_imm<E>(op, acc, p.insts[i].imm); break;
      case kKindAcc: chain_binary<E>(op, acc, acc); break;
      case kKindIn1: if constexpr (NIN > 1) chain_binary<E>(op, acc, x[0]); break;
      case kKindIn1 + 1: if constexpr (NIN > 2) chain_binary<E>(op, acc, x[1]); break;
      default: if constexpr (NIN > 3) chain_binary<E>(op, acc, x[2]); break;
    }
  }
  u32x4* dst = (u32x4*)p.out + v;
  if constexpr (NT) __builtin_nontemporal_store(pack_typed<DT>(acc), dst);
  else *dst = pack_typed<DT>(acc);
}

// Rewrites a program into accumulator form if it is a straight line.  On success fills chain[] (op, b = kind,
// imm), slot[] (original input index held by each slot) and the counts.
bool linearize(const llc_ew_program* prog, size_t n_inputs, llc_ew_inst* chain, int* n_chain, int* slot, int* n_slots) {
  if (prog->integer || prog->n_insts == 0) return false;
  auto is_in = [&](int s) { return s >= LLC_EW_IN0 && s < LLC_EW_IN0 + (int)n_inputs; };
  auto swapped = [](int op) {
    switch (op) {
      case LLC_EW_SUB: return (int)kOpRSub;
      case LLC_EW_DIV: return (int)kOpRDiv;
      case LLC_EW_POW: return (int)kOpRPow;
      case LLC_EW_CMP_GE: return (int)LLC_EW_CMP_LE;
      case LLC_EW_CMP_LE: return (int)LLC_EW_CMP_GE;
      case LLC_EW_CMP_GT: return (int)LLC_EW_CMP_LT;
      case LLC_EW_CMP_LT: return (int)LLC_EW_CMP_GT;
      default: return op;  // commutative
    }
  };
  *n_slots = 1;
  slot[0] = -1;
  auto slot_of = [&](int input) {  // slots 1.. hold the operands; the seed of acc always has slot 0 to itself
    for (int k = 1; k < *n_slots; ++k)
      if (slot[k] == input) return k;
    if (*n_slots >= 4) return -1;
    slot[*n_slots] = input;
    return (*n_slots)++;
  };
  int cur = -1;  // register that holds acc
  for (int i = 0; i < prog->n_insts; ++i) {
    const llc_ew_inst& in = prog->insts[i];
    llc_ew_inst& o = chain[i];
    o = in;
    if (in.op == LLC_EW_WHERE) return false;
    const bool binary = in.op >= LLC_EW_ADD;
    int a = in.a, b = binary ? in.b : -1;
    auto is_acc = [&](int s) { return i == 0 ? false : s == cur; };
    if (i == 0) {
      // seed: an input operand becomes acc
      if (!is_in(a)) {
        if (!binary || !is_in(b)) return false;
        const int t = a;
        a = b;
        b = t;
        o.op = swapped(in.op);
      }
      slot[0] = a - LLC_EW_IN0;
      if (binary && b == a) b = -2;  // both operands are the seed
    } else {
      if (!is_acc(a)) {
        if (!binary || !is_acc(b)) return false;
        const int t = a;
        a = b;
        b = t;
        o.op = swapped(in.op);
      }
      if (binary && is_acc(b)) b = -2;
    }
    if (!binary) {
      o.b = kKindNone;
    } else if (b == -2) {
      o.b = kKindAcc;
    } else if (b == LLC_EW_IMM) {
      o.b = kKindImm;
    } else if (is_in(b)) {
      const int k = slot_of(b - LLC_EW_IN0);
      if (k < 0) return false;
      o.b = kKindIn1 + (k - 1);
    } else {
      return false;  // an older register: not a straight line
    }
    cur = in.dst;
  }
  if (prog->result != cur) return false;
  *n_chain = prog->n_insts;
  return true;
}

bool float_compute_dtype(int t) {
  return t == LLC_FLOAT32 || t == LLC_BFLOAT16 || t == LLC_FLOAT16 || t == LLC_INT64 || t == LLC_INT32 ||
         t == LLC_INT1 || t == LLC_INT8;
}

int validate_program(const llc_ew_program* prog, size_t n_inputs) {
  if (prog->n_insts < 0 || prog->n_insts > LLC_EW_MAX_INSTS)
    return set_error(LLC_ERR_BAD_ARG, "elementwise: %d instructions (max %d)", prog->n_insts, LLC_EW_MAX_INSTS);
  auto sel_ok = [&](int s) {
    return (s >= 0 && s < LLC_EW_MAX_REGS) || (s >= LLC_EW_IN0 && s < LLC_EW_IN0 + (int)n_inputs) || s == LLC_EW_IMM;
  };
  for (int i = 0; i < prog->n_insts; ++i) {
    const llc_ew_inst& in = prog->insts[i];
    bool known = (in.op >= LLC_EW_ABS && in.op <= LLC_EW_RECIP) || in.op == LLC_EW_MOV ||
                 (in.op >= LLC_EW_ADD && in.op <= LLC_EW_POW) || (in.op >= LLC_EW_CMP_EQ && in.op <= LLC_EW_CMP_NE) ||
                 in.op == LLC_EW_WHERE;
    if (!known) return set_error(LLC_ERR_BAD_ARG, "elementwise: instruction %d has unknown opcode %d", i, in.op);
    if (in.dst < 0 || in.dst >= LLC_EW_MAX_REGS)
      return set_error(LLC_ERR_BAD_ARG, "elementwise: instruction %d writes register %d", i, in.dst);
    if (!sel_ok(in.a) || (in.op >= LLC_EW_ADD && !sel_ok(in.b)) || (in.op == LLC_EW_WHERE && !sel_ok(in.c)))
      return set_error(LLC_ERR_BAD_ARG, "elementwise: instruction %d has a bad operand selector", i);
    if (prog->integer) {
      bool int_ok = in.op == LLC_EW_ABS || in.op == LLC_EW_RELU || in.op == LLC_EW_NEG || in.op == LLC_EW_MOV ||
                    (in.op >= LLC_EW_ADD && in.op <= LLC_EW_MIN) || (in.op >= LLC_EW_CMP_EQ && in.op <= LLC_EW_CMP_NE) ||
                    in.op == LLC_EW_WHERE;
      if (!int_ok) return set_error(LLC_ERR_UNSUPPORTED, "elementwise: opcode %d has no int64 form", in.op);
    }
  }
  if (!sel_ok(prog->result)) return set_error(LLC_ERR_BAD_ARG, "elementwise: bad result selector %d", prog->result);
  return LLC_OK;
}

template <int VEC, int U, typename CT>
void launch_vec(const EwKernelParams& p, hipStream_t stream) {
  const uint32_t per_block = 256u * U;
  const uint32_t blocks = (p.hot.n_vec + per_block - 1) / per_block;  // exact cover, no grid-stride loop
  if (p.hot.streaming) {
    if (p.hot.n_inputs <= 2) hipLaunchKernelGGL((ew_kernel<VEC, U, 2, CT, true>), dim3(blocks), dim3(256), 0, stream, p);
    else hipLaunchKernelGGL((ew_kernel<VEC, U, LLC_EW_MAX_INPUTS, CT, true>), dim3(blocks), dim3(256), 0, stream, p);
  } else {
    if (p.hot.n_inputs <= 2) hipLaunchKernelGGL((ew_kernel<VEC, U, 2, CT, false>), dim3(blocks), dim3(256), 0, stream, p);
    else hipLaunchKernelGGL((ew_kernel<VEC, U, LLC_EW_MAX_INPUTS, CT, false>), dim3(blocks), dim3(256), 0, stream, p);
  }
}

template <typename CT>
int launch(const EwKernelParams& p, int vec, hipStream_t stream) {
  // one vector per lane measured best for the 16-byte widths
  if constexpr (sizeof(CT) == 4) {
    switch (vec) {
      case 8: launch_vec<8, 1, CT>(p, stream); break;
      case 4: launch_vec<4, 1, CT>(p, stream); break;
      case 2: launch_vec<2, 2, CT>(p, stream); break;
      default: launch_vec<1, 2, CT>(p, stream); break;
    }
  } else {
    if (vec >= 2) launch_vec<2, 2, CT>(p, stream);
    else launch_vec<1, 2, CT>(p, stream);
  }
  return check_launch("ew_kernel");
}

template <int VEC, bool NT>
void launch_chain_vec(const EwKernelParams& p, hipStream_t stream) {
  const uint32_t blocks = (p.hot.n_vec + 255u) / 256u;  // exact cover: one vector per lane
  if (p.hot.n_inputs <= 1) hipLaunchKernelGGL((ew_chain_kernel<VEC, 1, NT>), dim3(blocks), dim3(256), 0, stream, p);
  else if (p.hot.n_inputs == 2) hipLaunchKernelGGL((ew_chain_kernel<VEC, 2, NT>), dim3(blocks), dim3(256), 0, stream, p);
  else hipLaunchKernelGGL((ew_chain_kernel<VEC, 4, NT>), dim3(blocks), dim3(256), 0, stream, p);
}

template <bool NT>
void launch_chain_nt(const EwKernelParams& p, int vec, hipStream_t stream) {
  switch (vec) {
    case 8: launch_chain_vec<8, NT>(p, stream); break;
    case 4: launch_chain_vec<4, NT>(p, stream); break;
    case 2: launch_chain_vec<2, NT>(p, stream); break;
    default: launch_chain_vec<1, NT>(p, stream); break;
  }
}

template <int DT, bool NT>
void launch_chain_typed(const EwKernelParams& p, hipStream_t stream) {
  const uint32_t blocks = (p.hot.n_vec + 255u) / 256u;
  switch (p.hot.n_inputs) {
    case 0:
    case 1: hipLaunchKernelGGL((ew_chain_typed_kernel<DT, 1, NT>), dim3(blocks), dim3(256), 0, stream, p); break;
    case 2: hipLaunchKernelGGL((ew_chain_typed_kernel<DT, 2, NT>), dim3(blocks), dim3(256), 0, stream, p); break;
    case 3: hipLaunchKernelGGL((ew_chain_typed_kernel<DT, 3, NT>), dim3(blocks), dim3(256), 0, stream, p); break;
    default: hipLaunchKernelGGL((ew_chain_typed_kernel<DT, 4, NT>), dim3(blocks), dim3(256), 0, stream, p); break;
  }
}

// Whether the typed chain kernel takes this launch: same-shape contiguous operands of the result's floating type, 16 bytes a lane
bool chain_typed_ok(const EwKernelParams& p, int vec) {
  const int dt = p.hot.out_dtype;
  if (dt != LLC_FLOAT32 && dt != LLC_BFLOAT16 && dt != LLC_FLOAT16) return false;
  if (!p.hot.flat || p.hot.n_inputs < 1 || p.hot.n_inputs > 4 || vec != (dt == LLC_FLOAT32 ? 4 : 8)) return false;
  for (int k = 0; k < p.hot.n_inputs; ++k)
    if (p.hot.in_dtype[k] != dt || p.hot.in_inner[k] != 1) return false;
  return true;
}

int launch_chain(const EwKernelParams& p, int vec, hipStream_t stream) {
  if (chain_typed_ok(p, vec)) {
    const bool nt = p.hot.streaming != 0;
    switch (p.hot.out_dtype) {
      case LLC_FLOAT32: nt ? launch_chain_typed<LLC_FLOAT32, true>(p, stream) : launch_chain_typed<LLC_FLOAT32, false>(p, stream); break;
      case LLC_BFLOAT16: nt ? launch_chain_typed<LLC_BFLOAT16, true>(p, stream) : launch_chain_typed<LLC_BFLOAT16, false>(p, stream); break;
      default: nt ? launch_chain_typed<LLC_FLOAT16, true>(p, stream) : launch_chain_typed<LLC_FLOAT16, false>(p, stream); break;
    }
    return check_launch("ew_chain_typed_kernel");
  }
  if (p.hot.streaming) launch_chain_nt<true>(p, vec, stream);
  else launch_chain_nt<false>(p, vec, stream);
  return check_launch("ew_chain_kernel");
}

}  // namespace
}  // namespace llc

using namespace llc;

int llc_impl_elementwise(const llc_ew_program* prog, const llc_tensor* const* inputs, size_t n_inputs,
                                   llc_tensor* out, void* stream) {
  if (!prog || !out || (n_inputs && !inputs)) return set_error(LLC_ERR_BAD_ARG, "elementwise: null argument");
  if (n_inputs > LLC_EW_MAX_INPUTS)
    return set_error(LLC_ERR_UNSUPPORTED, "elementwise: %zu inputs (max %d)", n_inputs, LLC_EW_MAX_INPUTS);
  LLC_TRY(validate_program(prog, n_inputs));
  View o;
  LLC_TRY(make_view(out, "elementwise out", &o));
  if (!o.contiguous()) return set_error(LLC_ERR_LAYOUT, "elementwise: output must be contiguous");
  View in[LLC_EW_MAX_INPUTS];
  for (size_t k = 0; k < n_inputs; ++k) {
    LLC_TRY(make_view(inputs[k], "elementwise input", &in[k]));
    if (in[k].rank != o.rank)
      return set_error(LLC_ERR_SHAPE, "elementwise: input %zu has rank %d, output rank %d", k, in[k].rank, o.rank);
    for (int d = 0; d < o.rank; ++d)
      if (in[k].size[d] != o.size[d] && in[k].size[d] != 1)
        return set_error(LLC_ERR_SHAPE, "elementwise: input %zu extent %lld at dim %d does not broadcast to %lld", k,
                         (long long)in[k].size[d], d, (long long)o.size[d]);
    if (!float_compute_dtype(in[k].dtype))
      return set_error(LLC_ERR_DTYPE, "elementwise: input %zu has unsupported type %d", k, in[k].dtype);
  }
  if (!float_compute_dtype(o.dtype)) return set_error(LLC_ERR_DTYPE, "elementwise: unsupported output type %d", o.dtype);
  const int64_t total = o.numel();
  if (total == 0) return LLC_OK;
  if (total >= (int64_t)1 << 31) return set_error(LLC_ERR_TOO_LARGE, "elementwise: %lld elements (max 2^31-1)", (long long)total);

  // a straight-line program runs in accumulator form on the inputs it names, seed first
  llc_ew_inst chain[LLC_EW_MAX_INSTS];
  int n_chain = 0, slot[4], n_slots = 0;
  const bool linear = linearize(prog, n_inputs, chain, &n_chain, slot, &n_slots);
  View ine[LLC_EW_MAX_INPUTS];
  size_t ne = linear ? (size_t)n_slots : n_inputs;
  for (size_t k = 0; k < ne; ++k) ine[k] = linear ? in[slot[k]] : in[k];

  // effective strides (0 on broadcast dims), then collapse adjacent dims that stay affine for all inputs
  int64_t est[LLC_EW_MAX_INPUTS][LLC_MAX_RANK];
  for (size_t k = 0; k < ne; ++k)
    for (int d = 0; d < o.rank; ++d) est[k][d] = (ine[k].size[d] == 1 && o.size[d] != 1) ? 0 : (ine[k].size[d] == 1 ? 0 : ine[k].stride[d]);
  int64_t cdim[LLC_MAX_RANK];
  int64_t cst[LLC_EW_MAX_INPUTS][LLC_MAX_RANK];
  int nc = 0;
  for (int d = 0; d < o.rank; ++d) {
    if (o.size[d] == 1) continue;
    bool merge = nc > 0;
    if (merge)
      for (size_t k = 0; k < ne; ++k)
        if (cst[k][nc - 1] != est[k][d] * o.size[d]) { merge = false; break; }
    if (merge) {
      cdim[nc - 1] *= o.size[d];
      for (size_t k = 0; k < ne; ++k) cst[k][nc - 1] = est[k][d];
    } else {
      cdim[nc] = o.size[d];
      for (size_t k = 0; k < ne; ++k) cst[k][nc] = est[k][d];
      ++nc;
    }
  }
  if (nc == 0) {
    cdim[0] = 1;
    for (size_t k = 0; k < ne; ++k) cst[k][0] = 0;
    nc = 1;
  }
  if (nc > kMaxDims)
    return set_error(LLC_ERR_LAYOUT, "elementwise: broadcast pattern needs %d index dims (max %d)", nc, kMaxDims);

  EwKernelParams p{};
  for (int i = 0; i < prog->n_insts; ++i) p.insts[i] = linear ? chain[i] : prog->insts[i];
  p.hot.n_insts = prog->n_insts;
  p.hot.result = prog->result;
  p.hot.integer = prog->integer;
  p.hot.n_inputs = (int)ne;
  p.out = o.ptr;
  p.hot.out_dtype = o.dtype;
  for (int d = 0; d < kMaxDims; ++d) p.hot.dims[d] = 1;
  for (int d = 0; d < nc; ++d) p.hot.dims[kMaxDims - nc + d] = (uint32_t)cdim[d];
  bool flat = nc == 1;
  // widest vector: 16 bytes of the output type, shrunk until every access stays aligned and inside a row
  int vec = prog->integer ? 2 : (o.esize() <= 2 ? 8 : 4);
  auto aligned = [](const void* ptr, size_t bytes) { return ((uintptr_t)ptr % bytes) == 0; };
  for (size_t k = 0; k < ne; ++k) {
    p.in[k] = ine[k].ptr;
    p.hot.in_dtype[k] = ine[k].dtype;
    for (int d = 0; d < kMaxDims; ++d) p.in_stride[k][d] = 0;
    for (int d = 0; d < nc; ++d) {
      if (cst[k][d] >= (int64_t)1 << 31 || cst[k][d] < 0)
        return set_error(LLC_ERR_LAYOUT, "elementwise: input %zu stride out of range", k);
      p.in_stride[k][kMaxDims - nc + d] = (int32_t)cst[k][d];
    }
    const int inner = p.in_stride[k][kMaxDims - 1];
    if (inner != 0 && inner != 1) vec = 1;  // strided innermost access: one element per load, index scaled by the stride
  }
  while (vec > 1) {
    bool ok = (p.hot.dims[kMaxDims - 1] % vec) == 0 && aligned(o.ptr, vec * o.esize());
    for (size_t k = 0; ok && k < ne; ++k) {
      if (p.in_stride[k][kMaxDims - 1] == 0) continue;
      ok = aligned(ine[k].ptr, vec * ine[k].esize());
      for (int d = 0; ok && d < kMaxDims - 1; ++d) ok = (p.in_stride[k][d] % vec) == 0;
    }
    if (ok) break;
    vec >>= 1;
  }
  for (size_t k = 0; k < ne; ++k) p.hot.in_inner[k] = p.in_stride[k][kMaxDims - 1];
  p.hot.flat = flat ? 1 : 0;
  p.hot.n_vec = (uint32_t)(total / vec);
  // streams far larger than the L2 are touched once: non-temporal accesses keep them out of the caches
  p.hot.streaming = (int64_t)total * (int64_t)o.esize() >= ((int64_t)32 << 20) ? 1 : 0;
  if (linear) return launch_chain(p, vec, as_stream(stream));
  return prog->integer ? launch<int64_t>(p, vec, as_stream(stream)) : launch<float>(p, vec, as_stream(stream));
}
