// Host-side plumbing shared by every entry point of the kernel library: status/error reporting,
// descriptor validation, dtype helpers and launch checks.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>

#include <atomic>
#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "llc_hip.h"
#include "entries.hpp"

namespace llc {

int set_error(int status, const char* fmt, ...);

inline size_t dtype_size(size_t t) {
  switch (t) {
    case LLC_INT8: case LLC_INT1: return 1;
    case LLC_INT16: case LLC_BFLOAT16: case LLC_FLOAT16: return 2;
    case LLC_INT32: case LLC_FLOAT32: return 4;
    case LLC_INT64: case LLC_DOUBLE64: return 8;
  }
  return 0;
}
inline bool is_float_dtype(size_t t) { return t == LLC_FLOAT32 || t == LLC_BFLOAT16 || t == LLC_FLOAT16; }

// Validated view of an llc_tensor: extents/strides as int64, data pointer with `offset` applied.
struct View {
  char* ptr = nullptr;
  int dtype = -1;
  int rank = 0;
  int64_t size[LLC_MAX_RANK];
  int64_t stride[LLC_MAX_RANK];
  int64_t numel() const {
    int64_t n = 1;
    for (int i = 0; i < rank; ++i) n *= size[i];
    return n;
  }
  bool contiguous() const {
    int64_t s = 1;
    for (int i = rank - 1; i >= 0; --i) {
      if (size[i] == 0) return true;  // no elements: nothing is addressed, whatever the strides say
      if (size[i] != 1 && stride[i] != s) return false;
      s *= size[i];
    }
    return true;
  }
  size_t esize() const { return dtype_size((size_t)dtype); }
};

// Fills `v` from `t`; returns LLC_OK or sets the error (naming `what`).
int make_view(const llc_tensor* t, const char* what, View* v);

inline hipStream_t as_stream(void* s) { return reinterpret_cast<hipStream_t>(s); }

int check_launch(const char* kernel);

// Scratch device memory for kernels that keep partial results (split reductions).  Where it comes from, in
// this order: (1) a WorkspaceScope alive on the calling thread (a plan replaying with memory of its own, or the
// allocation-free entry point with the library's static array): that memory is handed out and nothing is ever
// allocated, a request beyond its capacity is an error; (2) one buffer per (device, stream), grown on demand.
// Growing allocates a new buffer and retires the old one (launches already queued, or a captured graph, may still
// address it) until scratch_trim frees it after a device synchronisation; it never synchronises by itself and is
// refused while `stream` is being captured.  Kernels of one stream run in order, so successive calls on a stream
// share that stream's buffer; calls on different streams never share one.
int get_workspace(size_t bytes, void** out, hipStream_t stream);

int scratch_bytes(int dev, size_t* live, size_t* retired);
int scratch_trim(int all);

struct WorkspaceScope {
  WorkspaceScope(void* ptr, size_t capacity);
  ~WorkspaceScope();
  WorkspaceScope(const WorkspaceScope&) = delete;
  WorkspaceScope& operator=(const WorkspaceScope&) = delete;

 private:
  void* prev_ptr_;
  size_t prev_cap_;
  bool prev_active_;
};
// While `high_water` is set on this thread, every get_workspace request raises *high_water to its size (a plan
// being recorded learns how much scratch memory its steps need).  Null stops it.
void workspace_track(size_t* high_water);

// A kernel that takes more than 64 KB of dynamic LDS must be allowed to, once per device: `done` (one per kernel
// instantiation, static at the call site) keeps a bit per device ordinal.
int allow_dynamic_lds(const void* kernel, int bytes, std::atomic<uint32_t>& done);

// Convolution on channels-last 16-bit tensors as an implicit GEMM on the wide-tile matmul kernel (gemm.hip):
// out[pixel, f] = sum over (tap, c) of x[pixel's window at tap, c] * w[f, tap, c].
struct ConvWideGeom {
  int32_t C, H, W, OH, OW, KH, KW;
  int32_t sh, sw, ph, pw, dh, dw;
  int32_t ncols;                    // N * OH * OW output pixels
  int32_t cblocks;                  // C / 64: k-tiles per tap
  uint32_t cblocks_magic, kw_magic; // for d = cblocks, KW: floor(2^32 / d) + 1, so that n / d == (n * magic) >> 32 for
                                    // the small n that occur; 0 when d == 1
};
// Runs it and returns LLC_OK (or an error); returns 1 without doing anything when the shape is not one the wide-tile
// kernel takes (the caller then uses its own kernels).
int conv_wide_16bit(int dtype, const char* x, const char* w, char* y, const char* bias, const char* residual, int F,
                    const ConvWideGeom& g, float alpha, int act, hipStream_t s);

#define LLC_TRY(expr)              \
  do {                             \
    int _st = (expr);              \
    if (_st != LLC_OK) return _st; \
  } while (0)

#define LLC_HIP_TRY(expr)                                                                       \
  do {                                                                                          \
    hipError_t _e = (expr);                                                                     \
    if (_e != hipSuccess) return ::llc::set_error(LLC_ERR_HIP, "%s: %s", #expr, hipGetErrorString(_e)); \
  } while (0)

// ---- device helpers ----
__device__ __forceinline__ float bf16_bits_to_f32(uint16_t h) { return __uint_as_float(((uint32_t)h) << 16); }
// round to nearest even, NaN stays NaN: gfx950 converts in hardware (v_cvt_pk_bf16_f32)
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
  const __bf16 b = static_cast<__bf16>(f);
  return __builtin_bit_cast(uint16_t, b);
}
__device__ __forceinline__ float f16_bits_to_f32(uint16_t h) { return __half2float(__ushort_as_half(h)); }
__device__ __forceinline__ uint16_t f32_to_f16_bits(float f) { return __half_as_ushort(__float2half_rn(f)); }

// two fp32 values rounded to the 16-bit storage type `dtype` (LLC_BFLOAT16 or LLC_FLOAT16), `lo` in the low half of the
// word: one v_cvt_pk_bf16_f32 / v_cvt_pk_f16_f32 (round to nearest even) instead of two conversions, a shift and an or
template <int DTYPE>
__device__ __forceinline__ uint32_t pack_pair(float lo, float hi) {
  typedef float f2_t __attribute__((ext_vector_type(2)));
  if constexpr (DTYPE == LLC_BFLOAT16) {
    typedef __bf16 bf2_t __attribute__((ext_vector_type(2)));
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f2_t{lo, hi}, bf2_t));
  } else {
    typedef _Float16 h2_t __attribute__((ext_vector_type(2)));
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f2_t{lo, hi}, h2_t));
  }
}

typedef uint32_t raw16_t __attribute__((ext_vector_type(4)));

// 16 bytes of storage type DT as fp32 values, and back (DT known when compiling: no branch between the loads and their use)
template <int DT>
__device__ __forceinline__ void unpack_typed(const raw16_t& raw, float* dst) {
  if constexpr (DT == LLC_FLOAT32) {
#pragma unroll
    for (int j = 0; j < 4; ++j) dst[j] = __uint_as_float(raw[j]);
  } else if constexpr (DT == LLC_BFLOAT16) {
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
template <int DT>
__device__ __forceinline__ raw16_t pack_typed(const float* src) {
  raw16_t r;
  if constexpr (DT == LLC_FLOAT32) {
#pragma unroll
    for (int j = 0; j < 4; ++j) r[j] = __float_as_uint(src[j]);
  } else {
#pragma unroll
    for (int j = 0; j < 4; ++j) r[j] = pack_pair<DT>(src[2 * j], src[2 * j + 1]);
  }
  return r;
}

// erf-based GELU, 0.5 x (1 + erf(x / sqrt 2)).  erf comes from the rational approximation 7.1.26 of
// Abramowitz & Stegun (absolute error below 1.5e-7) on the hardware reciprocal and exp2: the result stays
// within 5e-7 of the exactly rounded one over the whole range, a fortieth of the fp32 tolerance, at a third
// of the instructions of the library erff (this runs in GEMM epilogues, on every output element).
__device__ __forceinline__ float gelu_exact(float x) {
  const float z = fabsf(x) * 0.70710678118654752440f;
  const float t = __builtin_amdgcn_rcpf(1.0f + 0.3275911f * z);
  const float poly = t * (0.254829592f + t * (-0.284496736f + t * (1.421413741f + t * (-1.453152027f + t * 1.061405429f))));
  const float e = __builtin_amdgcn_exp2f(-z * z * 1.4426950408889634f);
  const float er = copysignf(1.0f - poly * e, x);
  return 0.5f * x * (1.0f + er);
}

// GELU for results that are rounded to a 16-bit storage type (the epilogues of the 16-bit products): x * Phi(x) with
// Phi(x) = 1 / (1 + 2^-t(x)), t an odd polynomial of degree 7 fitted to log2 of the odds Phi(x) / Phi(-x) so that
// the RELATIVE error of the result stays below 1.2e-3 for |x| <= 5 (half an ulp of bf16; absolute error below
// 2e-4 everywhere, results for x < -5 are below 1.5e-6 in magnitude either way).  Ten full-rate operations and two
// quarter-rate ones per value against the rational erf's sixteen and two: the epilogue of a product runs on one wave
// per SIMD with nothing to hide it behind, and a feed-forward layer applies this to every one of its outputs.
// fp32 results keep gelu_exact.
__device__ __forceinline__ float gelu_16bit(float x) {
  const float u = x * x;
  const float p = 2.2971660592200047f + u * (0.1095363857595901f + u * (-0.0014344055324419125f + u * 1.327634682739151e-05f));
  const float e = __builtin_amdgcn_exp2f(-x * p);
  return x * __builtin_amdgcn_rcpf(1.0f + e);
}
template <typename T>
__device__ __forceinline__ float gelu_for(float x) {
  if constexpr (sizeof(T) == 2) return gelu_16bit(x);
  else return gelu_exact(x);
}

constexpr int kWave = 64;

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, kWave));
  return v;
}

}  // namespace llc
