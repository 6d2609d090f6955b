// Fused elementwise chains: one launch evaluates a whole chain of LLH elementwise ops.
//
// The chain arrives as a tiny register program (llc_ew_program).  Every lane owns E = VEC*U
// consecutive-in-VEC output elements, loads all chain inputs first (16-byte vector loads, U of
// them in flight per input), then runs the program on registers and stores once.  Program control
// flow is uniform across the wave, so instruction decode runs on the scalar unit; the kernel is
// bound by HBM traffic: bytes moved = each distinct input once + the output once.
//
// Broadcast operands (llh.broadcast_to folded into the consumer) are read with stride 0; the host
// collapses the iteration space to at most four dims so that the common cases (same shape, bias
// over the last dim, per-channel NCHW, attention mask) need at most three integer divisions per
// vector.
#include "common.hpp"

namespace llc {
namespace {

constexpr int kMaxDims = 4;

struct EwKernelParams {
  llc_ew_program prog;
  const char* in[LLC_EW_MAX_INPUTS];
  int32_t in_dtype[LLC_EW_MAX_INPUTS];
  int32_t in_stride[LLC_EW_MAX_INPUTS][kMaxDims];  // elements; innermost is 0 or 1
  char* out;
  int32_t out_dtype;
  int32_t n_inputs;
  uint32_t dims[kMaxDims];  // collapsed output extents, dims[3] innermost
  int32_t flat;             // 1: every input is either same-shape contiguous or a scalar
  uint32_t n_vec;           // number of VEC-wide vectors in the output
};

// ---- typed loads: VEC consecutive elements (inner stride 1) or one element repeated (stride 0) ----
template <int VEC, typename CT>
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
      struct alignas(4 * VEC) P { float v[VEC]; };
      P p = *(const P*)(base + (size_t)off * 4);
#pragma unroll
      for (int j = 0; j < VEC; ++j) dst[j] = (CT)p.v[j];
    } break;
    case LLC_BFLOAT16: {
      struct alignas(2 * VEC) P { uint16_t v[VEC]; };
      P p = *(const P*)(base + (size_t)off * 2);
#pragma unroll
      for (int j = 0; j < VEC; ++j) dst[j] = (CT)bf16_bits_to_f32(p.v[j]);
    } break;
    case LLC_FLOAT16: {
      struct alignas(2 * VEC) P { uint16_t v[VEC]; };
      P p = *(const P*)(base + (size_t)off * 2);
#pragma unroll
      for (int j = 0; j < VEC; ++j) dst[j] = (CT)f16_bits_to_f32(p.v[j]);
    } break;
    case LLC_INT64: {
      struct alignas(VEC >= 2 ? 16 : 8) P { int64_t v[VEC]; };
      P p = *(const P*)(base + (size_t)off * 8);
#pragma unroll
      for (int j = 0; j < VEC; ++j) dst[j] = (CT)p.v[j];
    } break;
    case LLC_INT32: {
      struct alignas(4 * VEC) P { int32_t v[VEC]; };
      P p = *(const P*)(base + (size_t)off * 4);
#pragma unroll
      for (int j = 0; j < VEC; ++j) dst[j] = (CT)p.v[j];
    } break;
    default: {
      struct alignas(VEC) P { uint8_t v[VEC]; };
      P p = *(const P*)(base + (size_t)off);
#pragma unroll
      for (int j = 0; j < VEC; ++j) dst[j] = (CT)p.v[j];
    } break;
  }
}

template <int VEC, typename CT>
__device__ __forceinline__ void store_vec(char* base, int dtype, uint32_t off, const CT* src) {
  switch (dtype) {
    case LLC_FLOAT32: {
      struct alignas(4 * VEC) P { float v[VEC]; } p;
#pragma unroll
      for (int j = 0; j < VEC; ++j) p.v[j] = (float)src[j];
      *(P*)(base + (size_t)off * 4) = p;
    } break;
    case LLC_BFLOAT16: {
      struct alignas(2 * VEC) P { uint16_t v[VEC]; } p;
#pragma unroll
      for (int j = 0; j < VEC; ++j) p.v[j] = f32_to_bf16_bits((float)src[j]);
      *(P*)(base + (size_t)off * 2) = p;
    } break;
    case LLC_FLOAT16: {
      struct alignas(2 * VEC) P { uint16_t v[VEC]; } p;
#pragma unroll
      for (int j = 0; j < VEC; ++j) p.v[j] = f32_to_f16_bits((float)src[j]);
      *(P*)(base + (size_t)off * 2) = p;
    } break;
    case LLC_INT64: {
      struct alignas(VEC >= 2 ? 16 : 8) P { int64_t v[VEC]; } p;
#pragma unroll
      for (int j = 0; j < VEC; ++j) p.v[j] = (int64_t)src[j];
      *(P*)(base + (size_t)off * 8) = p;
    } break;
    case LLC_INT32: {
      struct alignas(4 * VEC) P { int32_t v[VEC]; } p;
#pragma unroll
      for (int j = 0; j < VEC; ++j) p.v[j] = (int32_t)src[j];
      *(P*)(base + (size_t)off * 4) = p;
    } break;
    case LLC_INT1: {
      struct alignas(VEC) P { uint8_t v[VEC]; } p;
#pragma unroll
      for (int j = 0; j < VEC; ++j) p.v[j] = src[j] != (CT)0 ? 1 : 0;
      *(P*)(base + (size_t)off) = p;
    } break;
    default: {
      struct alignas(VEC) P { int8_t v[VEC]; } p;
#pragma unroll
      for (int j = 0; j < VEC; ++j) p.v[j] = (int8_t)src[j];
      *(P*)(base + (size_t)off) = p;
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
    LLC_EW_CASE(LLC_EW_RELU, nanmax(a, 0.0f))
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

template <int VEC, int U, int MAXIN, typename CT>
__global__ __launch_bounds__(256) void ew_kernel(const EwKernelParams p) {
  constexpr int E = VEC * U;
  const uint32_t nthreads = gridDim.x * blockDim.x;
  for (uint32_t v0 = blockIdx.x * blockDim.x + threadIdx.x; v0 < p.n_vec; v0 += nthreads * U) {
    RegFile<E, CT> f;
    // ---- phase 1: issue every load ----
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const uint32_t v = v0 + u * nthreads;
      if (v < p.n_vec) {
        const uint32_t e = v * VEC;
        uint32_t idx0 = 0, idx1 = 0, idx2 = 0, idx3 = e;
        if (!p.flat) {
          uint32_t t = e;
          idx3 = t % p.dims[3];
          t /= p.dims[3];
          idx2 = t % p.dims[2];
          t /= p.dims[2];
          idx1 = t % p.dims[1];
          idx0 = t / p.dims[1];
        }
#define LLC_LOAD_INPUT(K, ARR)                                                                          \
  if (K < MAXIN && K < p.n_inputs) {                                                                    \
    uint32_t off = idx3 * (uint32_t)p.in_stride[K][3];                                                  \
    if (!p.flat)                                                                                        \
      off += idx0 * (uint32_t)p.in_stride[K][0] + idx1 * (uint32_t)p.in_stride[K][1] +                  \
             idx2 * (uint32_t)p.in_stride[K][2];                                                        \
    load_vec<VEC, CT>(p.in[K], p.in_dtype[K], off, p.in_stride[K][3], &ARR[u * VEC]);                   \
  }
        LLC_LOAD_INPUT(0, f.i0)
        LLC_LOAD_INPUT(1, f.i1)
        LLC_LOAD_INPUT(2, f.i2)
        LLC_LOAD_INPUT(3, f.i3)
        LLC_LOAD_INPUT(4, f.i4)
        LLC_LOAD_INPUT(5, f.i5)
#undef LLC_LOAD_INPUT
      }
    }
    // ---- phase 2: run the chain on registers ----
    for (int i = 0; i < p.prog.n_insts; ++i) {
      const llc_ew_inst inst = p.prog.insts[i];
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
    fetch<E, MAXIN, CT>(f, p.prog.result, (CT)0, res);
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const uint32_t v = v0 + u * nthreads;
      if (v < p.n_vec) store_vec<VEC, CT>(p.out, p.out_dtype, v * VEC, res + u * VEC);
    }
  }
}
#undef LLC_COPY

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
void launch_vec(const EwKernelParams& p, uint32_t blocks, hipStream_t stream) {
  if (p.n_inputs <= 2)
    hipLaunchKernelGGL((ew_kernel<VEC, U, 2, CT>), dim3(blocks), dim3(256), 0, stream, p);
  else
    hipLaunchKernelGGL((ew_kernel<VEC, U, LLC_EW_MAX_INPUTS, CT>), dim3(blocks), dim3(256), 0, stream, p);
}

template <typename CT>
int launch(const EwKernelParams& p, int vec, hipStream_t stream) {
  // lanes own 8 elements (4 for int64): two 16-byte loads per fp32 input, one per bf16/f16 input
  const int u = vec == 8 ? 1 : 2;
  // enough blocks to fill 256 CUs several times over, capped so each thread still loops a little
  uint64_t want = ((uint64_t)p.n_vec + (uint64_t)256 * u - 1) / ((uint64_t)256 * u);
  uint32_t blocks = (uint32_t)(want < 1 ? 1 : (want > 256u * 32u ? 256u * 32u : want));
  if constexpr (sizeof(CT) == 4) {
    switch (vec) {
      case 8: launch_vec<8, 1, CT>(p, blocks, stream); break;
      case 4: launch_vec<4, 2, CT>(p, blocks, stream); break;
      case 2: launch_vec<2, 2, CT>(p, blocks, stream); break;
      default: launch_vec<1, 2, CT>(p, blocks, stream); break;
    }
  } else {
    if (vec >= 2) launch_vec<2, 2, CT>(p, blocks, stream);
    else launch_vec<1, 2, CT>(p, blocks, stream);
  }
  return check_launch("ew_kernel");
}

}  // namespace
}  // namespace llc

using namespace llc;

extern "C" int llc_hip_elementwise(const llc_ew_program* prog, const llc_tensor* const* inputs, size_t n_inputs,
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

  // effective strides (0 on broadcast dims), then collapse adjacent dims that stay affine for all inputs
  int64_t est[LLC_EW_MAX_INPUTS][LLC_MAX_RANK];
  for (size_t k = 0; k < n_inputs; ++k)
    for (int d = 0; d < o.rank; ++d) est[k][d] = (in[k].size[d] == 1 && o.size[d] != 1) ? 0 : (in[k].size[d] == 1 ? 0 : in[k].stride[d]);
  int64_t cdim[LLC_MAX_RANK];
  int64_t cst[LLC_EW_MAX_INPUTS][LLC_MAX_RANK];
  int nc = 0;
  for (int d = 0; d < o.rank; ++d) {
    if (o.size[d] == 1) continue;
    bool merge = nc > 0;
    if (merge)
      for (size_t k = 0; k < n_inputs; ++k)
        if (cst[k][nc - 1] != est[k][d] * o.size[d]) { merge = false; break; }
    if (merge) {
      cdim[nc - 1] *= o.size[d];
      for (size_t k = 0; k < n_inputs; ++k) cst[k][nc - 1] = est[k][d];
    } else {
      cdim[nc] = o.size[d];
      for (size_t k = 0; k < n_inputs; ++k) cst[k][nc] = est[k][d];
      ++nc;
    }
  }
  if (nc == 0) {
    cdim[0] = 1;
    for (size_t k = 0; k < n_inputs; ++k) cst[k][0] = 0;
    nc = 1;
  }
  if (nc > kMaxDims)
    return set_error(LLC_ERR_LAYOUT, "elementwise: broadcast pattern needs %d index dims (max %d)", nc, kMaxDims);

  EwKernelParams p;
  p.prog = *prog;
  p.n_inputs = (int)n_inputs;
  p.out = o.ptr;
  p.out_dtype = o.dtype;
  for (int d = 0; d < kMaxDims; ++d) p.dims[d] = 1;
  for (int d = 0; d < nc; ++d) p.dims[kMaxDims - nc + d] = (uint32_t)cdim[d];
  bool flat = nc == 1;
  // widest vector: 16 bytes of the output type, shrunk until every access stays aligned and inside a row
  int vec = prog->integer ? 2 : (o.esize() <= 2 ? 8 : 4);
  auto aligned = [](const void* ptr, size_t bytes) { return ((uintptr_t)ptr % bytes) == 0; };
  for (size_t k = 0; k < n_inputs; ++k) {
    p.in[k] = in[k].ptr;
    p.in_dtype[k] = in[k].dtype;
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
    bool ok = (p.dims[kMaxDims - 1] % vec) == 0 && aligned(o.ptr, vec * o.esize());
    for (size_t k = 0; ok && k < n_inputs; ++k) {
      if (p.in_stride[k][kMaxDims - 1] == 0) continue;
      ok = aligned(in[k].ptr, vec * in[k].esize());
      for (int d = 0; ok && d < kMaxDims - 1; ++d) ok = (p.in_stride[k][d] % vec) == 0;
    }
    if (ok) break;
    vec >>= 1;
  }
  p.flat = flat ? 1 : 0;
  p.n_vec = (uint32_t)(total / vec);
  return prog->integer ? launch<int64_t>(p, vec, as_stream(stream)) : launch<float>(p, vec, as_stream(stream));
}
