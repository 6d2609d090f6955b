/*
 * llc_oracle.c -- CPU restatement of LLCompiler's compiled-op path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file is the parity checker for the HIP kernels: it is called from tests/, from
 * __graft_entry__.smoke() and from bench.py's cpu_baseline leg and from nowhere else.  The product
 * never routes through it.
 *
 * Every function restates, as plain single-threaded scalar loops, what the reference's lowering
 * emits for one LLH op (LLH -> StableHLO -> linalg -> affine loops -> LLVM, no tiling, no
 * vectorisation pass, fp32 accumulate, k ascending).  Build it with -ffp-contract=off: the
 * reference lowers to separate arith.mulf / arith.addf without a contract flag, so products are
 * rounded before they are added.
 *
 * Layouts: dense row-major, extents as int64.  NCHW activations, FCHW weights.
 *
 * Pinning: tests/test_oracle_pins.py holds every function here against an independent check (the
 * reference's own golden values, closed forms, float64 library routines, brute force on tiny inputs);
 * the docstring of each test there names the function it pins and the mistake it would catch.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define LLC_MAX_RANK 8

/* ---- op codes shared with tests (mirrors the order of LLHOps.td:345-393) ---- */
enum {
  LLC_U_ABS = 0, LLC_U_SQRT = 1, LLC_U_EXP = 2, LLC_U_RELU = 3, LLC_U_RSQRT = 4,
  LLC_U_NEG = 5, LLC_U_GELU = 6, LLC_U_TANH = 7, LLC_U_ERF = 8, LLC_U_SIGMOID = 9,
  LLC_U_LOG = 10, LLC_U_RECIP = 11
};
enum { LLC_B_ADD = 0, LLC_B_SUB = 1, LLC_B_MUL = 2, LLC_B_DIV = 3, LLC_B_MAX = 4, LLC_B_MIN = 5, LLC_B_POW = 6 };
/* CompareKind values of include/llcompiler/Dialect/LLH/IR/LLHEnums.td:111-116 */
enum { LLC_C_EQ = 1, LLC_C_GE = 2, LLC_C_LE = 3, LLC_C_GT = 4, LLC_C_LT = 5, LLC_C_NE = 6 };
enum { LLC_R_SUM = 0, LLC_R_MAX = 1, LLC_R_MIN = 2 };

/* ---- bf16 helpers: round-to-nearest-even, NaN kept quiet ---- */
uint16_t llc_ref_f32_to_bf16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}
float llc_ref_bf16_to_f32(uint16_t h) {
  uint32_t u = ((uint32_t)h) << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}
void llc_ref_round_bf16(const float* x, float* y, int64_t n) {
  for (int64_t i = 0; i < n; ++i) y[i] = llc_ref_bf16_to_f32(llc_ref_f32_to_bf16(x[i]));
}

/* ---- llh.matmul: LLHOps.td:438-444 -> stablehlo.dot (LLHToHLO.cpp:485) -> linalg.matmul ->
 *      three nested loops m, n, k with c += a*b in fp32 ---- */
void llc_ref_matmul_f32(const float* a, const float* b, float* c, int64_t M, int64_t N, int64_t K) {
  for (int64_t m = 0; m < M; ++m)
    for (int64_t n = 0; n < N; ++n) {
      float acc = 0.0f;
      for (int64_t k = 0; k < K; ++k) {
        float p = a[m * K + k] * b[k * N + n];
        acc = acc + p;
      }
      c[m * N + n] = acc;
    }
}

/* Same contraction with an fp64 accumulator: "what the mathematics fixes", used to budget the
 * rounding noise of any fp32 summation order. */
void llc_ref_matmul_f64acc(const float* a, const float* b, float* c, int64_t M, int64_t N, int64_t K) {
  for (int64_t m = 0; m < M; ++m)
    for (int64_t n = 0; n < N; ++n) {
      double acc = 0.0;
      for (int64_t k = 0; k < K; ++k) acc += (double)a[m * K + k] * (double)b[k * N + n];
      c[m * N + n] = (float)acc;
    }
}

/* Cache-friendlier m,k,n loop order; same per-element summation order as llc_ref_matmul_f32
 * (k ascending, rounded product then rounded add), so the results are bit-identical.  Only used
 * to finish big oracle cases in seconds. */
void llc_ref_matmul_f32_mkn(const float* a, const float* b, float* c, int64_t M, int64_t N, int64_t K) {
  for (int64_t m = 0; m < M; ++m) {
    float* crow = c + m * N;
    for (int64_t n = 0; n < N; ++n) crow[n] = 0.0f;
    for (int64_t k = 0; k < K; ++k) {
      float av = a[m * K + k];
      const float* brow = b + k * N;
      for (int64_t n = 0; n < N; ++n) {
        float p = av * brow[n];
        crow[n] = crow[n] + p;
      }
    }
  }
}

/* ---- llh.batch_matmul: LLHOps.td:446-452 -> stablehlo.dot_general batch {0}/{0}, contracting
 *      lhs dim 2 with rhs dim 1 (LLHToHLO.cpp:363-382) ---- */
void llc_ref_batch_matmul_f32(const float* a, const float* b, float* c, int64_t B, int64_t M, int64_t N,
                              int64_t K) {
  for (int64_t i = 0; i < B; ++i) llc_ref_matmul_f32(a + i * M * K, b + i * K * N, c + i * M * N, M, N, K);
}
void llc_ref_batch_matmul_f32_mkn(const float* a, const float* b, float* c, int64_t B, int64_t M, int64_t N,
                                  int64_t K) {
  for (int64_t i = 0; i < B; ++i) llc_ref_matmul_f32_mkn(a + i * M * K, b + i * K * N, c + i * M * N, M, N, K);
}

/* ---- output extent of conv / max_pool along one spatial dim:
 *      LLHinfersymbolShape.cpp:257-268  out = (in + pad_lo + pad_hi - dil*(k-1) - 1)/stride + 1 ---- */
int64_t llc_ref_window_out(int64_t in, int64_t pad_lo, int64_t pad_hi, int64_t dil, int64_t k, int64_t stride) {
  return (in + pad_lo + pad_hi - dil * (k - 1) - 1) / stride + 1;
}

/* ---- llh.conv: LLHOps.td:423-436 -> stablehlo.convolution [b,f,0,1]x[o,i,0,1]->[b,f,0,1]
 *      (LLHToHLO.cpp:214-270), window_strides=stride, rhs_dilation=dilation,
 *      feature_group_count=group.  pad = {h_lo, w_lo, h_hi, w_hi} as the shape rule reads it
 *      (LLHinfersymbolShape.cpp:257-268) and as the importer writes it (conv.py:48-70).
 *      Cross-correlation; loops n, f, oh, ow, c, kh, kw; padding contributes zero.
 *      bias may be NULL (llh.conv) or length F (llh.conv_bias, LLHOps.td:407-421). ---- */
void llc_ref_conv2d_f32(const float* x, const float* w, const float* bias, float* y, int64_t N, int64_t C,
                        int64_t H, int64_t W, int64_t F, int64_t KH, int64_t KW, const int64_t* pad,
                        const int64_t* stride, const int64_t* dil, int64_t group) {
  int64_t OH = llc_ref_window_out(H, pad[0], pad[2], dil[0], KH, stride[0]);
  int64_t OW = llc_ref_window_out(W, pad[1], pad[3], dil[1], KW, stride[1]);
  int64_t Cg = C / group, Fg = F / group;
  for (int64_t n = 0; n < N; ++n)
    for (int64_t f = 0; f < F; ++f) {
      int64_t g = f / Fg;
      for (int64_t oh = 0; oh < OH; ++oh)
        for (int64_t ow = 0; ow < OW; ++ow) {
          float acc = 0.0f;
          for (int64_t c = 0; c < Cg; ++c)
            for (int64_t kh = 0; kh < KH; ++kh) {
              int64_t ih = oh * stride[0] - pad[0] + kh * dil[0];
              if (ih < 0 || ih >= H) continue;
              for (int64_t kw = 0; kw < KW; ++kw) {
                int64_t iw = ow * stride[1] - pad[1] + kw * dil[1];
                if (iw < 0 || iw >= W) continue;
                float p = x[((n * C + g * Cg + c) * H + ih) * W + iw] * w[((f * Cg + c) * KH + kh) * KW + kw];
                acc = acc + p;
              }
            }
          if (bias) acc = acc + bias[f];
          y[((n * F + f) * OH + oh) * OW + ow] = acc;
        }
    }
}

/* ---- elementwise, same-shape operands (broadcast is explicit: llc_ref_broadcast_to) ----
 *  unary: abs/sqrt/exp/rsqrt LLHToHLO.cpp:486,488,490; relu = max(x, 0)
 *  (LLHPreprocessingForHLO.cpp:76-101).  gelu/tanh/erf/sigmoid/log/neg/recip are not LLH ops in the
 *  reference (those nodes run in torch eager there); they follow torch's definitions, gelu with
 *  approximate='none'. */
static float unary_f32(int op, float x) {
  switch (op) {
    case LLC_U_ABS: return fabsf(x);
    case LLC_U_SQRT: return sqrtf(x);
    case LLC_U_EXP: return expf(x);
    case LLC_U_RELU: return x > 0.0f ? x : (x != x ? x : 0.0f);
    case LLC_U_RSQRT: return 1.0f / sqrtf(x);
    case LLC_U_NEG: return -x;
    case LLC_U_GELU: return (float)(0.5 * (double)x * (1.0 + erf((double)x * 0.70710678118654752440)));
    case LLC_U_TANH: return tanhf(x);
    case LLC_U_ERF: return erff(x);
    case LLC_U_SIGMOID: return 1.0f / (1.0f + expf(-x));
    case LLC_U_LOG: return logf(x);
    case LLC_U_RECIP: return 1.0f / x;
  }
  return NAN;
}
void llc_ref_unary_f32(int op, const float* x, float* y, int64_t n) {
  for (int64_t i = 0; i < n; ++i) y[i] = unary_f32(op, x[i]);
}
/* binary: add/sub/mul/div/max LLHToHLO.cpp:480-484; min/pow are declared (LLHOps.td:381-393) and
 * follow IEEE / libm here.  max/min propagate NaN like stablehlo.maximum and torch.maximum. */
static float binary_f32(int op, float a, float b) {
  switch (op) {
    case LLC_B_ADD: return a + b;
    case LLC_B_SUB: return a - b;
    case LLC_B_MUL: return a * b;
    case LLC_B_DIV: return a / b;
    case LLC_B_MAX: return (a != a || b != b) ? NAN : (a > b ? a : b);
    case LLC_B_MIN: return (a != a || b != b) ? NAN : (a < b ? a : b);
    case LLC_B_POW: return powf(a, b);
  }
  return NAN;
}
void llc_ref_binary_f32(int op, const float* a, const float* b, float* y, int64_t n) {
  for (int64_t i = 0; i < n; ++i) y[i] = binary_f32(op, a[i], b[i]);
}
/* i64 flavour (symbol arithmetic and integer tensors, LLHToArith.cpp:112-144).  Division is
 * torch's floor division for non-negative operands, which is all the shape math ever sees; the
 * reference's arith.divui agrees there. */
void llc_ref_binary_i64(int op, const int64_t* a, const int64_t* b, int64_t* y, int64_t n) {
  for (int64_t i = 0; i < n; ++i) {
    int64_t r = 0;
    switch (op) {
      case LLC_B_ADD: r = a[i] + b[i]; break;
      case LLC_B_SUB: r = a[i] - b[i]; break;
      case LLC_B_MUL: r = a[i] * b[i]; break;
      case LLC_B_DIV: {
        int64_t q = a[i] / b[i];
        if ((a[i] % b[i] != 0) && ((a[i] < 0) != (b[i] < 0))) --q;
        r = q;
      } break;
      case LLC_B_MAX: r = a[i] > b[i] ? a[i] : b[i]; break;
      case LLC_B_MIN: r = a[i] < b[i] ? a[i] : b[i]; break;
    }
    y[i] = r;
  }
}
/* llh.compare: LLHToHLO.cpp:384-445, ordered float compare; result i1 stored as one byte */
void llc_ref_compare_f32(int kind, const float* a, const float* b, uint8_t* y, int64_t n) {
  for (int64_t i = 0; i < n; ++i) {
    int r = 0;
    switch (kind) {
      case LLC_C_EQ: r = a[i] == b[i]; break;
      case LLC_C_NE: r = a[i] != b[i]; break;
      case LLC_C_GE: r = a[i] >= b[i]; break;
      case LLC_C_GT: r = a[i] > b[i]; break;
      case LLC_C_LE: r = a[i] <= b[i]; break;
      case LLC_C_LT: r = a[i] < b[i]; break;
    }
    y[i] = (uint8_t)r;
  }
}
void llc_ref_compare_i64(int kind, const int64_t* a, const int64_t* b, uint8_t* y, int64_t n) {
  for (int64_t i = 0; i < n; ++i) {
    int r = 0;
    switch (kind) {
      case LLC_C_EQ: r = a[i] == b[i]; break;
      case LLC_C_NE: r = a[i] != b[i]; break;
      case LLC_C_GE: r = a[i] >= b[i]; break;
      case LLC_C_GT: r = a[i] > b[i]; break;
      case LLC_C_LE: r = a[i] <= b[i]; break;
      case LLC_C_LT: r = a[i] < b[i]; break;
    }
    y[i] = (uint8_t)r;
  }
}
/* llh.where -> stablehlo.select (LLHToHLO.cpp:487): pred ? on_true : on_false.  The reference's
 * importer passes on_true twice (where.py:48-49); this follows the op definition, i.e. torch. */
void llc_ref_where_f32(const uint8_t* pred, const float* t, const float* f, float* y, int64_t n) {
  for (int64_t i = 0; i < n; ++i) y[i] = pred[i] ? t[i] : f[i];
}
/* llh.convert_to -> stablehlo.convert (LLHToHLO.cpp:489) */
void llc_ref_convert_f32_to_i64(const float* x, int64_t* y, int64_t n) {
  for (int64_t i = 0; i < n; ++i) y[i] = (int64_t)x[i];
}
void llc_ref_convert_i64_to_f32(const int64_t* x, float* y, int64_t n) {
  for (int64_t i = 0; i < n; ++i) y[i] = (float)x[i];
}

/* ---- generic strided gather used by broadcast / transpose / slice:
 *      out[idx] = in[sum_d idx[d]*in_stride[d] + in_offset], elem bytes 1/2/4/8 ---- */
static void strided_copy(const void* in, void* out, int rank, const int64_t* out_shape,
                         const int64_t* in_stride, int64_t in_offset, int elem) {
  int64_t total = 1;
  for (int d = 0; d < rank; ++d) total *= out_shape[d];
  int64_t idx[LLC_MAX_RANK] = {0};
  const char* src = (const char*)in;
  char* dst = (char*)out;
  for (int64_t i = 0; i < total; ++i) {
    int64_t off = in_offset;
    for (int d = 0; d < rank; ++d) off += idx[d] * in_stride[d];
    memcpy(dst + i * elem, src + off * elem, (size_t)elem);
    for (int d = rank - 1; d >= 0; --d) {
      if (++idx[d] < out_shape[d]) break;
      idx[d] = 0;
    }
  }
}

/* llh.broadcast_to{cast_dims}: LLHOps.td:206-217 -> stablehlo.dynamic_broadcast_in_dim
 * (LLHToHLO.cpp:191-212).  Input and output have the same rank (the canonicaliser reshapes lower
 * ranks first, LLHUtilitys.cpp:80-150); every input dim of extent 1 is repeated. */
void llc_ref_broadcast_to(const void* in, void* out, int rank, const int64_t* in_shape,
                          const int64_t* out_shape, int elem) {
  int64_t st[LLC_MAX_RANK];
  int64_t s = 1;
  for (int d = rank - 1; d >= 0; --d) {
    st[d] = (in_shape[d] == 1 && out_shape[d] != 1) ? 0 : s;
    s *= in_shape[d];
  }
  strided_copy(in, out, rank, out_shape, st, 0, elem);
}

/* llh.transpose{perms}: LLHOps.td:343 -> stablehlo.transpose (LLHToHLO.td:24-26):
 * out.shape[i] = in.shape[perms[i]] */
void llc_ref_transpose(const void* in, void* out, int rank, const int64_t* in_shape, const int64_t* perms,
                       int elem) {
  int64_t in_st[LLC_MAX_RANK], st[LLC_MAX_RANK], oshape[LLC_MAX_RANK];
  int64_t s = 1;
  for (int d = rank - 1; d >= 0; --d) {
    in_st[d] = s;
    s *= in_shape[d];
  }
  for (int d = 0; d < rank; ++d) {
    st[d] = in_st[perms[d]];
    oshape[d] = in_shape[perms[d]];
  }
  strided_copy(in, out, rank, oshape, st, 0, elem);
}

/* llh.stride_slice: LLHOps.td:261-269 -> real_dynamic_slice -> tensor.extract_slice with
 * size = ceildiv(end - start, stride) (LLHToHLO.cpp:341-361,
 * StablehlotoLinalgExtension.cpp:64-118).  out_shape receives the sizes. */
void llc_ref_stride_slice(const void* in, void* out, int rank, const int64_t* in_shape, const int64_t* start,
                          const int64_t* end, const int64_t* step, int64_t* out_shape, int elem) {
  int64_t in_st[LLC_MAX_RANK], st[LLC_MAX_RANK];
  int64_t s = 1, off = 0;
  for (int d = rank - 1; d >= 0; --d) {
    in_st[d] = s;
    s *= in_shape[d];
  }
  for (int d = 0; d < rank; ++d) {
    out_shape[d] = (end[d] - start[d] + step[d] - 1) / step[d];
    if (out_shape[d] < 0) out_shape[d] = 0;
    st[d] = in_st[d] * step[d];
    off += start[d] * in_st[d];
  }
  if (out) strided_copy(in, out, rank, out_shape, st, off, elem);
}

/* llh.extract(input, index): row `index` of dim 0, dim dropped
 * (LLHPreprocessingForHLO.cpp:103-140); a negative index counts from the end
 * (LLHCanonicalize.cpp:337-354). */
void llc_ref_extract(const void* in, void* out, int rank, const int64_t* in_shape, int64_t index, int elem) {
  int64_t inner = 1;
  for (int d = 1; d < rank; ++d) inner *= in_shape[d];
  if (index < 0) index += in_shape[0];
  memcpy(out, (const char*)in + index * inner * elem, (size_t)(inner * elem));
}

/* gather of whole rows along dim 0 (embedding lookup, aten.index_select/embedding): not an LLH op
 * in the reference; torch semantics, negative indices not allowed. */
void llc_ref_gather_rows(const void* table, const int64_t* idx, void* out, int64_t n_idx, int64_t row_elems,
                         int elem) {
  for (int64_t i = 0; i < n_idx; ++i)
    memcpy((char*)out + i * row_elems * elem, (const char*)table + idx[i] * row_elems * elem,
           (size_t)(row_elems * elem));
}

/* ---- llh.reduce_sum/max/min{axis}: LLHOps.td:528-553 -> stablehlo.reduce with init 0 / -inf /
 *      +inf (LLHToHLO.cpp:81-133); result drops the reduced axes
 *      (LLHinfersymbolShape.cpp:185-212); elements are folded in ascending index order ---- */
void llc_ref_reduce_f32(int kind, const float* x, float* y, int rank, const int64_t* shape, const int64_t* axes,
                        int n_axes) {
  int reduced[LLC_MAX_RANK] = {0};
  for (int i = 0; i < n_axes; ++i) reduced[axes[i] < 0 ? axes[i] + rank : axes[i]] = 1;
  int64_t out_st[LLC_MAX_RANK];
  int64_t s = 1, total = 1;
  for (int d = rank - 1; d >= 0; --d) {
    if (reduced[d]) out_st[d] = 0;
    else {
      out_st[d] = s;
      s *= shape[d];
    }
    total *= shape[d];
  }
  float init = kind == LLC_R_SUM ? 0.0f : (kind == LLC_R_MAX ? -INFINITY : INFINITY);
  for (int64_t i = 0; i < s; ++i) y[i] = init;
  int64_t idx[LLC_MAX_RANK] = {0};
  for (int64_t i = 0; i < total; ++i) {
    int64_t o = 0;
    for (int d = 0; d < rank; ++d) o += idx[d] * out_st[d];
    float v = x[i];
    if (kind == LLC_R_SUM) y[o] = y[o] + v;
    else if (kind == LLC_R_MAX) y[o] = binary_f32(LLC_B_MAX, y[o], v);
    else y[o] = binary_f32(LLC_B_MIN, y[o], v);
    for (int d = rank - 1; d >= 0; --d) {
      if (++idx[d] < shape[d]) break;
      idx[d] = 0;
    }
  }
}

/* ---- softmax over the last dim.  No LLH op: ATen _softmax is decomposed
 *      (torch_compile_config.py:24) into amax -> sub -> exp -> sum -> div, five passes ---- */
void llc_ref_softmax_lastdim_f32(const float* x, float* y, int64_t rows, int64_t cols) {
  for (int64_t r = 0; r < rows; ++r) {
    const float* xr = x + r * cols;
    float* yr = y + r * cols;
    float mx = -INFINITY;
    for (int64_t c = 0; c < cols; ++c) mx = binary_f32(LLC_B_MAX, mx, xr[c]);
    for (int64_t c = 0; c < cols; ++c) yr[c] = xr[c] - mx;
    for (int64_t c = 0; c < cols; ++c) yr[c] = expf(yr[c]);
    float sum = 0.0f;
    for (int64_t c = 0; c < cols; ++c) sum = sum + yr[c];
    for (int64_t c = 0; c < cols; ++c) yr[c] = yr[c] / sum;
  }
}

/* ---- llh.layer_norm{epsilon, axis=-1}: LLHOps.td:454-463 (declared only in the reference; the
 *      node runs in torch eager there).  torch semantics: biased variance over the last dim,
 *      y = (x - mean) / sqrt(var + eps) * gamma + beta; statistics in fp32 ---- */
void llc_ref_layernorm_lastdim_f32(const float* x, const float* gamma, const float* beta, float* y, int64_t rows,
                                   int64_t cols, float eps) {
  for (int64_t r = 0; r < rows; ++r) {
    const float* xr = x + r * cols;
    float* yr = y + r * cols;
    float sum = 0.0f;
    for (int64_t c = 0; c < cols; ++c) sum = sum + xr[c];
    float mean = sum / (float)cols;
    float sq = 0.0f;
    for (int64_t c = 0; c < cols; ++c) {
      float d = xr[c] - mean;
      sq = sq + d * d;
    }
    float rstd = 1.0f / sqrtf(sq / (float)cols + eps);
    for (int64_t c = 0; c < cols; ++c) {
      float v = (xr[c] - mean) * rstd;
      if (gamma) v = v * gamma[c];
      if (beta) v = v + beta[c];
      yr[c] = v;
    }
  }
}

/* ---- llh.batch_norm_inference{feature_index=1}: decomposition of DecomposeOps.cpp:110-148:
 *      ((x - mean) * scale) / sqrt(var + eps) + bias, in that operation order ---- */
void llc_ref_batch_norm_inference_f32(const float* x, const float* scale, const float* bias, const float* mean,
                                      const float* var, float* y, int64_t N, int64_t C, int64_t HW, float eps) {
  for (int64_t n = 0; n < N; ++n)
    for (int64_t c = 0; c < C; ++c) {
      float sd = sqrtf(var[c] + eps);
      for (int64_t i = 0; i < HW; ++i) {
        int64_t o = (n * C + c) * HW + i;
        float v = x[o] - mean[c];
        v = v * scale[c];
        v = v / sd;
        y[o] = v + bias[c];
      }
    }
}

/* BN folded into the preceding conv (host-side, at plan time): w' = w * scale/sqrt(var+eps),
 * b' = (b - mean) * scale/sqrt(var+eps) + bias.  Algebraically the same affine map as
 * DecomposeOps.cpp:139-144 applied to the conv result. */
void llc_ref_fold_bn_into_conv_f32(const float* w, const float* b, const float* scale, const float* bias,
                                   const float* mean, const float* var, float* w_out, float* b_out, int64_t F,
                                   int64_t per_filter, float eps) {
  for (int64_t f = 0; f < F; ++f) {
    float k = scale[f] / sqrtf(var[f] + eps);
    for (int64_t i = 0; i < per_filter; ++i) w_out[f * per_filter + i] = w[f * per_filter + i] * k;
    b_out[f] = ((b ? b[f] : 0.0f) - mean[f]) * k + bias[f];
  }
}

/* ---- llh.max_pool: LLHOps.td:495-507 -> stablehlo.reduce_window max (LLHToHLO.cpp:295-339).
 *      init_zero=1 reproduces the reference's init value 0 (LLHToHLO.cpp:313-314: the result is
 *      max(0, window max) and padding acts as 0); init_zero=0 is torch's -inf padding.  pad =
 *      {h_lo, w_lo, h_hi, w_hi}; ceil_mode false ---- */
void llc_ref_maxpool2d_f32(const float* x, float* y, int64_t N, int64_t C, int64_t H, int64_t W, int64_t KH,
                           int64_t KW, const int64_t* pad, const int64_t* stride, const int64_t* dil,
                           int init_zero) {
  int64_t OH = llc_ref_window_out(H, pad[0], pad[2], dil[0], KH, stride[0]);
  int64_t OW = llc_ref_window_out(W, pad[1], pad[3], dil[1], KW, stride[1]);
  for (int64_t nc = 0; nc < N * C; ++nc)
    for (int64_t oh = 0; oh < OH; ++oh)
      for (int64_t ow = 0; ow < OW; ++ow) {
        float acc = init_zero ? 0.0f : -INFINITY;
        for (int64_t kh = 0; kh < KH; ++kh) {
          int64_t ih = oh * stride[0] - pad[0] + kh * dil[0];
          if (ih < 0 || ih >= H) continue;
          for (int64_t kw = 0; kw < KW; ++kw) {
            int64_t iw = ow * stride[1] - pad[1] + kw * dil[1];
            if (iw < 0 || iw >= W) continue;
            acc = binary_f32(LLC_B_MAX, acc, x[(nc * H + ih) * W + iw]);
          }
        }
        y[(nc * OH + oh) * OW + ow] = acc;
      }
}

/* ---- llh.adaptive_average_pool{out_size=(1,1)}: shape rule only in the reference
 *      (LLHinfersymbolShape.cpp:587-613); global average = reduce_sum over (2,3) then one divide ---- */
void llc_ref_global_avgpool_f32(const float* x, float* y, int64_t NC, int64_t HW) {
  for (int64_t i = 0; i < NC; ++i) {
    float s = 0.0f;
    for (int64_t j = 0; j < HW; ++j) s = s + x[i * HW + j];
    y[i] = s / (float)HW;
  }
}

/* ---- the two numeric known answers the reference's own runner tests hold ----
 *  test/RunnerTest/abs.mlir:5-10        abs(dense<-1.0> : tensor<2xf32>) prints [1, 1]
 *  test/RunnerTest/mlir-runner.mlir:11-25   i64 2*2 converted to f32 prints [4]          */
void llc_ref_golden_abs(float* out2) {
  float in[2] = {-1.0f, -1.0f};
  llc_ref_unary_f32(LLC_U_ABS, in, out2, 2);
}
void llc_ref_golden_i64_mul_to_f32(float* out1) {
  int64_t two = 2, prod;
  llc_ref_binary_i64(LLC_B_MUL, &two, &two, &prod, 1);
  llc_ref_convert_i64_to_f32(&prod, out1, 1);
}
