// llh.max_pool.  NCHW: one lane per output element, lanes consecutive along OW so that window
// rows are read as contiguous (stride-`stride_w`) runs; overlapping windows are served by L1/L2, so
// HBM traffic stays at input once + output once.  Channels-last (NHWC in memory): one lane per output
// pixel and 16-byte run of channels, lanes consecutive along the channels.
#include "common.hpp"

namespace llc {
namespace {

typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4_t;

struct PoolParams {
  const char* x;
  char* y;
  int32_t dtype;
  int32_t H, W, OH, OW;
  int32_t KH, KW, ph, pw, sh, sw, dh, dw;
  int32_t init_zero;
  int64_t total;  // N*C*OH*OW
  int32_t C;      // channels (the channels-last kernel)
};


// K > 0: a K x K window known at compile time.  All K*K loads are issued unconditionally from indices
// clamped into the plane, then combined (a load guarded by the window test compiles to a branch with a wait:
// one memory round trip per tap).  K == 0: any window, tap by tap.
template <int DT, int K>
__global__ __launch_bounds__(256) void max_pool_kernel(const PoolParams p) {
  const int64_t o = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (o >= p.total) return;
  const int ow = (int)(o % p.OW);
  int64_t t = o / p.OW;
  const int oh = (int)(t % p.OH);
  const int64_t nc = t / p.OH;
  const int64_t plane = nc * p.H * p.W;
  float acc = p.init_zero ? 0.0f : -INFINITY;
  if constexpr (K > 0) {
    float tap[K * K];
    bool ok[K * K];
#pragma unroll
    for (int kh = 0; kh < K; ++kh) {
      const int ih = oh * p.sh - p.ph + kh * p.dh;
      const int ch = ih < 0 ? 0 : (ih >= p.H ? p.H - 1 : ih);
#pragma unroll
      for (int kw = 0; kw < K; ++kw) {
        const int iw = ow * p.sw - p.pw + kw * p.dw;
        const int cw = iw < 0 ? 0 : (iw >= p.W ? p.W - 1 : iw);
        ok[kh * K + kw] = ih >= 0 && ih < p.H && iw >= 0 && iw < p.W;
        const int64_t i = plane + (int64_t)ch * p.W + cw;
        if constexpr (DT == LLC_FLOAT32) tap[kh * K + kw] = ((const float*)p.x)[i];
        else if constexpr (DT == LLC_BFLOAT16) tap[kh * K + kw] = bf16_bits_to_f32(((const uint16_t*)p.x)[i]);
        else tap[kh * K + kw] = f16_bits_to_f32(((const uint16_t*)p.x)[i]);
      }
    }
#pragma unroll
    for (int j = 0; j < K * K; ++j) {
      const float v = tap[j];
      const float m = (v > acc || v != v) ? v : acc;  // NaN propagates, like stablehlo.maximum / torch
      acc = ok[j] ? m : acc;
    }
  } else
  for (int kh = 0; kh < p.KH; ++kh) {
    const int ih = oh * p.sh - p.ph + kh * p.dh;
    if (ih < 0 || ih >= p.H) continue;
    for (int kw = 0; kw < p.KW; ++kw) {
      const int iw = ow * p.sw - p.pw + kw * p.dw;
      if (iw < 0 || iw >= p.W) continue;
      const int64_t i = plane + (int64_t)ih * p.W + iw;
      float v;
      if constexpr (DT == LLC_FLOAT32) v = ((const float*)p.x)[i];
      else if constexpr (DT == LLC_BFLOAT16) v = bf16_bits_to_f32(((const uint16_t*)p.x)[i]);
      else v = f16_bits_to_f32(((const uint16_t*)p.x)[i]);
      acc = (v > acc || v != v) ? v : acc;  // NaN propagates, like stablehlo.maximum / torch
    }
  }
  if constexpr (DT == LLC_FLOAT32) ((float*)p.y)[o] = acc;
  else if constexpr (DT == LLC_BFLOAT16) ((uint16_t*)p.y)[o] = f32_to_bf16_bits(acc);
  else ((uint16_t*)p.y)[o] = f32_to_f16_bits(acc);
}

// Channels-last.  `p.total` counts lanes: N*OH*OW*(C / V), V = 16 / element size values per lane.
template <int DT, int K>
__global__ __launch_bounds__(256) void max_pool_nhwc_kernel(const PoolParams p) {
  constexpr int V = DT == LLC_FLOAT32 ? 4 : 8;
  const int64_t o = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (o >= p.total) return;
  const int chunks = p.C / V;
  const int ck = (int)(o % chunks);
  int64_t t = o / chunks;
  const int ow = (int)(t % p.OW);
  t /= p.OW;
  const int oh = (int)(t % p.OH);
  const int64_t n = t / p.OH;
  const u32x4_t* img = (const u32x4_t*)p.x + n * p.H * p.W * chunks + ck;
  float acc[V];
#pragma unroll
  for (int e = 0; e < V; ++e) acc[e] = p.init_zero ? 0.0f : -INFINITY;
  auto combine = [&](const u32x4_t q, bool ok) {
#pragma unroll
    for (int e = 0; e < V; ++e) {
      float v;
      if constexpr (DT == LLC_FLOAT32) v = __uint_as_float(q[e]);
      else if constexpr (DT == LLC_BFLOAT16) v = __uint_as_float((e & 1) ? (q[e / 2] & 0xffff0000u) : (q[e / 2] << 16));
      else v = f16_bits_to_f32((uint16_t)(q[e / 2] >> (16 * (e & 1))));
      const float m = (v > acc[e] || v != v) ? v : acc[e];  // NaN propagates, like stablehlo.maximum / torch
      acc[e] = ok ? m : acc[e];
    }
  };
  if constexpr (K > 0) {
    // every tap is loaded from an index clamped into the image, then combined under its window test
    u32x4_t tap[K * K];
    bool ok[K * K];
#pragma unroll
    for (int kh = 0; kh < K; ++kh) {
      const int ih = oh * p.sh - p.ph + kh * p.dh;
      const int ch = ih < 0 ? 0 : (ih >= p.H ? p.H - 1 : ih);
#pragma unroll
      for (int kw = 0; kw < K; ++kw) {
        const int iw = ow * p.sw - p.pw + kw * p.dw;
        const int cw = iw < 0 ? 0 : (iw >= p.W ? p.W - 1 : iw);
        ok[kh * K + kw] = ih >= 0 && ih < p.H && iw >= 0 && iw < p.W;
        tap[kh * K + kw] = img[((int64_t)ch * p.W + cw) * chunks];
      }
    }
#pragma unroll
    for (int j = 0; j < K * K; ++j) combine(tap[j], ok[j]);
  } else {
    for (int kh = 0; kh < p.KH; ++kh) {
      const int ih = oh * p.sh - p.ph + kh * p.dh;
      if (ih < 0 || ih >= p.H) continue;
      for (int kw = 0; kw < p.KW; ++kw) {
        const int iw = ow * p.sw - p.pw + kw * p.dw;
        if (iw < 0 || iw >= p.W) continue;
        combine(img[((int64_t)ih * p.W + iw) * chunks], true);
      }
    }
  }
  u32x4_t r;
  if constexpr (DT == LLC_FLOAT32) r = u32x4_t{__float_as_uint(acc[0]), __float_as_uint(acc[1]), __float_as_uint(acc[2]), __float_as_uint(acc[3])};
  else
    r = u32x4_t{pack_pair<DT>(acc[0], acc[1]), pack_pair<DT>(acc[2], acc[3]), pack_pair<DT>(acc[4], acc[5]), pack_pair<DT>(acc[6], acc[7])};
  ((u32x4_t*)p.y)[o] = r;
}

}  // namespace
}  // namespace llc

using namespace llc;

int llc_impl_max_pool(const llc_tensor* x, const llc_pool_attrs* at, llc_tensor* out, void* stream) {
  View a, o;
  LLC_TRY(make_view(x, "max_pool input", &a));
  LLC_TRY(make_view(out, "max_pool output", &o));
  if (!at) return set_error(LLC_ERR_BAD_ARG, "max_pool: null attributes");
  if (a.dtype != o.dtype) return set_error(LLC_ERR_DTYPE, "max_pool: input and output types differ");
  if (a.dtype != LLC_FLOAT32 && a.dtype != LLC_BFLOAT16 && a.dtype != LLC_FLOAT16)
    return set_error(LLC_ERR_DTYPE, "max_pool: element type %d", a.dtype);
  if (a.rank != 4 || o.rank != 4) return set_error(LLC_ERR_SHAPE, "max_pool: NCHW tensors expected");
  // Layout travels in the strides, as for the convolution: both tensors NCHW-contiguous, or both channels-last.
  auto channels_last = [](const View& v) {
    const int64_t C = v.size[1], H = v.size[2], W = v.size[3];
    return (C == 1 || v.stride[1] == 1) && (W == 1 || v.stride[3] == C) && (H == 1 || v.stride[2] == W * C) &&
           (v.size[0] == 1 || v.stride[0] == H * W * C);
  };
  const bool nhwc = !(a.contiguous() && o.contiguous()) && channels_last(a) && channels_last(o);
  if (!nhwc && (!a.contiguous() || !o.contiguous()))
    return set_error(LLC_ERR_LAYOUT, "max_pool: tensors must both be contiguous (NCHW) or both channels-last");
  if (nhwc && (a.size[1] % (16 / a.esize()) != 0 || ((uintptr_t)a.ptr | (uintptr_t)o.ptr) % 16 != 0))
    return set_error(LLC_ERR_UNSUPPORTED, "max_pool: channels-last tensors need 16-byte runs of channels (C %% %d == 0) and 16-byte alignment",
                     (int)(16 / a.esize()));
  for (int i = 0; i < 2; ++i)
    if (at->kernel_shape[i] <= 0 || at->stride[i] <= 0 || at->dilation[i] <= 0 || at->pad[i] < 0 || at->pad[i + 2] < 0)
      return set_error(LLC_ERR_BAD_ARG, "max_pool: bad window attributes");
  // LLHinfersymbolShape.cpp:257-268 (the pooling rule shares the convolution formula)
  const int64_t OH = (a.size[2] + at->pad[0] + at->pad[2] - at->dilation[0] * (at->kernel_shape[0] - 1) - 1) / at->stride[0] + 1;
  const int64_t OW = (a.size[3] + at->pad[1] + at->pad[3] - at->dilation[1] * (at->kernel_shape[1] - 1) - 1) / at->stride[1] + 1;
  if (o.size[0] != a.size[0] || o.size[1] != a.size[1] || o.size[2] != OH || o.size[3] != OW)
    return set_error(LLC_ERR_SHAPE, "max_pool: output is %lldx%lldx%lldx%lld, expected %lldx%lldx%lldx%lld",
                     (long long)o.size[0], (long long)o.size[1], (long long)o.size[2], (long long)o.size[3],
                     (long long)a.size[0], (long long)a.size[1], (long long)OH, (long long)OW);
  PoolParams p{};
  p.x = a.ptr;
  p.y = o.ptr;
  p.dtype = a.dtype;
  p.H = (int)a.size[2];
  p.W = (int)a.size[3];
  p.OH = (int)OH;
  p.OW = (int)OW;
  p.KH = (int)at->kernel_shape[0];
  p.KW = (int)at->kernel_shape[1];
  p.ph = (int)at->pad[0];
  p.pw = (int)at->pad[1];
  p.sh = (int)at->stride[0];
  p.sw = (int)at->stride[1];
  p.dh = (int)at->dilation[0];
  p.dw = (int)at->dilation[1];
  p.init_zero = at->init_zero;
  p.total = o.numel();
  p.C = (int)a.size[1];
  if (p.total == 0) return LLC_OK;
  if (nhwc) p.total /= 16 / a.esize();
  const int64_t blocks = (p.total + 255) / 256;
  if (blocks > 0x7fffffff) return set_error(LLC_ERR_TOO_LARGE, "max_pool: output too large");
  hipStream_t s = as_stream(stream);
  const bool k3 = p.KH == 3 && p.KW == 3, k2 = p.KH == 2 && p.KW == 2;
  if (nhwc) {
#define LLC_POOL_LAUNCH_NHWC(DT)                                                                                    \
  if (k3) hipLaunchKernelGGL((max_pool_nhwc_kernel<DT, 3>), dim3((unsigned)blocks), dim3(256), 0, s, p);            \
  else if (k2) hipLaunchKernelGGL((max_pool_nhwc_kernel<DT, 2>), dim3((unsigned)blocks), dim3(256), 0, s, p);       \
  else hipLaunchKernelGGL((max_pool_nhwc_kernel<DT, 0>), dim3((unsigned)blocks), dim3(256), 0, s, p);
    if (a.dtype == LLC_FLOAT32) { LLC_POOL_LAUNCH_NHWC(LLC_FLOAT32) }
    else if (a.dtype == LLC_BFLOAT16) { LLC_POOL_LAUNCH_NHWC(LLC_BFLOAT16) }
    else { LLC_POOL_LAUNCH_NHWC(LLC_FLOAT16) }
#undef LLC_POOL_LAUNCH_NHWC
    return check_launch("max_pool_nhwc_kernel");
  }
#define LLC_POOL_LAUNCH(DT)                                                                                         \
  if (k3) hipLaunchKernelGGL((max_pool_kernel<DT, 3>), dim3((unsigned)blocks), dim3(256), 0, s, p);                 \
  else if (k2) hipLaunchKernelGGL((max_pool_kernel<DT, 2>), dim3((unsigned)blocks), dim3(256), 0, s, p);            \
  else hipLaunchKernelGGL((max_pool_kernel<DT, 0>), dim3((unsigned)blocks), dim3(256), 0, s, p);
  if (a.dtype == LLC_FLOAT32) { LLC_POOL_LAUNCH(LLC_FLOAT32) }
  else if (a.dtype == LLC_BFLOAT16) { LLC_POOL_LAUNCH(LLC_BFLOAT16) }
  else { LLC_POOL_LAUNCH(LLC_FLOAT16) }
#undef LLC_POOL_LAUNCH
  return check_launch("max_pool_kernel");
}
