// The first layer of an image network in fp32 NCHW: few input channels, a large window, stride 2 (3 x 7 x 7 -> 64 on
// 224 x 224).  Included by conv.hip inside namespace llc::{anonymous}.
//
// The reduction is only C*KH*KW = 147 long and the im2col matrix has no contiguous run longer than a window row, so
// the gather kernels spend their time on addresses.  Here nothing is gathered: a workgroup stays resident and walks
// output rows (n, oh); for each it needs the C*KH input rows under the window, which arrive as they lie in memory by
// direct-to-LDS loads (one row of up to 224 floats per wave instruction, lanes past the row's end fetch zeros, which
// is the right-hand padding and, seen from the next row, the left-hand one), double buffered.  The MFMA
// (v_mfma_f32_16x16x4_f32: 16 pixels x 16 filters x 4 k) takes its pixel operand straight from that patch: lane
// (pixel i, k slot kk) reads one float at  row(c, kh) * 1 KB + (2 (16 pb + i) + kw) * 4,  k = 4 s + kk, an address
// that is a per-lane constant for each k-step s plus an immediate for the pixel block pb.  Each of the 4 waves owns
// 16 filters and keeps their weights in 37 registers for the whole kernel; accumulators of a lane are 4 consecutive
// pixels of one filter, stored as 16 bytes into NCHW.
//
// 16-bit tensors take the same kernel (TO = their type): the image and the filters are first copied to fp32 in scratch
// memory (the image is 3 % of the layer's bytes), the products are the same fp32 ones the 16-bit matrix instruction
// would form, and the result is rounded once on its way out; the gather kernel this replaces takes twice as long.
//
// LDS reads are inline asm with hand-placed waits: with direct-to-LDS loads in flight the compiler would put
// s_waitcnt vmcnt(0) in front of every LDS read it knows about.

constexpr int kRowsSteps = 37;           // k-steps of 4: reductions up to 148
constexpr int kRowsPitch = 1024;         // bytes of LDS per input row (256 floats)
constexpr int kRowsLead = 128;           // zeroed bytes in front of the first row (the left padding of row 0)
constexpr int kRowsMaxRows = 21;         // C * KH
constexpr int kRowsBuf = kRowsLead + kRowsMaxRows * kRowsPitch;
constexpr int kRowsBlocks = 7;           // pixel blocks of 16 per output row: OW <= 112
constexpr int kRowsLds = 2 * kRowsBuf;

static __device__ __align__(256) unsigned char llc_conv_zero_row[256];

template <int OFF>
__device__ __forceinline__ void rows_lds_read(float& v, uint32_t addr) {
  asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF));
}
template <int N, typename F>
__device__ __forceinline__ void rows_static_for(F&& f) {
  if constexpr (N > 0) {
    rows_static_for<N - 1>(f);
    f(std::integral_constant<int, N - 1>{});
  }
}

template <typename TO>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void conv_rows_f32_kernel(const ConvParams p) {
  extern __shared__ __align__(16) char smem[];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave), lane = threadIdx.x % kWave;
  const int li = lane % 16, kk = lane / 16;
  const int nrows = p.C * p.KH;
  const float* X = (const float*)p.X;

  // ---- once: this wave's 16 filters (lane: filter 16 wave + li, k = 4 s + kk), its bias, the patch offset of every
  //      k-step; all of it in registers before the first direct-to-LDS load is issued ----
  const int f = 16 * wave + li;
  float bw[kRowsSteps];
  uint32_t kaddr[kRowsSteps];
  const uint32_t lds0 = (uint32_t)(uintptr_t)smem;
#pragma unroll
  for (int s = 0; s < kRowsSteps; ++s) {
    const int k = 4 * s + kk;
    const bool in = k < p.Kdim;
    bw[s] = in ? ((const float*)p.W)[(int64_t)f * p.Kdim + k] : 0.0f;
    const int kc = in ? k : 0;
    const int c = kc / (p.KH * p.KW), rem = kc - c * (p.KH * p.KW);
    const int kh = rem / p.KW, kw = rem - kh * p.KW;
    // pixel i of block 0 reads column 2 i + kw - pw of row (c, kh); a k past the reduction reads row 0 (times weight 0)
    kaddr[s] = lds0 + kRowsLead + (uint32_t)((c * p.KH + kh) * kRowsPitch) + (uint32_t)((2 * li + kw - p.pw) * 4);
  }
  const float bias = p.bias ? load_as_f32(p.bias, Elem<TO>::kDtype, f) : 0.0f;
  // the lead-in of both buffers and whatever the loads never write stays zero
  for (int i = threadIdx.x; i < kRowsLds / 4; i += 256) ((uint32_t*)smem)[i] = 0u;
  __builtin_amdgcn_s_waitcnt(0);  // weights and bias are here, the zeros are written
  float tie_b = bias;
  asm volatile("" : "+v"(tie_b));
#pragma unroll
  for (int s = 0; s < kRowsSteps; ++s) asm volatile("" : "+v"(bw[s]));
  __syncthreads();

  // ---- input rows of output row `r` into buffer `buf`: wave w brings patch rows w, w + 4, ... ----
  const int total = p.N * p.OH;
  auto fetch = [&](int r, int buf) {
    const int n = r / p.OH, oh = r - n * p.OH;
    const int ih0 = oh * p.sh - p.ph;
    for (int pr = wave; pr < nrows; pr += 4) {
      const int c = pr / p.KH, kh = pr - c * p.KH;
      const int ih = ih0 + kh;
      const bool in = ih >= 0 && ih < p.H && 4 * lane < p.Wd;
      const char* src = in ? (const char*)(X + (((int64_t)n * p.C + c) * p.H + ih) * p.Wd) + lane * 16
                           : (const char*)llc_conv_zero_row + (lane % 16) * 16;
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                       (__attribute__((address_space(3))) void*)(smem + buf * kRowsBuf + kRowsLead + pr * kRowsPitch),
                                       16, 0, 0);
    }
  };

  int r = blockIdx.x;
  if (r < total) fetch(r, 0);
  __builtin_amdgcn_s_waitcnt(0 | (7 << 4) | (15 << 8) | (0 << 14));  // vmcnt(0)
  int buf = 0;
  for (; r < total; r += gridDim.x, buf ^= 1) {
    // every wave has waited for its own loads of this row's patch, and has finished reading the other buffer
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    const int rn = r + gridDim.x;
    if (rn < total) fetch(rn, buf ^ 1);

    f32x4_t acc[kRowsBlocks];
#pragma unroll
    for (int b = 0; b < kRowsBlocks; ++b) acc[b] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
    // pixel operands of half a block (19 / 18 k-steps) at a time, the next half in flight under the MFMAs of this one
    constexpr int kHalf = (kRowsSteps + 1) / 2;
    float av[2][kHalf];
    auto read_half = [&](auto u_tag, auto buf_tag) {
      constexpr int U = decltype(u_tag)::value, PB = U / 2, S0 = (U % 2) * kHalf, BUF = decltype(buf_tag)::value;
      constexpr int CNT = (U % 2) ? kRowsSteps - kHalf : kHalf;
      rows_static_for<CNT>([&](auto s_tag) {
        constexpr int S = decltype(s_tag)::value;
        float& dst = av[U & 1][S];
        rows_lds_read<PB * 128 + BUF * kRowsBuf>(dst, kaddr[S0 + S]);
      });
    };
    auto row = [&](auto buf_tag) {
      read_half(std::integral_constant<int, 0>{}, buf_tag);
      rows_static_for<2 * kRowsBlocks>([&](auto u_tag) {
        constexpr int U = decltype(u_tag)::value, PB = U / 2, S0 = (U % 2) * kHalf;
        constexpr int CNT = (U % 2) ? kRowsSteps - kHalf : kHalf;
        __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
#pragma unroll
        for (int s = 0; s < CNT; ++s) asm volatile("" : "+v"(av[U & 1][s]));
        if constexpr (U + 1 < 2 * kRowsBlocks) read_half(std::integral_constant<int, U + 1>{}, buf_tag);
#pragma unroll
        for (int s = 0; s < CNT; ++s) acc[PB] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[U & 1][s], bw[S0 + s], acc[PB], 0, 0, 0);
      });
    };
    if (buf == 0) row(std::integral_constant<int, 0>{});
    else row(std::integral_constant<int, 1>{});

    // The next row's loads went out a whole row of MFMAs ago and the previous row's stores before them: waiting for
    // all of them here costs nothing, and leaves only this row's stores in flight at the barrier.
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_waitcnt(0 | (7 << 4) | (15 << 8) | (0 << 14));  // vmcnt(0)
    __builtin_amdgcn_sched_barrier(0);
    // ---- act(alpha acc + bias) -> y[n][f][oh][16 pb + 4 kk .. + 3] ----
    const int n = r / p.OH, oh = r - n * p.OH;
    TO* yrow = (TO*)p.Y + (((int64_t)n * p.F + f) * p.OH + oh) * p.OW;
#pragma unroll
    for (int b = 0; b < kRowsBlocks; ++b) {
      const int ow = 16 * b + 4 * kk;
      f32x4_t o;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float v = acc[b][e] * p.alpha + tie_b;
        if (p.act == LLC_ACT_RELU) v = v < 0.0f ? 0.0f : v;
        else if (p.act == LLC_ACT_GELU) v = gelu_exact(v);
        o[e] = v;
      }
      if (ow < p.OW) {
        if constexpr (sizeof(TO) == 4) *(f32x4_t*)(yrow + ow) = o;
        else *(uint2*)(yrow + ow) = uint2{pack_pair<Elem<TO>::kDtype>(o[0], o[1]), pack_pair<Elem<TO>::kDtype>(o[2], o[3])};
      }
    }
  }
}

// Whether the row kernel takes this convolution (NCHW, contiguous, checked by the caller).
inline bool conv_rows_ok(const ConvParams& p, int groups) {
  if (groups != 1 || p.F != 64 || p.Kdim > 4 * kRowsSteps || p.C * p.KH > kRowsMaxRows || p.residual) return false;
  if (p.sw != 2 || p.dh != 1 || p.dw != 1) return false;
  // a row and its right-hand zeros fit a 256-float slot whose tail is also the next row's left-hand padding
  if (p.Wd % 4 != 0 || p.Wd > 224 || p.pw > 256 - p.Wd || p.pw * 4 > kRowsLead) return false;
  if (p.OW % 4 != 0 || p.OW > 16 * kRowsBlocks || 2 * (16 * kRowsBlocks - 1) + p.KW - 1 - p.pw > 255) return false;
  if (((uintptr_t)p.X % 16) != 0 || ((uintptr_t)p.Y % 16) != 0) return false;
  return (int64_t)p.N * p.OH >= 256;  // rows enough for every CU
}

template <typename TO>
int launch_conv_rows(const ConvParams& p, hipStream_t s) {
  auto kern = conv_rows_f32_kernel<TO>;
  static std::atomic<uint32_t> lds_allowed{0};
  LLC_TRY(allow_dynamic_lds((const void*)kern, kRowsLds, lds_allowed));
  const int64_t total = (int64_t)p.N * p.OH;
  const unsigned wgs = (unsigned)(total < 512 ? total : 512);  // two workgroups per CU, each walking rows wgs apart
  hipLaunchKernelGGL(kern, dim3(wgs), dim3(256), kRowsLds, s, p);
  return check_launch("conv_rows_f32_kernel");
}

// 16-bit values to fp32, 8 per lane
template <typename T>
__global__ __launch_bounds__(256) void widen_to_f32_kernel(const T* __restrict__ in, float* __restrict__ out, int64_t n) {
  const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 8;
  if (i + 8 <= n) {
    const u32x4_t v = *(const u32x4_t*)(in + i);
    float f[8];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      if constexpr (Elem<T>::kDtype == LLC_BFLOAT16) {
        f[2 * e] = __uint_as_float(v[e] << 16);
        f[2 * e + 1] = __uint_as_float(v[e] & 0xffff0000u);
      } else {
        f[2 * e] = f16_bits_to_f32((uint16_t)(v[e] & 0xffffu));
        f[2 * e + 1] = f16_bits_to_f32((uint16_t)(v[e] >> 16));
      }
    }
    *(f32x4_t*)(out + i) = f32x4_t{f[0], f[1], f[2], f[3]};
    *(f32x4_t*)(out + i + 4) = f32x4_t{f[4], f[5], f[6], f[7]};
  } else {
    for (int64_t j = i; j < n; ++j) out[j] = load_as_f32((const char*)in, Elem<T>::kDtype, j);
  }
}

// The 16-bit form: fp32 copies of the image and the filters in scratch memory, then the row kernel with a 16-bit result.
template <typename T>
int launch_conv_rows_16bit(const ConvParams& p, hipStream_t s) {
  const int64_t nx = (int64_t)p.N * p.C * p.H * p.Wd, nw = (int64_t)p.F * p.Kdim;
  const size_t xbytes = ((size_t)nx * 4 + 255) / 256 * 256;
  void* ws = nullptr;
  LLC_TRY(get_workspace(xbytes + (size_t)nw * 4, &ws, s));
  float* x32 = (float*)ws;
  float* w32 = (float*)((char*)ws + xbytes);
  hipLaunchKernelGGL(widen_to_f32_kernel<T>, dim3((unsigned)((nx + 2047) / 2048)), dim3(256), 0, s, (const T*)p.X, x32, nx);
  hipLaunchKernelGGL(widen_to_f32_kernel<T>, dim3((unsigned)((nw + 2047) / 2048)), dim3(256), 0, s, (const T*)p.W, w32, nw);
  LLC_TRY(check_launch("widen_to_f32_kernel"));
  ConvParams q = p;
  q.X = (const char*)x32;
  q.W = (const char*)w32;
  return launch_conv_rows<T>(q, s);
}
