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
constexpr int kRowsLdsAll = kRowsLds + 256;  // and the bias of the channels-last form

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

template <typename TO, bool NHWC>
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
    const int kc = in ? k : 0;
    // every load is issued, from an index inside the filter: a load under a test would be a branch with its own wait
    const float wv = ((const float*)p.W)[(int64_t)f * p.Kdim + kc];
    bw[s] = in ? wv : 0.0f;
    const int c = kc / (p.KH * p.KW), rem = kc - c * (p.KH * p.KW);
    const int kh = rem / p.KW, kw = rem - kh * p.KW;
    // pixel i of block 0 reads column 2 i + kw - pw of row (c, kh); a k past the reduction reads row 0 (times weight 0)
    kaddr[s] = lds0 + kRowsLead + (uint32_t)((c * p.KH + kh) * kRowsPitch) + (uint32_t)((2 * li + kw - p.pw) * 4);
  }
  // channels-last results: the operands trade places, so a lane's four accumulators of a block are filters
  // 16 wave + 4 kk .. + 3 of pixel li, 16 bytes of that pixel's 256
  // (their bias waits in LDS behind the row buffers: four more registers would not fit)
  float tie_b = (p.bias && !NHWC) ? load_as_f32(p.bias, Elem<TO>::kDtype, f) : 0.0f;
  if (NHWC && threadIdx.x < 64) ((float*)(smem + kRowsLds))[threadIdx.x] = p.bias ? load_as_f32(p.bias, Elem<TO>::kDtype, threadIdx.x) : 0.0f;
  // the lead-in of both buffers and whatever the loads never write stays zero
  for (int i = threadIdx.x; i < kRowsLds / 4; i += 256) ((uint32_t*)smem)[i] = 0u;
  __builtin_amdgcn_s_waitcnt(0);  // weights and bias are here, the zeros are written
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

  // Workgroups are dealt to the eight XCDs in turn (workgroup b runs on XCD b % 8), and neighbouring output rows share
  // most of their input rows: each XCD walks one contiguous eighth of the rows, so that the shared input rows meet in
  // its L2 (with rows b, b + 512, ... per workgroup every XCD fetched input rows none of its other rows needed: 34 MB
  // for 9.6 MB of image).
  const bool by_xcd = gridDim.x % 8 == 0;
  const int share = by_xcd ? (total + 7) / 8 : total, stride = by_xcd ? (int)gridDim.x / 8 : (int)gridDim.x;
  const int r_first = by_xcd ? ((int)blockIdx.x % 8) * share : 0;
  const int r_end = r_first + share < total ? r_first + share : total;
  int r = r_first + (by_xcd ? (int)blockIdx.x / 8 : (int)blockIdx.x);
  if (r < r_end) fetch(r, 0);
  __builtin_amdgcn_s_waitcnt(0 | (7 << 4) | (15 << 8) | (0 << 14));  // vmcnt(0)
  int buf = 0;
  for (; r < r_end; r += stride, buf ^= 1) {
    // every wave has waited for its own loads of this row's patch, and has finished reading the other buffer
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    const int rn = r + stride;
    if (rn < r_end) fetch(rn, buf ^ 1);

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
        for (int s = 0; s < CNT; ++s) {
          if constexpr (NHWC) acc[PB] = __builtin_amdgcn_mfma_f32_16x16x4f32(bw[S0 + s], av[U & 1][s], acc[PB], 0, 0, 0);
          else acc[PB] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[U & 1][s], bw[S0 + s], acc[PB], 0, 0, 0);
        }
      });
    };
    if (buf == 0) row(std::integral_constant<int, 0>{});
    else row(std::integral_constant<int, 1>{});

    // The next row's loads went out a whole row of MFMAs ago and the previous row's stores before them: waiting for
    // all of them here costs nothing, and leaves only this row's stores in flight at the barrier.
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_waitcnt(0 | (7 << 4) | (15 << 8) | (0 << 14));  // vmcnt(0)
    __builtin_amdgcn_sched_barrier(0);
    // ---- act(alpha acc + bias) -> y[n][f][oh][16 pb + 4 kk .. + 3], or y[n][oh][16 pb + li][16 wave + 4 kk .. + 3] ----
    const int n = r / p.OH, oh = r - n * p.OH;
    TO* yrow = NHWC ? (TO*)p.Y + ((int64_t)r * p.OW) * p.F + 16 * wave + 4 * kk
                    : (TO*)p.Y + (((int64_t)n * p.F + f) * p.OH + oh) * p.OW;
    f32x4_t b4 = {tie_b, tie_b, tie_b, tie_b};
    if constexpr (NHWC) b4 = *(const f32x4_t*)(smem + kRowsLds + (16 * wave + 4 * kk) * 4);
#pragma unroll
    for (int b = 0; b < kRowsBlocks; ++b) {
      const int ow = NHWC ? 16 * b + li : 16 * b + 4 * kk;
      f32x4_t o;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float v = acc[b][e] * p.alpha + b4[e];
        if (p.act == LLC_ACT_RELU) v = v < 0.0f ? 0.0f : v;
        else if (p.act == LLC_ACT_GELU) v = gelu_exact(v);
        o[e] = v;
      }
      if (ow < p.OW) {
        TO* dst = NHWC ? yrow + (int64_t)ow * p.F : yrow + ow;
        if constexpr (sizeof(TO) == 4) *(f32x4_t*)dst = o;
        else *(uint2*)dst = uint2{pack_pair<Elem<TO>::kDtype>(o[0], o[1]), pack_pair<Elem<TO>::kDtype>(o[2], o[3])};
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

template <typename TO, bool NHWC>
int launch_conv_rows_as(const ConvParams& p, hipStream_t s) {
  auto kern = conv_rows_f32_kernel<TO, NHWC>;
  static std::atomic<uint32_t> lds_allowed{0};
  LLC_TRY(allow_dynamic_lds((const void*)kern, kRowsLdsAll, lds_allowed));
  const int64_t total = (int64_t)p.N * p.OH;
  const unsigned wgs = (unsigned)(total < 512 ? total : 512);  // two workgroups per CU, each walking rows wgs apart
  hipLaunchKernelGGL(kern, dim3(wgs), dim3(256), kRowsLdsAll, s, p);
  return check_launch("conv_rows_f32_kernel");
}
template <typename TO>
int launch_conv_rows(const ConvParams& p, hipStream_t s) {
  return p.y_nhwc ? launch_conv_rows_as<TO, true>(p, s) : launch_conv_rows_as<TO, false>(p, s);
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

// ---- the same layer in 16-bit storage, on the 16-bit matrix instruction ----
//
// v_mfma_f32_16x16x32 takes eight consecutive k per lane.  With k ordered (channel, window row, window column) those
// eight are the window columns of one (channel, window row): 16 consecutive bytes of that input row in LDS, starting at
// column 2 pixel - pad.  The start has to be a whole dword, so for an odd pad the run begins one column early and the
// filters carry a zero in front (a 7-wide window with pad 3 fills the eight slots exactly); columns of the run outside
// the window are also cleared in the pixel operand, so that an Inf or NaN next to a window does not reach its sum.  A
// k-step is four (channel, window row) pairs, one per quarter wave, and there are always six k-steps: pairs past the
// last are rows of LDS nothing is loaded into.  Each wave owns pixel blocks wave and wave + 4 of the output row and all 64 filters (96 registers of
// filters, read once through LDS), so the pixel operand is read once per block.  Input rows arrive two per wave
// instruction (a row slot is 512 bytes: 256 values).  The matrix instructions of a row take a fraction of a memory
// round trip, so the rows of the next three iterations are in flight (a ring of four row buffers); every wave issues
// the same three loads per row, also for rows past the end (they fetch zeros), which is what lets the wait in front
// of a row be a count: all but the loads of the two rows behind it.
constexpr int kRows16Slots = 24;
constexpr int kRows16Pitch = 512;
constexpr int kRows16Lead = 128;
constexpr int kRows16Buf = kRows16Lead + kRows16Slots * kRows16Pitch;
constexpr int kRows16Ring = 4;            // row buffers: the rows three iterations ahead are in flight
constexpr int kRows16Loads = kRows16Slots / 8;  // direct-to-LDS loads per wave and row (two slots each, four waves)
constexpr int kRows16Lds = kRows16Ring * kRows16Buf;
static_assert(64 * kRows16Slots * 16 <= kRows16Lds, "the filters pass through the row buffers");

typedef uint32_t rows_u32x2_t __attribute__((ext_vector_type(2)));

__device__ __forceinline__ void rows16_read(rows_u32x2_t& lo, rows_u32x2_t& hi, uint32_t addr) {
  asm volatile("ds_read2_b32 %0, %2 offset1:1\n\tds_read2_b32 %1, %2 offset0:2 offset1:3" : "=&v"(lo), "=&v"(hi) : "v"(addr));
}

template <typename T, bool NHWC>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void conv_rows_16bit_kernel(const ConvParams p) {
  constexpr int DT = Elem<T>::kDtype;
  extern __shared__ __align__(16) char smem[];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave), lane = threadIdx.x % kWave;
  const int li = lane % 16, g = lane / 16;
  const int nrows = p.C * p.KH, shift = p.pw & 1;

  // ---- once: the filters as [64][24] runs of eight (zeros where the run leaves the window or the reduction) ----
#pragma unroll
  for (int v0 = 0; v0 < 64 * kRows16Slots; v0 += 256) {
    const int v = v0 + threadIdx.x;
    const int f = v / kRows16Slots, r = v - f * kRows16Slots;
    uint32_t e[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int kw = j - shift;
      const bool in = r < nrows && kw >= 0 && kw < p.KW;
      // every load is issued, from an index inside the filters: a load under a test would be a branch with its own wait
      const uint32_t wv = ((const uint16_t*)p.W)[in ? (int64_t)f * p.Kdim + r * p.KW + kw : 0];
      e[j] = in ? wv : 0u;
    }
    ((u32x4_t*)smem)[v] = u32x4_t{e[0] | e[1] << 16, e[2] | e[3] << 16, e[4] | e[5] << 16, e[6] | e[7] << 16};
  }
  __syncthreads();
  // filter operand of group fg, k-step s.  Channels-last results: the filters are the rows of the product, row li of
  // group fg is filter 16 (li / 4) + 4 fg + li % 4, which leaves a lane with 16 consecutive filters of one pixel.
  u32x4_t w[4][6];
#pragma unroll
  for (int fg = 0; fg < 4; ++fg) {
    const int fl = NHWC ? 16 * (li / 4) + 4 * fg + (li % 4) : 16 * fg + li;
#pragma unroll
    for (int s = 0; s < 6; ++s) w[fg][s] = ((const u32x4_t*)smem)[fl * kRows16Slots + 4 * s + g];
  }
  float bias[NHWC ? 16 : 4];
#pragma unroll
  for (int e = 0; e < (NHWC ? 16 : 4); ++e) bias[e] = 0.0f;
  if (p.bias) {  // one test around all the loads: they are in flight together
#pragma unroll
    for (int e = 0; e < (NHWC ? 16 : 4); ++e) bias[e] = load_as_f32(p.bias, DT, NHWC ? 16 * g + e : 16 * e + li);
  }
  // which halves of the run's four dwords lie inside the window
  uint32_t km[4];
#pragma unroll
  for (int d = 0; d < 4; ++d) {
    const int k0 = 2 * d - shift, k1 = 2 * d + 1 - shift;
    km[d] = ((k0 >= 0 && k0 < p.KW) ? 0x0000ffffu : 0u) | ((k1 >= 0 && k1 < p.KW) ? 0xffff0000u : 0u);
  }
  __syncthreads();
  // the lead-in of both buffers, the rows past the reduction and whatever the loads never write stay zero
  for (int i = threadIdx.x; i < kRows16Lds / 16; i += 256) ((u32x4_t*)smem)[i] = u32x4_t{0u, 0u, 0u, 0u};
  __builtin_amdgcn_s_waitcnt(0);
#pragma unroll
  for (int fg = 0; fg < 4; ++fg)
#pragma unroll
    for (int s = 0; s < 6; ++s) asm volatile("" : "+v"(w[fg][s]));
#pragma unroll
  for (int e = 0; e < (NHWC ? 16 : 4); ++e) asm volatile("" : "+v"(bias[e]));
  __syncthreads();

  const uint32_t lds0 = (uint32_t)(uintptr_t)smem;
  // pixel li of block 0, k-step 0: row slot g, column 2 li - pad - shift
  const uint32_t lane_addr = lds0 + kRows16Lead + (uint32_t)(g * kRows16Pitch) + (uint32_t)((2 * li - p.pw - shift) * 2);

  // ---- input rows of output row `r` into buffer `buf`: two patch rows per wave instruction, three instructions per
  //      wave whatever the row (slots past the reduction and rows past the end fetch zeros) ----
  const int total = p.N * p.OH;
  int row_limit = total;  // rows from here on fetch zeros (set below to the end of this workgroup's share)
  const int hl = lane / 32, l32 = lane % 32;
  auto fetch = [&](int r, int buf) {
    const int n = r / p.OH, oh = r - n * p.OH;
    const int ih0 = oh * p.sh - p.ph;
#pragma unroll
    for (int j = 0; j < kRows16Loads; ++j) {
      const int q = wave + 4 * j;
      const int pr = 2 * q + hl;
      const int c = pr / p.KH, kh = pr - c * p.KH;
      const int ih = ih0 + kh;
      const bool in = r < row_limit && pr < nrows && ih >= 0 && ih < p.H && 8 * l32 < p.Wd;
      const char* src = in ? p.X + ((((int64_t)n * p.C + c) * p.H + ih) * p.Wd) * 2 + l32 * 16
                           : (const char*)llc_conv_zero_row + (lane % 16) * 16;
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                       (__attribute__((address_space(3))) void*)(smem + buf * kRows16Buf + kRows16Lead + 2 * q * kRows16Pitch),
                                       16, 0, 0);
    }
  };
  const int nblk = (p.OW + 15) / 16;
  auto mma = [&](f32x4_t (&a)[4], const rows_u32x2_t (&lo)[6], const rows_u32x2_t (&hi)[6]) {
#pragma unroll
    for (int s = 0; s < 6; ++s) {
      const u32x4_t px = u32x4_t{lo[s][0] & km[0], lo[s][1] & km[1], hi[s][0] & km[2], hi[s][1] & km[3]};
#pragma unroll
      for (int fg = 0; fg < 4; ++fg) {
        if constexpr (DT == LLC_BFLOAT16) {
          if constexpr (NHWC)
            a[fg] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, w[fg][s]), __builtin_bit_cast(bf16x8_t, px), a[fg], 0, 0, 0);
          else
            a[fg] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, px), __builtin_bit_cast(bf16x8_t, w[fg][s]), a[fg], 0, 0, 0);
        } else {
          if constexpr (NHWC)
            a[fg] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_t, w[fg][s]), __builtin_bit_cast(f16x8_t, px), a[fg], 0, 0, 0);
          else
            a[fg] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_t, px), __builtin_bit_cast(f16x8_t, w[fg][s]), a[fg], 0, 0, 0);
        }
      }
    }
  };

  // Workgroups are dealt to the eight XCDs in turn (workgroup b runs on XCD b % 8), and neighbouring output rows share
  // six of their seven input rows per channel: each XCD walks one contiguous eighth of the rows, so that the shared input
  // rows meet in its L2 (with rows b, b + 512, ... per workgroup every XCD read input rows no other row of its own needed:
  // 17.4 MB fetched for 4.8 MB of image).
  const bool by_xcd = gridDim.x % 8 == 0;
  const int share = by_xcd ? (total + 7) / 8 : total, stride = by_xcd ? (int)gridDim.x / 8 : (int)gridDim.x;
  const int r_first = by_xcd ? ((int)blockIdx.x % 8) * share : 0;
  const int r_end = r_first + share < total ? r_first + share : total;
  row_limit = r_end;
  int r = r_first + (by_xcd ? (int)blockIdx.x / 8 : (int)blockIdx.x);
#pragma unroll
  for (int d = 0; d < kRows16Ring - 1; ++d) fetch(r + d * stride, d);
  int buf = 0;
  const bool two = wave + 4 < nblk;  // this wave's second pixel block exists
  // Vector memory operations leave the counter in the order they were issued.  Behind the loads of a row this wave has
  // issued the loads of the next two rows and the stores of the last two rows it finished (of fewer at the start):
  // the row is here when no more than those are still counted.  A block's stores are always issued (a block has at
  // least one pixel inside the row), 2 per block channels-last and 4 otherwise.
  const int row_stores = (two ? 2 : 1) * (NHWC ? 2 : 4);
  int done = 0;  // rows this wave has stored, up to 2
  for (; r < r_end; r += stride, buf = buf + 1 == kRows16Ring ? 0 : buf + 1) {
    __builtin_amdgcn_sched_barrier(0);
    switch (2 * kRows16Loads + done * row_stores) {
      case 6: __builtin_amdgcn_s_waitcnt(6 | (7 << 4) | (15 << 8)); break;
      case 8: __builtin_amdgcn_s_waitcnt(8 | (7 << 4) | (15 << 8)); break;
      case 10: __builtin_amdgcn_s_waitcnt(10 | (7 << 4) | (15 << 8)); break;
      case 14: __builtin_amdgcn_s_waitcnt(14 | (7 << 4) | (15 << 8)); break;
      case 22: __builtin_amdgcn_s_waitcnt((22 & 15) | (7 << 4) | (15 << 8) | ((22 >> 4) << 14)); break;
      default: __builtin_amdgcn_s_waitcnt(0 | (7 << 4) | (15 << 8)); break;
    }
    done = done < 2 ? done + 1 : 2;
    // past the barrier every wave's loads of the row are here, and every wave has read the previous row for the last time
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);

    f32x4_t acc[2][4];
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int fg = 0; fg < 4; ++fg) acc[b][fg] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
    const uint32_t row_addr = lane_addr + (uint32_t)(buf * kRows16Buf) + (uint32_t)(wave * 64);
    rows_u32x2_t lo0[6], hi0[6], lo1[6], hi1[6];
#pragma unroll
    for (int s = 0; s < 6; ++s) rows16_read(lo0[s], hi0[s], row_addr + (uint32_t)(s * 4 * kRows16Pitch));
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
#pragma unroll
    for (int s = 0; s < 6; ++s) asm volatile("" : "+v"(lo0[s]), "+v"(hi0[s]));
    // the second block's operand is on its way under the matrix instructions of the first
    if (two) {
#pragma unroll
      for (int s = 0; s < 6; ++s) rows16_read(lo1[s], hi1[s], row_addr + (uint32_t)(4 * 64 + s * 4 * kRows16Pitch));
    }
    mma(acc[0], lo0, hi0);
    if (two) {
      __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
#pragma unroll
      for (int s = 0; s < 6; ++s) asm volatile("" : "+v"(lo1[s]), "+v"(hi1[s]));
      mma(acc[1], lo1, hi1);
    }
    __builtin_amdgcn_sched_barrier(0);
    const int n = r / p.OH, oh = r - n * p.OH;
    // one test of the activation per row, not one per element
    auto finish = [&](auto act_tag) {
    constexpr int ACT = decltype(act_tag)::value;
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      const int pb = wave + 4 * b;
      if (pb >= nblk) continue;
      if constexpr (NHWC) {
        // lane: pixel 16 pb + li, filters 16 g .. 16 g + 15 (group fg, element e is filter 16 g + 4 fg + e)
        const int ow = 16 * pb + li;
        uint32_t o[8];
#pragma unroll
        for (int fg = 0; fg < 4; ++fg) {
          float v[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            float x = acc[b][fg][e] * p.alpha + bias[4 * fg + e];
            if constexpr (ACT == LLC_ACT_RELU) x = x < 0.0f ? 0.0f : x;
            else if constexpr (ACT == LLC_ACT_GELU) x = gelu_for<T>(x);
            v[e] = x;
          }
          o[2 * fg] = pack_pair<DT>(v[0], v[1]);
          o[2 * fg + 1] = pack_pair<DT>(v[2], v[3]);
        }
        if (ow < p.OW) {
          T* dst = (T*)p.Y + ((int64_t)r * p.OW + ow) * p.F + 16 * g;
          *(u32x4_t*)dst = u32x4_t{o[0], o[1], o[2], o[3]};
          *(u32x4_t*)(dst + 8) = u32x4_t{o[4], o[5], o[6], o[7]};
        }
      } else {
        // lane: filter 16 fg + li, pixels 16 pb + 4 g .. + 3
        const int ow = 16 * pb + 4 * g;
#pragma unroll
        for (int fg = 0; fg < 4; ++fg) {
          float v[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            float x = acc[b][fg][e] * p.alpha + bias[fg];
            if constexpr (ACT == LLC_ACT_RELU) x = x < 0.0f ? 0.0f : x;
            else if constexpr (ACT == LLC_ACT_GELU) x = gelu_for<T>(x);
            v[e] = x;
          }
          if (ow < p.OW)
            *(uint2*)((T*)p.Y + (((int64_t)n * p.F + 16 * fg + li) * p.OH + oh) * p.OW + ow) =
                uint2{pack_pair<DT>(v[0], v[1]), pack_pair<DT>(v[2], v[3])};
        }
      }
    }
    };
    if (p.act == LLC_ACT_RELU) finish(std::integral_constant<int, LLC_ACT_RELU>{});
    else if (p.act == LLC_ACT_GELU) finish(std::integral_constant<int, LLC_ACT_GELU>{});
    else finish(std::integral_constant<int, LLC_ACT_NONE>{});
    // into the buffer of the previous row, which every wave has left (the barrier above)
    __builtin_amdgcn_sched_barrier(0);
    fetch(r + (kRows16Ring - 1) * stride, buf == 0 ? kRows16Ring - 1 : buf - 1);
  }
  __builtin_amdgcn_s_waitcnt(0 | (7 << 4) | (15 << 8) | (0 << 14));  // the loads past the end have landed
}

// Whether the 16-bit row kernel takes this convolution (NCHW input, contiguous, checked by the caller).
inline bool conv_rows_16bit_ok(const ConvParams& p, int groups) {
  const int shift = p.pw & 1;
  if (groups != 1 || p.F != 64 || p.C * p.KH > kRows16Slots || p.KW + shift > 8 || p.residual) return false;
  if (p.sw != 2 || p.dh != 1 || p.dw != 1) return false;
  // a row and its right-hand zeros fit a 256-value slot whose tail is also the next row's left-hand padding
  if (p.Wd % 8 != 0 || p.Wd > 256 - (p.pw + shift) || (p.pw + shift) * 2 > kRows16Lead) return false;
  if (p.OW % 4 != 0 || p.OW > 128 || 2 * (16 * ((p.OW + 15) / 16) - 1) - p.pw - shift + 7 > 255) return false;
  if (((uintptr_t)p.X % 16) != 0 || ((uintptr_t)p.Y % 16) != 0 || ((uintptr_t)p.W % 2) != 0 ||
      (p.bias && ((uintptr_t)p.bias % 2) != 0))
    return false;
  return (int64_t)p.N * p.OH >= 256;  // rows enough for every CU
}

template <typename T, bool NHWC>
int launch_conv_rows_16bit_mfma_as(const ConvParams& p, hipStream_t s) {
  auto kern = conv_rows_16bit_kernel<T, NHWC>;
  const int64_t total = (int64_t)p.N * p.OH;
  const unsigned wgs = (unsigned)(total < 512 ? total : 512);
  hipLaunchKernelGGL(kern, dim3(wgs), dim3(256), kRows16Lds, s, p);
  return check_launch("conv_rows_16bit_kernel");
}
template <typename T>
int launch_conv_rows_16bit_mfma(const ConvParams& p, hipStream_t s) {
  return p.y_nhwc ? launch_conv_rows_16bit_mfma_as<T, true>(p, s) : launch_conv_rows_16bit_mfma_as<T, false>(p, s);
}
