// Channels-last convolutions with stride 1 (the 3x3 layers inside a ResNet stage), any element type.  Included by
// conv.hip inside namespace llc::{anonymous}, after conv_rows.hpp.
//
// An implicit GEMM whose k-tiles are (tap, 128-byte channel block) reads every input element once per tap: nine times
// for a 3x3 window, from L2, which is what bounds the small layers (64 channels on 56 x 56 at batch 16 in bf16: 58 MB of
// gathered rows for 6.4 MB of image).  Here a workgroup owns 128 consecutive output pixels of one image and 64 filters,
// and parks the input patch under those pixels (their rows, the window's extra rows and columns, one 128-byte channel
// block per pixel) in LDS once per channel block: the pixel operand of tap (kh, kw) is then the same patch read at an
// address shifted by kh patch rows and kw pixels, a constant for the whole workgroup.  Only the filters still stream:
// a ring of 8 KB tiles (64 filters x 128 bytes of one tap and channel block), direct to LDS, a few taps ahead.
//
// Patch pixel q = (input row - first row) * PW + (input column + pad), PW = OW + KW - 1, lies at byte 128 q with its
// eight 16-byte chunks XOR-swizzled like the rows of a GEMM tile (consecutive pixels, which the 32 lanes of a fragment
// read, then fall in different banks); pixels outside the image are loaded from a row of zeros.  4 waves, wave tile 64 pixels x 32
// filters.  The filters' loads are counted by hand (two per wave and tile); the patch is waited for completely.

constexpr int kPatchMaxPix = 352;                      // patch pixels that fit: 44 KB
constexpr int kPatchBytes = kPatchMaxPix * 128;
constexpr int kPatchStages = 4;                        // filter tiles in the ring
constexpr int kPatchBTile = 64 * 128;
constexpr int kPatchLds = kPatchBytes + kPatchStages * kPatchBTile;
constexpr int kPatchOutPitch = 68;                     // floats per row of the epilogue's staging tile
static_assert(128 * kPatchOutPitch * 4 <= kPatchBytes, "the staging tile reuses the patch");

#define LLC_PATCH_GPTR(p) ((const __attribute__((address_space(1))) void*)(p))
#define LLC_PATCH_LPTR(p) ((__attribute__((address_space(3))) void*)(p))
// vmcnt <= VM and lgkmcnt <= 0 (gfx9 encoding), expcnt untouched
#define LLC_PATCH_WAIT(VM) __builtin_amdgcn_s_waitcnt(((VM) & 15) | (7 << 4) | (0 << 8) | (((VM) >> 4) << 14))

template <typename T>
__global__ __launch_bounds__(256) void conv_patch_kernel(const ConvParams p, int tiles_per_image, uint32_t pw_magic) {
  constexpr int ES = (int)sizeof(T);
  constexpr int CBE = 128 / ES;  // channels per block
  extern __shared__ __align__(16) char smem[];
  char* patch = smem;
  char* ring = smem + kPatchBytes;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave), lane = threadIdx.x % kWave;
  const int wm = wave >> 1, wn = wave & 1;
  const int li = lane % 32, lh = lane / 32;
  const int n = blockIdx.x / tiles_per_image, tp = blockIdx.x - n * tiles_per_image;
  const int f0 = blockIdx.y * 64;
  const int ohw = p.OH * p.OW;
  const int p0 = tp * 128;                                   // first output pixel of the tile, inside image n
  const int p_last = (p0 + 127 < ohw ? p0 + 127 : ohw - 1);
  const int r_first = p0 / p.OW, r_last = p_last / p.OW;
  const int PW = p.OW + p.KW - 1;
  const int prows = r_last - r_first + p.KH;                 // patch rows
  const int npix = prows * PW;                               // patch pixels (<= kPatchMaxPix, checked by the host)
  const int ir0 = r_first - p.ph;                            // input row of patch row 0 (stride 1)
  const int ntaps = p.KH * p.KW, ncb = p.C / CBE;
  const char* Ximg = p.X + (int64_t)n * p.H * p.Wd * p.C * ES;

  // ---- fragment addresses.  Row block i of this wave: output pixel p0 + 64 wm + 32 i + li (the last tile of an image
  //      may run past its end: those lanes read the last pixel and store nothing) ----
  int pb[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    int m = p0 + wm * 64 + i * 32 + li;
    m = m < ohw ? m : ohw - 1;
    const int r = m / p.OW, c = m - r * p.OW;
    pb[i] = (r - r_first) * PW + c;
  }
  int ob[4];
#pragma unroll
  for (int s = 0; s < 4; ++s) {
    const int rb = wn * 32 + li;
    ob[s] = rb * 128 + (((2 * s + lh) ^ lds_swz(rb)) << 4);
  }
  // filter tile loads: rows 8 (wave + 4 j) + lane / 8 of the 64 filters, j = 0, 1
  const char* gb[2];
  int lb[2];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int row = (wave + 4 * j) * 8 + lane / 8;
    gb[j] = p.W + ((int64_t)(f0 + row) * p.Kdim) * ES + (((lane % 8) ^ lds_swz(row)) << 4);
    lb[j] = (wave + 4 * j) * 8 * 128;
  }
  auto issue_b = [&](int stage, int tap, int cb) {
    const int64_t koff = ((int64_t)tap * p.C + cb * CBE) * ES;
#pragma unroll
    for (int j = 0; j < 2; ++j)
      __builtin_amdgcn_global_load_lds(LLC_PATCH_GPTR(gb[j] + koff), LLC_PATCH_LPTR(ring + stage * kPatchBTile + lb[j]), 16, 0, 0);
  };
  // the patch of channel block cb: 8 pixels per wave instruction, instructions dealt to the waves in turn
  auto issue_patch = [&](int cb) {
    for (int g = wave; g * 8 < npix; g += 4) {
      const int q = g * 8 + lane / 8;
      const int prow = (int)(((uint32_t)q * pw_magic) >> 16), pcol = q - prow * PW;
      const int ir = ir0 + prow, ic = pcol - p.pw;
      const bool inside = q < npix && ir >= 0 && ir < p.H && ic >= 0 && ic < p.Wd;
      const char* src = inside ? Ximg + (((int64_t)ir * p.Wd + ic) * p.C + cb * CBE) * ES + (((lane % 8) ^ lds_swz(q)) << 4)
                               : (const char*)llc_conv_zero_row + (lane % 8) * 16;
      __builtin_amdgcn_global_load_lds(LLC_PATCH_GPTR(src), LLC_PATCH_LPTR(patch + g * 1024), 16, 0, 0);
    }
  };
  auto wait_tiles = [&](int tiles) {  // at most `tiles` filter tiles of this wave's loads (two each) still in flight
    switch (tiles) {
      case 1: LLC_PATCH_WAIT(2); break;
      case 2: LLC_PATCH_WAIT(4); break;
      case 3: LLC_PATCH_WAIT(6); break;
      default: LLC_PATCH_WAIT(0); break;
    }
  };

  f32x16_t acc[2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[i][r] = 0.0f;
  u32x4_t fa[2][4][2], fb[2][4];  // [set][k step][row block]

  // fragments of tap `tap` (filter tile in ring stage `stage`) into set SET
#define LLC_PATCH_READ(SET, TAP, STAGE)                                                                  \
  {                                                                                                      \
    const int kh_ = (TAP) / p.KW, kw_ = (TAP) - kh_ * p.KW;                                              \
    const int shift_ = kh_ * PW + kw_;                                                                   \
    const char* bt_ = ring + (STAGE) * kPatchBTile;                                                      \
    _Pragma("unroll") for (int i = 0; i < 2; ++i) {                                                      \
      const int q_ = pb[i] + shift_;                                                                     \
      const char* row_ = patch + q_ * 128;                                                               \
      const int key_ = lds_swz(q_);                                                                      \
      _Pragma("unroll") for (int s = 0; s < 4; ++s)                                                      \
          fa[SET][s][i] = *(const u32x4_t*)(row_ + (((2 * s + lh) ^ key_) << 4));                        \
    }                                                                                                    \
    _Pragma("unroll") for (int s = 0; s < 4; ++s) fb[SET][s] = *(const u32x4_t*)(bt_ + ob[s]);           \
  }
#define LLC_PATCH_MMA(SET)                                                                               \
  _Pragma("unroll") for (int s = 0; s < 4; ++s) {                                                        \
    if constexpr (ES == 4) {                                                                             \
      /* consecutive MFMAs write different accumulators: none waits for the one before it */            \
      _Pragma("unroll") for (int q = 0; q < 4; ++q) _Pragma("unroll") for (int i = 0; i < 2; ++i)        \
          acc[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(fa[SET][s][i][q]),               \
                                                        __uint_as_float(fb[SET][s][q]), acc[i], 0, 0, 0); \
    } else {                                                                                             \
      _Pragma("unroll") for (int i = 0; i < 2; ++i) mfma_step<T>(fa[SET][s][i], fb[SET][s], acc[i]);     \
    }                                                                                                    \
  }
#define LLC_PATCH_STEP(TT, SET)                                                                          \
  {                                                                                                      \
    const int issued_ = (TT) + kPatchStages < ntaps ? (TT) + kPatchStages : ntaps;                       \
    const int behind_ = issued_ - ((TT) + 2);                                                            \
    wait_tiles(behind_ > 0 ? behind_ : 0);                                                               \
    __builtin_amdgcn_s_barrier();                                                                        \
    if ((TT) + kPatchStages < ntaps) issue_b(st, (TT) + kPatchStages, cb);                               \
    st = st + 1 == kPatchStages ? 0 : st + 1;                                                            \
    if ((TT) + 1 < ntaps) LLC_PATCH_READ((SET) ^ 1, (TT) + 1, st)                                        \
    LLC_PATCH_MMA(SET)                                                                                   \
  }

  for (int cb = 0; cb < ncb; ++cb) {
    // every wave has read the previous patch and filter tiles for the last time
    if (cb > 0) {
      LLC_PATCH_WAIT(0);
      __builtin_amdgcn_s_barrier();
    }
    issue_patch(cb);
#pragma unroll
    for (int x = 0; x < kPatchStages; ++x)
      if (x < ntaps) issue_b(x, x, cb);
    LLC_PATCH_WAIT(0);
    __builtin_amdgcn_s_barrier();
    LLC_PATCH_READ(0, 0, 0)
    int st = 0;
    for (int t = 0; t < ntaps; t += 2) {
      LLC_PATCH_STEP(t, 0)
      if (t + 1 < ntaps) LLC_PATCH_STEP(t + 1, 1)
    }
  }
#undef LLC_PATCH_READ
#undef LLC_PATCH_MMA
#undef LLC_PATCH_STEP

  // ---- epilogue: the tile to LDS as fp32 [128][kPatchOutPitch] over the patch, then whole 16-byte stores along the
  //      filters of a pixel ----
  LLC_PATCH_WAIT(0);
  __syncthreads();  // every wave has read the patch for the last time
  float* stage = (float*)smem;
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int row = wm * 64 + i * 32 + (r / 4) * 8 + lh * 4 + (r % 4);
      stage[row * kPatchOutPitch + wn * 32 + li] = acc[i][r];
    }
  __syncthreads();
  constexpr int EPV = 16 / ES;           // outputs per 16-byte store
  constexpr int CPR = 64 / EPV;          // stores per pixel
  const int64_t img_off = (int64_t)n * ohw;
  // bias and residual of every pass are requested before the first pass stores: inside the loop each pass's loads waited
  // behind the stores of the pass before, which may alias them (a lane's filters are the same in every pass; rows past
  // the image read its last pixel and are not stored)
  constexpr int NIT = 128 * CPR / 256;
  u32x4_t bq_all = {0, 0, 0, 0}, rq_all[NIT];
#pragma unroll
  for (int it = 0; it < NIT; ++it) rq_all[it] = u32x4_t{0, 0, 0, 0};
  {
    const int lc0 = (threadIdx.x % CPR) * EPV;
    if (p.bias) bq_all = *(const u32x4_t*)((const char*)p.bias + (int64_t)(f0 + lc0) * ES);
    if (p.residual) {
#pragma unroll
      for (int it = 0; it < NIT; ++it) {
        const int prow = p0 + it * (256 / CPR) + threadIdx.x / CPR;
        rq_all[it] = *(const u32x4_t*)((const char*)p.residual + ((img_off + (prow < ohw ? prow : ohw - 1)) * p.F + f0 + lc0) * ES);
      }
    }
  }
#pragma unroll
  for (int it = 0; it < NIT; ++it) {
    const int vid = it * 256 + threadIdx.x;
    const int row = vid / CPR, c0 = (vid % CPR) * EPV;
    if (p0 + row >= ohw) continue;
    const float* s0 = stage + row * kPatchOutPitch + c0;
    const int64_t o = (img_off + p0 + row) * p.F + f0 + c0;
    if constexpr (ES == 4) {
      const f32x4_t x = *(const f32x4_t*)s0;
      const f32x4_t b = __builtin_bit_cast(f32x4_t, bq_all), rr = __builtin_bit_cast(f32x4_t, rq_all[it]);
      f32x4_t outv;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float v = x[e] * p.alpha + b[e] + rr[e];
        if (p.act == LLC_ACT_RELU) v = v < 0.0f ? 0.0f : v;
        else if (p.act == LLC_ACT_GELU) v = gelu_exact(v);
        outv[e] = v;
      }
      *(f32x4_t*)((float*)p.Y + o) = outv;
    } else {
      const f32x4_t x0 = *(const f32x4_t*)s0, x1 = *(const f32x4_t*)(s0 + 4);
      const float v[8] = {x0[0], x0[1], x0[2], x0[3], x1[0], x1[1], x1[2], x1[3]};
      const u32x4_t bq = bq_all, rq = rq_all[it];
      float xs[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const uint16_t bb = (uint16_t)(bq[e / 2] >> (16 * (e & 1))), rb = (uint16_t)(rq[e / 2] >> (16 * (e & 1)));
        float x = v[e] * p.alpha;
        if constexpr (Elem<T>::kDtype == LLC_BFLOAT16) x += bf16_bits_to_f32(bb);
        else x += f16_bits_to_f32(bb);
        if (p.residual) x += (Elem<T>::kDtype == LLC_BFLOAT16) ? bf16_bits_to_f32(rb) : f16_bits_to_f32(rb);
        if (p.act == LLC_ACT_RELU) x = x < 0.0f ? 0.0f : x;
        else if (p.act == LLC_ACT_GELU) x = gelu_exact(x);
        xs[e] = x;
      }
      *(u32x4_t*)((T*)p.Y + o) = u32x4_t{pack_pair<Elem<T>::kDtype>(xs[0], xs[1]), pack_pair<Elem<T>::kDtype>(xs[2], xs[3]),
                                        pack_pair<Elem<T>::kDtype>(xs[4], xs[5]), pack_pair<Elem<T>::kDtype>(xs[6], xs[7])};
    }
  }
}

// Whether the patch kernel takes this channels-last convolution (group 1 and 16-byte alignment checked by the caller).
template <typename T>
inline bool conv_patch_ok(const ConvParams& p) {
  constexpr int CBE = 128 / (int)sizeof(T);
  if (p.sh != 1 || p.sw != 1 || p.dh != 1 || p.dw != 1 || p.KH * p.KW < 2 || p.KH * p.KW > 25) return false;
  // measured against conv_nhwc_kernel at batch 16: 64 channels in 16-bit storage (one channel block) on 56 x 56 13.9
  // against 17.0 us; two blocks (128 channels in 16 bits on 28 x 28: 17.9 against 17.3 us; 64 channels in fp32 on
  // 56 x 56: 51.9 against 53.2 us, 128 on 28 x 28: 57.7 against 53.5 us) gain nothing: one block only
  if (p.C != CBE || sizeof(T) != 2 || p.F % 64 != 0) return false;
  const int ohw = p.OH * p.OW;
  if (ohw < 128) return false;
  const int PW = p.OW + p.KW - 1;
  const int span = (127 + p.OW - 1) / p.OW + 1;  // output rows 128 consecutive pixels can touch
  if ((span + p.KH - 1) * PW > kPatchMaxPix) return false;
  const int64_t tiles = (int64_t)p.N * ((ohw + 127) / 128) * (p.F / 64);
  // enough workgroups for the chip, and few enough steps per workgroup that the walk stays short
  return tiles >= 192 && tiles <= 0x7fffffff && (int64_t)p.KH * p.KW * (p.C / CBE) <= 40 && p.F / 64 <= 65535;
}

template <typename T>
int launch_conv_patch(const ConvParams& p, hipStream_t s) {
  auto kern = conv_patch_kernel<T>;
  static std::atomic<uint32_t> lds_allowed{0};
  LLC_TRY(allow_dynamic_lds((const void*)kern, kPatchLds, lds_allowed));
  const int tpi = (p.OH * p.OW + 127) / 128;
  const int PW = p.OW + p.KW - 1;
  const uint32_t magic = (65536u + (uint32_t)PW - 1u) / (uint32_t)PW;  // q / PW == (q * magic) >> 16 for q < 512
  hipLaunchKernelGGL(kern, dim3((unsigned)(p.N * tpi), (unsigned)(p.F / 64)), dim3(256), kPatchLds, s, p, tpi, magic);
  return check_launch("conv_patch_kernel");
}
