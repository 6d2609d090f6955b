// Small 16-bit products whose time is latency, not arithmetic: x [M, K] times a linear layer's weight [N, K] with a few
// hundred rows (an encoder block at a batch of one: 512 x 768 x 768 is 0.6 GFLOP, 0.3 us of matrix time).  Included by
// gemm.hip inside namespace llc::{anonymous}.
//
// The 64 x 64 tile kernel keeps one k-tile in flight ahead of the one it multiplies, so every k-tile costs most of a
// trip to L2 (0.8 us measured; 12 of them at K = 768).  Here a workgroup (4 waves, 32 x 32 each) owns the same 64 x 64
// tile but a ring of NS stages of 16 KB (64 rows x 128 bytes of A, then of B, 16-byte chunks XOR-swizzled by the row)
// filled by direct-to-LDS loads: NS - 1 k-tiles are on their way while one is multiplied, the trip is paid once, and a
// k-tile then costs its LDS reads, four MFMAs and a barrier.  Every wave issues exactly four loads per k-tile (rows
// 8 (wave + 4 j) + lane / 8 of A and of B, j = 0, 1), so "k-tile t + 1 has landed" is a count of this wave's loads still
// allowed in flight, waited for by hand, followed by the barrier that makes it true for the other waves' loads.

constexpr int kDeepStage = 16384;  // bytes of one stage: A tile, then B tile
constexpr int kDeepBOff = 8192;
constexpr int kDeepOutPitch = 68;  // floats per row of the epilogue's staging tile

template <typename T, int NS>
__global__ __launch_bounds__(256) void gemm_deep_kernel(const GemmParams p) {
  static_assert(sizeof(T) == 2, "16-bit operands");
  static_assert(NS >= 3 && NS <= 8, "wait_tiles knows up to seven k-tiles in flight");
  extern __shared__ __align__(16) char smem[];
  int tile_m, tile_n, z;
  tile_and_batch_of_block(p.tiles_m, p.tiles_n, tile_m, tile_n, z);
  const int m0 = tile_m * 64, n0 = tile_n * 64;
  const int z0 = z / p.bdiv, z1 = z - z0 * p.bdiv;
  const T* A = (const T*)p.A + (int64_t)z0 * p.a_sb + (int64_t)z1 * p.a_sb1;
  const T* B = (const T*)p.B + (int64_t)z0 * p.b_sb + (int64_t)z1 * p.b_sb1;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave), lane = threadIdx.x % kWave;
  const int wm = wave >> 1, wn = wave & 1;
  const int li = lane % 32, lh = lane / 32;

  const char* ga[2];
  const char* gb[2];
  int la[2], oa[4], ob[4];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int r0 = (wave + 4 * j) * 8, row = r0 + lane / 8;
    const int chunk = ((lane % 8) ^ lds_swz(row)) << 3;  // elements
    ga[j] = (const char*)(A + (int64_t)(m0 + row) * p.a_sm + chunk);
    gb[j] = (const char*)(B + (int64_t)(n0 + row) * p.b_sn + chunk);
    la[j] = r0 * kRowStride;
  }
#pragma unroll
  for (int s = 0; s < 4; ++s) {
    const int ra = wm * 32 + li, rb = wn * 32 + li, chunk = 2 * s + lh;
    oa[s] = ra * kRowStride + ((chunk ^ lds_swz(ra)) << 4);
    ob[s] = kDeepBOff + rb * kRowStride + ((chunk ^ lds_swz(rb)) << 4);
  }
  auto issue = [&](int stage) {
    char* base = smem + stage * kDeepStage;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      __builtin_amdgcn_global_load_lds(LLC_GPTR(ga[j]), LLC_LPTR(base + la[j]), 16, 0, 0);
      ga[j] += 128;
    }
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      __builtin_amdgcn_global_load_lds(LLC_GPTR(gb[j]), LLC_LPTR(base + kDeepBOff + la[j]), 16, 0, 0);
      gb[j] += 128;
    }
  };
  // at most `tiles` k-tiles of this wave's loads (four each) may still be in flight; LDS reads are complete
  auto wait_tiles = [&](int tiles) {
    switch (tiles) {
      case 1: LLC_WAIT_VM_LGKM0(4); break;
      case 2: LLC_WAIT_VM_LGKM0(8); break;
      case 3: LLC_WAIT_VM_LGKM0(12); break;
      case 4: LLC_WAIT_VM_LGKM0(16); break;
      case 5: LLC_WAIT_VM_LGKM0(20); break;
      case 6: LLC_WAIT_VM_LGKM0(24); break;
      case 7: LLC_WAIT_VM_LGKM0(28); break;
      default: LLC_WAIT_VM_LGKM0(0); break;
    }
  };

  f32x16_t acc;
#pragma unroll
  for (int r = 0; r < 16; ++r) acc[r] = 0.0f;
  u32x4_t fa[2][4], fb[2][4];

  const int nk = p.K / 64;
#pragma unroll
  for (int x = 0; x < NS; ++x)
    if (x < nk) issue(x);
  wait_tiles((nk < NS ? nk : NS) - 1);  // tile 0 has landed: the tiles issued behind it may be in flight
  __builtin_amdgcn_s_barrier();
#define LLC_DEEP_READ(SET, STAGE)                                          \
  {                                                                        \
    const char* base = smem + (STAGE) * kDeepStage;                        \
    _Pragma("unroll") for (int s = 0; s < 4; ++s) {                        \
      fa[SET][s] = *(const u32x4_t*)(base + oa[s]);                        \
      fb[SET][s] = *(const u32x4_t*)(base + ob[s]);                        \
    }                                                                      \
  }
  LLC_DEEP_READ(0, 0)
  // Iteration t: tile t's fragments are in registers (set t & 1).  Tiles up to min(nk, t + NS) - 1 have been issued;
  // tile t + 1 has landed when no more than the tiles behind it are in flight.  After the barrier every wave has read
  // stage t % NS, which takes tile t + NS.
  int st = 0;
#define LLC_DEEP_STEP(TT, SET)                                             \
  {                                                                        \
    const int issued = (TT) + NS < nk ? (TT) + NS : nk;                    \
    const int behind = issued - ((TT) + 2);                                \
    wait_tiles(behind > 0 ? behind : 0);                                   \
    __builtin_amdgcn_s_barrier();                                          \
    if ((TT) + NS < nk) issue(st);                                         \
    st = st + 1 == NS ? 0 : st + 1;                                        \
    if ((TT) + 1 < nk) LLC_DEEP_READ((SET) ^ 1, st)                        \
    _Pragma("unroll") for (int s = 0; s < 4; ++s) mfma_step<T>(fa[SET][s], fb[SET][s], acc); \
  }
  for (int t = 0; t < nk; t += 2) {
    LLC_DEEP_STEP(t, 0)
    if (t + 1 < nk) LLC_DEEP_STEP(t + 1, 1)
  }
#undef LLC_DEEP_READ
#undef LLC_DEEP_STEP

  // ---- epilogue: the tile to LDS as fp32 [64][kDeepOutPitch], then row-major 16-byte stores.  The last barrier came
  //      after every wave's last fragment read, and no load is in flight. ----
  float* stage = (float*)smem;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int row = wm * 32 + (r / 4) * 8 + lh * 4 + (r % 4);
    stage[row * kDeepOutPitch + wn * 32 + li] = acc[r];
  }
  __syncthreads();
  const int64_t c_off = (int64_t)z0 * p.c_sb + (int64_t)z1 * p.c_sb1;
  T* C = (T*)p.C + c_off;
  const T* res = p.residual ? (const T*)p.residual + c_off : nullptr;
  // bias and residual of both passes are requested before the first pass stores (inside the loop the second pass's loads
  // waited behind the first pass's stores, which may alias them); a lane's eight columns are the same in both passes
  u32x4_t bq_all = {0, 0, 0, 0}, rq_all[2] = {{0, 0, 0, 0}, {0, 0, 0, 0}};
  if (p.bias) bq_all = *(const u32x4_t*)((const T*)p.bias + (int64_t)z0 * p.bias_sb + n0 + (threadIdx.x % 8) * 8);
  if (res) {
#pragma unroll
    for (int it = 0; it < 2; ++it)
      rq_all[it] = *(const u32x4_t*)(res + (int64_t)(m0 + it * 32 + threadIdx.x / 8) * p.c_sm + n0 + (threadIdx.x % 8) * 8);
  }
#pragma unroll
  for (int it = 0; it < 2; ++it) {
    const int vid = it * 256 + threadIdx.x;
    const int row = vid / 8, c0 = (vid % 8) * 8;
    const float* s0 = stage + row * kDeepOutPitch + c0;
    const float4 x0 = *(const float4*)s0, x1 = *(const float4*)(s0 + 4);
    const float v[8] = {x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w};
    const int64_t o = (int64_t)(m0 + row) * p.c_sm + n0 + c0;
    const u32x4_t bq = bq_all, rq = rq_all[it];
    float xs[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const uint16_t bb = (uint16_t)(bq[e / 2] >> (16 * (e & 1))), rb = (uint16_t)(rq[e / 2] >> (16 * (e & 1)));
      float x = v[e] * p.alpha;
      if constexpr (Elem<T>::kDtype == LLC_BFLOAT16) x += bf16_bits_to_f32(bb);
      else x += f16_bits_to_f32(bb);
      if (res) x += (Elem<T>::kDtype == LLC_BFLOAT16) ? bf16_bits_to_f32(rb) : f16_bits_to_f32(rb);
      if (p.act == LLC_ACT_RELU) x = x < 0.0f ? 0.0f : x;
      else if (p.act == LLC_ACT_GELU) x = gelu_for<T>(x);
      xs[e] = x;
    }
    *(u32x4_t*)(C + o) = u32x4_t{pack_pair<Elem<T>::kDtype>(xs[0], xs[1]), pack_pair<Elem<T>::kDtype>(xs[2], xs[3]),
                                pack_pair<Elem<T>::kDtype>(xs[4], xs[5]), pack_pair<Elem<T>::kDtype>(xs[6], xs[7])};
  }
}

// Whether the product is one of the small ones this kernel is for (the caller has checked 16-byte alignment of every
// operand, k-contiguous rows of both, and K % 64 == 0).
inline bool deep_ok(const GemmParams& p, int batch) {
  if (p.M % 64 != 0 || p.N % 64 != 0 || p.K < 256 || p.c_f32) return false;
  const int64_t tiles = (int64_t)(p.M / 64) * (p.N / 64) * batch;
  return tiles >= 1 && tiles <= 1024 && batch <= 65535;
}

template <typename T>
int launch_deep(const GemmParams& p0, int batch, hipStream_t s) {
  GemmParams p = p0;
  p.tiles_m = p.M / 64;
  p.tiles_n = p.N / 64;
  const int64_t tiles = (int64_t)p.tiles_m * p.tiles_n * batch;
  // up to one tile per CU: the whole LDS for the ring; more: two workgroups per CU with half the ring each
  if (tiles <= 256) {
    auto kern = gemm_deep_kernel<T, 8>;
    static std::atomic<uint32_t> lds_allowed{0};
    LLC_TRY(allow_dynamic_lds((const void*)kern, 8 * kDeepStage, lds_allowed));
    hipLaunchKernelGGL(kern, dim3((unsigned)(p.tiles_m * p.tiles_n), 1, (unsigned)batch), dim3(256), 8 * kDeepStage, s, p);
  } else {
    auto kern = gemm_deep_kernel<T, 4>;
    static std::atomic<uint32_t> lds_allowed{0};
    LLC_TRY(allow_dynamic_lds((const void*)kern, 4 * kDeepStage, lds_allowed));
    hipLaunchKernelGGL(kern, dim3((unsigned)(p.tiles_m * p.tiles_n), 1, (unsigned)batch), dim3(256), 4 * kDeepStage, s, p);
  }
  return check_launch("gemm_deep_kernel");
}
