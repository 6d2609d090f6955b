// llh.matmul / llh.batch_matmul on the CDNA4 matrix cores.
//
//   C[z][m][n] = act(alpha * sum_k A[z][m][k] * B[z][k][n] + bias[n] + residual[z][m][n])
//
// bf16 / f16 operands use v_mfma_f32_32x32x16_{bf16,f16}; fp32 operands use
// v_mfma_f32_32x32x2_f32 (fp32 products, fp32 accumulate) so that fp32 graphs keep fp32 accuracy.
// Accumulation is always fp32.
//
// Data path per workgroup (256 lanes = 4 waves in a 2x2 grid, macro tile BM x BN):
//   HBM/L2 --16-byte global loads--> registers --> LDS tile [row][128 bytes of k] whose 16-byte
//   chunks are XOR-swizzled by the row (no padding; fragment reads, row copies and transposing
//   stores all spread over the banks) --> ds_read_b128 fragments --> MFMA.  Two LDS buffers and two
//   register stages: global loads for k-tile t+2 are issued before the MFMAs of tile t, tile t+1 is
//   written to the other buffer after them, one barrier per tile.
// A fragment is "8 consecutive k of one row" for both operands.  Operands whose unit-stride dim is
// k (row-major A; B given as [N,K], i.e. a transposed weight view) are copied as they are; a
// row-major B (unit stride along n) is transposed in registers on its way to LDS.  Anything else
// (odd strides, extents that break 16-byte alignment) takes an element-wise loader.
//
// Workgroup -> tile mapping is XCD aware: consecutive workgroup ids are dealt round-robin to the 8
// XCDs by the hardware, so ids are first regrouped per XCD and then walked in column-grouped order,
// which gives each XCD's L2 a compact patch of the output (few distinct A row-panels / B
// column-panels).
#include "gemm_core.hpp"

namespace llc {
using namespace gemm;
namespace {

struct GemmParams {
  const char* A;
  const char* B;
  char* C;
  const char* bias;      // [N] or null, same type as C
  const char* residual;  // [batch, M, N] contiguous or null, same type as C
  int32_t M, N, K;
  int64_t a_sm, a_sk, a_sb;  // element strides of A along m, k, batch
  int64_t b_sk, b_sn, b_sb;  // element strides of B along k, n, batch
  int64_t c_sb;              // batch stride of C (rows are contiguous, pitch N)
  float alpha;
  int32_t act;
  int32_t tiles_m, tiles_n;
};

template <typename T, int BM, int BN, int LA, int LB, bool FULL>
__global__ __launch_bounds__(256) void gemm_kernel(const GemmParams p) {
  constexpr int BK = kRowBytes / sizeof(T);
  constexpr int WTM = BM / 2, WTN = BN / 2;  // wave tile
  constexpr int TM = WTM / 32, TN = WTN / 32;
  constexpr int kABytes = BM * kRowStride, kBBytes = BN * kRowStride;
  constexpr int kBufBytes = kABytes + kBBytes;  // buffer b: A tile at b*kBufBytes, B tile right after it
  extern __shared__ __align__(16) char smem[];

  int tile_m, tile_n;
  tile_of_block(p.tiles_m, p.tiles_n, tile_m, tile_n);
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  const int z = blockIdx.z;
  const T* A = (const T*)p.A + (int64_t)z * p.a_sb;
  const T* B = (const T*)p.B + (int64_t)z * p.b_sb;

  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int wm = wave / 2, wn = wave % 2;
  const int li = lane % 32, lh = lane / 32;

  f32x16_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  // Two register stages: the global loads of k-tile t+2 are issued before the MFMAs of tile t, tile t+1
  // (issued one iteration earlier) is written to the other LDS buffer after them.  The loop is unrolled
  // by two so that the stage index is a compile-time constant (register arrays, not scratch).
  TileLoader<T, BM, LA> la0, la1;
  TileLoader<T, BN, LB> lb0, lb1;
  const int nk = (p.K + BK - 1) / BK;
  la0.template load<FULL>(A, m0, p.M, 0, p.K, p.a_sm, p.a_sk);
  lb0.template load<FULL>(B, n0, p.N, 0, p.K, p.b_sn, p.b_sk);
  if (nk > 1) {
    la1.template load<FULL>(A, m0, p.M, BK, p.K, p.a_sm, p.a_sk);
    lb1.template load<FULL>(B, n0, p.N, BK, p.K, p.b_sn, p.b_sk);
  }
  la0.store(smem);
  lb0.store(smem + kABytes);
  __syncthreads();

#define LLC_GEMM_STEP(KT, CUR, LA2, LB2, LA1, LB1, GUARDED)                                                     \
  {                                                                                                             \
    /* LA2/LB2: stage that held tile KT (now in LDS) and receives tile KT+2; LA1/LB1 hold tile KT+1 */          \
    if (!(GUARDED) || (KT) + 2 < nk) {                                                                          \
      LA2.template load<FULL>(A, m0, p.M, ((KT) + 2) * BK, p.K, p.a_sm, p.a_sk);                                \
      LB2.template load<FULL>(B, n0, p.N, ((KT) + 2) * BK, p.K, p.b_sn, p.b_sk);                                \
    }                                                                                                           \
    mma_tile<T, TM, TN>(smem + (CUR) * kBufBytes, wm * WTM + li, smem + (CUR) * kBufBytes + kABytes,            \
                        wn * WTN + li, lh, acc);                                                                \
    if (!(GUARDED) || (KT) + 1 < nk) {                                                                          \
      LA1.store(smem + ((CUR) ^ 1) * kBufBytes);                                                                \
      LB1.store(smem + ((CUR) ^ 1) * kBufBytes + kABytes);                                                      \
    }                                                                                                           \
    __syncthreads();                                                                                            \
  }
  // steady state: no control flow inside the body (every load and store is known to be needed), so the
  // accumulators stay where the MFMAs leave them; the last up to three tiles run the guarded form
  int kt = 0;
  for (; kt + 3 < nk; kt += 2) {
    LLC_GEMM_STEP(kt, 0, la0, lb0, la1, lb1, false)
    LLC_GEMM_STEP(kt + 1, 1, la1, lb1, la0, lb0, false)
  }
  for (; kt < nk; kt += 2) {
    LLC_GEMM_STEP(kt, 0, la0, lb0, la1, lb1, true)
    if (kt + 1 < nk) LLC_GEMM_STEP(kt + 1, 1, la1, lb1, la0, lb0, true)
  }
#undef LLC_GEMM_STEP

  // ---- epilogue.  32x32 accumulator layout: register r of lane (li, lh) is row 8*(r/4) + 4*lh + r%4,
  //      column li: for fixed r, 32 lanes store 32 consecutive columns of one row. ----
  T* C = (T*)p.C + (int64_t)z * p.c_sb;
  const char* res = p.residual ? p.residual + (int64_t)z * p.c_sb * (int64_t)sizeof(T) : nullptr;
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int col = n0 + wn * WTN + j * 32 + li;
    if (!FULL && col >= p.N) continue;
    const float bv = p.bias ? load_as_f32(p.bias, Elem<T>::kDtype, col) : 0.0f;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = m0 + wm * WTM + i * 32 + (r / 4) * 8 + lh * 4 + (r % 4);
        if (!FULL && row >= p.M) continue;
        epilogue_store<T>(C, (int64_t)row * p.N + col, acc[i][j][r], p.alpha, bv, res, p.act);
      }
    }
  }
}

template <typename T, int BM, int BN, int LA, int LB>
int launch_cfg(const GemmParams& p0, int batch, hipStream_t s) {
  GemmParams p = p0;
  p.tiles_m = (p.M + BM - 1) / BM;
  p.tiles_n = (p.N + BN - 1) / BN;
  const size_t lds = 2 * (size_t)(BM + BN) * kRowStride;
  static bool attr_set[2] = {false, false};  // per instantiation
  // every tile complete: the unguarded instantiation (no per-access branches in the main loop)
  const bool full = p.M % BM == 0 && p.N % BN == 0 && p.K % (kRowBytes / (int)sizeof(T)) == 0;
  auto kern = full ? gemm_kernel<T, BM, BN, LA, LB, true> : gemm_kernel<T, BM, BN, LA, LB, false>;
  if (!attr_set[full]) {
    LLC_HIP_TRY(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    attr_set[full] = true;
  }
  const int64_t tiles = (int64_t)p.tiles_m * p.tiles_n;
  if (tiles > 0x7fffffff || batch > 65535) return set_error(LLC_ERR_TOO_LARGE, "matmul: grid too large");
  hipLaunchKernelGGL(kern, dim3((unsigned)tiles, 1, (unsigned)batch), dim3(256), lds, s, p);
  return check_launch("gemm_kernel");
}

template <typename T, int LA, int LB>
int launch_tiles(const GemmParams& p, int batch, hipStream_t s) {
  // 128x128 while it still yields enough workgroups for 256 CUs, smaller tiles for skinny outputs
  const int64_t t128 = (int64_t)((p.M + 127) / 128) * ((p.N + 127) / 128) * batch;
  if (p.N > 64 && p.M > 64 && t128 >= 128) return launch_cfg<T, 128, 128, LA, LB>(p, batch, s);
  if (p.N <= 64 && p.M > 64) return launch_cfg<T, 128, 64, LA, LB>(p, batch, s);
  return launch_cfg<T, 64, 64, LA, LB>(p, batch, s);
}

template <typename T>
int launch_loaders(const GemmParams& p, int batch, hipStream_t s) {
  constexpr int EPV = 16 / sizeof(T);
  auto al16 = [](const void* q) { return ((uintptr_t)q % 16) == 0; };
  const bool a_kvec = p.a_sk == 1 && p.a_sm % EPV == 0 && p.a_sb % EPV == 0 && p.K % EPV == 0 && al16(p.A);
  const bool b_kvec = p.b_sk == 1 && p.b_sn % EPV == 0 && p.b_sb % EPV == 0 && p.K % EPV == 0 && al16(p.B);
  const bool b_rvec = p.b_sn == 1 && p.b_sk % EPV == 0 && p.b_sb % EPV == 0 && p.N % EPV == 0 && al16(p.B);
  if (a_kvec && b_kvec) return launch_tiles<T, kLoadKVec, kLoadKVec>(p, batch, s);
  if (a_kvec && b_rvec) return launch_tiles<T, kLoadKVec, kLoadRVec>(p, batch, s);
  return launch_tiles<T, kLoadGeneric, kLoadGeneric>(p, batch, s);
}

}  // namespace

namespace {
int gemm_dispatch(int dtype, const GemmParams& p, int batch, hipStream_t s) {
  if (p.M == 0 || p.N == 0 || batch == 0) return LLC_OK;
  switch (dtype) {
    case LLC_FLOAT32: return launch_loaders<float>(p, batch, s);
    case LLC_BFLOAT16: return launch_loaders<__bf16>(p, batch, s);
    case LLC_FLOAT16: return launch_loaders<_Float16>(p, batch, s);
  }
  return set_error(LLC_ERR_DTYPE, "matmul: element type %d (f32, bf16 or f16 expected)", dtype);
}

int fill_epilogue(const llc_epilogue* epi, const View& o, int64_t n_cols, GemmParams* p) {
  p->alpha = 1.0f;
  p->act = LLC_ACT_NONE;
  p->bias = nullptr;
  p->residual = nullptr;
  if (!epi) return LLC_OK;
  p->alpha = epi->alpha;
  if (epi->act < LLC_ACT_NONE || epi->act > LLC_ACT_GELU) return set_error(LLC_ERR_BAD_ARG, "epilogue: activation %d", epi->act);
  p->act = epi->act;
  if (epi->bias) {
    View b;
    LLC_TRY(make_view(epi->bias, "epilogue bias", &b));
    if (b.dtype != o.dtype) return set_error(LLC_ERR_DTYPE, "epilogue: bias type differs from output");
    if (b.numel() != n_cols || !b.contiguous()) return set_error(LLC_ERR_SHAPE, "epilogue: bias must hold %lld contiguous values", (long long)n_cols);
    p->bias = b.ptr;
  }
  if (epi->residual) {
    View r;
    LLC_TRY(make_view(epi->residual, "epilogue residual", &r));
    if (r.dtype != o.dtype) return set_error(LLC_ERR_DTYPE, "epilogue: residual type differs from output");
    if (r.numel() != o.numel() || !r.contiguous()) return set_error(LLC_ERR_SHAPE, "epilogue: residual must match the output and be contiguous");
    p->residual = r.ptr;
  }
  return LLC_OK;
}

}  // namespace
}  // namespace llc

using namespace llc;

extern "C" int llc_hip_matmul(const llc_tensor* lhs, const llc_tensor* rhs, const llc_epilogue* epi, llc_tensor* out,
                              void* stream) {
  View a, b, o;
  LLC_TRY(make_view(lhs, "matmul lhs", &a));
  LLC_TRY(make_view(rhs, "matmul rhs", &b));
  LLC_TRY(make_view(out, "matmul out", &o));
  if (a.rank != 2 || b.rank != 2 || o.rank != 2) return set_error(LLC_ERR_SHAPE, "matmul: rank-2 tensors expected (LLH_2DTensor)");
  if (a.dtype != b.dtype || a.dtype != o.dtype) return set_error(LLC_ERR_DTYPE, "matmul: operand types differ");
  if (a.size[1] != b.size[0] || o.size[0] != a.size[0] || o.size[1] != b.size[1])
    return set_error(LLC_ERR_SHAPE, "matmul: [%lld,%lld] x [%lld,%lld] -> [%lld,%lld]", (long long)a.size[0], (long long)a.size[1],
                     (long long)b.size[0], (long long)b.size[1], (long long)o.size[0], (long long)o.size[1]);
  if (!o.contiguous()) return set_error(LLC_ERR_LAYOUT, "matmul: output must be contiguous");
  if (a.size[0] > 0x7fffffff || a.size[1] > 0x7fffffff || b.size[1] > 0x7fffffff) return set_error(LLC_ERR_TOO_LARGE, "matmul: extent too large");
  GemmParams p{};
  p.A = a.ptr;
  p.B = b.ptr;
  p.C = o.ptr;
  p.M = (int)a.size[0];
  p.K = (int)a.size[1];
  p.N = (int)b.size[1];
  p.a_sm = a.stride[0];
  p.a_sk = a.stride[1];
  p.b_sk = b.stride[0];
  p.b_sn = b.stride[1];
  LLC_TRY(fill_epilogue(epi, o, p.N, &p));
  return gemm_dispatch(a.dtype, p, 1, as_stream(stream));
}

extern "C" int llc_hip_batch_matmul(const llc_tensor* lhs, const llc_tensor* rhs, const llc_epilogue* epi,
                                    llc_tensor* out, void* stream) {
  View a, b, o;
  LLC_TRY(make_view(lhs, "batch_matmul lhs", &a));
  LLC_TRY(make_view(rhs, "batch_matmul rhs", &b));
  LLC_TRY(make_view(out, "batch_matmul out", &o));
  if (a.rank != 3 || b.rank != 3 || o.rank != 3) return set_error(LLC_ERR_SHAPE, "batch_matmul: rank-3 tensors expected (LLH_3DTensor)");
  if (a.dtype != b.dtype || a.dtype != o.dtype) return set_error(LLC_ERR_DTYPE, "batch_matmul: operand types differ");
  if (a.size[0] != b.size[0] || o.size[0] != a.size[0] || a.size[2] != b.size[1] || o.size[1] != a.size[1] || o.size[2] != b.size[2])
    return set_error(LLC_ERR_SHAPE, "batch_matmul: [%lld,%lld,%lld] x [%lld,%lld,%lld] -> [%lld,%lld,%lld]", (long long)a.size[0],
                     (long long)a.size[1], (long long)a.size[2], (long long)b.size[0], (long long)b.size[1], (long long)b.size[2],
                     (long long)o.size[0], (long long)o.size[1], (long long)o.size[2]);
  if (!o.contiguous()) return set_error(LLC_ERR_LAYOUT, "batch_matmul: output must be contiguous");
  if (a.size[1] > 0x7fffffff || a.size[2] > 0x7fffffff || b.size[2] > 0x7fffffff) return set_error(LLC_ERR_TOO_LARGE, "batch_matmul: extent too large");
  GemmParams p{};
  p.A = a.ptr;
  p.B = b.ptr;
  p.C = o.ptr;
  p.M = (int)a.size[1];
  p.K = (int)a.size[2];
  p.N = (int)b.size[2];
  p.a_sb = a.stride[0];
  p.a_sm = a.stride[1];
  p.a_sk = a.stride[2];
  p.b_sb = b.stride[0];
  p.b_sk = b.stride[1];
  p.b_sn = b.stride[2];
  p.c_sb = (int64_t)p.M * p.N;
  LLC_TRY(fill_epilogue(epi, o, p.N, &p));
  // blockIdx.z carries the batch; larger batches are issued in slices
  hipStream_t s = as_stream(stream);
  const int64_t nb = a.size[0];
  for (int64_t z0 = 0; z0 < nb; z0 += 65535) {
    GemmParams q = p;
    const int cnt = (int)((nb - z0) < 65535 ? (nb - z0) : 65535);
    q.A = p.A + z0 * p.a_sb * (int64_t)a.esize();
    q.B = p.B + z0 * p.b_sb * (int64_t)a.esize();
    q.C = p.C + z0 * p.c_sb * (int64_t)a.esize();
    if (p.residual) q.residual = p.residual + z0 * p.c_sb * (int64_t)a.esize();
    LLC_TRY(gemm_dispatch(a.dtype, q, cnt, s));
  }
  return LLC_OK;
}
