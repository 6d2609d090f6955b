// Data-movement ops, bit exact for 1/2/4/8-byte elements: transpose, stride_slice, broadcast_to,
// strided copy, row gather and convert.
//
// Everything except gather is "contiguous output <- strided input".  Two kernels cover it:
//  * strided_copy_kernel: lanes walk the output linearly; when the input's innermost stride is 1
//    both sides move 16-byte vectors (head split/merge of attention, slices, broadcasts).
//  * tile_transpose_kernel: when the input's unit-stride dim is not the output's innermost dim, a
//    64x64 tile goes through LDS so that reads are coalesced along the input's unit-stride dim and
//    writes along the output's (2-D and batched transposes).
#include "common.hpp"

namespace llc {
namespace {

constexpr int kCopyDims = 6;

struct CopyParams {
  const char* in;
  char* out;
  uint32_t dims[kCopyDims];      // collapsed output extents, dims[kCopyDims-1] innermost
  int64_t in_stride[kCopyDims];  // elements
  int64_t n_vec;
};

template <typename T, int VEC>
__global__ __launch_bounds__(256) void strided_copy_kernel(const CopyParams p) {
  struct alignas(sizeof(T) * VEC) Pack { T v[VEC]; };
  const int64_t nthreads = (int64_t)gridDim.x * blockDim.x;
  for (int64_t v = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; v < p.n_vec; v += nthreads) {
    uint32_t t = (uint32_t)(v * VEC);  // the host rejects outputs of 2^32 elements or more
    int64_t off = 0;
#pragma unroll
    for (int d = kCopyDims - 1; d > 0; --d) {
      if (p.dims[d] != 1) {
        off += (int64_t)(t % p.dims[d]) * p.in_stride[d];
        t /= p.dims[d];
      }
    }
    off += (int64_t)t * p.in_stride[0];
    const T* src = (const T*)p.in + off;
    Pack pk;
    if constexpr (VEC == 1) pk.v[0] = *src;
    else pk = *(const Pack*)src;  // innermost input stride is 1 on this path
    *((Pack*)p.out + v) = pk;
  }
}

struct TransposeParams {
  const char* in;
  char* out;
  uint32_t bdims[kCopyDims];       // batch dims (everything except I and J), outermost first
  int64_t b_in_stride[kCopyDims];  // elements
  int64_t b_out_stride[kCopyDims];
  int32_t n_bdims;
  int64_t NI, NJ;  // I: output-innermost dim; J: input unit-stride dim
  int64_t sI;      // input stride of I
  int64_t oJ;      // output stride of J
  uint32_t tiles_i, tiles_j;
};

template <typename T>
__global__ __launch_bounds__(256) void tile_transpose_kernel(const TransposeParams p) {
  __shared__ T tile[64][65];
  uint32_t b = blockIdx.x;
  const uint32_t tj = b % p.tiles_j;
  b /= p.tiles_j;
  const uint32_t ti = b % p.tiles_i;
  b /= p.tiles_i;
  int64_t in_base = 0, out_base = 0;
  for (int d = p.n_bdims - 1; d >= 0; --d) {
    const uint32_t id = b % p.bdims[d];
    b /= p.bdims[d];
    in_base += id * p.b_in_stride[d];
    out_base += id * p.b_out_stride[d];
  }
  const int64_t i0 = (int64_t)ti * 64, j0 = (int64_t)tj * 64;
  const int tx = threadIdx.x % 64, ty = threadIdx.x / 64;
  const T* in = (const T*)p.in + in_base;
  T* out = (T*)p.out + out_base;
#pragma unroll 4
  for (int r = 0; r < 16; ++r) {
    const int i = r * 4 + ty;
    if (i0 + i < p.NI && j0 + tx < p.NJ) tile[i][tx] = in[(i0 + i) * p.sI + (j0 + tx)];
  }
  __syncthreads();
#pragma unroll 4
  for (int r = 0; r < 16; ++r) {
    const int j = r * 4 + ty;
    if (i0 + tx < p.NI && j0 + j < p.NJ) out[(j0 + j) * p.oJ + (i0 + tx)] = tile[tx][j];
  }
}

// Collapsed "contiguous out <- strided in" description shared by the entry points.
struct Collapsed {
  int n = 0;
  int64_t dim[LLC_MAX_RANK];
  int64_t ist[LLC_MAX_RANK];
};

Collapsed collapse(int rank, const int64_t* size, const int64_t* in_stride) {
  Collapsed c;
  for (int d = 0; d < rank; ++d) {
    if (size[d] == 1) continue;
    if (c.n > 0 && c.ist[c.n - 1] == in_stride[d] * size[d]) {
      c.dim[c.n - 1] *= size[d];
      c.ist[c.n - 1] = in_stride[d];
    } else {
      c.dim[c.n] = size[d];
      c.ist[c.n] = in_stride[d];
      ++c.n;
    }
  }
  if (c.n == 0) {
    c.dim[0] = 1;
    c.ist[0] = 1;
    c.n = 1;
  }
  return c;
}

template <typename T>
int launch_copy_t(const CopyParams& p0, int vec, hipStream_t s) {
  CopyParams p = p0;
  p.n_vec = p0.n_vec / vec;
  int64_t want = (p.n_vec + 255) / 256;
  unsigned blocks = (unsigned)(want > 256 * 64 ? 256 * 64 : (want < 1 ? 1 : want));
  constexpr int kMaxVec = 16 / sizeof(T);
  if (vec == kMaxVec && kMaxVec > 1) hipLaunchKernelGGL((strided_copy_kernel<T, kMaxVec>), dim3(blocks), dim3(256), 0, s, p);
  else hipLaunchKernelGGL((strided_copy_kernel<T, 1>), dim3(blocks), dim3(256), 0, s, p);
  return check_launch("strided_copy_kernel");
}

template <typename T>
int launch_transpose_t(const TransposeParams& p, hipStream_t s) {
  uint64_t blocks = (uint64_t)p.tiles_i * p.tiles_j;
  for (int d = 0; d < p.n_bdims; ++d) blocks *= p.bdims[d];
  if (blocks > 0x7fffffffull) return set_error(LLC_ERR_TOO_LARGE, "transpose: too many tiles");
  hipLaunchKernelGGL((tile_transpose_kernel<T>), dim3((unsigned)blocks), dim3(256), 0, s, p);
  return check_launch("tile_transpose_kernel");
}

// out (contiguous, shape `size`) <- in read through `in_stride` (elements) from `in_ptr`.
int strided_to_contiguous(const char* in_ptr, char* out_ptr, int rank, const int64_t* size, const int64_t* in_stride,
                          size_t es, hipStream_t s) {
  int64_t total = 1;
  for (int d = 0; d < rank; ++d) total *= size[d];
  if (total == 0) return LLC_OK;
  if (total >= (int64_t)1 << 32) return set_error(LLC_ERR_TOO_LARGE, "copy: %lld elements (max 2^32-1)", (long long)total);
  Collapsed c = collapse(rank, size, in_stride);
  if (c.n > kCopyDims) return set_error(LLC_ERR_LAYOUT, "copy: view needs %d index dims (max %d)", c.n, kCopyDims);
  for (int d = 0; d < c.n; ++d)
    if (c.dim[d] >= (int64_t)1 << 32) return set_error(LLC_ERR_TOO_LARGE, "copy: extent %lld", (long long)c.dim[d]);

  const int64_t inner_stride = c.ist[c.n - 1];
  // ---- LDS-tiled path: the input's unit-stride dim is a different dim than the output's innermost ----
  int jdim = -1;
  if (inner_stride != 1 && c.dim[c.n - 1] >= 16) {
    for (int d = 0; d < c.n - 1; ++d)
      if (c.ist[d] == 1 && c.dim[d] >= 16) jdim = d;
  }
  if (jdim >= 0) {
    TransposeParams t{};
    t.in = in_ptr;
    t.out = out_ptr;
    int64_t ost[LLC_MAX_RANK];
    int64_t acc = 1;
    for (int d = c.n - 1; d >= 0; --d) {
      ost[d] = acc;
      acc *= c.dim[d];
    }
    t.NI = c.dim[c.n - 1];
    t.sI = inner_stride;
    t.NJ = c.dim[jdim];
    t.oJ = ost[jdim];
    t.tiles_i = (uint32_t)((t.NI + 63) / 64);
    t.tiles_j = (uint32_t)((t.NJ + 63) / 64);
    for (int d = 0; d < c.n - 1; ++d) {
      if (d == jdim) continue;
      t.bdims[t.n_bdims] = (uint32_t)c.dim[d];
      t.b_in_stride[t.n_bdims] = c.ist[d];
      t.b_out_stride[t.n_bdims] = ost[d];
      ++t.n_bdims;
    }
    switch (es) {
      case 1: return launch_transpose_t<uint8_t>(t, s);
      case 2: return launch_transpose_t<uint16_t>(t, s);
      case 4: return launch_transpose_t<uint32_t>(t, s);
      default: return launch_transpose_t<uint64_t>(t, s);
    }
  }

  CopyParams p{};
  p.in = in_ptr;
  p.out = out_ptr;
  for (int d = 0; d < kCopyDims; ++d) {
    p.dims[d] = 1;
    p.in_stride[d] = 0;
  }
  for (int d = 0; d < c.n; ++d) {
    p.dims[kCopyDims - c.n + d] = (uint32_t)c.dim[d];
    p.in_stride[kCopyDims - c.n + d] = c.ist[d];
  }
  p.n_vec = total;
  int vec = 1;
  const int wide = (int)(16 / es);
  if (inner_stride == 1 && wide > 1 && c.dim[c.n - 1] % wide == 0 && ((uintptr_t)in_ptr % 16) == 0 &&
      ((uintptr_t)out_ptr % 16) == 0) {
    bool ok = true;
    for (int d = 0; d < c.n - 1; ++d) ok = ok && (c.ist[d] % wide) == 0;
    if (ok) vec = wide;
  }
  switch (es) {
    case 1: return launch_copy_t<uint8_t>(p, vec, s);
    case 2: return launch_copy_t<uint16_t>(p, vec, s);
    case 4: return launch_copy_t<uint32_t>(p, vec, s);
    default: return launch_copy_t<uint64_t>(p, vec, s);
  }
}

int same_dtype(const View& a, const View& o, const char* what) {
  if (a.dtype != o.dtype) return set_error(LLC_ERR_DTYPE, "%s: input type %d, output type %d", what, a.dtype, o.dtype);
  return LLC_OK;
}
int out_contiguous(const View& o, const char* what) {
  if (!o.contiguous()) return set_error(LLC_ERR_LAYOUT, "%s: output must be contiguous", what);
  return LLC_OK;
}

template <typename T, int VEC>
__global__ __launch_bounds__(256) void gather_rows_kernel(const T* table, const int64_t* idx, T* out, int64_t n_idx,
                                                         int64_t row_vecs, int64_t table_rows) {
  struct alignas(sizeof(T) * VEC) Pack { T v[VEC]; };
  const int64_t total = n_idx * row_vecs;
  for (int64_t v = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; v < total; v += (int64_t)gridDim.x * blockDim.x) {
    const int64_t r = v / row_vecs, c = v % row_vecs;
    int64_t src = idx[r];
    // indices outside the table would be a fault in the caller's program; clamp instead of faulting
    src = src < 0 ? 0 : (src >= table_rows ? table_rows - 1 : src);
    *((Pack*)out + v) = *((const Pack*)table + src * row_vecs + c);
  }
}

}  // namespace
}  // namespace llc

using namespace llc;

int llc_impl_copy(const llc_tensor* x, llc_tensor* out, void* stream) {
  View a, o;
  LLC_TRY(make_view(x, "copy input", &a));
  LLC_TRY(make_view(out, "copy output", &o));
  LLC_TRY(same_dtype(a, o, "copy"));
  LLC_TRY(out_contiguous(o, "copy"));
  if (a.rank != o.rank) return set_error(LLC_ERR_SHAPE, "copy: rank mismatch");
  for (int d = 0; d < a.rank; ++d)
    if (a.size[d] != o.size[d]) return set_error(LLC_ERR_SHAPE, "copy: extent mismatch at dim %d", d);
  return strided_to_contiguous(a.ptr, o.ptr, a.rank, a.size, a.stride, a.esize(), as_stream(stream));
}

int llc_impl_transpose(const llc_tensor* x, const int64_t* perms, llc_tensor* out, void* stream) {
  View a, o;
  LLC_TRY(make_view(x, "transpose input", &a));
  LLC_TRY(make_view(out, "transpose output", &o));
  LLC_TRY(same_dtype(a, o, "transpose"));
  LLC_TRY(out_contiguous(o, "transpose"));
  if (!perms) return set_error(LLC_ERR_BAD_ARG, "transpose: null perms");
  if (a.rank != o.rank) return set_error(LLC_ERR_SHAPE, "transpose: rank mismatch");
  bool seen[LLC_MAX_RANK] = {false};
  int64_t st[LLC_MAX_RANK];
  for (int d = 0; d < a.rank; ++d) {
    int64_t pd = perms[d];
    if (pd < 0 || pd >= a.rank || seen[pd]) return set_error(LLC_ERR_BAD_ARG, "transpose: perms is not a permutation");
    seen[pd] = true;
    if (o.size[d] != a.size[pd])
      return set_error(LLC_ERR_SHAPE, "transpose: out extent %lld at dim %d, expected %lld", (long long)o.size[d], d,
                       (long long)a.size[pd]);
    st[d] = a.stride[pd];
  }
  return strided_to_contiguous(a.ptr, o.ptr, a.rank, o.size, st, a.esize(), as_stream(stream));
}

int llc_impl_stride_slice(const llc_tensor* x, const int64_t* start, const int64_t* end, const int64_t* step,
                                    llc_tensor* out, void* stream) {
  View a, o;
  LLC_TRY(make_view(x, "stride_slice input", &a));
  LLC_TRY(make_view(out, "stride_slice output", &o));
  LLC_TRY(same_dtype(a, o, "stride_slice"));
  LLC_TRY(out_contiguous(o, "stride_slice"));
  if (!start || !end || !step) return set_error(LLC_ERR_BAD_ARG, "stride_slice: null index array");
  int64_t size[LLC_MAX_RANK], st[LLC_MAX_RANK];
  int64_t off = 0, total = 1;
  for (int d = 0; d < a.rank; ++d) {
    if (step[d] <= 0) return set_error(LLC_ERR_BAD_ARG, "stride_slice: step %lld at dim %d", (long long)step[d], d);
    if (start[d] < 0 || end[d] > a.size[d])
      return set_error(LLC_ERR_SHAPE, "stride_slice: [%lld, %lld) leaves extent %lld at dim %d", (long long)start[d],
                       (long long)end[d], (long long)a.size[d], d);
    int64_t n = (end[d] - start[d] + step[d] - 1) / step[d];  // ceildiv, StablehlotoLinalgExtension.cpp:68-118
    size[d] = n < 0 ? 0 : n;
    st[d] = a.stride[d] * step[d];
    off += start[d] * a.stride[d];
    total *= size[d];
  }
  if (o.numel() != total)
    return set_error(LLC_ERR_SHAPE, "stride_slice: output holds %lld elements, expected %lld", (long long)o.numel(), (long long)total);
  return strided_to_contiguous(a.ptr + off * (int64_t)a.esize(), o.ptr, a.rank, size, st, a.esize(), as_stream(stream));
}

int llc_impl_broadcast_to(const llc_tensor* x, llc_tensor* out, void* stream) {
  View a, o;
  LLC_TRY(make_view(x, "broadcast_to input", &a));
  LLC_TRY(make_view(out, "broadcast_to output", &o));
  LLC_TRY(same_dtype(a, o, "broadcast_to"));
  LLC_TRY(out_contiguous(o, "broadcast_to"));
  if (a.rank != o.rank) return set_error(LLC_ERR_SHAPE, "broadcast_to: rank %d -> %d (reshape first)", a.rank, o.rank);
  int64_t st[LLC_MAX_RANK];
  for (int d = 0; d < a.rank; ++d) {
    if (a.size[d] == o.size[d]) st[d] = a.stride[d];
    else if (a.size[d] == 1) st[d] = 0;
    else return set_error(LLC_ERR_SHAPE, "broadcast_to: extent %lld -> %lld at dim %d", (long long)a.size[d], (long long)o.size[d], d);
  }
  return strided_to_contiguous(a.ptr, o.ptr, a.rank, o.size, st, a.esize(), as_stream(stream));
}

int llc_impl_gather_rows(const llc_tensor* table, const llc_tensor* idx, llc_tensor* out, void* stream) {
  View t, i, o;
  LLC_TRY(make_view(table, "gather_rows table", &t));
  LLC_TRY(make_view(idx, "gather_rows indices", &i));
  LLC_TRY(make_view(out, "gather_rows output", &o));
  LLC_TRY(same_dtype(t, o, "gather_rows"));
  if (i.dtype != LLC_INT64) return set_error(LLC_ERR_DTYPE, "gather_rows: indices must be int64");
  if (!t.contiguous() || !i.contiguous() || !o.contiguous()) return set_error(LLC_ERR_LAYOUT, "gather_rows: contiguous tensors expected");
  if (t.rank < 1) return set_error(LLC_ERR_SHAPE, "gather_rows: table needs rank >= 1");
  const int64_t rows = t.size[0];
  const int64_t row_elems = rows ? t.numel() / rows : 0;
  const int64_t n_idx = i.numel();
  if (o.numel() != n_idx * row_elems) return set_error(LLC_ERR_SHAPE, "gather_rows: output holds %lld elements, expected %lld", (long long)o.numel(), (long long)(n_idx * row_elems));
  if (n_idx == 0 || row_elems == 0) return LLC_OK;
  if (rows == 0) return set_error(LLC_ERR_SHAPE, "gather_rows: empty table");
  const size_t row_bytes = (size_t)row_elems * t.esize();
  hipStream_t s = as_stream(stream);
  if (row_bytes % 16 == 0 && (uintptr_t)t.ptr % 16 == 0 && (uintptr_t)o.ptr % 16 == 0) {
    const int64_t rv = (int64_t)(row_bytes / 16);
    int64_t want = (n_idx * rv + 255) / 256;
    unsigned blocks = (unsigned)(want > 256 * 64 ? 256 * 64 : want);
    hipLaunchKernelGGL((gather_rows_kernel<uint32_t, 4>), dim3(blocks), dim3(256), 0, s, (const uint32_t*)t.ptr,
                       (const int64_t*)i.ptr, (uint32_t*)o.ptr, n_idx, rv, rows);
  } else {
    const int64_t rv = (int64_t)row_bytes;
    int64_t want = (n_idx * rv + 255) / 256;
    unsigned blocks = (unsigned)(want > 256 * 64 ? 256 * 64 : want);
    hipLaunchKernelGGL((gather_rows_kernel<uint8_t, 1>), dim3(blocks), dim3(256), 0, s, (const uint8_t*)t.ptr,
                       (const int64_t*)i.ptr, (uint8_t*)o.ptr, n_idx, rv, rows);
  }
  return check_launch("gather_rows_kernel");
}

int llc_impl_convert(const llc_tensor* x, llc_tensor* out, void* stream) {
  if (!x || !out) return set_error(LLC_ERR_BAD_ARG, "convert: null tensor");
  llc_ew_program prog{};
  prog.n_insts = 1;
  prog.result = 0;
  const bool int_in = x->type == LLC_INT64 || x->type == LLC_INT32 || x->type == LLC_INT8 || x->type == LLC_INT1;
  const bool int_out = out->type == LLC_INT64 || out->type == LLC_INT32 || out->type == LLC_INT8 || out->type == LLC_INT1;
  prog.integer = (int_in && int_out) ? 1 : 0;
  prog.insts[0].op = LLC_EW_MOV;
  prog.insts[0].dst = 0;
  prog.insts[0].a = LLC_EW_IN0;
  const llc_tensor* ins[1] = {x};
  return llc_impl_elementwise(&prog, ins, 1, out, stream);
}
