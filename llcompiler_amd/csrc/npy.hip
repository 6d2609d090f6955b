// Weight files: NumPy .npy, the format the reference's importer writes with np.save
// (llcompiler/importer/fx_translate.py:427-430) and its LoadWeight pass parses
// (src/Dialect/LLH/Transforms/LoadWeight.cpp:58-132: 10-byte preamble, the header dictionary with 'descr',
// 'fortran_order' and 'shape', then the raw little-endian data in C order).  The reference reads '<f4' and
// '<i8' and turns the data into constants of the compiled object; here the data is uploaded into memory owned
// by a plan, and the 16-bit and small integer types are read as well ('<u2' carries bf16 bit patterns: NumPy
// has no bf16, so the expected element type comes from the caller, as the reference takes it from the op's
// result type).
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "common.hpp"

using namespace llc;

namespace {

struct NpyInfo {
  std::string descr;
  bool fortran = false;
  std::vector<size_t> shape;
  size_t data_offset = 0;
};

int parse_header(FILE* fp, const char* path, NpyInfo* info) {
  unsigned char pre[12];
  if (fread(pre, 1, 10, fp) != 10 || memcmp(pre, "\x93NUMPY", 6) != 0)
    return set_error(LLC_ERR_BAD_ARG, "npy: %s is not a .npy file", path);
  const int major = pre[6];
  size_t hlen = pre[8] | ((size_t)pre[9] << 8), hoff = 10;
  if (major >= 2) {  // version 2/3: four-byte header length
    if (fread(pre + 10, 1, 2, fp) != 2) return set_error(LLC_ERR_BAD_ARG, "npy: %s: truncated preamble", path);
    hlen |= ((size_t)pre[10] << 16) | ((size_t)pre[11] << 24);
    hoff = 12;
  } else if (major != 1) {
    return set_error(LLC_ERR_UNSUPPORTED, "npy: %s: format version %d", path, major);
  }
  if (hlen == 0 || hlen > (1u << 20)) return set_error(LLC_ERR_BAD_ARG, "npy: %s: header length %zu", path, hlen);
  std::string h(hlen, '\0');
  if (fread(&h[0], 1, hlen, fp) != hlen) return set_error(LLC_ERR_BAD_ARG, "npy: %s: truncated header", path);
  info->data_offset = hoff + hlen;
  size_t at = h.find("'descr'");
  if (at == std::string::npos) return set_error(LLC_ERR_BAD_ARG, "npy: %s: no 'descr' in the header", path);
  size_t q0 = h.find('\'', at + 7);
  size_t q1 = q0 == std::string::npos ? q0 : h.find('\'', q0 + 1);
  if (q1 == std::string::npos) return set_error(LLC_ERR_BAD_ARG, "npy: %s: malformed 'descr'", path);
  info->descr = h.substr(q0 + 1, q1 - q0 - 1);
  at = h.find("'fortran_order'");
  if (at == std::string::npos) return set_error(LLC_ERR_BAD_ARG, "npy: %s: no 'fortran_order' in the header", path);
  const size_t fv = h.find_first_not_of(": ", at + 15);
  if (fv == std::string::npos) return set_error(LLC_ERR_BAD_ARG, "npy: %s: 'fortran_order' has no value", path);
  info->fortran = h.compare(fv, 4, "True") == 0;
  at = h.find("'shape'");
  size_t p0 = at == std::string::npos ? at : h.find('(', at);
  size_t p1 = p0 == std::string::npos ? p0 : h.find(')', p0);
  if (p1 == std::string::npos) return set_error(LLC_ERR_BAD_ARG, "npy: %s: no 'shape' tuple in the header", path);
  info->shape.clear();
  size_t i = p0 + 1;
  while (i < p1) {
    if (h[i] >= '0' && h[i] <= '9') {
      size_t v = 0;
      while (i < p1 && h[i] >= '0' && h[i] <= '9') v = v * 10 + (size_t)(h[i++] - '0');
      info->shape.push_back(v);
    } else {
      ++i;
    }
  }
  if (info->shape.size() > LLC_MAX_RANK) return set_error(LLC_ERR_SHAPE, "npy: %s: rank %zu", path, info->shape.size());
  return LLC_OK;
}

// element type of a descr, or -1.  expect (an llc_dtype or -1) resolves what the file cannot say.
int dtype_of(const std::string& d, int expect) {
  if (d.size() < 3 || d[0] == '>') return -1;  // big-endian data is not converted
  const std::string t = d.substr(1);
  if (t == "f4") return LLC_FLOAT32;
  if (t == "i8") return LLC_INT64;
  if (t == "f8") return LLC_DOUBLE64;
  if (t == "f2") return LLC_FLOAT16;
  if (t == "i4") return LLC_INT32;
  if (t == "i2") return LLC_INT16;
  if (t == "i1") return LLC_INT8;
  if (t == "b1") return LLC_INT1;
  if (t == "u2") return expect == LLC_BFLOAT16 ? LLC_BFLOAT16 : -1;  // bf16 bit patterns
  return -1;
}

}  // namespace

extern "C" int llc_npy_info(const char* path, int expect_dtype, size_t* dtype, size_t* rank, size_t* size,
                            size_t* data_offset) {
  if (!path || !dtype || !rank || !size || !data_offset) return set_error(LLC_ERR_BAD_ARG, "npy_info: null argument");
  FILE* fp = fopen(path, "rb");
  if (!fp) return set_error(LLC_ERR_BAD_ARG, "npy: cannot open %s", path);
  NpyInfo info;
  int st = parse_header(fp, path, &info);
  fclose(fp);
  LLC_TRY(st);
  // the reference assumes C order without looking (LoadWeight.cpp reads the flag and ignores it); a
  // Fortran-ordered file would be read transposed, so it is refused here
  if (info.fortran && info.shape.size() > 1) return set_error(LLC_ERR_LAYOUT, "npy: %s is in Fortran order", path);
  const int dt = dtype_of(info.descr, expect_dtype);
  if (dt < 0) return set_error(LLC_ERR_DTYPE, "npy: %s: element type '%s' is not read", path, info.descr.c_str());
  if (expect_dtype >= 0 && dt != expect_dtype)
    return set_error(LLC_ERR_DTYPE, "npy: %s holds type code %d, %d expected", path, dt, expect_dtype);
  *dtype = (size_t)dt;
  *rank = info.shape.size();
  for (size_t i = 0; i < info.shape.size(); ++i) size[i] = info.shape[i];
  *data_offset = info.data_offset;
  return LLC_OK;
}

extern "C" int llc_plan_load_npy(llc_plan_t* plan, const char* path, int expect_dtype, llc_tensor* out, size_t* size_out,
                                 size_t* stride_out) {
  if (!plan || !out || !size_out || !stride_out) return set_error(LLC_ERR_BAD_ARG, "plan_load_npy: null argument");
  size_t dtype = 0, rank = 0, off = 0;
  LLC_TRY(llc_npy_info(path, expect_dtype, &dtype, &rank, size_out, &off));
  size_t n = 1;
  for (size_t i = rank; i-- > 0;) {
    stride_out[i] = n;
    if (size_out[i] != 0 && n > SIZE_MAX / 16 / size_out[i]) return set_error(LLC_ERR_TOO_LARGE, "npy: %s: shape overflows", path);
    n *= size_out[i];
  }
  const size_t bytes = n * dtype_size(dtype);
  FILE* fp = fopen(path, "rb");
  if (!fp) return set_error(LLC_ERR_BAD_ARG, "npy: cannot open %s", path);
  // the header's shape is not trusted before the file is seen to hold that much data (a damaged header must not
  // become a huge allocation)
  if (fseek(fp, 0, SEEK_END) != 0 || ftell(fp) < 0 || (size_t)ftell(fp) < off || (size_t)ftell(fp) - off < bytes) {
    fclose(fp);
    return set_error(LLC_ERR_BAD_ARG, "npy: %s holds fewer than %zu bytes of data", path, bytes);
  }
  std::vector<char> host;
  try {
    host.resize(bytes ? bytes : 1);
  } catch (...) {
    fclose(fp);
    return set_error(LLC_ERR_TOO_LARGE, "npy: %s: no host memory for %zu bytes", path, bytes);
  }
  const bool ok = fseek(fp, (long)off, SEEK_SET) == 0 && fread(host.data(), 1, bytes, fp) == bytes;
  fclose(fp);
  if (!ok) return set_error(LLC_ERR_BAD_ARG, "npy: %s holds fewer than %zu bytes of data", path, bytes);
  void* dev = nullptr;
  LLC_TRY(llc_plan_upload(plan, host.data(), bytes, &dev));
  out->data = out->base = dev;
  out->type = dtype;
  out->offset = 0;
  out->rank = rank;
  out->size = size_out;
  out->stride = stride_out;
  return LLC_OK;
}
