/* llc_run_plan: a host in plain C that runs a plan file through the C-ABI alone (no Python, no torch, no HIP
 * headers): the part the reference's C++ `Execution` plays for its compiled shared object
 * (src/Compiler/Execution.cpp:12-66: load, pack the tensors into the void** block, call the entry).
 *
 *   llc_run_plan PLAN IN0.npy [IN1.npy ...] -o OUT0.npy [OUT1.npy ...]
 *
 * Inputs are NumPy .npy files in the order of the plan's parameter block; they must have the type and extents
 * the plan was recorded for.  Outputs are written as .npy (bf16 as '<u2' bit patterns).  Exit status 0 on
 * success; 1 with a message on stderr otherwise. */
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "llc_hip.h"

static void die(const char* what) {
  fprintf(stderr, "llc_run_plan: %s: %s\n", what, llc_hip_last_error());
  exit(1);
}

static const char* npy_descr(size_t type) {
  switch (type) {
    case LLC_INT8: return "|i1";
    case LLC_INT16: return "<i2";
    case LLC_INT32: return "<i4";
    case LLC_INT64: return "<i8";
    case LLC_FLOAT32: return "<f4";
    case LLC_DOUBLE64: return "<f8";
    case LLC_INT1: return "|b1";
    case LLC_BFLOAT16: return "<u2";
    case LLC_FLOAT16: return "<f2";
  }
  return NULL;
}

static size_t type_bytes(size_t type) {
  switch (type) {
    case LLC_INT8: case LLC_INT1: return 1;
    case LLC_INT16: case LLC_BFLOAT16: case LLC_FLOAT16: return 2;
    case LLC_INT32: case LLC_FLOAT32: return 4;
    default: return 8;
  }
}

/* .npy format 1.0: magic, version, little-endian u16 header length, a Python dict literal padded with
 * spaces to a multiple of 64 bytes and ended by a newline, then the data in C order. */
static int write_npy(const char* path, size_t type, size_t rank, const size_t* size, const void* data, size_t bytes) {
  char dict[512];
  int n = snprintf(dict, sizeof(dict), "{'descr': '%s', 'fortran_order': False, 'shape': (", npy_descr(type));
  for (size_t d = 0; d < rank; ++d) n += snprintf(dict + n, sizeof(dict) - n, "%zu%s", size[d], (rank == 1 || d + 1 < rank) ? ", " : "");
  n += snprintf(dict + n, sizeof(dict) - n, "), }");
  size_t total = 10 + (size_t)n + 1;
  size_t pad = (64 - total % 64) % 64;
  unsigned short hlen = (unsigned short)(n + pad + 1);
  FILE* f = fopen(path, "wb");
  if (!f) return -1;
  fwrite("\x93NUMPY\x01\x00", 1, 8, f);
  fputc(hlen & 0xff, f);
  fputc(hlen >> 8, f);
  fwrite(dict, 1, (size_t)n, f);
  for (size_t i = 0; i < pad; ++i) fputc(' ', f);
  fputc('\n', f);
  if (bytes && fwrite(data, 1, bytes, f) != bytes) {
    fclose(f);
    return -1;
  }
  return fclose(f);
}

int main(int argc, char** argv) {
  int split = -1;
  for (int i = 2; i < argc; ++i)
    if (strcmp(argv[i], "-o") == 0) split = i;
  if (argc < 2 || split < 0) {
    fprintf(stderr, "usage: llc_run_plan PLAN IN0.npy [IN1.npy ...] -o OUT0.npy [OUT1.npy ...]\n");
    return 1;
  }
  if (llc_hip_init(0) != LLC_OK) die("no usable device");
  llc_plan_t* plan = NULL;
  if (llc_plan_load(argv[1], &plan) != LLC_OK) die("loading the plan");
  size_t n_in = 0, n_out = 0;
  llc_plan_num_io(plan, &n_in, &n_out);
  if ((size_t)(split - 2) != n_in || (size_t)(argc - split - 1) != n_out) {
    fprintf(stderr, "llc_run_plan: the plan takes %zu inputs and gives %zu outputs\n", n_in, n_out);
    return 1;
  }
  const size_t n = n_in + n_out;
  /* the reference's block: slot 0 the symbol values, then per tensor base, data, &offset, sizes, strides */
  void** params = (void**)calloc(1 + 5 * n, sizeof(void*));
  size_t* sizes = (size_t*)calloc(n * LLC_MAX_RANK, sizeof(size_t));
  size_t* strides = (size_t*)calloc(n * LLC_MAX_RANK, sizeof(size_t));
  size_t* offsets = (size_t*)calloc(n, sizeof(size_t));
  llc_tensor* like = (llc_tensor*)calloc(n, sizeof(llc_tensor));
  size_t* out_bytes = (size_t*)calloc(n, sizeof(size_t));
  for (size_t k = 0; k < n; ++k) {
    size_t* sz = sizes + k * LLC_MAX_RANK;
    size_t* st = strides + k * LLC_MAX_RANK;
    if (llc_plan_io_info(plan, k, &like[k], sz, st) != LLC_OK) die("reading the plan's tensors");
    void* dev = NULL;
    if (k < n_in) {
      llc_tensor got;
      size_t gsz[LLC_MAX_RANK], gst[LLC_MAX_RANK];
      if (llc_plan_load_npy(plan, argv[2 + k], (int)like[k].type, &got, gsz, gst) != LLC_OK) die(argv[2 + k]);
      int same = got.rank == like[k].rank;
      for (size_t d = 0; same && d < got.rank; ++d) same = gsz[d] == sz[d] && (sz[d] <= 1 || gst[d] == st[d]);
      if (!same) {
        fprintf(stderr, "llc_run_plan: %s does not have the extents (or the plan not the dense layout) of input %zu\n", argv[2 + k], k);
        return 1;
      }
      dev = got.data;
    } else {
      size_t count = 1, span = 1;
      for (size_t d = 0; d < like[k].rank; ++d) {
        count *= sz[d];
        if (sz[d]) span += (sz[d] - 1) * st[d];
      }
      if (count && span != count) {
        fprintf(stderr, "llc_run_plan: output %zu is not dense in memory\n", k - n_in);
        return 1;
      }
      out_bytes[k] = count * type_bytes(like[k].type);
      if (llc_plan_alloc(plan, out_bytes[k], &dev) != LLC_OK) die("allocating an output");
    }
    params[1 + 5 * k] = dev;
    params[2 + 5 * k] = dev;
    params[3 + 5 * k] = &offsets[k];
    params[4 + 5 * k] = sz;
    params[5 + 5 * k] = st;
  }
  if (llc_hip_run(plan, params, NULL) != LLC_OK) die("running the plan");
  for (size_t k = n_in; k < n; ++k) {
    void* host = malloc(out_bytes[k] ? out_bytes[k] : 1);
    if (llc_hip_download(host, params[2 + 5 * k], out_bytes[k], NULL) != LLC_OK) die("reading an output back");
    /* a dense output may still be a permutation of C order: written in C order only when the strides say so */
    size_t expect = 1;
    int c_order = 1;
    for (size_t d = like[k].rank; d-- > 0;) {
      const size_t* sz = sizes + k * LLC_MAX_RANK;
      const size_t* st = strides + k * LLC_MAX_RANK;
      if (sz[d] > 1 && st[d] != expect) c_order = 0;
      expect *= sz[d];
    }
    if (!c_order) {
      fprintf(stderr, "llc_run_plan: output %zu is not in C order\n", k - n_in);
      return 1;
    }
    if (write_npy(argv[split + 1 + (k - n_in)], like[k].type, like[k].rank, sizes + k * LLC_MAX_RANK, host, out_bytes[k]) != 0) {
      fprintf(stderr, "llc_run_plan: cannot write %s\n", argv[split + 1 + (k - n_in)]);
      return 1;
    }
    free(host);
  }
  llc_plan_destroy(plan);
  return 0;
}
