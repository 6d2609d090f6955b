// Model-level boundary: a plan is a recorded sequence of kernel calls that is replayed from the reference's
// packed `main(void** params)` block (src/Compiler/Execution.cpp:21-66).
//
// The per-op entry points of the C-ABI are defined here as wrappers around the launchers (entries.hpp).
// Between llc_plan_begin and llc_plan_end every successful call made by the recording thread is also
// appended to the plan, with deep copies of its descriptors and attributes.  An operand whose address lies
// inside a declared input or output tensor is bound to that tensor: llc_hip_run re-bases it on the pointer
// the params block carries for the tensor; every other address (weights uploaded into the plan, its arena,
// caller-owned constants) is replayed as recorded.  A replay allocates nothing and makes no host-device
// synchronisation: it is the list of kernel launches, in order, on the given stream.
#include <algorithm>
#include <cstdio>
#include <cstring>
#include <memory>
#include <mutex>
#include <utility>
#include <vector>

#include "common.hpp"

using namespace llc;

namespace {

enum OpCode {
  kMatmul, kBatchMatmul, kConv2d, kElementwise, kReduce, kSoftmax, kLayerNorm, kMaxPool, kGlobalAvgPool,
  kTranspose, kStrideSlice, kBroadcastTo, kCopy, kGatherRows, kConvert, kAttention,
};

// Owned copy of a tensor descriptor.
struct Operand {
  llc_tensor t{};
  size_t size[LLC_MAX_RANK];
  size_t stride[LLC_MAX_RANK];
  bool present = false;
  int io = -1;        // index among the params tensors (inputs, then outputs); -1 = fixed address
  int64_t delta = 0;  // bytes from that tensor's first element

  // Copies *src; `offset` is folded into the data pointer.  Returns false for a malformed descriptor.
  bool assign(const llc_tensor* src) {
    if (!src) return true;  // stays absent
    const size_t es = dtype_size(src->type);
    if (src->rank > LLC_MAX_RANK || es == 0 || (src->rank && (!src->size || !src->stride))) return false;
    present = true;
    t = *src;
    for (size_t i = 0; i < src->rank; ++i) {
      size[i] = src->size[i];
      stride[i] = src->stride[i];
    }
    t.size = size;
    t.stride = stride;
    t.data = src->data ? (char*)src->data + src->offset * es : nullptr;
    t.base = t.data;
    t.offset = 0;
    return true;
  }
  llc_tensor* ptr() { return present ? &t : nullptr; }
  // bytes from the first element to one past the last addressed element
  size_t span_bytes() const {
    size_t last = 0;
    for (size_t i = 0; i < t.rank; ++i) {
      if (size[i] == 0) return 0;
      last += (size[i] - 1) * stride[i];
    }
    return (last + 1) * dtype_size(t.type);
  }
};

struct Step {
  int op = 0;
  std::vector<Operand> opnd;  // element addresses stay put when the step moves
  bool has_epi = false;
  float alpha = 1.0f;
  int act = 0;
  int kind = 0;
  double eps = 0.0;
  size_t n_ints = 0;
  int64_t ints[3 * LLC_MAX_RANK];
  union {
    llc_conv_attrs conv;
    llc_pool_attrs pool;
  };
  std::unique_ptr<llc_ew_program> prog;
  Step() { memset(&conv, 0, sizeof(conv)); }
};

struct Io {
  Operand like;
  char* lo = nullptr;  // address range the tensor occupied while the plan was recorded
  char* hi = nullptr;
  bool output = false;
  // address of the first element modulo 16 while the plan was recorded: kernels were chosen for that alignment
  // (16-byte vector and direct-to-LDS paths, split reductions), so a run must bind the same class
  unsigned align16 = 0;
};

struct Overlap {
  int first, second;
  int64_t diff;  // recorded address of `second` minus that of `first`
};

enum State { kOpen, kRecording, kReady, kBroken };

}  // namespace

struct llc_plan {
  int device = 0;
  State state = kOpen;
  std::vector<Io> io;
  size_t n_inputs = 0;
  std::vector<Step> steps;
  std::vector<void*> owned;
  std::vector<int64_t> symbols;
  std::vector<Overlap> overlaps;
  std::vector<char*> bound;  // per run: first element of every params tensor
  // scratch memory of the steps that split a reduction: sized while recording (the largest request), allocated
  // by llc_plan_end / llc_plan_load, handed to the kernels by llc_hip_run (which therefore never allocates)
  void* ws = nullptr;
  size_t ws_bytes = 0;
  std::mutex mu;
};

namespace {

thread_local llc_plan* t_rec = nullptr;

// ---- recording ----
int bind(llc_plan* p, Operand& o) {
  if (!o.present || !o.t.data) return LLC_OK;
  char* a = (char*)o.t.data;
  for (size_t k = 0; k < p->io.size(); ++k) {
    const Io& io = p->io[k];
    if (a >= io.lo && a < io.hi) {
      o.io = (int)k;
      o.delta = a - io.lo;
      return LLC_OK;
    }
  }
  return LLC_OK;
}

struct Recorder {
  llc_plan* p;
  Step st;
  bool ok = true;
  Recorder(int op, size_t n_operands) : p(t_rec) {
    st.op = op;
    st.opnd.resize(n_operands);
  }
  void tensor(size_t i, const llc_tensor* t) {
    if (!st.opnd[i].assign(t)) ok = false;
    bind(p, st.opnd[i]);
  }
  void epilogue(const llc_epilogue* e, size_t bias_at) {
    if (!e) return;
    st.has_epi = true;
    st.alpha = e->alpha;
    st.act = e->act;
    tensor(bias_at, e->bias);
    tensor(bias_at + 1, e->residual);
  }
  void ints(const int64_t* v, size_t n) {
    if (st.n_ints + n > sizeof(st.ints) / sizeof(st.ints[0]) || (n && !v)) {
      ok = false;
      return;
    }
    for (size_t i = 0; i < n; ++i) st.ints[st.n_ints++] = v[i];
  }
  int commit() {
    if (!ok) {
      p->state = kBroken;
      t_rec = nullptr;
      workspace_track(nullptr);
      return set_error(LLC_ERR_BAD_ARG, "plan: a call could not be recorded (descriptor rank or attribute count)");
    }
    p->steps.push_back(std::move(st));
    return LLC_OK;
  }
};

// ---- replay ----
inline void rebase(Step& s, char* const* bound) {
  for (Operand& o : s.opnd)
    if (o.io >= 0) o.t.data = o.t.base = bound[o.io] + o.delta;
}

// Operand count every step code is recorded with (0: variable, the elementwise program's inputs + 1).  A plan
// file whose step disagrees is refused: replay() indexes the operands by position.
int operands_of(int op) {
  switch (op) {
    case kMatmul: case kBatchMatmul: case kConv2d: case kAttention: return 5;
    case kLayerNorm: return 4;
    case kGatherRows: return 3;
    case kElementwise: return 0;
    default: return 2;
  }
}

// The shape of a loaded step: operand count, required operands present, integer attributes sized by the
// operand's rank.  Returns null when it is what the recorder would have written, else what is wrong.
const char* step_defect(const Step& s) {
  const size_t n = s.opnd.size();
  if (s.op == kElementwise) {
    if (!s.prog) return "elementwise step without a program";
    if (n < 1 || n > LLC_EW_MAX_INPUTS + 1) return "elementwise step with too many operands";
    for (const Operand& o : s.opnd)
      if (!o.present) return "elementwise step with an absent operand";
    return nullptr;
  }
  if (s.prog) return "a program on a step that is not elementwise";
  if (n != (size_t)operands_of(s.op)) return "operand count does not fit the step code";
  auto need = [&](size_t i) { return s.opnd[i].present; };
  switch (s.op) {
    case kMatmul: case kBatchMatmul: case kConv2d:
      if (!need(0) || !need(1) || !need(4)) return "contraction without lhs, rhs or output";
      break;
    case kAttention:
      if (!need(0) || !need(1) || !need(2) || !need(4)) return "attention without q, k, v or output";
      break;
    case kLayerNorm:
      if (!need(0) || !need(3)) return "layer_norm without input or output";
      break;
    case kGatherRows:
      if (!need(0) || !need(1) || !need(2)) return "gather without table, indices or output";
      break;
    default:
      if (!need(0) || !need(1)) return "step without input or output";
  }
  const size_t rank0 = s.opnd[0].t.rank;
  if (s.op == kTranspose && s.n_ints != rank0) return "transpose: one permutation entry per dim expected";
  if (s.op == kStrideSlice && s.n_ints != 3 * rank0) return "stride_slice: start, end and step per dim expected";
  if (s.op == kReduce && (s.n_ints == 0 || s.n_ints > rank0)) return "reduce: axis list does not fit the operand";
  return nullptr;
}

int replay(Step& s, void* stream) {
  Operand* o = s.opnd.data();
  llc_epilogue epi;
  const llc_epilogue* e = nullptr;
  switch (s.op) {
    case kMatmul:
    case kBatchMatmul:
    case kConv2d:
      if (s.has_epi) {
        epi.alpha = s.alpha;
        epi.bias = o[2].ptr();
        epi.residual = o[3].ptr();
        epi.act = s.act;
        e = &epi;
      }
      if (s.op == kMatmul) return llc_impl_matmul(o[0].ptr(), o[1].ptr(), e, o[4].ptr(), stream);
      if (s.op == kBatchMatmul) return llc_impl_batch_matmul(o[0].ptr(), o[1].ptr(), e, o[4].ptr(), stream);
      return llc_impl_conv2d(o[0].ptr(), o[1].ptr(), &s.conv, e, o[4].ptr(), stream);
    case kElementwise: {
      const llc_tensor* ins[LLC_EW_MAX_INPUTS];
      const size_t n = s.opnd.size() - 1;
      if (n > LLC_EW_MAX_INPUTS) return set_error(LLC_ERR_BAD_ARG, "plan: elementwise step with %zu inputs", n);
      for (size_t i = 0; i < n; ++i) ins[i] = o[i].ptr();
      return llc_impl_elementwise(s.prog.get(), ins, n, o[n].ptr(), stream);
    }
    case kReduce: return llc_impl_reduce(s.kind, o[0].ptr(), s.ints, s.n_ints, o[1].ptr(), stream);
    case kSoftmax: return llc_impl_softmax(o[0].ptr(), o[1].ptr(), stream);
    case kLayerNorm: return llc_impl_layer_norm(o[0].ptr(), o[1].ptr(), o[2].ptr(), s.eps, o[3].ptr(), stream);
    case kMaxPool: return llc_impl_max_pool(o[0].ptr(), &s.pool, o[1].ptr(), stream);
    case kGlobalAvgPool: return llc_impl_global_avg_pool(o[0].ptr(), o[1].ptr(), stream);
    case kTranspose: return llc_impl_transpose(o[0].ptr(), s.ints, o[1].ptr(), stream);
    case kStrideSlice: {
      const size_t r = s.n_ints / 3;
      return llc_impl_stride_slice(o[0].ptr(), s.ints, s.ints + r, s.ints + 2 * r, o[1].ptr(), stream);
    }
    case kBroadcastTo: return llc_impl_broadcast_to(o[0].ptr(), o[1].ptr(), stream);
    case kCopy: return llc_impl_copy(o[0].ptr(), o[1].ptr(), stream);
    case kGatherRows: return llc_impl_gather_rows(o[0].ptr(), o[1].ptr(), o[2].ptr(), stream);
    case kConvert: return llc_impl_convert(o[0].ptr(), o[1].ptr(), stream);
    case kAttention: return llc_impl_attention(o[0].ptr(), o[1].ptr(), o[2].ptr(), o[3].ptr(), s.alpha, o[4].ptr(), stream);
  }
  return set_error(LLC_ERR_BAD_ARG, "plan: unknown step code %d", s.op);
}

int check_device(llc_plan* p, const char* what) {
  int dev = -1;
  LLC_HIP_TRY(hipGetDevice(&dev));
  if (dev != p->device)
    return set_error(LLC_ERR_BAD_ARG, "%s: the plan belongs to device %d, the current device is %d", what, p->device, dev);
  return LLC_OK;
}

}  // namespace

// ---- per-op entry points: launch, then record if a plan is recording on this thread ----
extern "C" int llc_hip_matmul(const llc_tensor* lhs, const llc_tensor* rhs, const llc_epilogue* epi, llc_tensor* out,
                              void* stream) {
  LLC_TRY(llc_impl_matmul(lhs, rhs, epi, out, stream));
  if (!t_rec) return LLC_OK;
  Recorder r(kMatmul, 5);
  r.tensor(0, lhs), r.tensor(1, rhs), r.epilogue(epi, 2), r.tensor(4, out);
  return r.commit();
}

extern "C" int llc_hip_batch_matmul(const llc_tensor* lhs, const llc_tensor* rhs, const llc_epilogue* epi,
                                    llc_tensor* out, void* stream) {
  LLC_TRY(llc_impl_batch_matmul(lhs, rhs, epi, out, stream));
  if (!t_rec) return LLC_OK;
  Recorder r(kBatchMatmul, 5);
  r.tensor(0, lhs), r.tensor(1, rhs), r.epilogue(epi, 2), r.tensor(4, out);
  return r.commit();
}

extern "C" int llc_hip_conv2d(const llc_tensor* x, const llc_tensor* w, const llc_conv_attrs* attrs,
                              const llc_epilogue* epi, llc_tensor* out, void* stream) {
  LLC_TRY(llc_impl_conv2d(x, w, attrs, epi, out, stream));
  if (!t_rec) return LLC_OK;
  Recorder r(kConv2d, 5);
  r.tensor(0, x), r.tensor(1, w), r.epilogue(epi, 2), r.tensor(4, out);
  r.st.conv = *attrs;
  return r.commit();
}

extern "C" int llc_hip_elementwise(const llc_ew_program* prog, const llc_tensor* const* inputs, size_t n_inputs,
                                   llc_tensor* out, void* stream) {
  LLC_TRY(llc_impl_elementwise(prog, inputs, n_inputs, out, stream));
  if (!t_rec) return LLC_OK;
  Recorder r(kElementwise, n_inputs + 1);
  for (size_t i = 0; i < n_inputs; ++i) r.tensor(i, inputs[i]);
  r.tensor(n_inputs, out);
  r.st.prog.reset(new llc_ew_program(*prog));
  return r.commit();
}

extern "C" int llc_hip_reduce(int kind, const llc_tensor* x, const int64_t* axes, size_t n_axes, llc_tensor* out,
                              void* stream) {
  LLC_TRY(llc_impl_reduce(kind, x, axes, n_axes, out, stream));
  if (!t_rec) return LLC_OK;
  Recorder r(kReduce, 2);
  r.tensor(0, x), r.tensor(1, out), r.ints(axes, n_axes);
  r.st.kind = kind;
  return r.commit();
}

extern "C" int llc_hip_softmax(const llc_tensor* x, llc_tensor* out, void* stream) {
  LLC_TRY(llc_impl_softmax(x, out, stream));
  if (!t_rec) return LLC_OK;
  Recorder r(kSoftmax, 2);
  r.tensor(0, x), r.tensor(1, out);
  return r.commit();
}

extern "C" int llc_hip_layer_norm(const llc_tensor* x, const llc_tensor* scale, const llc_tensor* bias, double epsilon,
                                  llc_tensor* out, void* stream) {
  LLC_TRY(llc_impl_layer_norm(x, scale, bias, epsilon, out, stream));
  if (!t_rec) return LLC_OK;
  Recorder r(kLayerNorm, 4);
  r.tensor(0, x), r.tensor(1, scale), r.tensor(2, bias), r.tensor(3, out);
  r.st.eps = epsilon;
  return r.commit();
}

extern "C" int llc_hip_max_pool(const llc_tensor* x, const llc_pool_attrs* attrs, llc_tensor* out, void* stream) {
  LLC_TRY(llc_impl_max_pool(x, attrs, out, stream));
  if (!t_rec) return LLC_OK;
  Recorder r(kMaxPool, 2);
  r.tensor(0, x), r.tensor(1, out);
  r.st.pool = *attrs;
  return r.commit();
}

extern "C" int llc_hip_global_avg_pool(const llc_tensor* x, llc_tensor* out, void* stream) {
  LLC_TRY(llc_impl_global_avg_pool(x, out, stream));
  if (!t_rec) return LLC_OK;
  Recorder r(kGlobalAvgPool, 2);
  r.tensor(0, x), r.tensor(1, out);
  return r.commit();
}

extern "C" int llc_hip_transpose(const llc_tensor* x, const int64_t* perms, llc_tensor* out, void* stream) {
  LLC_TRY(llc_impl_transpose(x, perms, out, stream));
  if (!t_rec) return LLC_OK;
  Recorder r(kTranspose, 2);
  r.tensor(0, x), r.tensor(1, out), r.ints(perms, x->rank);
  return r.commit();
}

extern "C" int llc_hip_stride_slice(const llc_tensor* x, const int64_t* start, const int64_t* end, const int64_t* step,
                                    llc_tensor* out, void* stream) {
  LLC_TRY(llc_impl_stride_slice(x, start, end, step, out, stream));
  if (!t_rec) return LLC_OK;
  Recorder r(kStrideSlice, 2);
  r.tensor(0, x), r.tensor(1, out);
  r.ints(start, x->rank), r.ints(end, x->rank), r.ints(step, x->rank);
  return r.commit();
}

extern "C" int llc_hip_broadcast_to(const llc_tensor* x, llc_tensor* out, void* stream) {
  LLC_TRY(llc_impl_broadcast_to(x, out, stream));
  if (!t_rec) return LLC_OK;
  Recorder r(kBroadcastTo, 2);
  r.tensor(0, x), r.tensor(1, out);
  return r.commit();
}

extern "C" int llc_hip_copy(const llc_tensor* x, llc_tensor* out, void* stream) {
  LLC_TRY(llc_impl_copy(x, out, stream));
  if (!t_rec) return LLC_OK;
  Recorder r(kCopy, 2);
  r.tensor(0, x), r.tensor(1, out);
  return r.commit();
}

extern "C" int llc_hip_gather_rows(const llc_tensor* table, const llc_tensor* idx, llc_tensor* out, void* stream) {
  LLC_TRY(llc_impl_gather_rows(table, idx, out, stream));
  if (!t_rec) return LLC_OK;
  Recorder r(kGatherRows, 3);
  r.tensor(0, table), r.tensor(1, idx), r.tensor(2, out);
  return r.commit();
}

extern "C" int llc_hip_convert(const llc_tensor* x, llc_tensor* out, void* stream) {
  LLC_TRY(llc_impl_convert(x, out, stream));
  if (!t_rec) return LLC_OK;
  Recorder r(kConvert, 2);
  r.tensor(0, x), r.tensor(1, out);
  return r.commit();
}

extern "C" int llc_hip_attention(const llc_tensor* q, const llc_tensor* k, const llc_tensor* v, const llc_tensor* mask,
                                 float scale, llc_tensor* out, void* stream) {
  LLC_TRY(llc_impl_attention(q, k, v, mask, scale, out, stream));
  if (!t_rec) return LLC_OK;
  Recorder r(kAttention, 5);
  r.tensor(0, q), r.tensor(1, k), r.tensor(2, v), r.tensor(3, mask), r.tensor(4, out);
  r.st.alpha = scale;
  return r.commit();
}

// ---- plan life cycle ----
extern "C" int llc_plan_create(llc_plan_t** plan) {
  if (!plan) return set_error(LLC_ERR_BAD_ARG, "plan_create: null argument");
  int dev = -1;
  LLC_HIP_TRY(hipGetDevice(&dev));
  llc_plan* p = new llc_plan();
  p->device = dev;
  *plan = p;
  return LLC_OK;
}

extern "C" int llc_plan_destroy(llc_plan_t* p) {
  if (!p) return LLC_OK;
  if (t_rec == p) {
    t_rec = nullptr;
    workspace_track(nullptr);
  }
  int status = LLC_OK;
  for (void* m : p->owned) {
    hipError_t e = hipFree(m);  // waits for the device to finish with the memory
    if (e != hipSuccess) status = set_error(LLC_ERR_HIP, "plan_destroy: hipFree: %s", hipGetErrorString(e));
  }
  delete p;
  return status;
}

extern "C" int llc_plan_alloc(llc_plan_t* p, size_t bytes, void** device_ptr) {
  if (!p || !device_ptr) return set_error(LLC_ERR_BAD_ARG, "plan_alloc: null argument");
  LLC_TRY(check_device(p, "plan_alloc"));
  void* m = nullptr;
  LLC_HIP_TRY(hipMalloc(&m, bytes ? bytes : 1));
  p->owned.push_back(m);
  *device_ptr = m;
  return LLC_OK;
}

extern "C" int llc_plan_upload(llc_plan_t* p, const void* host, size_t bytes, void** device_ptr) {
  if (!host && bytes) return set_error(LLC_ERR_BAD_ARG, "plan_upload: null host pointer");
  LLC_TRY(llc_plan_alloc(p, bytes, device_ptr));
  if (bytes) LLC_HIP_TRY(hipMemcpy(*device_ptr, host, bytes, hipMemcpyHostToDevice));
  return LLC_OK;
}

extern "C" int llc_plan_declare_io(llc_plan_t* p, int is_output, const llc_tensor* like) {
  if (!p || !like) return set_error(LLC_ERR_BAD_ARG, "plan_declare_io: null argument");
  if (p->state != kOpen) return set_error(LLC_ERR_BAD_ARG, "plan_declare_io: tensors are declared before recording starts");
  if (!is_output && p->io.size() != p->n_inputs)
    return set_error(LLC_ERR_BAD_ARG, "plan_declare_io: inputs are declared before outputs");
  Io io;
  if (!io.like.assign(like)) return set_error(LLC_ERR_BAD_ARG, "plan_declare_io: malformed descriptor");
  io.output = is_output != 0;
  io.lo = (char*)io.like.t.data;
  io.hi = io.lo ? io.lo + io.like.span_bytes() : nullptr;
  io.align16 = (unsigned)((uintptr_t)io.lo % 16);
  p->io.push_back(std::move(io));
  Io& mine = p->io.back();
  mine.like.t.size = mine.like.t.stride = nullptr;  // the arrays moved with the copy; only like.size/.stride are read
  if (!is_output) p->n_inputs++;
  // a tensor that shares addresses with an earlier one: operands inside the shared range bind to the earlier
  // tensor, which is only right while the two keep their distance
  const int k = (int)p->io.size() - 1;
  for (int j = 0; j < k; ++j) {
    const Io& other = p->io[j];
    if (mine.lo && other.lo && mine.lo < other.hi && other.lo < mine.hi)
      p->overlaps.push_back({j, k, (int64_t)(mine.lo - other.lo)});
  }
  return LLC_OK;
}

extern "C" int llc_plan_expect_symbols(llc_plan_t* p, const int64_t* values, size_t n) {
  if (!p || (n && !values)) return set_error(LLC_ERR_BAD_ARG, "plan_expect_symbols: null argument");
  p->symbols.assign(values, values + n);
  return LLC_OK;
}

extern "C" int llc_plan_begin(llc_plan_t* p) {
  if (!p) return set_error(LLC_ERR_BAD_ARG, "plan_begin: null plan");
  if (t_rec) return set_error(LLC_ERR_BAD_ARG, "plan_begin: this thread is already recording a plan");
  if (p->state != kOpen) return set_error(LLC_ERR_BAD_ARG, "plan_begin: the plan has been recorded already");
  LLC_TRY(check_device(p, "plan_begin"));
  p->state = kRecording;
  p->ws_bytes = 0;
  workspace_track(&p->ws_bytes);
  t_rec = p;
  return LLC_OK;
}

extern "C" int llc_plan_end(llc_plan_t* p) {
  if (!p) return set_error(LLC_ERR_BAD_ARG, "plan_end: null plan");
  if (p->state == kBroken) return set_error(LLC_ERR_BAD_ARG, "plan_end: recording failed earlier");
  if (t_rec != p || p->state != kRecording) return set_error(LLC_ERR_BAD_ARG, "plan_end: the plan is not recording on this thread");
  t_rec = nullptr;
  workspace_track(nullptr);
  if (p->ws_bytes) {
    p->state = kBroken;  // until the scratch memory is there
    LLC_HIP_TRY(hipMalloc(&p->ws, p->ws_bytes));
    p->owned.push_back(p->ws);
  }
  p->state = kReady;
  p->bound.assign(p->io.size(), nullptr);
  return LLC_OK;
}

extern "C" int64_t llc_plan_num_steps(const llc_plan_t* p) { return p ? (int64_t)p->steps.size() : -1; }

extern "C" int64_t llc_plan_num_params(const llc_plan_t* p) { return p ? (int64_t)(1 + 5 * p->io.size()) : -1; }

// ---- replay from the packed parameter block ----
extern "C" int llc_hip_run(llc_plan_t* p, void* const* params, void* stream) {
  if (!p || !params) return set_error(LLC_ERR_BAD_ARG, "run: null argument");
  if (p->state != kReady) return set_error(LLC_ERR_BAD_ARG, "run: the plan has not been recorded (begin .. end)");
  if (t_rec) return set_error(LLC_ERR_BAD_ARG, "run: this thread is recording a plan");
  std::lock_guard<std::mutex> lock(p->mu);
  if (!p->symbols.empty()) {
    const int64_t* sym = (const int64_t*)params[0];
    if (!sym) return set_error(LLC_ERR_BAD_ARG, "run: the plan expects %zu symbol values, slot 0 is null", p->symbols.size());
    for (size_t i = 0; i < p->symbols.size(); ++i)
      if (sym[i] != p->symbols[i])
        return set_error(LLC_ERR_SHAPE, "run: symbol %zu is %lld, the plan was specialised for %lld", i, (long long)sym[i],
                         (long long)p->symbols[i]);
  }
  size_t slot = 1;
  for (size_t k = 0; k < p->io.size(); ++k, slot += 5) {
    const Operand& like = p->io[k].like;
    char* data = (char*)params[slot + 1];
    const size_t* off = (const size_t*)params[slot + 2];
    const size_t* size = (const size_t*)params[slot + 3];
    const size_t* stride = (const size_t*)params[slot + 4];
    if (!off || (like.t.rank && (!size || !stride)))
      return set_error(LLC_ERR_BAD_ARG, "run: tensor %zu has a null offset, size or stride slot", k);
    bool empty = false;
    for (size_t d = 0; d < like.t.rank; ++d) {
      if (size[d] != like.size[d])
        return set_error(LLC_ERR_SHAPE, "run: tensor %zu has extent %zu in dim %zu, the plan was specialised for %zu", k,
                         size[d], d, like.size[d]);
      if (size[d] > 1 && stride[d] != like.stride[d])
        return set_error(LLC_ERR_LAYOUT, "run: tensor %zu has stride %zu in dim %zu, the plan was specialised for %zu", k,
                         stride[d], d, like.stride[d]);
      empty |= size[d] == 0;
    }
    if (!data && !empty) return set_error(LLC_ERR_BAD_ARG, "run: tensor %zu has a null data pointer", k);
    p->bound[k] = data ? data + *off * dtype_size(like.t.type) : nullptr;
    if (p->bound[k] && (uintptr_t)p->bound[k] % 16 != p->io[k].align16)
      return set_error(LLC_ERR_LAYOUT, "run: tensor %zu lies at an address that is %u modulo 16, the plan was recorded with %u "
                       "(its kernels and scratch memory were chosen for that alignment)", k,
                       (unsigned)((uintptr_t)p->bound[k] % 16), p->io[k].align16);
  }
  for (const Overlap& ov : p->overlaps)
    if (p->bound[ov.second] - p->bound[ov.first] != ov.diff)
      return set_error(LLC_ERR_LAYOUT, "run: tensors %d and %d shared memory when the plan was recorded and do not now", ov.first,
                       ov.second);
  WorkspaceScope scratch(p->ws, p->ws_bytes);  // the steps use the plan's own scratch memory: nothing is allocated here
  for (Step& s : p->steps) {
    rebase(s, p->bound.data());
    LLC_TRY(replay(s, stream));
  }
  return LLC_OK;
}

// ---- `void main(void**)` convention: one plan bound per process ----
namespace {
llc_plan* g_entry_plan = nullptr;
void* g_entry_stream = nullptr;
int g_entry_status = LLC_OK;
}  // namespace

extern "C" int llc_hip_bind_entry(llc_plan_t* p, void* stream) {
  if (p && p->state != kReady) return set_error(LLC_ERR_BAD_ARG, "bind_entry: the plan has not been recorded");
  g_entry_plan = p;
  g_entry_stream = stream;
  g_entry_status = LLC_OK;
  return LLC_OK;
}

extern "C" void llc_hip_entry(void** params) {
  if (!g_entry_plan) {
    g_entry_status = set_error(LLC_ERR_BAD_ARG, "entry: no plan is bound (llc_hip_bind_entry)");
  } else {
    g_entry_status = llc_hip_run(g_entry_plan, params, g_entry_stream);
  }
  // the reference's entry returns nothing and its failures are only logged (Logger.h:132-134)
  if (g_entry_status != LLC_OK) fprintf(stderr, "llc_hip_entry: %s\n", llc_hip_last_error());
}

extern "C" int llc_hip_entry_status(void) { return g_entry_status; }

// ---- plans on disk --------------------------------------------------------------------------------------
// The reference's compile step leaves a shared object with the weights baked in, which Execution loads and
// runs later (src/Compiler/Compiler.cpp:306-330, src/Compiler/Execution.cpp:21-66).  The counterpart here is
// a plan file: the recorded steps, the declared tensors, and the device memory the steps address outside
// those tensors.  That memory is cut into regions (maximal runs of overlapping operand ranges); a region
// whose every byte is written by a step before a step reads it is scratch and only its size is kept, any
// other region (constants, weights uploaded into the plan) is stored with its contents as they are when the
// plan is saved.  Loading allocates the regions in memory owned by the new plan, at the same address modulo
// 256, and points the operands into them.
namespace {

constexpr char kPlanMagic[8] = {'L', 'L', 'C', 'P', 'L', 'A', 'N', '1'};

struct Region {
  char* lo;
  char* hi;
  bool keep = false;                                // contents are part of the plan
  std::vector<std::pair<char*, char*>> written;     // ranges known to be fully written by earlier steps
};

struct Writer {
  FILE* f;
  bool ok = true;
  void raw(const void* p, size_t n) {
    if (ok && n && fwrite(p, 1, n, f) != n) ok = false;
  }
  template <typename T>
  void pod(const T& v) { raw(&v, sizeof(T)); }
  void u64(uint64_t v) { pod(v); }
  void i64(int64_t v) { pod(v); }
};

struct Reader {
  FILE* f;
  bool ok = true;
  void raw(void* p, size_t n) {
    if (ok && n && fread(p, 1, n, f) != n) ok = false;
  }
  template <typename T>
  void pod(T& v) { raw(&v, sizeof(T)); }
  uint64_t u64() {
    uint64_t v = 0;
    pod(v);
    return v;
  }
  int64_t i64() {
    int64_t v = 0;
    pod(v);
    return v;
  }
};

void write_operand_shape(Writer& w, const Operand& o) {
  w.u64(o.present ? 1 : 0);
  if (!o.present) return;
  w.u64(o.t.type);
  w.u64(o.t.rank);
  for (size_t i = 0; i < o.t.rank; ++i) w.u64(o.size[i]), w.u64(o.stride[i]);
}

bool read_operand_shape(Reader& r, Operand& o) {
  o.present = r.u64() != 0;
  if (!o.present) return r.ok;
  memset(&o.t, 0, sizeof(o.t));
  o.t.type = (size_t)r.u64();
  o.t.rank = (size_t)r.u64();
  if (!r.ok || o.t.rank > LLC_MAX_RANK || dtype_size(o.t.type) == 0) return false;
  // extents and strides small enough that the byte span below cannot wrap: a file is not trusted
  unsigned __int128 last = 0;
  for (size_t i = 0; i < o.t.rank; ++i) {
    o.size[i] = (size_t)r.u64(), o.stride[i] = (size_t)r.u64();
    if (o.size[i] > ((uint64_t)1 << 40) || o.stride[i] > ((uint64_t)1 << 40)) return false;
    if (o.size[i]) last += (unsigned __int128)(o.size[i] - 1) * o.stride[i];
  }
  if (last > ((uint64_t)1 << 44)) return false;
  o.t.size = o.size;
  o.t.stride = o.stride;
  return r.ok;
}

bool covered(const Region& g, char* lo, char* hi) {
  // written ranges are few (one per intermediate): a linear walk over the sorted, merged list
  for (const auto& w : g.written)
    if (w.first <= lo && hi <= w.second) return true;
  return false;
}

void add_written(Region& g, char* lo, char* hi) {
  g.written.emplace_back(lo, hi);
  std::sort(g.written.begin(), g.written.end());
  std::vector<std::pair<char*, char*>> merged;
  for (const auto& w : g.written) {
    if (!merged.empty() && w.first <= merged.back().second) merged.back().second = std::max(merged.back().second, w.second);
    else merged.push_back(w);
  }
  g.written.swap(merged);
}

// index of the last operand of a step that is written (the result); everything before it is read
inline size_t result_index(const Step& s) { return s.opnd.size() - 1; }

}  // namespace

extern "C" int llc_plan_save(llc_plan_t* p, const char* path) {
  if (!p || !path) return set_error(LLC_ERR_BAD_ARG, "plan_save: null argument");
  if (p->state != kReady) return set_error(LLC_ERR_BAD_ARG, "plan_save: the plan has not been recorded (begin .. end)");
  LLC_TRY(check_device(p, "plan_save"));
  std::lock_guard<std::mutex> lock(p->mu);
  // regions of fixed-address memory
  std::vector<std::pair<char*, char*>> spans;
  for (const Step& s : p->steps)
    for (const Operand& o : s.opnd)
      if (o.present && o.io < 0 && o.t.data && o.span_bytes()) spans.emplace_back((char*)o.t.data, (char*)o.t.data + o.span_bytes());
  std::sort(spans.begin(), spans.end());
  std::vector<Region> regions;
  for (const auto& sp : spans) {
    if (!regions.empty() && sp.first < regions.back().hi) regions.back().hi = std::max(regions.back().hi, sp.second);
    else regions.push_back(Region{sp.first, sp.second});
  }
  auto region_of = [&](const char* a) -> int {
    size_t lo = 0, hi = regions.size();
    while (lo < hi) {
      const size_t mid = (lo + hi) / 2;
      if (regions[mid].hi <= a) lo = mid + 1;
      else hi = mid;
    }
    return (lo < regions.size() && regions[lo].lo <= a) ? (int)lo : -1;
  };
  // which regions are read before they are written
  for (const Step& s : p->steps) {
    const size_t res = result_index(s);
    for (size_t i = 0; i < s.opnd.size(); ++i) {
      const Operand& o = s.opnd[i];
      if (!o.present || o.io >= 0 || !o.t.data || !o.span_bytes()) continue;
      Region& g = regions[region_of((char*)o.t.data)];
      char* lo = (char*)o.t.data;
      char* hi = lo + o.span_bytes();
      if (i != res) {
        if (!covered(g, lo, hi)) g.keep = true;
      } else {
        size_t n = dtype_size(o.t.type);
        for (size_t d = 0; d < o.t.rank; ++d) n *= o.size[d];
        if (n == o.span_bytes()) add_written(g, lo, hi);  // a dense result covers its range; a strided one may leave gaps
      }
    }
  }
  LLC_HIP_TRY(hipDeviceSynchronize());
  FILE* f = fopen(path, "wb");
  if (!f) return set_error(LLC_ERR_BAD_ARG, "plan_save: cannot open %s for writing", path);
  Writer w{f};
  w.raw(kPlanMagic, 8);
  w.u64((uint64_t)LLC_HIP_ABI_VERSION);
  w.u64(p->io.size());
  w.u64(p->n_inputs);
  for (const Io& io : p->io) {
    write_operand_shape(w, io.like);
    w.u64((io.output ? 1u : 0u) | ((uint64_t)io.align16 << 8));
  }
  w.u64(p->symbols.size());
  for (int64_t v : p->symbols) w.i64(v);
  w.u64(p->overlaps.size());
  for (const Overlap& ov : p->overlaps) w.i64(ov.first), w.i64(ov.second), w.i64(ov.diff);
  w.u64(p->ws_bytes);
  w.u64(regions.size());
  std::vector<char> host;
  for (const Region& g : regions) {
    const size_t bytes = (size_t)(g.hi - g.lo);
    w.u64(bytes);
    w.u64((uint64_t)((uintptr_t)g.lo % 256));
    w.u64(g.keep ? 1 : 0);
    if (g.keep) {
      host.resize(bytes);
      const hipError_t e = hipMemcpy(host.data(), g.lo, bytes, hipMemcpyDeviceToHost);
      if (e != hipSuccess) {
        fclose(f);
        return set_error(LLC_ERR_HIP, "plan_save: reading %zu bytes of device memory failed: %s", bytes, hipGetErrorString(e));
      }
      w.raw(host.data(), bytes);
    }
  }
  w.u64(p->steps.size());
  for (const Step& s : p->steps) {
    w.i64(s.op);
    w.u64(s.has_epi ? 1 : 0);
    w.pod(s.alpha);
    w.i64(s.act);
    w.i64(s.kind);
    w.pod(s.eps);
    w.u64(s.n_ints);
    for (size_t i = 0; i < s.n_ints; ++i) w.i64(s.ints[i]);
    w.pod(s.conv);
    w.pod(s.pool);
    w.u64(s.prog ? 1 : 0);
    if (s.prog) w.pod(*s.prog);
    w.u64(s.opnd.size());
    for (const Operand& o : s.opnd) {
      write_operand_shape(w, o);
      if (!o.present) continue;
      w.i64(o.io);
      w.i64(o.delta);
      int reg = -1;
      int64_t off = 0;
      if (o.io < 0 && o.t.data && o.span_bytes()) {
        reg = region_of((char*)o.t.data);
        off = (char*)o.t.data - regions[reg].lo;
      }
      w.i64(reg);
      w.i64(off);
    }
  }
  const bool ok = w.ok && fclose(f) == 0;
  if (!ok) return set_error(LLC_ERR_BAD_ARG, "plan_save: writing %s failed", path);
  return LLC_OK;
}

extern "C" int llc_plan_load(const char* path, llc_plan_t** out) {
  if (!path || !out) return set_error(LLC_ERR_BAD_ARG, "plan_load: null argument");
  *out = nullptr;
  FILE* f = fopen(path, "rb");
  if (!f) return set_error(LLC_ERR_BAD_ARG, "plan_load: cannot open %s", path);
  struct Closer {
    FILE* f;
    ~Closer() { fclose(f); }
  } closer{f};
  Reader r{f};
  uint64_t file_bytes = 0;
  if (fseek(f, 0, SEEK_END) == 0) {
    const long end = ftell(f);
    file_bytes = end > 0 ? (uint64_t)end : 0;
  }
  rewind(f);
  char magic[8] = {0};
  r.raw(magic, 8);
  if (!r.ok || memcmp(magic, kPlanMagic, 8) != 0) return set_error(LLC_ERR_BAD_ARG, "plan_load: %s is not a plan file", path);
  const uint64_t abi = r.u64();
  if (abi != (uint64_t)LLC_HIP_ABI_VERSION)
    return set_error(LLC_ERR_UNSUPPORTED, "plan_load: %s was written by ABI version %llu, this library is version %d", path,
                     (unsigned long long)abi, LLC_HIP_ABI_VERSION);
  llc_plan_t* p = nullptr;
  LLC_TRY(llc_plan_create(&p));
  std::unique_ptr<llc_plan_t, int (*)(llc_plan_t*)> guard(p, llc_plan_destroy);
  auto bad = [&](const char* what) { return set_error(LLC_ERR_BAD_ARG, "plan_load: %s: %s", path, what); };
  const uint64_t n_io = r.u64();
  p->n_inputs = (size_t)r.u64();
  if (!r.ok || n_io > (1u << 20) || p->n_inputs > n_io) return bad("truncated or corrupt header");
  p->io.resize((size_t)n_io);
  for (Io& io : p->io) {
    if (!read_operand_shape(r, io.like) || !io.like.present) return bad("malformed tensor declaration");
    io.like.t.size = io.like.t.stride = nullptr;  // as after llc_plan_declare_io: only like.size / like.stride are read
    const uint64_t flags = r.u64();
    io.output = (flags & 1) != 0;
    io.align16 = (unsigned)((flags >> 8) & 15);
  }
  const uint64_t n_sym = r.u64();
  if (!r.ok || n_sym > (1u << 20)) return bad("truncated symbol list");
  p->symbols.resize((size_t)n_sym);
  for (int64_t& v : p->symbols) v = r.i64();
  const uint64_t n_ov = r.u64();
  if (!r.ok || n_ov > (1u << 20)) return bad("truncated overlap list");
  for (uint64_t i = 0; i < n_ov; ++i) {
    Overlap ov;
    ov.first = (int)r.i64(), ov.second = (int)r.i64(), ov.diff = r.i64();
    if (!r.ok || ov.first < 0 || ov.second < 0 || (uint64_t)ov.first >= n_io || (uint64_t)ov.second >= n_io) return bad("malformed overlap entry");
    p->overlaps.push_back(ov);
  }
  const uint64_t ws_bytes = r.u64();
  if (!r.ok || ws_bytes > ((uint64_t)1 << 36)) return bad("malformed scratch size");
  if (ws_bytes) {
    LLC_TRY(llc_plan_alloc(p, (size_t)ws_bytes, &p->ws));
    p->ws_bytes = (size_t)ws_bytes;
  }
  const uint64_t n_reg = r.u64();
  if (!r.ok || n_reg > (1u << 24)) return bad("truncated region list");
  std::vector<std::pair<char*, size_t>> regions;
  std::vector<char> host;
  for (uint64_t i = 0; i < n_reg; ++i) {
    const uint64_t bytes = r.u64(), mis = r.u64(), keep = r.u64();
    if (!r.ok || mis >= 256 || bytes > ((uint64_t)1 << 40) || (keep && bytes > file_bytes)) return bad("malformed region entry");
    void* m = nullptr;
    LLC_TRY(llc_plan_alloc(p, (size_t)(bytes + mis), &m));
    char* base = (char*)m + mis;
    if (keep) {
      host.resize((size_t)bytes);
      r.raw(host.data(), (size_t)bytes);
      if (!r.ok) return bad("truncated region contents");
      if (bytes) LLC_HIP_TRY(hipMemcpy(base, host.data(), (size_t)bytes, hipMemcpyHostToDevice));
    } else if (bytes) {
      LLC_HIP_TRY(hipMemset(base, 0, (size_t)bytes));
    }
    regions.emplace_back(base, (size_t)bytes);
  }
  const uint64_t n_steps = r.u64();
  if (!r.ok || n_steps > (1u << 24)) return bad("truncated step list");
  p->steps.resize((size_t)n_steps);
  for (Step& s : p->steps) {
    s.op = (int)r.i64();
    s.has_epi = r.u64() != 0;
    r.pod(s.alpha);
    s.act = (int)r.i64();
    s.kind = (int)r.i64();
    r.pod(s.eps);
    s.n_ints = (size_t)r.u64();
    if (!r.ok || s.n_ints > sizeof(s.ints) / sizeof(s.ints[0]) || s.op < kMatmul || s.op > kAttention) return bad("malformed step");
    for (size_t i = 0; i < s.n_ints; ++i) s.ints[i] = r.i64();
    llc_conv_attrs conv;
    llc_pool_attrs pool;
    r.pod(conv);
    r.pod(pool);
    if (s.op == kMaxPool) s.pool = pool;
    else s.conv = conv;
    if (r.u64()) {
      s.prog.reset(new llc_ew_program);
      r.pod(*s.prog);
    }
    const uint64_t n_op = r.u64();
    if (!r.ok || n_op == 0 || n_op > LLC_EW_MAX_INPUTS + 8) return bad("malformed operand list");
    if ((s.op == kElementwise) != (s.prog != nullptr)) return bad("elementwise step without a program (or a program elsewhere)");
    s.opnd.resize((size_t)n_op);
    for (Operand& o : s.opnd) {
      if (!read_operand_shape(r, o)) return bad("malformed operand");
      if (!o.present) continue;
      o.io = (int)r.i64();
      o.delta = r.i64();
      const int64_t reg = r.i64(), off = r.i64();
      if (!r.ok || o.io >= (int64_t)n_io) return bad("operand bound to an undeclared tensor");
      if (o.io >= 0) {
        // bound at run time to a tensor of the parameter block, `delta` bytes into it: it starts inside that
        // tensor, and ends inside it too unless tensors of the block share memory (then it may run on into the next)
        const uint64_t io_bytes = p->io[(size_t)o.io].like.span_bytes();
        if (o.delta < 0 || (o.span_bytes() && (uint64_t)o.delta >= io_bytes) ||
            (p->overlaps.empty() && (uint64_t)o.delta + o.span_bytes() > io_bytes))
          return bad("operand outside the tensor it is bound to");
      } else if (reg >= 0) {
        if ((uint64_t)reg >= regions.size() || off < 0 || (uint64_t)off + o.span_bytes() > regions[(size_t)reg].second)
          return bad("operand outside its memory region");
        o.t.data = o.t.base = regions[(size_t)reg].first + off;
      } else if (o.span_bytes()) {
        return bad("operand with elements but no memory");
      }
    }
  }
  if (!r.ok) return bad("truncated file");
  for (const Step& s : p->steps)
    if (const char* why = step_defect(s)) return bad(why);
  p->state = kReady;
  p->bound.assign(p->io.size(), nullptr);
  *out = guard.release();
  return LLC_OK;
}

// ---- what a host needs to run a loaded plan without any other description of it ----
extern "C" int llc_plan_num_io(const llc_plan_t* p, size_t* n_inputs, size_t* n_outputs) {
  if (!p || !n_inputs || !n_outputs) return set_error(LLC_ERR_BAD_ARG, "plan_num_io: null argument");
  *n_inputs = p->n_inputs;
  *n_outputs = p->io.size() - p->n_inputs;
  return LLC_OK;
}

extern "C" int llc_plan_io_info(const llc_plan_t* p, size_t index, llc_tensor* like, size_t* size_out, size_t* stride_out) {
  if (!p || !like || !size_out || !stride_out) return set_error(LLC_ERR_BAD_ARG, "plan_io_info: null argument");
  if (index >= p->io.size()) return set_error(LLC_ERR_BAD_ARG, "plan_io_info: the plan declares %zu tensors, index %zu", p->io.size(), index);
  const Operand& o = p->io[index].like;
  memset(like, 0, sizeof(*like));
  like->type = o.t.type;
  like->rank = o.t.rank;
  for (size_t d = 0; d < o.t.rank; ++d) size_out[d] = o.size[d], stride_out[d] = o.stride[d];
  like->size = size_out;
  like->stride = stride_out;
  return LLC_OK;
}

extern "C" int llc_hip_download(void* host, const void* device, size_t bytes, void* stream) {
  if (bytes && (!host || !device)) return set_error(LLC_ERR_BAD_ARG, "download: null pointer");
  LLC_HIP_TRY(hipStreamSynchronize(as_stream(stream)));
  if (bytes) LLC_HIP_TRY(hipMemcpy(host, device, bytes, hipMemcpyDeviceToHost));
  return LLC_OK;
}
