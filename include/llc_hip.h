/*
 * llc_hip.h -- C-ABI of the gfx950 (MI355X) kernel library behind LLCompiler's compiled-op path.
 *
 * The reference lowers LLH ops to CPU loop nests inside a generated `main(void**)`; its runtime
 * op library is an empty placeholder (ops/cpu/ops.h, 0 bytes).  This header is the `ops/hip`
 * sibling: one entry point per LLH op (or per fused group the reference's pipeline forms), plus
 * the model-level entry that keeps the reference's packed-pointer convention.
 *
 * Conventions
 *  - plain C: pointers, sizes, no C++ or torch types.
 *  - every `data`/`base` pointer is a DEVICE pointer; `size`/`stride` arrays and attribute structs
 *    live on the host.  Strides are in ELEMENTS, like the reference's Tensor
 *    (include/llcompiler/Compiler/Tensor.h:36-48).
 *  - the caller owns every input and output buffer (Tensor.h:35: the descriptor allocates nothing).
 *  - `stream` is a hipStream_t passed as void*; NULL = the default stream.  Calls only enqueue
 *    work; the caller synchronises.
 *  - kernels that split a reduction (convolutions with few output tiles, matmuls with a long K) keep partial
 *    sums in scratch device memory.  A plan owns its scratch memory (sized while it is recorded, allocated by
 *    llc_plan_end / llc_plan_load), so llc_hip_run allocates nothing and plans replayed on different streams do
 *    not share any.  An op entry point called outside a plan uses a buffer per (device, stream) that grows on
 *    demand, which is the only allocation an op entry point ever makes (nothing is synchronised; an outgrown
 *    buffer is kept until llc_hip_trim, since queued launches may still address it; growing is refused with
 *    LLC_ERR_UNSUPPORTED while the stream is being captured: run the call once on that stream ahead of the
 *    capture, and keep the stream to the graph).  Calls on one stream follow each other, calls on
 *    different streams use different buffers: op entry points are re-entrant per stream, like plans.  Two host
 *    threads must not issue work to the SAME stream at the same time.  llc_hip_matmul_static never allocates
 *    (see there).
 *  - every entry returns an llc_status (0 = ok, negative = error) and leaves a message for
 *    llc_hip_last_error() (thread local).  The reference only logs on failure
 *    (include/llcompiler/Support/Logger.h:132-134); returning a status is a deliberate tightening.
 */
#ifndef LLC_HIP_H_
#define LLC_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define LLC_HIP_ABI_VERSION 3
#define LLC_MAX_RANK 8

/* Element type codes.  0-6 are the reference's `enum Type` (Tensor.h:25-33, and the Python map
 * llcompiler/executor/engine.py:11); 7 and 8 are new. */
typedef enum llc_dtype {
  LLC_INT8 = 0,
  LLC_INT16 = 1,
  LLC_INT32 = 2,
  LLC_INT64 = 3,
  LLC_FLOAT32 = 4,
  LLC_DOUBLE64 = 5,
  LLC_INT1 = 6, /* one byte per element, 0 or 1 (torch.bool) */
  LLC_BFLOAT16 = 7,
  LLC_FLOAT16 = 8
} llc_dtype;

/* Non-owning tensor descriptor; same fields in the same order as the reference's
 * `struct Tensor` (Tensor.h:42-47) with the two std::vectors flattened to rank + pointers.
 * The element at index (i0, i1, ...) is at  data + (offset + sum_k i_k * stride[k]) elements. */
typedef struct llc_tensor {
  void* data;
  void* base;
  size_t type;   /* llc_dtype */
  size_t offset; /* elements */
  size_t rank;
  const size_t* size;
  const size_t* stride;
} llc_tensor;

typedef enum llc_status {
  LLC_OK = 0,
  LLC_ERR_BAD_ARG = -1,     /* null pointer, bad enum value */
  LLC_ERR_DTYPE = -2,       /* unsupported or mismatched element types */
  LLC_ERR_SHAPE = -3,       /* rank / extent mismatch between operands */
  LLC_ERR_LAYOUT = -4,      /* strides the kernel cannot address */
  LLC_ERR_UNSUPPORTED = -5, /* attribute combination not implemented */
  LLC_ERR_HIP = -6,         /* a HIP runtime call failed */
  LLC_ERR_NO_DEVICE = -7,
  LLC_ERR_TOO_LARGE = -8
} llc_status;

/* ---- library ---- */
int llc_hip_abi_version(void);
/* Selects the device and checks that it is a gfx950 part. */
int llc_hip_init(int device);
const char* llc_hip_last_error(void);
const char* llc_hip_status_string(int status);
/* Scratch memory the op entry points hold on `device` outside plans: in use (one buffer per stream that needed
 * one) and retired (outgrown, not yet freed).  Either pointer may be NULL. */
int llc_hip_scratch_bytes(int device, size_t* live_bytes, size_t* retired_bytes);
/* Waits for the current device to finish everything queued, then frees the retired scratch buffers and, with
 * release_live != 0, the live ones too (the next call that needs one allocates again).  For a host that wants
 * the memory back after a one-off large product; never called by the library itself. */
int llc_hip_trim(int release_live);

/* ---- fused epilogue of the contractions.  The reference's pipeline fuses the elementwise
 * consumers of a linalg op into it (linalg-fuse-elementwise-ops,
 * include/llcompiler/TransformLibrary/linalg_include.mlir:50-53); here the same chain
 *   out = act(alpha * acc + bias + residual)
 * is applied to the accumulator tile before it is stored. ---- */
typedef enum llc_activation { LLC_ACT_NONE = 0, LLC_ACT_RELU = 1, LLC_ACT_GELU = 2 } llc_activation;
typedef struct llc_epilogue {
  float alpha;                /* applied to the fp32 accumulator; 1.0f = none */
  const llc_tensor* bias;     /* rank 1, one value per output column / filter; may be NULL.  batch_matmul with two
                                 batch dims also takes rank 2, [B0, N]: one row per outer batch (an attention
                                 mask [B,1,1,S] added to scores [B,H,S,S]) */
  const llc_tensor* residual; /* same shape as the output, contiguous; may be NULL.  It may be the output tensor itself
                                 (an in-place add: every kernel reads an element's residual before it stores that
                                 element); any other overlap with the output is undefined */
  int act;                    /* llc_activation */
} llc_epilogue;

/* llh.matmul (include/llcompiler/Dialect/LLH/IR/LLHOps.td:438-444; lowered at
 * src/Conversion/LLHToHLO/LLHToHLO.cpp:485): out[m,n] = sum_k lhs[m,k] * rhs[k,n], rank 2,
 * fp32 accumulate.  f32, bf16 or f16 operands (all three the same type).  Either operand may be a
 * transposed view (stride[0] == 1), which is how llh.transpose{perms=[1,0]} of a weight
 * (llcompiler/importer/fx_op_translate/transpose.py:39-48) is consumed without a copy.
 * `epi` may be NULL.  Products with a long reduction and few output tiles sum the reduction in
 * chunks through the library's scratch buffer of this stream (grown on demand by this call); the order
 * of the sum is fixed, so results are the same bits on every run. */
int llc_hip_matmul(const llc_tensor* lhs, const llc_tensor* rhs, const llc_epilogue* epi, llc_tensor* out,
                   void* stream);

/* llc_hip_matmul for callers that cannot allocate device memory: code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference.  Same arguments, same kernels
 * and the same bits as llc_hip_matmul; the partial sums of a split reduction go to a 32 MiB array that is part of
 * the library's code object (each GPU the library runs on holds it until the process ends) instead of the
 * per-stream buffer that llc_hip_matmul grows on demand.  The call never allocates or frees; a product whose
 * partial sums need more than 32 MiB is refused with LLC_ERR_TOO_LARGE (use llc_hip_matmul or a plan).  Every call
 * on a GPU shares that GPU's array (nothing in it has to start at zero: partial sums are written before they are
 * read): calls that overlap on different streams of one GPU race (llc_hip_matmul's do not).  The call is not recorded
 * into a plan (a plan owns its scratch memory anyway). */
int llc_hip_matmul_static(const llc_tensor* lhs, const llc_tensor* rhs, const llc_epilogue* epi, llc_tensor* out,
                          void* stream);

/* llh.batch_matmul (LLHOps.td:446-452; LLHToHLO.cpp:363-382: batch dims {0}/{0}, contracting lhs
 * dim 2 with rhs dim 1): rank 3.  The two inner dims of each operand may be a transposed view.
 * Extension: either operand (and the contiguous output) may be rank 4, [B0, B1, rows, cols], with any
 * strides on the two batch dims; batch b of the op is (b / B1, b % B1).  The head split of an attention
 * layer, [B, S, H*D] viewed as [B, H, S, D], is then read in place instead of being copied first.  A rank-4
 * output may also be strided (unit stride on its last dim; no residual then): the head merge back to
 * [B, S, H*D] is written in place. */
int llc_hip_batch_matmul(const llc_tensor* lhs, const llc_tensor* rhs, const llc_epilogue* epi, llc_tensor* out,
                         void* stream);

/* llh.conv / llh.conv_bias attributes (LLHOps.td:407-436).  NCHW x FCHW -> NCHW.
 * pad = {h_lo, w_lo, h_hi, w_hi}: the order the shape rule reads
 * (src/Dialect/LLH/IR/LLHinfersymbolShape.cpp:257-268) and the importer writes
 * (llcompiler/importer/fx_op_translate/conv.py:48-70). */
typedef struct llc_conv_attrs {
  int64_t dilation[2];
  int64_t kernel_shape[2];
  int64_t pad[4];
  int64_t stride[2];
  int64_t group;
} llc_conv_attrs;
/* Cross-correlation as implicit GEMM (LLHToHLO.cpp:214-270).  conv_bias is `epi->bias`.
 * Layout travels in the strides, as in torch: either every tensor (x, w, out, epilogue residual) is contiguous
 * NCHW / FCHW, or every one is channels-last (NHWC in memory: strides (H W C, 1, W C, C) under the same
 * logical shape), which takes a kernel of its own (group 1, C a multiple of 128 bytes' worth of values: 32 fp32,
 * 64 bf16 / f16; F % 4 == 0, at most 64 taps; LLC_ERR_UNSUPPORTED otherwise).  One mixed form is taken: contiguous x
 * and w with a channels-last out, for an image network's first layer, whose result the channels-last layers behind it
 * read (64 filters, stride 2 along w, C * KH at most 21 (24 for the 16-bit types) input rows under a window, rows of
 * at most 224 values, no residual; LLC_ERR_UNSUPPORTED otherwise).  Other mixed layouts are refused (LLC_ERR_LAYOUT). */
int llc_hip_conv2d(const llc_tensor* x, const llc_tensor* w, const llc_conv_attrs* attrs, const llc_epilogue* epi,
                   llc_tensor* out, void* stream);

/* ---- fused elementwise chain.  One launch evaluates a whole chain of LLH elementwise ops, the
 * unit the reference forms with linalg-fuse-elementwise-ops (linalg_include.mlir:50-53,94).
 * Unary abs/sqrt/exp/relu/rsqrt (LLHOps.td:345-355), binary add/sub/mul/div/max/min/pow
 * (LLHOps.td:357-393), compare (LLHOps.td:395-405), where (LLHOps.td:509-517), convert_to
 * (LLHOps.td:329-335); neg/gelu/tanh/erf/sigmoid/log/recip are added for the nodes the
 * reference leaves to torch eager.  llh.broadcast_to (LLHOps.td:206-217) is never materialised:
 * an input whose extent is 1 where the output's is not is read with stride 0. ---- */
typedef enum llc_ew_opcode {
  LLC_EW_ABS = 0, LLC_EW_SQRT = 1, LLC_EW_EXP = 2, LLC_EW_RELU = 3, LLC_EW_RSQRT = 4, LLC_EW_NEG = 5,
  LLC_EW_GELU = 6, LLC_EW_TANH = 7, LLC_EW_ERF = 8, LLC_EW_SIGMOID = 9, LLC_EW_LOG = 10, LLC_EW_RECIP = 11,
  LLC_EW_MOV = 15,
  LLC_EW_ADD = 16, LLC_EW_SUB = 17, LLC_EW_MUL = 18, LLC_EW_DIV = 19, LLC_EW_MAX = 20, LLC_EW_MIN = 21,
  LLC_EW_POW = 22,
  /* 32 + the reference's CompareKind value (include/llcompiler/Dialect/LLH/IR/LLHEnums.td:111-116) */
  LLC_EW_CMP_EQ = 33, LLC_EW_CMP_GE = 34, LLC_EW_CMP_LE = 35, LLC_EW_CMP_GT = 36, LLC_EW_CMP_LT = 37,
  LLC_EW_CMP_NE = 38,
  LLC_EW_WHERE = 48 /* dst = a != 0 ? b : c */
} llc_ew_opcode;
/* operand selectors: 0..LLC_EW_MAX_REGS-1 = register, LLC_EW_IN0 + k = input k, LLC_EW_IMM = imm */
#define LLC_EW_MAX_REGS 4
#define LLC_EW_MAX_INPUTS 6
#define LLC_EW_MAX_INSTS 24
#define LLC_EW_IN0 16
#define LLC_EW_IMM 64
typedef struct llc_ew_inst {
  int32_t op;  /* llc_ew_opcode */
  int32_t dst; /* register written */
  int32_t a, b, c;
  float imm;
} llc_ew_inst;
typedef struct llc_ew_program {
  int32_t n_insts;
  int32_t result; /* register holding the chain's value */
  int32_t integer; /* 0: compute in fp32; 1: compute in int64 (imm is rounded to an integer) */
  llc_ew_inst insts[LLC_EW_MAX_INSTS];
} llc_ew_program;
/* Every input must have the output's rank with each extent equal to the output's or 1.  The
 * output is contiguous. */
int llc_hip_elementwise(const llc_ew_program* prog, const llc_tensor* const* inputs, size_t n_inputs,
                        llc_tensor* out, void* stream);

/* llh.reduce_sum / reduce_max / reduce_min {axis} (LLHOps.td:528-553; LLHToHLO.cpp:81-171,
 * 448-464): init 0 / -inf / +inf, the result drops the reduced axes
 * (LLHinfersymbolShape.cpp:185-212).  Any set of axes: runs of adjacent reduced axes are reduced one kernel
 * each, innermost first, partial results in scratch memory (two runs or more only). */
typedef enum llc_reduce_kind { LLC_REDUCE_SUM = 0, LLC_REDUCE_MAX = 1, LLC_REDUCE_MIN = 2 } llc_reduce_kind;
int llc_hip_reduce(int kind, const llc_tensor* x, const int64_t* axes, size_t n_axes, llc_tensor* out,
                   void* stream);

/* softmax over the last dim: the amax -> sub -> exp -> sum -> div group that ATen `_softmax`
 * decomposes to (llcompiler/compiler/torch_compile_config.py:24), as one kernel.  fp32
 * statistics for every storage type. */
int llc_hip_softmax(const llc_tensor* x, llc_tensor* out, void* stream);

/* llh.layer_norm{epsilon, axis} (LLHOps.td:454-463) over the last dim; biased variance, fp32
 * statistics; scale / bias may be NULL. */
int llc_hip_layer_norm(const llc_tensor* x, const llc_tensor* scale, const llc_tensor* bias, double epsilon,
                       llc_tensor* out, void* stream);

/* llh.max_pool (LLHOps.td:495-507; LLHToHLO.cpp:295-339), NCHW, ceil_mode false.
 * init_zero = 1 reproduces the reference's reduce_window init value 0 (LLHToHLO.cpp:313-314);
 * init_zero = 0 is torch's -inf padding.  x and out are both contiguous or both channels-last (strides as for
 * llc_hip_conv2d; C a multiple of 16 bytes' worth of values then, LLC_ERR_UNSUPPORTED otherwise). */
typedef struct llc_pool_attrs {
  int64_t dilation[2];
  int64_t kernel_shape[2];
  int64_t pad[4]; /* h_lo, w_lo, h_hi, w_hi */
  int64_t stride[2];
  int32_t init_zero;
} llc_pool_attrs;
int llc_hip_max_pool(const llc_tensor* x, const llc_pool_attrs* attrs, llc_tensor* out, void* stream);

/* llh.adaptive_average_pool{out_size=(1,1)} (LLHOps.td:337-339; shape rule
 * LLHinfersymbolShape.cpp:587-613): [N,C,H,W] -> [N,C] (or [N,C,1,1]); x contiguous or channels-last. */
int llc_hip_global_avg_pool(const llc_tensor* x, llc_tensor* out, void* stream);

/* ---- data movement, bit exact for every element size (1, 2, 4, 8 bytes) ---- */
/* llh.transpose{perms} (LLHOps.td:343; LLHToHLO.td:24-26): out.size[i] = x.size[perms[i]] */
int llc_hip_transpose(const llc_tensor* x, const int64_t* perms, llc_tensor* out, void* stream);
/* llh.stride_slice (LLHOps.td:261-269; LLHToHLO.cpp:341-361;
 * src/Conversion/StablehlotoLinalgExtension/StablehlotoLinalgExtension.cpp:64-118):
 * out.size[d] = ceildiv(end[d] - start[d], step[d]).  llh.extract (LLHOps.td:252-259) is the
 * rank-dropping special case and is expressed by the caller through `out`'s descriptor. */
int llc_hip_stride_slice(const llc_tensor* x, const int64_t* start, const int64_t* end, const int64_t* step,
                         llc_tensor* out, void* stream);
/* llh.broadcast_to (LLHOps.td:206-217; LLHToHLO.cpp:191-212), materialised: same rank, input
 * extents 1 are repeated. */
int llc_hip_broadcast_to(const llc_tensor* x, llc_tensor* out, void* stream);
/* Strided -> contiguous copy of any view (the materialising half of reshape, LLHOps.td:281-289). */
int llc_hip_copy(const llc_tensor* x, llc_tensor* out, void* stream);
/* Row gather along dim 0 with int64 indices (aten.embedding / index_select, left to torch eager
 * by the reference): out[i, ...] = table[idx[i], ...]. */
int llc_hip_gather_rows(const llc_tensor* table, const llc_tensor* idx, llc_tensor* out, void* stream);
/* Fused attention: out = softmax(scale * q k^T + mask) v over the key dim, for the op group the importer
 * produces from an attention layer: llh.batch_matmul (LLHOps.td:446-452) of q with the transposed keys, the
 * scaling mul/div and the mask add (LLHOps.td:357-393), the softmax chain (amax, sub, exp, sum, div;
 * llcompiler/compiler/torch_compile_config.py:24) and the llh.batch_matmul with v.  The reference lowers each
 * of these to its own loop nest; the fused form never writes the [B, H, Sq, Skv] scores.
 * q, out: [B, H, Sq, D]; k, v: [B, H, Skv, D] with head dim D = 64, or 32 or 128 in the 16-bit types
 * (LLC_ERR_UNSUPPORTED otherwise); f32, bf16 or f16 (f32 operands run on the fp32 MFMA and keep
 * fp32 probabilities; 16-bit operands round the probabilities to the storage type before the second
 * product, as the unfused group does); the last dim contiguous, the other strides
 * free (multiples of 8 elements), so head-split views of [B, S, H*D] activations are read and written in
 * place.  mask: NULL or [B, Skv] of the same type, added to every head and query row.  scale > 0. */
int llc_hip_attention(const llc_tensor* q, const llc_tensor* k, const llc_tensor* v, const llc_tensor* mask, float scale,
                      llc_tensor* out, void* stream);

/* llh.convert_to (LLHOps.td:329-335; LLHToHLO.cpp:489) between f32, bf16, f16, i64, i32, i1. */
int llc_hip_convert(const llc_tensor* x, llc_tensor* out, void* stream);

/* ---- model-level entry: the reference's `main(void** params)` convention
 * (src/Compiler/Execution.cpp:21-66; unpacked by
 * src/Dialect/LLVMExtension/Transforms/AdaptEntryParmsForEngine.cpp:188-284):
 *   params[0]            int64_t* symbols, or NULL
 *   then per input, then per output, five slots:
 *     base*, data*, size_t* offset, size_t* size[rank], size_t* stride[rank]
 * llc_hip_unpack_params turns that array into descriptors (ranks are known to the plan, as they
 * are baked into the reference's compiled prologue).  `types` gives the element type of each
 * tensor.  Returns the number of slots consumed, or a negative llc_status. */
int llc_hip_unpack_params(void* const* params, size_t n_tensors, const size_t* ranks, const size_t* types,
                          llc_tensor* tensors_out, const int64_t** symbols_out);

/* ---- model-level entry: a recorded plan run from the packed block.
 *
 * The reference compiles a graph into one `void main(void** params)` (entry type
 * include/llcompiler/Compiler/Execution.h:23; called at src/Compiler/Execution.cpp:21-66) whose prologue
 * unpacks the block (AdaptEntryParmsForEngine.cpp:154-242), whose constants are baked into the object and
 * whose temporaries it allocates itself.  The counterpart here is a plan: the ordered kernel calls of one
 * graph specialised to concrete extents (one plan per binding of the symbols), recorded once and replayed
 * by llc_hip_run from the same block.  The caller owns inputs and outputs (Tensor.h:35); the plan owns what
 * llc_plan_alloc / llc_plan_upload hand out (weights, the arena of intermediates) until llc_plan_destroy.
 *
 *   llc_plan_create(&p);
 *   llc_plan_upload(p, host_weights, bytes, &w);  llc_plan_alloc(p, arena_bytes, &arena);
 *   llc_plan_declare_io(p, 0, &in0); ...          inputs first, then outputs, in params order
 *   llc_plan_declare_io(p, 1, &out0); ...
 *   llc_plan_begin(p);
 *     llc_hip_matmul(...); llc_hip_elementwise(...); ...   each call runs AND is appended to the plan
 *   llc_plan_end(p);
 *   llc_hip_run(p, params, stream);                        any number of times, any input/output addresses
 *
 * While recording, an operand whose address lies inside a declared tensor is bound to it and follows the
 * pointer the block carries at run time; any other address is replayed as recorded.  llc_hip_run launches
 * only: no allocation, no host-device synchronisation.  One run at a time per plan (runs of one plan are
 * serialised by a lock; different plans are independent). ---- */
typedef struct llc_plan llc_plan_t;
/* The plan belongs to the current device. */
int llc_plan_create(llc_plan_t** plan);
/* Frees the plan and the device memory it owns (waits for the device to be done with it). */
int llc_plan_destroy(llc_plan_t* plan);
/* Device memory owned by the plan: the stand-in for the reference's baked constants
 * (src/Dialect/LLH/Transforms/LoadWeight.cpp:58-171) and its malloc'ed temporaries
 * (include/llcompiler/TransformLibrary/memref_include.mlir:6-8). */
int llc_plan_alloc(llc_plan_t* plan, size_t bytes, void** device_ptr);
int llc_plan_upload(llc_plan_t* plan, const void* host, size_t bytes, void** device_ptr);
/* llh.weight{weight_file} (LLHOps.td:219-227): the reference's importer saves parameters with np.save
 * (llcompiler/importer/fx_translate.py:427-430) and its LoadWeight pass (LoadWeight.cpp:58-171) parses the
 * .npy file ('<f4', '<i8', C order assumed) and bakes the data into the compiled object.  llc_npy_info reads
 * the header (format versions 1 to 3): element type, rank, extents and where the data starts;
 * llc_plan_load_npy uploads the data into memory owned by the plan and fills `out` (contiguous, with
 * size_out / stride_out as its arrays, LLC_MAX_RANK entries each).  Read: f4, i8, f8, f2, i4, i2, i1, b1, and
 * u2 as bf16 bit patterns when expect_dtype says LLC_BFLOAT16.  expect_dtype < 0 takes what the file says;
 * otherwise a file of another type is refused (LLC_ERR_DTYPE).  Fortran-ordered files of rank > 1 are refused
 * (the reference reads them as if they were C ordered). */
int llc_npy_info(const char* path, int expect_dtype, size_t* dtype, size_t* rank, size_t* size, size_t* data_offset);
int llc_plan_load_npy(llc_plan_t* plan, const char* path, int expect_dtype, llc_tensor* out, size_t* size_out,
                      size_t* stride_out);
/* Declares the next tensor of the params block: type, rank, extents and strides it will have on every run,
 * and (data + offset) = where it lives while the plan is recorded. */
int llc_plan_declare_io(llc_plan_t* plan, int is_output, const llc_tensor* like);
/* The symbol values the plan was specialised for; llc_hip_run then checks params[0] against them
 * (the reference passes them in slot 0, Execution.cpp:24,46-49). */
int llc_plan_expect_symbols(llc_plan_t* plan, const int64_t* values, size_t n);
int llc_plan_begin(llc_plan_t* plan);
int llc_plan_end(llc_plan_t* plan);
int64_t llc_plan_num_steps(const llc_plan_t* plan);
/* Number of slots llc_hip_run reads from `params`: 1 + 5 per declared tensor. */
int64_t llc_plan_num_params(const llc_plan_t* plan);
/* Replays the plan.  `params` has the layout described above llc_hip_unpack_params; base/data are device
 * pointers.  Extents must equal the declared ones, strides too, and every tensor must lie at the same address
 * modulo 16 as when the plan was recorded (the kernels and the scratch memory of a plan are chosen for that
 * alignment) (LLC_ERR_SHAPE / LLC_ERR_LAYOUT otherwise: the caller then picks or records the plan for that
 * binding). */
int llc_hip_run(llc_plan_t* plan, void* const* params, void* stream);
/* Plans on disk.  The reference's compile step leaves a shared object with the weights baked in
 * (src/Compiler/Compiler.cpp:306-330: the object is named after a hash of the module text) that a later process
 * loads and runs (src/Compiler/Execution.cpp:21-66).  llc_plan_save writes a recorded plan: the declared tensors,
 * the expected symbol values, the steps, and the device memory the steps address outside the declared tensors
 * (constants and weights with their contents as they are now; memory that every run writes before it reads
 * it, i.e. intermediates, only by size).  llc_plan_load gives a plan of its own memory on the current device
 * that llc_hip_run replays like the original.  A file written by another ABI version is refused
 * (LLC_ERR_UNSUPPORTED), a truncated or malformed one LLC_ERR_BAD_ARG. */
int llc_plan_save(llc_plan_t* plan, const char* path);
int llc_plan_load(const char* path, llc_plan_t** plan);
/* What a host needs to run a plan it did not record (the reference's Execution gets the same from the
 * tensors its caller passes, Execution.cpp:21-45): how many tensors the block holds, and type, rank, extents
 * and strides of each (index < n_inputs: an input).  `like` is filled with size_out / stride_out as its
 * arrays (LLC_MAX_RANK entries each) and a null data pointer. */
int llc_plan_num_io(const llc_plan_t* plan, size_t* n_inputs, size_t* n_outputs);
int llc_plan_io_info(const llc_plan_t* plan, size_t index, llc_tensor* like, size_t* size_out, size_t* stride_out);
/* Waits for `stream`, then copies device memory to the host: results for a host that has no GPU runtime of
 * its own (the counterpart of llc_plan_upload). */
int llc_hip_download(void* host, const void* device, size_t bytes, void* stream);
/* The reference's loader resolves a symbol of type void(void**) (Execution.cpp:12-16).  llc_hip_entry has
 * that type and runs the plan bound with llc_hip_bind_entry (one per process; NULL unbinds) on the stream
 * given there; like the reference's entry it returns nothing and logs failures
 * (include/llcompiler/Support/Logger.h:132-134), and llc_hip_entry_status() returns the status of the last
 * call.  libllc_entry.so exports the same function under the name `main` for a loader that looks that
 * name up. */
int llc_hip_bind_entry(llc_plan_t* plan, void* stream);
void llc_hip_entry(void** params);
int llc_hip_entry_status(void);


#ifdef __cplusplus
}
#endif
#endif /* LLC_HIP_H_ */
