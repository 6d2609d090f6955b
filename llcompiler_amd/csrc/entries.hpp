// The kernel launchers behind the per-op entry points.  Each llc_hip_<op> of the C-ABI is a thin wrapper
// (plan.hip) that calls the matching llc_impl_<op> and, while a plan is being recorded on the calling
// thread, appends the call to that plan.  A plan replays through these functions directly.
#pragma once
#include "llc_hip.h"

int llc_impl_matmul(const llc_tensor* lhs, const llc_tensor* rhs, const llc_epilogue* epi, llc_tensor* out, void* stream);
int llc_impl_batch_matmul(const llc_tensor* lhs, const llc_tensor* rhs, const llc_epilogue* epi, llc_tensor* out,
                          void* stream);
int llc_impl_conv2d(const llc_tensor* x, const llc_tensor* w, const llc_conv_attrs* attrs, const llc_epilogue* epi,
                    llc_tensor* out, void* stream);
int llc_impl_elementwise(const llc_ew_program* prog, const llc_tensor* const* inputs, size_t n_inputs, llc_tensor* out,
                         void* stream);
int llc_impl_reduce(int kind, const llc_tensor* x, const int64_t* axes, size_t n_axes, llc_tensor* out, void* stream);
int llc_impl_softmax(const llc_tensor* x, llc_tensor* out, void* stream);
int llc_impl_layer_norm(const llc_tensor* x, const llc_tensor* scale, const llc_tensor* bias, double epsilon,
                        llc_tensor* out, void* stream);
int llc_impl_max_pool(const llc_tensor* x, const llc_pool_attrs* attrs, llc_tensor* out, void* stream);
int llc_impl_global_avg_pool(const llc_tensor* x, llc_tensor* out, void* stream);
int llc_impl_transpose(const llc_tensor* x, const int64_t* perms, llc_tensor* out, void* stream);
int llc_impl_stride_slice(const llc_tensor* x, const int64_t* start, const int64_t* end, const int64_t* step,
                          llc_tensor* out, void* stream);
int llc_impl_broadcast_to(const llc_tensor* x, llc_tensor* out, void* stream);
int llc_impl_copy(const llc_tensor* x, llc_tensor* out, void* stream);
int llc_impl_gather_rows(const llc_tensor* table, const llc_tensor* idx, llc_tensor* out, void* stream);
int llc_impl_convert(const llc_tensor* x, llc_tensor* out, void* stream);
int llc_impl_attention(const llc_tensor* q, const llc_tensor* k, const llc_tensor* v, const llc_tensor* mask, float scale,
                       llc_tensor* out, void* stream);
// Looks up, for the current device, the address of the scratch array behind llc_hip_matmul_static (gemm.hip).
int llc_impl_static_scratch_setup(void);
