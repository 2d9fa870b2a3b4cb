/*
 * ppml_hip_backend.h -- C ABI over the C++ host side (ppml_hip_backend.hpp): build a few tensor
 * nodes, bind device memory, run them through the backend's graph executor.
 *
 * This is the shape the reference's own tests use (tests/test_cuda.cpp:39-51, 108-110: make device
 * leaves, make one node, graph_compute, synchronize, copy back), exposed without C++ types so that
 * tests and other languages can drive the executor.  It has no counterpart among the reference's
 * launcher functions; those are in ppml_hip.h.
 *
 * Status values returned by graph_compute / pack_weight are the reference's
 * enum class Status {SUCCESS = 0, ALLOC_FAILED, NOT_SUPPORTED, ABORTED} (include/ppml/Backend.h:168-173).
 */
#ifndef PPML_HIP_BACKEND_H
#define PPML_HIP_BACKEND_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct ppml_hip_backend ppml_hip_backend;
typedef struct ppml_hip_tensor ppml_hip_tensor;

ppml_hip_backend *ppml_hip_backend_create(int device);
void ppml_hip_backend_destroy(ppml_hip_backend *b);
const char *ppml_hip_backend_name(const ppml_hip_backend *b);
const char *ppml_hip_backend_last_error(const ppml_hip_backend *b);
int ppml_hip_backend_priority(const ppml_hip_backend *b);
void ppml_hip_backend_synchronize(ppml_hip_backend *b);

/* op / type are the reference's tensor_op / tensor_type values; dims[0] is the innermost dimension */
ppml_hip_tensor *ppml_hip_tensor_create(int op, int type, int ndim, const int64_t *dims);
void ppml_hip_tensor_destroy(ppml_hip_tensor *t);
void ppml_hip_tensor_set_src(ppml_hip_tensor *t, int slot, ppml_hip_tensor *src);
void ppml_hip_tensor_set_data(ppml_hip_tensor *t, void *device_ptr);
void ppml_hip_tensor_set_view(ppml_hip_tensor *t, ppml_hip_tensor *view_src, size_t byte_offset);
/* op_params as in the reference's node (include/ppml/Tensor.h:449-450): 32-bit integers, floats stored by bit pattern */
void ppml_hip_tensor_set_param(ppml_hip_tensor *t, int index, float value);
void ppml_hip_tensor_set_param_i32(ppml_hip_tensor *t, int index, int value);
/* the node's flag bits (include/ppml/Tensor.h:19-22: INPUT = 1, OUTPUT = 2); a tensor marked OUTPUT is never
 * folded into a neighbouring node by graph_compute */
void ppml_hip_tensor_set_flag(ppml_hip_tensor *t, int flag);
size_t ppml_hip_tensor_nbytes(const ppml_hip_tensor *t);
int ppml_hip_tensor_type(const ppml_hip_tensor *t);
/* allocate device storage through the backend's BufferType and copy host data in / out */
int ppml_hip_tensor_upload(ppml_hip_backend *b, ppml_hip_tensor *t, const void *host, size_t nbytes);
int ppml_hip_tensor_download(ppml_hip_backend *b, const ppml_hip_tensor *t, void *host, size_t nbytes);

/* The rule is a function of the node alone: b may be NULL, which lets a scheduler on a host without
 * a device ask the question (Backend::supports_op, include/ppml/Backend.h:571). */
int ppml_hip_backend_supports_op(const ppml_hip_backend *b, const ppml_hip_tensor *node);
/* 1: a scheduler owns allocation, graph_compute allocates nothing (Backend.h skip_alloc_) */
void ppml_hip_backend_set_skip_alloc(ppml_hip_backend *b, int on);
/* 0: quantize activations with the Q8_0 rule (default, the CPU contract); 1: with the Q8_1 rule of
 * the reference's CUDA launcher (src/cuda/MulMatQ8Kernel.cu:483-527) */
void ppml_hip_backend_set_q8_1_activations(ppml_hip_backend *b, int on);
/* 1: graph_compute does not execute the {1,0,2,3} permutations the reference's builder wraps around a fused
 * attention node (src/core/ComputeGraphHelper.cpp:456-458, 483) when the attention node is their only
 * reader / they are its only reader; the attention kernel takes the other layout itself and the skipped
 * tensors are never written.  0 (default): every node is executed as it stands. */
void ppml_hip_backend_set_fuse_attention_bridges(ppml_hip_backend *b, int on);
/* Folding of element-wise nodes into the contraction beside them.  The rule is the reference's own for eliminating
 * an intermediate (exactly one reader in the graph, include/ppml/ComputeGraph.h:73-87), plus "not marked OUTPUT";
 * a folded tensor is never written.
 *   relu_into_q8 (default 1): an OP_UNARY/RELU read only -- directly or through whole OP_VIEW / OP_RESHAPE nodes --
 *     by the activation side of a quantized OP_MUL_MAT is applied by that matmul's quantizer
 *     (src/modules/Attention.cpp:1097-1104); same bits as the two nodes run one after the other.
 *   scale_into_out_prod (default 1): an OP_SCALE whose source is an OP_OUT_PROD nobody else reads runs as one
 *     scaled contraction (src/modules/Attention.cpp:264-270); same bits.
 *   attention_chain (default 0): out_prod(K,Q) -> scale -> [add bias] -> softmax -> permute / permute(V) ->
 *     out_prod (src/modules/Attention.cpp:264-281) runs as one fused attention launch when no intermediate has
 *     another reader -- what the reference does itself under PPML_FLASH_ATTN (Attention.cpp:232-262); agrees with
 *     the node-by-node chain to rounding, not bit for bit. */
void ppml_hip_backend_set_fuse_relu_into_q8(ppml_hip_backend *b, int on);
void ppml_hip_backend_set_fuse_scale_into_out_prod(ppml_hip_backend *b, int on);
void ppml_hip_backend_set_fuse_attention_chain(ppml_hip_backend *b, int on);
/*   add_into_soft_max (default 1): an OP_ADD read only by an OP_SOFT_MAX (first operand of the result's size, second
 *     operand whole rows of the softmax: the attention bias, src/modules/Attention.cpp:271-276) is added on the
 *     softmax kernel's way in; same bits.
 *   permutes_into_out_prod (default 1): an OP_OUT_PROD whose operands are both {1,0,2,3} permutations nobody else
 *     reads (src/modules/Attention.cpp:277-281) contracts the unpermuted tensors over their innermost dimension;
 *     same bits, two copies less. */
void ppml_hip_backend_set_fuse_add_into_soft_max(ppml_hip_backend *b, int on);
void ppml_hip_backend_set_fuse_permutes_into_out_prod(ppml_hip_backend *b, int on);
/*   permutes_into_mul_mat (default 1): an F32 OP_MUL_MAT without bias whose operands are both matrix transpositions
 *     nobody else reads -- the weight gradient of a LinearLayer, mul_mat(mat_transpose(grad), mat_transpose(x)),
 *     src/core/ComputeGraph.cpp:733-738 -- contracts the untransposed matrices over their rows; same bits, and the
 *     copies of the activations and of their gradient are not made. */
void ppml_hip_backend_set_fuse_permutes_into_mul_mat(ppml_hip_backend *b, int on);
/* how many nodes the last graph_compute folded into a neighbour and did not execute */
int ppml_hip_backend_nodes_fused_away(const ppml_hip_backend *b);
/* Matrix pipe of this backend's f32 contractions for the length of each graph_compute: 0 = bf16 pipe through
 * the exact three-way split, 1 = fp32 pipe, anything else = the calling thread's ppml_hip_set_f32_arithmetic
 * choice (default).  A field of the backend object, so backends with different settings do not interfere. */
void ppml_hip_backend_set_f32_arithmetic(ppml_hip_backend *b, int mode);
/* graph_compute in single-backend mode (skip_alloc off) copies sources bound to HOST memory to the device for
 * the duration of the call and puts the tensors' fields back afterwards (ensure_host_shadow /
 * release_host_shadows, src/backend/CUDABackend.cpp:521-577, 824-830); ppml_hip_tensor_set_data accepts such a
 * host pointer.  Returns how many sources the last graph_compute covered this way. */
int ppml_hip_backend_host_shadows_made(const ppml_hip_backend *b);
int ppml_hip_backend_graph_compute(ppml_hip_backend *b, ppml_hip_tensor **nodes, int n);
int ppml_hip_backend_pack_weight(ppml_hip_backend *b, ppml_hip_tensor *weight);

#ifdef __cplusplus
}
#endif
#endif
