// ppml_hip_backend.hpp -- C++ host side of the gfx950 backend, above the C ABI of ppml_hip.h.
//
// It mirrors the part of the reference's backend plug-in interface that the matrix-multiplication
// path goes through (include/ppml/Backend.h:550-605 `Backend`, 252-329 `BufferType`/`Buffer`,
// 168-173 `Status`) on a field-compatible subset of the reference's tensor node
// (include/ppml/Tensor.h:443-464: op, type, dims, src[], data, buffer, view_src, op_params), so that
// the executor logic -- which nodes are skipped, how views are resolved, what is rejected, how
// failures map to Status -- can be exercised without the rest of the reference.  A maintainer of
// the reference needs only the C ABI; this class shows what the adapter around it does.
#pragma once

#include <cstddef>
#include <cstdint>
#include <cstring>
#include <memory>
#include <string>
#include <vector>

namespace ppmlhip {

// numeric values of the reference's enums (include/ppml/Tensor.h:35-64 and 136-278)
enum TensorType : int {
    TENSOR_TYPE_F32 = 0,
    TENSOR_TYPE_F16 = 1,
    TENSOR_TYPE_Q8_0 = 8,
    TENSOR_TYPE_Q8_1 = 9,
    TENSOR_TYPE_Q8_0R = 19,
    TENSOR_TYPE_Q8_0M = 64,   // this backend's MFMA-fragment layout; never leaves the device
};

enum TensorOp : int {
    OP_NONE = 0,
    OP_ADD = 2,
    OP_SUB = 6,
    OP_MUL = 7,
    OP_DIV = 8,
    OP_REPEAT_BACK = 21,
    OP_MUL_MAT = 30,
    OP_OUT_PROD = 32,
    OP_SCALE = 33,
    OP_RESHAPE = 37,
    OP_VIEW = 38,
    OP_PERMUTE = 39,
    OP_TRANSPOSE = 40,
    OP_SOFT_MAX = 47,
    OP_FLASH_ATTN_EXT = 75,
    OP_FLASH_ATTN_BACK = 76,
    OP_UNARY = 88,
    OP_TRI_MUL = 100,
    OP_TRI_MUL_BACK = 101,
    OP_OUTER_PROD_MEAN = 102,
    OP_OUTER_PROD_MEAN_BACK = 103,
};

// include/ppml/ComputeGraph.h:20-39: the sub-type of an OP_UNARY node, kept in op_params[0]
enum UnaryOp : int { UNARY_OP_RELU = 4 };

// include/ppml/Tensor.h:19-22
enum TensorFlag : int { TENSOR_FLAG_INPUT = 1, TENSOR_FLAG_OUTPUT = 2 };

// include/ppml/Backend.h:168-173
enum class Status : int { SUCCESS = 0, ALLOC_FAILED, NOT_SUPPORTED, ABORTED };

// include/ppml/Tensor.h:72-133
bool is_quantized_type(int t);
bool is_quantized_type_supported(int t);
int quant_block_elems(int t);
size_t quant_block_bytes(int t);

class Buffer;

// The fields of the reference's tensor node that this path reads.
struct Tensor {
    int op = OP_NONE;
    int type = TENSOR_TYPE_F32;
    int ndim = 0;
    int64_t dims[4] = {1, 1, 1, 1};       // dims[0] innermost
    Tensor* src[10] = {nullptr};
    void* data = nullptr;
    Buffer* buffer = nullptr;
    size_t buffer_offs = 0;
    Tensor* view_src = nullptr;           // OP_VIEW / OP_RESHAPE share their source's storage
    size_t view_offs = 0;
    int32_t op_params[16] = {0};          // as in the reference: integers, or the bit pattern of a float
    int32_t flag = 0;                     // TensorFlag bits; a tensor marked OUTPUT is never fused away

    float param_f32(int i) const { float f; std::memcpy(&f, &op_params[i], sizeof f); return f; }
    void set_param_f32(int i, float f) { std::memcpy(&op_params[i], &f, sizeof f); }

    int64_t numel() const { return dims[0] * dims[1] * dims[2] * dims[3]; }
    // include/ppml/Tensor.h:327-352
    bool quant_shape_valid() const;
    size_t nbytes() const;
};

// include/ppml/Backend.h:252-272
class BufferType {
public:
    const char* get_name() const { return "HIP"; }
    void* alloc(size_t size) const;
    void free(void* p) const;
    size_t get_alignment() const { return 128; }
    size_t get_alloc_size(const Tensor* t) const { return t->nbytes(); }
    bool is_host() const { return false; }
    static const BufferType* instance();
};

// include/ppml/Backend.h:275-329, 355-432 (device semantics: blocking copies)
class Buffer {
public:
    Buffer(const BufferType* type, size_t size);
    ~Buffer();
    Buffer(const Buffer&) = delete;
    Buffer& operator=(const Buffer&) = delete;
    void* data() const { return base_; }
    size_t size() const { return size_; }
    bool is_host() const { return false; }
    bool set_tensor(Tensor* t, const void* host, size_t offs, size_t n);
    bool get_tensor(const Tensor* t, void* host, size_t offs, size_t n) const;
    bool memset_tensor(Tensor* t, int value, size_t offs, size_t n);
    bool contains(const void* p, size_t n) const;

private:
    const BufferType* type_;
    void* base_ = nullptr;
    size_t size_ = 0;
};

using ComputeGraph = std::vector<Tensor*>;   // nodes in evaluation order

// src/backend/CUDABackend.cpp:121-163 (OP_MUL_MAT, OP_OUT_PROD), 410-421 (OP_OUTER_PROD_MEAN, OP_OUTER_PROD_MEAN_BACK),
// 113-119 (OP_PERMUTE, OP_TRANSPOSE), 395-409 (OP_TRI_MUL, OP_TRI_MUL_BACK), 457-471 (OP_FLASH_ATTN_EXT, OP_FLASH_ATTN_BACK),
// 94-98 (OP_ADD, OP_SUB, OP_MUL, OP_DIV), 236-237 (OP_SOFT_MAX), 340-344 (OP_SCALE), 470-493 (OP_UNARY); a function of
// the node alone, so it can be asked without a device
bool node_supported(const Tensor* node);

// include/ppml/Backend.h:550-605; executor obligations of src/backend/CUDABackend.cpp:708-1086
class HipBackend {
public:
    explicit HipBackend(int device);
    ~HipBackend();
    const char* get_name() const { return "HIP-gfx950"; }
    Status graph_compute(ComputeGraph* graph);
    void synchronize();
    bool supports_op(const Tensor* node) const { return node_supported(node); }
    const BufferType* buffer_type() const { return BufferType::instance(); }
    bool supports_buffer_type(const BufferType* t) const { return t == BufferType::instance(); }
    int priority() const { return 1; }                   // include/ppml/Backend.h:949
    bool vram_budgeted() const { return true; }
    bool skip_alloc() const { return skip_alloc_; }
    void set_skip_alloc(bool v) { skip_alloc_ = v; }
    const std::string& last_error() const { return error_; }
    // Rule the quantized mul_mat uses for its activations: false = Q8_0 (quantize_q8_0_host, the CPU
    // contract), true = Q8_1 (what the reference's CUDA launcher does, src/cuda/MulMatQ8Kernel.cu:483-527).
    void set_q8_1_activations(bool v) { q8_1_activations_ = v; }
    bool q8_1_activations() const { return q8_1_activations_; }
    // Off by default.  On: a permutation {1,0,2,3} whose only reader is a fused attention node (all three of
    // Q, K, V), or that is the only reader of its result, is not executed -- the attention kernel takes that
    // layout directly -- and the skipped permutation's own tensor is never written.  Only for graphs whose
    // every reader of those tensors is inside the graph handed to graph_compute.
    void set_fuse_attention_bridges(bool v) { fuse_attention_bridges_ = v; }
    bool fuse_attention_bridges() const { return fuse_attention_bridges_; }

    // Fusion of the element-wise nodes into the contraction beside them.  The legality rule is the reference's own
    // for eliminating an intermediate (include/ppml/ComputeGraph.h:73-87): the tensor has exactly one reader in the
    // graph handed to graph_compute; here it must also not be marked TENSOR_FLAG_OUTPUT.  A fused-away tensor is
    // never written.  Both are ON by default and give the same bits as the nodes run one by one:
    //   relu   -- an OP_UNARY/RELU node read only (directly or through whole OP_VIEW / OP_RESHAPE nodes) by the
    //             activation side of a quantized OP_MUL_MAT is not executed; the matmul's quantizer applies it
    //             (src/modules/Attention.cpp:1097-1104: linear1 -> relu -> linear2 of the pair feed-forward);
    //   scale  -- an OP_SCALE whose source is an OP_OUT_PROD nobody else reads runs as one scaled contraction
    //             (src/modules/Attention.cpp:264-270: the attention logits and their 1/sqrt(D)).
    void set_fuse_relu_into_q8(bool v) { fuse_relu_into_q8_ = v; }
    bool fuse_relu_into_q8() const { return fuse_relu_into_q8_; }
    void set_fuse_scale_into_out_prod(bool v) { fuse_scale_into_out_prod_ = v; }
    bool fuse_scale_into_out_prod() const { return fuse_scale_into_out_prod_; }
    // Two more of the same kind, ON by default, same bits as the nodes run one by one; together with `scale` they turn
    // the reference's default attention chain (src/modules/Attention.cpp:264-281) from seven launches into three:
    //   add      -- an OP_ADD read only by an OP_SOFT_MAX, whose first operand has the result's size and whose second
    //               is whole rows of the softmax (the attention bias), is added on the softmax kernel's way in;
    //   permutes -- an OP_OUT_PROD both of whose operands are {1,0,2,3} permutations nobody else reads contracts
    //               the unpermuted tensors over their innermost dimension instead (the permutation is a copy in the
    //               reference, src/core/ComputeGraphHelper.cpp:700-729).
    void set_fuse_add_into_soft_max(bool v) { fuse_add_into_soft_max_ = v; }
    bool fuse_add_into_soft_max() const { return fuse_add_into_soft_max_; }
    void set_fuse_permutes_into_out_prod(bool v) { fuse_permutes_into_out_prod_ = v; }
    bool fuse_permutes_into_out_prod() const { return fuse_permutes_into_out_prod_; }
    // The same for the weight gradient of a LinearLayer, dW = mul_mat(mat_transpose(grad), mat_transpose(x))
    // (src/core/ComputeGraph.cpp:733-738): an F32 OP_MUL_MAT without bias both of whose operands are matrix
    // transpositions nobody else reads contracts the untransposed matrices over their rows (mul_mat_tn_hip); the two
    // copies -- of the activations and of their gradient, the largest tensors of the backward pass -- are not made.
    // ON by default; same bits as the nodes run one by one.
    void set_fuse_permutes_into_mul_mat(bool v) { fuse_permutes_into_mul_mat_ = v; }
    bool fuse_permutes_into_mul_mat() const { return fuse_permutes_into_mul_mat_; }
    // Off by default.  On: the reference's default attention chain (src/modules/Attention.cpp:264-281)
    //   out_prod(K, Q) -> scale -> [add bias] -> softmax -> permute{1,0,2,3} ; permute{1,0,2,3}(V) -> out_prod
    // whose intermediates have no other reader runs as one fused attention launch on the graph's own layouts
    // (what the reference does itself under PPML_FLASH_ATTN, Attention.cpp:232-262).  Results then agree with the
    // node-by-node chain to rounding, not bit for bit (the softmax sums are formed in another order).
    void set_fuse_attention_chain(bool v) { fuse_attention_chain_ = v; }
    bool fuse_attention_chain() const { return fuse_attention_chain_; }
    // How many nodes the last graph_compute folded into a neighbour and did not execute.
    size_t nodes_fused_away() const { return nodes_fused_away_; }

    // Matrix pipe of this backend's f32 contractions: 0 = bf16 pipe through the exact three-way split, 1 = fp32
    // pipe, -1 (default) = whatever the calling thread has chosen with ppml_hip_set_f32_arithmetic.  Applied
    // for the length of each graph_compute and put back afterwards, so two backends (or threads) with different
    // settings do not disturb each other.
    void set_f32_arithmetic(int mode) { f32_arithmetic_ = (mode == 0 || mode == 1) ? mode : -1; }
    int f32_arithmetic() const { return f32_arithmetic_; }
    // Host-resident sources the last graph_compute copied to the device for its duration
    // (src/backend/CUDABackend.cpp:521-577; single-backend mode only, i.e. not under skip_alloc).
    size_t host_shadows_made() const { return host_shadows_made_; }

    // Once-per-weight step of src/model/PPML.cpp:4504-4528: turns a Q8_0 / Q8_1 / Q8_0R weight node
    // into the MFMA-fragment layout in a buffer owned by this backend.
    Status pack_weight(Tensor* weight);

private:
    Status dispatch_node(Tensor* node);                  // src/backend/CUDAKernels.cpp:351-, 717-847
    Status kernel_mul_mat(Tensor* node);
    Status kernel_out_prod(Tensor* node);
    Status kernel_outer_prod_mean(Tensor* node);
    Status kernel_flash_attn_ext(Tensor* node);
    Status kernel_flash_attn_back(Tensor* node);
    Status kernel_permute(Tensor* node);
    Status kernel_repeat_back(Tensor* node);
    Status kernel_tri_mul(Tensor* node);
    Status kernel_tri_mul_back(Tensor* node);
    Status kernel_outer_prod_mean_back(Tensor* node);
    Status kernel_scale(Tensor* node);
    Status kernel_unary(Tensor* node);
    Status kernel_elemwise(Tensor* node);
    Status kernel_soft_max(Tensor* node);
    bool resolve_views(Tensor* node);                    // src/backend/CUDABackend.cpp:800-819
    bool device_pointer_ok(const Tensor* t) const;       // src/backend/CUDABackend.cpp:894-973
    Status fail(Status s, const std::string& why);

    int device_;
    bool skip_alloc_ = false;
    bool q8_1_activations_ = false;
    bool fuse_attention_bridges_ = false;
    int f32_arithmetic_ = -1;
    size_t host_shadows_made_ = 0;
    bool fuse_relu_into_q8_ = true;
    bool fuse_scale_into_out_prod_ = true;
    bool fuse_attention_chain_ = false;
    bool fuse_add_into_soft_max_ = true;
    bool fuse_permutes_into_out_prod_ = true;
    bool fuse_permutes_into_mul_mat_ = true;
    size_t nodes_fused_away_ = 0;
    int attn_layout_ = 0;                                // layout bits of the attention node being dispatched
    bool relu_in_quantizer_ = false;                     // the matmul being dispatched applies a fused-away ReLU
    float out_prod_alpha_ = 1.0f;                        // scale of a fused-away OP_SCALE behind the out_prod being dispatched
    bool out_prod_scaled_ = false;
    bool out_prod_transposed_ = false;                   // the out_prod being dispatched reads the sources of two fused-away permutations
    bool mul_mat_transposed_ = false;                    // the same for the mul_mat being dispatched
    const Tensor* soft_max_bias_ = nullptr;              // second operand of a fused-away OP_ADD in front of the softmax being dispatched
    std::string error_;
    std::vector<std::unique_ptr<Buffer>> owned_;         // node outputs allocated here, packed weights
};

}  // namespace ppmlhip
