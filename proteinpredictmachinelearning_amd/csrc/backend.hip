// Host side of the gfx950 backend: the executor that walks a list of tensor nodes and hands the
// matrix-multiplication ops to the launchers of ppml_hip.h.  No kernels in this file.
//
// What it mirrors of the reference:
//   supports_op      src/backend/CUDABackend.cpp:121-163 (OP_MUL_MAT, OP_OUT_PROD), 410-416 (OP_OUTER_PROD_MEAN)
//   graph_compute    src/backend/CUDABackend.cpp:708-1086 (skip no-op nodes, resolve view sources,
//                    refuse host / out-of-buffer pointers, dispatch, launch error -> ABORTED)
//   node -> launcher src/backend/CUDAKernels.cpp:717-847 (mul_mat), 1537-1565 (out_prod), 1204-1221 (outer_prod_mean),
//                    666-712 (unary, element-wise binary ops), 849-857 (softmax), 992-1004 (scale)
//
// Two deliberate differences, both on failure paths only:
//   * the reference's quantized mul_mat prints and returns normally when the launcher fails, so the
//     node is silently left unwritten (CUDAKernels.cpp:735-763); here every launcher failure ends
//     graph_compute with NOT_SUPPORTED (bad arguments) or ABORTED (device error);
//   * a view source is bound to root data PLUS the accumulated view offsets; the reference binds the
//     root pointer itself (CUDABackend.cpp:812-819) and relies on its allocator having bound offset
//     views beforehand.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstring>
#include <new>
#include <unordered_map>
#include <unordered_set>

#include "../../include/ppml_hip.h"
#include "../../include/ppml_hip_backend.h"
#include "../../include/ppml_hip_backend.hpp"

namespace ppmlhip {

// ------------------------------------------------------------------------------------------------
// type helpers (include/ppml/Tensor.h:72-133)
bool is_quantized_type(int t) {
    return t == TENSOR_TYPE_Q8_0 || t == TENSOR_TYPE_Q8_1 || t == TENSOR_TYPE_Q8_0R || t == TENSOR_TYPE_Q8_0M;
}
bool is_quantized_type_supported(int t) { return is_quantized_type(t); }
int quant_block_elems(int t) { return is_quantized_type(t) ? 32 : 1; }
size_t quant_block_bytes(int t) {
    switch (t) {
        case TENSOR_TYPE_Q8_0:
        case TENSOR_TYPE_Q8_0R:
        case TENSOR_TYPE_Q8_0M: return 34;
        case TENSOR_TYPE_Q8_1: return 36;
        case TENSOR_TYPE_F16: return 2;
        default: return 4;
    }
}

bool Tensor::quant_shape_valid() const {
    if (!is_quantized_type(type)) return true;
    return ndim >= 1 && dims[0] > 0 && dims[0] % quant_block_elems(type) == 0;
}

size_t Tensor::nbytes() const {
    const int64_t n = numel();
    if (n <= 0) return 0;
    if (type == TENSOR_TYPE_Q8_0M) {
        if (!quant_shape_valid()) return 0;
        return q8_weight_packed_bytes_hip(static_cast<int>(n / dims[0]), static_cast<int>(dims[0]));
    }
    if (is_quantized_type(type)) {
        if (!quant_shape_valid()) return 0;
        return static_cast<size_t>(n / quant_block_elems(type)) * quant_block_bytes(type);
    }
    return static_cast<size_t>(n) * quant_block_bytes(type);
}

// ------------------------------------------------------------------------------------------------
// BufferType / Buffer (include/ppml/Backend.h:252-329)
void* BufferType::alloc(size_t size) const {
    void* p = nullptr;
    if (size == 0) size = get_alignment();
    if (hipMalloc(&p, size) != hipSuccess) {
        (void)hipGetLastError();
        return nullptr;
    }
    return p;
}
void BufferType::free(void* p) const {
    if (p) (void)hipFree(p);
}
const BufferType* BufferType::instance() {
    static const BufferType t;
    return &t;
}

Buffer::Buffer(const BufferType* type, size_t size) : type_(type), size_(size) { base_ = type_->alloc(size); }
Buffer::~Buffer() { type_->free(base_); }

bool Buffer::contains(const void* p, size_t n) const {
    const char* b = static_cast<const char*>(base_);
    const char* q = static_cast<const char*>(p);
    return base_ && q >= b && n <= size_ && q + n <= b + size_;
}
bool Buffer::set_tensor(Tensor* t, const void* host, size_t offs, size_t n) {
    if (!t || !t->data || !host || !contains(static_cast<char*>(t->data) + offs, n)) return false;
    return hipMemcpy(static_cast<char*>(t->data) + offs, host, n, hipMemcpyHostToDevice) == hipSuccess;
}
bool Buffer::get_tensor(const Tensor* t, void* host, size_t offs, size_t n) const {
    if (!t || !t->data || !host || !contains(static_cast<const char*>(t->data) + offs, n)) return false;
    return hipMemcpy(host, static_cast<const char*>(t->data) + offs, n, hipMemcpyDeviceToHost) == hipSuccess;
}
bool Buffer::memset_tensor(Tensor* t, int value, size_t offs, size_t n) {
    if (!t || !t->data || !contains(static_cast<char*>(t->data) + offs, n)) return false;
    return hipMemset(static_cast<char*>(t->data) + offs, value, n) == hipSuccess;
}

// ------------------------------------------------------------------------------------------------
HipBackend::HipBackend(int device) : device_(device) {
    if (ppml_hip_init(device) != 0) error_ = ppml_hip_last_error();
}
HipBackend::~HipBackend() {
    (void)hipSetDevice(device_);
    (void)hipDeviceSynchronize();
}

Status HipBackend::fail(Status s, const std::string& why) {
    error_ = why;
    return s;
}

void HipBackend::synchronize() {
    (void)hipSetDevice(device_);
    (void)hipDeviceSynchronize();
}

// The operand combinations OP_MUL_MAT takes (src/backend/CUDABackend.cpp:121-157), one row each: the result
// is always F32, a bias (src[2]) rides along on the all-F32 row only, and a quantized operand is the weight of
// a product whose other side is F32 activations.
enum OperandClass { OPERAND_F32, OPERAND_F16, OPERAND_Q8, OPERAND_OTHER };
static OperandClass operand_class(int type) {
    if (type == TENSOR_TYPE_F32) return OPERAND_F32;
    if (type == TENSOR_TYPE_F16) return OPERAND_F16;
    return is_quantized_type(type) ? OPERAND_Q8 : OPERAND_OTHER;
}
struct MulMatCombo { OperandClass src0, src1; bool bias; };
static const MulMatCombo MUL_MAT_COMBOS[] = {
    {OPERAND_F32, OPERAND_F32, true},
    {OPERAND_F16, OPERAND_F16, false},
    {OPERAND_Q8, OPERAND_F32, false},
    {OPERAND_F32, OPERAND_Q8, false},
};

bool node_supported(const Tensor* node) {
    if (!node) return false;
    const Tensor* src0 = node->src[0];
    const Tensor* src1 = node->src[1];
    switch (node->op) {
        case OP_NONE:
        case OP_VIEW:
        case OP_RESHAPE:
            return true;
        case OP_MUL_MAT: {
            if (!src1) return true;              // nothing to multiply with yet: the reference lets such a node pass
            if (!src0 || node->type != TENSOR_TYPE_F32) return false;
            const OperandClass c0 = operand_class(src0->type), c1 = operand_class(src1->type);
            for (const MulMatCombo& combo : MUL_MAT_COMBOS) {
                if (combo.src0 != c0 || combo.src1 != c1) continue;
                if (node->src[2] && !combo.bias) return false;
                const Tensor* w = c0 == OPERAND_Q8 ? src0 : c1 == OPERAND_Q8 ? src1 : nullptr;
                return !w || (w->quant_shape_valid() && is_quantized_type_supported(w->type));
            }
            return false;
        }
        case OP_OUT_PROD:
            return src0 && src1 && src0->type == TENSOR_TYPE_F32 && src1->type == TENSOR_TYPE_F32 &&
                   node->type == TENSOR_TYPE_F32;
        case OP_SCALE:
            // src/backend/CUDABackend.cpp:340-344
            return src0 && src0->type == TENSOR_TYPE_F32 && node->type == TENSOR_TYPE_F32;
        case OP_UNARY:
            // src/backend/CUDABackend.cpp:470-493 lists the sub-types its unary kernel has; of those, this
            // backend has the one that sits between two matrix multiplications
            return src0 && src0->type == TENSOR_TYPE_F32 && node->type == TENSOR_TYPE_F32 &&
                   node->op_params[0] == UNARY_OP_RELU;
        case OP_ADD:
        case OP_SUB:
        case OP_MUL:
        case OP_DIV:
            // src/backend/CUDABackend.cpp:94-98 says yes to all four without looking; the kernel behind them is
            // f32 with operands that repeat along the result's flat order (CUDAKernels.cpp:678-712)
            return src0 && src1 && src0->type == TENSOR_TYPE_F32 && src1->type == TENSOR_TYPE_F32 &&
                   node->type == TENSOR_TYPE_F32;
        case OP_SOFT_MAX:
            // src/backend/CUDABackend.cpp:236-237 (unconditional there)
            return src0 && src0->type == TENSOR_TYPE_F32 && node->type == TENSOR_TYPE_F32 && node->dims[0] > 0;
        case OP_TRI_MUL:
            // src/backend/CUDABackend.cpp:395-402: left, right and the result all 4-D f32
            if (!src0 || !src1) return false;
            if (src0->type != TENSOR_TYPE_F32 || src1->type != TENSOR_TYPE_F32 || node->type != TENSOR_TYPE_F32) return false;
            return src0->ndim == 4 && src1->ndim == 4 && node->ndim == 4;
        case OP_FLASH_ATTN_BACK: {
            // src/backend/CUDABackend.cpp:465-471 (there: d <= 32; this kernel takes the forward's range)
            if (!src0 || src0->type != TENSOR_TYPE_F32) return false;
            const int64_t d = src0->dims[0];
            return d > 0 && d <= 64 && (d % 4) == 0;
        }
        case OP_OUTER_PROD_MEAN_BACK:           // src/backend/CUDABackend.cpp:418-421, the same rule
        case OP_TRI_MUL_BACK:
            // src/backend/CUDABackend.cpp:404-409: grad, left, right present, at least one of the two outputs
            if (!src0 || !src1 || !node->src[2]) return false;
            if (!node->src[3] && !node->src[4]) return false;
            return src0->type == TENSOR_TYPE_F32 && node->type == TENSOR_TYPE_F32;
        case OP_REPEAT_BACK:
            // src/backend/CUDABackend.cpp:317-330: F32 in and out, at most four dimensions either side
            return src0 && src0->type == TENSOR_TYPE_F32 && node->type == TENSOR_TYPE_F32 &&
                   src0->ndim >= 1 && src0->ndim <= 4 && node->ndim >= 1 && node->ndim <= 4;
        case OP_PERMUTE:
        case OP_TRANSPOSE:
            // src/backend/CUDABackend.cpp:113-119
            return src0 && src0->type == TENSOR_TYPE_F32 && node->type == TENSOR_TYPE_F32;
        case OP_FLASH_ATTN_EXT: {
            // src/backend/CUDABackend.cpp:457-463: f32, head dimension (dims[0] of the [d,L,h,B] layout)
            // a multiple of 4 and at most 64
            if (!src0 || !src1 || !node->src[2]) return false;
            if (src0->type != TENSOR_TYPE_F32) return false;
            const int64_t d = src0->dims[0];
            return d > 0 && d <= 64 && (d % 4) == 0;
        }
        case OP_OUTER_PROD_MEAN:
            if (!src0 || !src1) return false;
            if (src0->type != TENSOR_TYPE_F32 || src1->type != TENSOR_TYPE_F32 || node->type != TENSOR_TYPE_F32) return false;
            return src0->ndim == 4 && src1->ndim == 4 && src0->dims[0] > 0 && src0->dims[2] > 0;
        default:
            return false;
    }
}

// Follows view_src (or, for OP_VIEW / OP_RESHAPE nodes built with only src[0] set, src[0]) to the
// tensor that carries the storage and binds every unbound source of `node` to it.
bool HipBackend::resolve_views(Tensor* node) {
    for (Tensor* src : node->src) {
        if (!src || src->data) continue;
        Tensor* r = src;
        size_t offs = 0;
        for (int guard = 0; guard < 64; ++guard) {
            Tensor* nxt = r->view_src;
            if (!nxt && (r->op == OP_VIEW || r->op == OP_RESHAPE)) nxt = r->src[0];
            if (!nxt) break;
            offs += r->view_offs;
            r = nxt;
        }
        if (r == src || !r->data) continue;
        src->data = static_cast<char*>(r->data) + offs;
        src->buffer = r->buffer;
        src->buffer_offs = r->buffer_offs + offs;
    }
    return true;
}

bool HipBackend::device_pointer_ok(const Tensor* t) const {
    if (!t || !t->data) return false;
    hipPointerAttribute_t attr{};
    if (hipPointerGetAttributes(&attr, t->data) != hipSuccess) {
        (void)hipGetLastError();
        return false;
    }
    if (attr.type != hipMemoryTypeDevice && attr.type != hipMemoryTypeManaged) return false;
    if (t->buffer) {
        const size_t need = t->nbytes();
        if (!t->buffer->contains(t->data, need)) return false;
    }
    return true;
}

// Single-backend mode has no scheduler to copy host-resident leaves (embedding tables, constant masks, any
// tensor bound to host memory) to the device, so the executor does it: every such source gets a device copy
// for the duration of graph_compute, and the tensor's own fields are put back afterwards
// (src/backend/CUDABackend.cpp:521-577, 824-830).
namespace {
bool is_device_memory(const void* p) {
    hipPointerAttribute_t attr{};
    if (hipPointerGetAttributes(&attr, p) != hipSuccess) {
        (void)hipGetLastError();                        // an ordinary host pointer: not an error to report later
        return false;
    }
    return attr.type == hipMemoryTypeDevice || attr.type == hipMemoryTypeManaged;
}
}  // namespace

class HostShadows {
public:
    ~HostShadows() {
        for (const Saved& s : saved_) {
            s.t->data = s.data;
            s.t->buffer = s.buffer;
            s.t->buffer_offs = s.offs;
        }
        // views that were bound to a copy while it existed go back to unbound (only unbound sources get bound)
        for (Tensor* t : borrowed_) {
            t->data = nullptr;
            t->buffer = nullptr;
            t->buffer_offs = 0;
        }
        for (const Saved& s : saved_) (void)hipFree(s.dev);      // waits for the kernels that read it
    }
    // Leaves `t` bound to device memory if that can be arranged; a tensor it cannot help is left as it is,
    // and the executor's pointer check names it.
    void cover(Tensor* t) {
        if (!t || !t->data) return;
        for (const Saved& s : saved_) {
            if (s.t == t) return;
            const char* p = static_cast<const char*>(t->data);
            if (p >= static_cast<const char*>(s.dev) && p < static_cast<const char*>(s.dev) + s.bytes) {
                // a view of a covered leaf, resolved while the copy is the leaf's storage
                if (std::find(borrowed_.begin(), borrowed_.end(), t) == borrowed_.end()) borrowed_.push_back(t);
                return;
            }
        }
        if (t->buffer ? !t->buffer->is_host() : is_device_memory(t->data)) return;
        size_t bytes = t->nbytes();
        if (bytes == 0) return;
        void* dev = nullptr;
        if (hipMalloc(&dev, bytes) != hipSuccess) { (void)hipGetLastError(); return; }
        if (hipMemcpy(dev, t->data, bytes, hipMemcpyHostToDevice) != hipSuccess) {
            (void)hipGetLastError();
            (void)hipFree(dev);
            return;
        }
        saved_.push_back(Saved{t, t->data, t->buffer, t->buffer_offs, dev, bytes});
        t->data = dev;
        t->buffer = nullptr;                            // the copy belongs to no Buffer
        t->buffer_offs = 0;
    }
    size_t count() const { return saved_.size(); }

private:
    struct Saved { Tensor* t; void* data; Buffer* buffer; size_t offs; void* dev; size_t bytes; };
    std::vector<Saved> saved_;
    std::vector<Tensor*> borrowed_;
};

static Status status_of_rc(int rc) {
    if (rc == 0) return Status::SUCCESS;
    if (rc == 3) return Status::ALLOC_FAILED;
    if (rc == 6 || rc == 7) return Status::ABORTED;
    return Status::NOT_SUPPORTED;
}

Status HipBackend::kernel_mul_mat(Tensor* node) {
    Tensor* s0 = node->src[0];
    Tensor* s1 = node->src[1];
    if (!s0 || !s1) return fail(Status::NOT_SUPPORTED, "mul_mat: missing source");
    if (mul_mat_transposed_) {
        // s0, s1 are the sources of the two folded transpositions: [M, K] and [N, K] in the reference's order of
        // dimensions, i.e. K rows of M and of N elements; the node is [N, M]
        const int64_t M = node->dims[1], N = node->dims[0], K = s0->dims[1];
        if (s0->type != TENSOR_TYPE_F32 || s1->type != TENSOR_TYPE_F32 || node->type != TENSOR_TYPE_F32 || node->src[2] ||
            s0->dims[0] != M || s1->dims[0] != N || s1->dims[1] != K || s0->numel() != M * K || s1->numel() != N * K)
            return fail(Status::ABORTED, "mul_mat: the folded transpositions do not fit the node");
        const int rc = mul_mat_tn_hip(static_cast<const float*>(s0->data), static_cast<const float*>(s1->data), static_cast<float*>(node->data),
                                      static_cast<int>(M), static_cast<int>(K), static_cast<int>(N), 1.0f, nullptr);
        if (rc != 0) return fail(status_of_rc(rc), std::string("mul_mat: ") + ppml_hip_last_error());
        return Status::SUCCESS;
    }
    const int64_t M = node->dims[1], N = node->dims[0], K = s0->dims[0];
    if (s1->dims[0] != K) return fail(Status::NOT_SUPPORTED, "mul_mat: inner dimensions differ");
    if (s0->numel() != M * K || s1->numel() != N * K)
        return fail(Status::NOT_SUPPORTED, "mul_mat: source shapes do not match the node's [N, M]");
    const float* bias = node->src[2] ? static_cast<const float*>(node->src[2]->data) : nullptr;
    if (node->src[2] && node->src[2]->numel() != N) return fail(Status::NOT_SUPPORTED, "mul_mat: bias length is not N");

    const bool q0 = is_quantized_type(s0->type), q1 = is_quantized_type(s1->type);
    int rc;
    if (q0 || q1) {
        if (bias) return fail(Status::NOT_SUPPORTED, "mul_mat: the quantized path has no bias epilogue");
        if (q0 == q1) return fail(Status::NOT_SUPPORTED, "mul_mat: exactly one side may be quantized");
        Tensor* w = q0 ? s0 : s1;
        Tensor* a = q0 ? s1 : s0;
        if (!w->quant_shape_valid() || a->type != TENSOR_TYPE_F32 || node->type != TENSOR_TYPE_F32 || K % 32 != 0)
            return fail(Status::NOT_SUPPORTED, "mul_mat: unsupported quantized combination");
        const int wtype = w->type == TENSOR_TYPE_Q8_1 ? PPML_WTYPE_Q8_1
                        : w->type == TENSOR_TYPE_Q8_0R ? PPML_WTYPE_Q8_0R
                        : w->type == TENSOR_TYPE_Q8_0M ? PPML_WTYPE_Q8_0M : PPML_WTYPE_Q8_0;
        // weight rows are the out features: with the weight in src0 they index the node's dims[1]
        const int64_t Mq = q0 ? M : N, Nq = q0 ? N : M;
        const int c_trans = q0 ? 0 : 1;
        rc = mul_mat_q8_ex_hip(w->data, static_cast<const float*>(a->data), static_cast<float*>(node->data),
                               static_cast<int>(Mq), static_cast<int>(Nq), static_cast<int>(K), wtype, c_trans,
                               (q8_1_activations_ ? PPML_Q8_FLAG_Q8_1_ACTIVATIONS : 0) | (relu_in_quantizer_ ? PPML_Q8_FLAG_RELU : 0),
                               nullptr, nullptr, nullptr);
    } else if (relu_in_quantizer_) {
        return fail(Status::ABORTED, "mul_mat: a ReLU was folded into a matmul that has no quantizer");
    } else if (s0->type == TENSOR_TYPE_F16 && s1->type == TENSOR_TYPE_F16) {
        // src/backend/CUDAKernels.cpp:794-821: F16 x F16 -> F32, no bias epilogue on this path
        if (bias) return fail(Status::NOT_SUPPORTED, "mul_mat: the F16 path has no bias epilogue");
        if (node->type != TENSOR_TYPE_F32) return fail(Status::NOT_SUPPORTED, "mul_mat: F16 x F16 gives F32");
        rc = mul_mat_f16_hip(s0->data, s1->data, static_cast<float*>(node->data), static_cast<int>(M),
                             static_cast<int>(K), static_cast<int>(N), nullptr, nullptr);
    } else {
        if (s0->type != TENSOR_TYPE_F32 || s1->type != TENSOR_TYPE_F32 || node->type != TENSOR_TYPE_F32)
            return fail(Status::NOT_SUPPORTED, "mul_mat: F32 x F32 or F16 x F16 -> F32 besides the quantized path");
        rc = mul_mat_hip(static_cast<const float*>(s0->data), static_cast<const float*>(s1->data),
                         static_cast<float*>(node->data), static_cast<int>(M), static_cast<int>(K),
                         static_cast<int>(N), bias, nullptr);
    }
    if (rc != 0) return fail(status_of_rc(rc), std::string("mul_mat: ") + ppml_hip_last_error());
    return Status::SUCCESS;
}

static inline int64_t dim_or_1(const Tensor* t, int i) { return t->ndim > i ? t->dims[i] : 1; }

Status HipBackend::kernel_out_prod(Tensor* node) {
    const Tensor* a = node->src[0];
    const Tensor* b = node->src[1];
    if (!a || !b) return fail(Status::NOT_SUPPORTED, "out_prod: missing source");
    // the reference clears dst first and accumulates; the launcher overwrites dst instead
    if (out_prod_transposed_) {
        // a, b are the sources of the two folded permutations: [k, i0, ..] and [k, i1, ..]
        const int rc = out_prod_tt_hip(static_cast<const float*>(a->data), static_cast<const float*>(b->data), static_cast<float*>(node->data),
                                       a->dims[0], a->dims[1], dim_or_1(a, 2), dim_or_1(a, 3),
                                       b->dims[0], b->dims[1], dim_or_1(b, 2), dim_or_1(b, 3),
                                       node->dims[0], node->dims[1], dim_or_1(node, 2), dim_or_1(node, 3), nullptr);
        if (rc != 0) return fail(status_of_rc(rc), std::string("out_prod: ") + ppml_hip_last_error());
        return Status::SUCCESS;
    }
    const int rc = out_prod_scaled_ ? out_prod_scaled_hip(static_cast<const float*>(a->data), static_cast<const float*>(b->data),
                                static_cast<float*>(node->data),
                                a->dims[0], a->dims[1], dim_or_1(a, 2), dim_or_1(a, 3),
                                b->dims[0], b->dims[1], dim_or_1(b, 2), dim_or_1(b, 3),
                                node->dims[0], node->dims[1], dim_or_1(node, 2), dim_or_1(node, 3), out_prod_alpha_, nullptr)
                                    : out_prod_hip(static_cast<const float*>(a->data), static_cast<const float*>(b->data),
                                static_cast<float*>(node->data),
                                a->dims[0], a->dims[1], dim_or_1(a, 2), dim_or_1(a, 3),
                                b->dims[0], b->dims[1], dim_or_1(b, 2), dim_or_1(b, 3),
                                node->dims[0], node->dims[1], dim_or_1(node, 2), dim_or_1(node, 3), nullptr);
    if (rc != 0) return fail(status_of_rc(rc), std::string("out_prod: ") + ppml_hip_last_error());
    return Status::SUCCESS;
}

Status HipBackend::kernel_outer_prod_mean(Tensor* node) {
    const Tensor* l = node->src[0];
    const Tensor* r = node->src[1];
    if (!l || !r || !l->data || !r->data || !node->data) return fail(Status::NOT_SUPPORTED, "outer_prod_mean: unbound tensor");
    const int64_t D = l->dims[0], L = l->dims[1], N = l->dims[2], B = l->dims[3];
    if (N <= 0) return fail(Status::NOT_SUPPORTED, "outer_prod_mean: N must be positive");
    if (r->numel() != l->numel() || node->numel() != D * D * L * L * B)
        return fail(Status::NOT_SUPPORTED, "outer_prod_mean: shapes are not [D,L,N,B] x [D,L,N,B] -> [D*D,L,L,B]");
    const int rc = outer_prod_mean_hip(static_cast<const float*>(l->data), static_cast<const float*>(r->data),
                                       static_cast<float*>(node->data), D, L, N, B, 1.0f / static_cast<float>(N),
                                       nullptr);
    if (rc != 0) return fail(status_of_rc(rc), std::string("outer_prod_mean: ") + ppml_hip_last_error());
    return Status::SUCCESS;
}

// src/backend/CUDAKernels.cpp:894-903 with the configuration of CPUKernels.cpp:1384-1398:
// src 0..2 = Q, K, V in the [d, L, h, B] layout, src 3 = bias or null, src 4 = LSE output or null;
// op_params: 0 scale (f32), 1 causal, 2 softmax eps (f32), 3 Br, 4 Bc.
Status HipBackend::kernel_flash_attn_ext(Tensor* node) {
    const Tensor* q = node->src[0];
    const Tensor* k = node->src[1];
    const Tensor* v = node->src[2];
    if (!q || !k || !v || !q->data || !k->data || !v->data || !node->data)
        return fail(Status::NOT_SUPPORTED, "flash_attn_ext: unbound tensor");
    // with the leading bridges fused away the sources are still [L, D, h, B]
    const int64_t d = (attn_layout_ & 1) ? q->dims[1] : q->dims[0], L = (attn_layout_ & 1) ? q->dims[0] : q->dims[1];
    const int64_t h = dim_or_1(q, 2), B = dim_or_1(q, 3);
    if (k->numel() != q->numel() || v->numel() != q->numel() || node->numel() != q->numel())
        return fail(Status::NOT_SUPPORTED, "flash_attn_ext: Q, K, V and O differ in size");
    const Tensor* bias = node->src[3];
    if (bias && (!bias->data || bias->numel() != B * h * L * L))
        return fail(Status::NOT_SUPPORTED, "flash_attn_ext: bias is not [L, L, h, B]");
    Tensor* lse = node->src[4];
    if (lse && lse->numel() != B * h * L) return fail(Status::NOT_SUPPORTED, "flash_attn_ext: LSE is not [L, h, B]");
    if (lse && !lse->data) return fail(Status::NOT_SUPPORTED, "flash_attn_ext: LSE buffer is unbound");
    const int rc = flash_attn_forward_ex_hip(static_cast<int>(B), static_cast<int>(h), static_cast<int>(L), static_cast<int>(d),
                                             node->op_params[1] != 0, node->param_f32(0), node->param_f32(2), node->op_params[4],
                                             static_cast<const float*>(q->data), static_cast<const float*>(k->data),
                                             static_cast<const float*>(v->data), bias ? static_cast<const float*>(bias->data) : nullptr,
                                             static_cast<float*>(node->data), lse ? static_cast<float*>(lse->data) : nullptr,
                                             attn_layout_, nullptr);
    if (rc != 0) return fail(status_of_rc(rc), std::string("flash_attn_ext: ") + ppml_hip_last_error());
    return Status::SUCCESS;
}

// src/backend/CUDAKernels.cpp:1344-1390: OP_PERMUTE and OP_TRANSPOSE both carry the axis map in
// op_params[0..ndim) (dimension p of the node is dimension op_params[p] of src[0]); a map with an entry
// outside the tensor's dimensions is refused.
Status HipBackend::kernel_permute(Tensor* node) {
    const Tensor* a = node->src[0];
    if (!a || !a->data || !node->data) return fail(Status::NOT_SUPPORTED, "permute: unbound tensor");
    const int ndim = a->ndim;
    if (ndim < 1 || ndim > 4 || node->numel() != a->numel()) return fail(Status::NOT_SUPPORTED, "permute: sizes differ");
    int32_t ax[4] = {0, 1, 2, 3};
    int64_t sd[4] = {1, 1, 1, 1}, dd[4] = {1, 1, 1, 1};
    for (int i = 0; i < ndim; ++i) {
        ax[i] = node->op_params[i];
        if (ax[i] < 0 || ax[i] >= ndim) return fail(Status::NOT_SUPPORTED, "permute: axis map outside the tensor's dimensions");
        sd[i] = a->dims[i];
        dd[i] = node->dims[i];
    }
    const int rc = permute_hip(static_cast<const float*>(a->data), static_cast<float*>(node->data), node->numel(), ndim,
                               ax[0], ax[1], ax[2], ax[3], sd[0], sd[1], sd[2], sd[3], dd[0], dd[1], dd[2], dd[3], nullptr);
    if (rc != 0) return fail(status_of_rc(rc), std::string("permute: ") + ppml_hip_last_error());
    return Status::SUCCESS;
}

// src/backend/CUDAKernels.cpp:1146-1170: the node is [D, I, J, B]; op_params[0] holds L as a float,
// the low byte of op_params[4] the outgoing flag (ComputeGraphHelper.cpp:409-411); the contracted length
// is left.dims[2] (outgoing) or left.dims[1] (incoming); L == 0 is refused.
Status HipBackend::kernel_tri_mul(Tensor* node) {
    const Tensor* l = node->src[0];
    const Tensor* r = node->src[1];
    if (!l || !r || !l->data || !r->data || !node->data) return fail(Status::NOT_SUPPORTED, "tri_mul: unbound tensor");
    const float L = node->param_f32(0);
    const bool outgoing = (node->op_params[4] & 0xff) != 0;
    if (L == 0.0f) return fail(Status::NOT_SUPPORTED, "tri_mul: L is zero");
    const int64_t D = node->dims[0], I = node->dims[1], J = node->dims[2], B = node->dims[3];
    const int64_t K = outgoing ? l->dims[2] : l->dims[1];
    if (l->numel() != D * I * K * B || r->numel() != D * J * K * B)
        return fail(Status::NOT_SUPPORTED, "tri_mul: operand sizes do not match [D,I,J,B] and the contracted length");
    const int rc = tri_mul_hip(static_cast<const float*>(l->data), static_cast<const float*>(r->data),
                               static_cast<float*>(node->data), D, I, J, K, B, 1.0f / L, outgoing ? 1 : 0, nullptr);
    if (rc != 0) return fail(status_of_rc(rc), std::string("tri_mul: ") + ppml_hip_last_error());
    return Status::SUCCESS;
}

// src/backend/CUDAKernels.cpp:1172-1201: src 0 grad [D,I,J,B], 1 left, 2 right, 3 gradient of left (or null),
// 4 gradient of right (or null); L and the outgoing flag as in the forward node.
Status HipBackend::kernel_tri_mul_back(Tensor* node) {
    const Tensor* g = node->src[0];
    const Tensor* l = node->src[1];
    const Tensor* r = node->src[2];
    Tensor* gl = node->src[3];
    Tensor* gr = node->src[4];
    if (!g || !l || !r || !g->data || !l->data || !r->data || (!gl && !gr) || (gl && !gl->data) || (gr && !gr->data))
        return fail(Status::NOT_SUPPORTED, "tri_mul_back: unbound tensor");
    const float L = node->param_f32(0);
    const bool outgoing = (node->op_params[4] & 0xff) != 0;
    if (L == 0.0f) return fail(Status::NOT_SUPPORTED, "tri_mul_back: L is zero");
    const int64_t D = l->dims[0], B = l->dims[3];
    const int64_t I = outgoing ? l->dims[1] : l->dims[2], J = outgoing ? r->dims[1] : r->dims[2];
    const int64_t K = outgoing ? l->dims[2] : l->dims[1];
    if (g->numel() != D * I * J * B || r->numel() != D * J * K * B || (gl && gl->numel() != l->numel()) || (gr && gr->numel() != r->numel()))
        return fail(Status::NOT_SUPPORTED, "tri_mul_back: tensor sizes do not match each other");
    const int rc = tri_mul_back_hip(static_cast<const float*>(g->data), static_cast<const float*>(l->data),
                                    static_cast<const float*>(r->data), gl ? static_cast<float*>(gl->data) : nullptr,
                                    gr ? static_cast<float*>(gr->data) : nullptr, D, I, J, K, B, 1.0f / L, outgoing ? 1 : 0, nullptr);
    if (rc != 0) return fail(status_of_rc(rc), std::string("tri_mul_back: ") + ppml_hip_last_error());
    return Status::SUCCESS;
}

// src/backend/CUDAKernels.cpp:1223-1245: src 0 grad [D*D,L,L,B], 1 left, 2 right [D,L,N,B], 3 / 4 the gradients
Status HipBackend::kernel_outer_prod_mean_back(Tensor* node) {
    const Tensor* g = node->src[0];
    const Tensor* l = node->src[1];
    const Tensor* r = node->src[2];
    Tensor* gl = node->src[3];
    Tensor* gr = node->src[4];
    if (!g || !l || !r || !g->data || !l->data || !r->data || (!gl && !gr) || (gl && !gl->data) || (gr && !gr->data))
        return fail(Status::NOT_SUPPORTED, "outer_prod_mean_back: unbound tensor");
    const int64_t D = l->dims[0], L = l->dims[1], N = l->dims[2], B = l->dims[3];
    if (N <= 0) return fail(Status::NOT_SUPPORTED, "outer_prod_mean_back: N must be positive");
    if (g->numel() != D * D * L * L * B || r->numel() != l->numel() || (gl && gl->numel() != l->numel()) || (gr && gr->numel() != l->numel()))
        return fail(Status::NOT_SUPPORTED, "outer_prod_mean_back: tensor sizes do not match each other");
    const int rc = outer_prod_mean_back_hip(static_cast<const float*>(g->data), static_cast<const float*>(l->data),
                                            static_cast<const float*>(r->data), gl ? static_cast<float*>(gl->data) : nullptr,
                                            gr ? static_cast<float*>(gr->data) : nullptr, D, L, N, B, 1.0f / static_cast<float>(N), nullptr);
    if (rc != 0) return fail(status_of_rc(rc), std::string("outer_prod_mean_back: ") + ppml_hip_last_error());
    return Status::SUCCESS;
}

// src/backend/CUDAKernels.cpp:905-924: src 0..2 Q, K, V ([d, L, h, B]), 3 bias or null, 4 O, 5 dO, 6 LSE,
// 7..9 dQ, dK, dV (each may be null); the node itself receives dbias when op_params[5] != 0.
Status HipBackend::kernel_flash_attn_back(Tensor* node) {
    const Tensor* q = node->src[0];
    const Tensor* k = node->src[1];
    const Tensor* v = node->src[2];
    const Tensor* bias = node->src[3];
    const Tensor* o = node->src[4];
    const Tensor* dout = node->src[5];
    const Tensor* lse = node->src[6];
    Tensor* dq = node->src[7];
    Tensor* dk = node->src[8];
    Tensor* dv = node->src[9];
    if (!q || !k || !v || !o || !dout || !lse || !q->data || !k->data || !v->data || !o->data || !dout->data || !lse->data)
        return fail(Status::NOT_SUPPORTED, "flash_attn_back: unbound tensor");
    const bool want_dbias = node->op_params[5] != 0;
    if ((dq && !dq->data) || (dk && !dk->data) || (dv && !dv->data) || (want_dbias && !node->data) || (bias && !bias->data))
        return fail(Status::NOT_SUPPORTED, "flash_attn_back: unbound output");
    const int64_t d = q->dims[0], L = q->dims[1], h = dim_or_1(q, 2), B = dim_or_1(q, 3);
    const int64_t n = q->numel();
    if (k->numel() != n || v->numel() != n || o->numel() != n || dout->numel() != n || lse->numel() != B * h * L ||
        (dq && dq->numel() != n) || (dk && dk->numel() != n) || (dv && dv->numel() != n) ||
        (bias && bias->numel() != B * h * L * L) || (want_dbias && node->numel() != B * h * L * L))
        return fail(Status::NOT_SUPPORTED, "flash_attn_back: tensor sizes do not match each other");
    const auto f = [](const Tensor* t) { return t ? static_cast<float*>(t->data) : nullptr; };
    const int rc = flash_attn_backward_hip(static_cast<int>(B), static_cast<int>(h), static_cast<int>(L), static_cast<int>(d),
                                           node->op_params[1] != 0, node->param_f32(0), f(q), f(k), f(v), f(bias), f(o), f(dout), f(lse),
                                           f(dq), f(dk), f(dv), want_dbias ? static_cast<float*>(node->data) : nullptr, nullptr);
    if (rc != 0) return fail(status_of_rc(rc), std::string("flash_attn_back: ") + ppml_hip_last_error());
    return Status::SUCCESS;
}

// src/backend/CUDAKernels.cpp:1290-1320 (kernel_repeat_back_cross_cuda): dimension d of the node meets
// dimension d of src[0] (only a node of higher rank is right-aligned), copies = integer quotient of the sizes.
Status HipBackend::kernel_repeat_back(Tensor* node) {
    const Tensor* a = node->src[0];
    if (!a || !a->data || !node->data) return fail(Status::NOT_SUPPORTED, "repeat_back: unbound tensor");
    const int off = a->ndim >= node->ndim ? 0 : a->ndim - node->ndim;
    int64_t sd[4] = {1, 1, 1, 1}, dd[4] = {1, 1, 1, 1}, rd[4] = {1, 1, 1, 1};
    for (int d = 0; d < node->ndim && d < 4; ++d) dd[d] = node->dims[d];
    for (int d = 0; d < a->ndim && d < 4; ++d) sd[d] = a->dims[d];
    for (int d = 0; d < 4; ++d) {
        const int si = d + off;
        const int64_t sdim = (si >= 0 && si < 4) ? sd[si] : 1;
        rd[d] = dd[d] > 0 ? sdim / dd[d] : 1;
    }
    const int rc = repeat_back_hip(static_cast<const float*>(a->data), static_cast<float*>(node->data),
                                   sd[0], sd[1], sd[2], sd[3], dd[0], dd[1], dd[2], dd[3], rd[0], rd[1], rd[2], rd[3], nullptr);
    if (rc != 0) return fail(status_of_rc(rc), std::string("repeat_back: ") + ppml_hip_last_error());
    return Status::SUCCESS;
}

// src/backend/CUDAKernels.cpp:992-1004: dst = src * s, s the float in op_params[0]
Status HipBackend::kernel_scale(Tensor* node) {
    const Tensor* a = node->src[0];
    if (!a || !a->data || !node->data) return fail(Status::NOT_SUPPORTED, "scale: unbound tensor");
    if (a->numel() != node->numel()) return fail(Status::NOT_SUPPORTED, "scale: source and result differ in size");
    const int rc = scale_hip(static_cast<const float*>(a->data), static_cast<float*>(node->data), node->param_f32(0), node->numel(), nullptr);
    if (rc != 0) return fail(status_of_rc(rc), std::string("scale: ") + ppml_hip_last_error());
    return Status::SUCCESS;
}

// src/backend/CUDAKernels.cpp:666-672: the sub-type rides in op_params[0]
Status HipBackend::kernel_unary(Tensor* node) {
    const Tensor* a = node->src[0];
    if (!a || !a->data || !node->data) return fail(Status::NOT_SUPPORTED, "unary: unbound tensor");
    if (a->numel() != node->numel()) return fail(Status::NOT_SUPPORTED, "unary: source and result differ in size");
    const int rc = unary_hip(static_cast<const float*>(a->data), static_cast<float*>(node->data), node->numel(), node->op_params[0], nullptr);
    if (rc != 0) return fail(status_of_rc(rc), std::string("unary: ") + ppml_hip_last_error());
    return Status::SUCCESS;
}

// src/backend/CUDAKernels.cpp:678-712: n, an, bn are the element counts of the node and of its two sources
Status HipBackend::kernel_elemwise(Tensor* node) {
    const Tensor* a = node->src[0];
    const Tensor* b = node->src[1];
    if (!a || !b || !a->data || !b->data || !node->data) return fail(Status::NOT_SUPPORTED, "elemwise: unbound tensor");
    const int eop = node->op == OP_ADD ? 0 : node->op == OP_SUB ? 1 : node->op == OP_MUL ? 2 : 3;
    const int rc = bcast_elemwise_hip(static_cast<const float*>(a->data), static_cast<const float*>(b->data),
                                      static_cast<float*>(node->data), node->numel(), a->numel(), b->numel(), eop, nullptr);
    if (rc != 0) return fail(status_of_rc(rc), std::string("elemwise: ") + ppml_hip_last_error());
    return Status::SUCCESS;
}

// src/backend/CUDAKernels.cpp:849-857: rows of dims[0] values
Status HipBackend::kernel_soft_max(Tensor* node) {
    const Tensor* a = node->src[0];
    if (!a || !a->data || !node->data) return fail(Status::NOT_SUPPORTED, "soft_max: unbound tensor");
    const int64_t N = node->dims[0], M = N > 0 ? node->numel() / N : 0;
    if (a->numel() != node->numel() || N <= 0 || N > 0x7fffffffLL || M > 0x7fffffffLL)
        return fail(Status::NOT_SUPPORTED, "soft_max: sizes outside what one launch takes");
    int rc;
    if (soft_max_bias_) {
        const Tensor* bias = soft_max_bias_;
        if (!bias->data || bias->numel() <= 0 || bias->numel() % N != 0 || M % (bias->numel() / N) != 0)
            return fail(Status::NOT_SUPPORTED, "soft_max: the folded bias is not whole rows of the softmax");
        rc = softmax_add_hip(static_cast<const float*>(a->data), static_cast<const float*>(bias->data), static_cast<float*>(node->data),
                             static_cast<int>(M), static_cast<int>(N), static_cast<int>(bias->numel() / N), nullptr);
    } else {
        rc = softmax_hip(static_cast<const float*>(a->data), static_cast<float*>(node->data), static_cast<int>(M), static_cast<int>(N), nullptr);
    }
    if (rc != 0) return fail(status_of_rc(rc), std::string("soft_max: ") + ppml_hip_last_error());
    return Status::SUCCESS;
}

Status HipBackend::dispatch_node(Tensor* node) {
    switch (node->op) {
        case OP_MUL_MAT: return kernel_mul_mat(node);
        case OP_OUT_PROD: return kernel_out_prod(node);
        case OP_OUTER_PROD_MEAN: return kernel_outer_prod_mean(node);
        case OP_FLASH_ATTN_EXT: return kernel_flash_attn_ext(node);
        case OP_FLASH_ATTN_BACK: return kernel_flash_attn_back(node);
        case OP_PERMUTE:
        case OP_TRANSPOSE: return kernel_permute(node);
        case OP_REPEAT_BACK: return kernel_repeat_back(node);
        case OP_TRI_MUL: return kernel_tri_mul(node);
        case OP_TRI_MUL_BACK: return kernel_tri_mul_back(node);
        case OP_OUTER_PROD_MEAN_BACK: return kernel_outer_prod_mean_back(node);
        case OP_SCALE: return kernel_scale(node);
        case OP_UNARY: return kernel_unary(node);
        case OP_ADD:
        case OP_SUB:
        case OP_MUL:
        case OP_DIV: return kernel_elemwise(node);
        case OP_SOFT_MAX: return kernel_soft_max(node);
        default: return fail(Status::NOT_SUPPORTED, "no kernel for op " + std::to_string(node->op));
    }
}

Status HipBackend::graph_compute(ComputeGraph* graph) {
    if (!graph) return fail(Status::NOT_SUPPORTED, "null graph");
    if (hipSetDevice(device_) != hipSuccess) {
        (void)hipGetLastError();
        return fail(Status::ABORTED, "cannot select device " + std::to_string(device_));
    }
    error_.clear();

    // ---- fusion plan.  Legality is the reference's own rule for eliminating an intermediate: exactly one reader
    // in this graph (include/ppml/ComputeGraph.h:73-87), and here also no TENSOR_FLAG_OUTPUT.  A tensor fused away
    // is never written.
    struct Plan {
        bool bridges_in = false;            // fused attention node: the three leading {1,0,2,3} permutations are skipped
        Tensor* bridge_out = nullptr;       // ... and this trailing one, whose storage the node writes
        int relu_slot = -1;                 // quantized mul_mat: activation slot whose chain ends in a skipped ReLU
        Tensor* relu = nullptr;
        Tensor* out_prod = nullptr;         // OP_SCALE node that runs as the (skipped) out_prod it reads, scaled
        Tensor* added = nullptr;            // OP_SOFT_MAX node that adds the second operand of this (skipped) OP_ADD on its way in
        bool transposed = false;            // OP_OUT_PROD / OP_MUL_MAT that reads the sources of its two (skipped) {1,0,2,3} permutations
        bool chain = false;                 // out_prod(attn_t, V_t) that runs as the whole attention chain
        Tensor *q = nullptr, *k = nullptr, *v = nullptr, *bias = nullptr;
        float scale = 1.0f;
    };
    std::unordered_map<const Tensor*, Plan> plans;
    std::unordered_set<const Tensor*> skipped;
    nodes_fused_away_ = 0;
    if (fuse_attention_bridges_ || fuse_relu_into_q8_ || fuse_scale_into_out_prod_ || fuse_attention_chain_ ||
        fuse_add_into_soft_max_ || fuse_permutes_into_out_prod_ || fuse_permutes_into_mul_mat_) {
        std::unordered_map<const Tensor*, int> uses, position;
        std::unordered_map<const Tensor*, Tensor*> single_user;
        int pos = 0;
        for (Tensor* n : *graph) {
            if (!n) continue;
            position[n] = pos++;
            bool view_counted = false;
            for (Tensor* s : n->src) if (s) { ++uses[s]; single_user[s] = n; view_counted = view_counted || s == n->view_src; }
            if (n->view_src && !view_counted) { ++uses[n->view_src]; single_user[n->view_src] = n; }
        }
        const auto before = [&](const Tensor* a, const Tensor* b) {
            const auto ia = position.find(a), ib = position.find(b);
            return ia != position.end() && ib != position.end() && ia->second < ib->second;
        };
        // an intermediate this graph computes that only `reader` reads and nobody outside is promised
        const auto private_to = [&](const Tensor* t, const Tensor* reader) {
            return t && !(t->flag & TENSOR_FLAG_OUTPUT) && !t->view_src && t->type == TENSOR_TYPE_F32 && uses[t] == 1 &&
                   before(t, reader) && !skipped.count(t);
        };
        const auto is_bridge = [](const Tensor* t) {
            if (!t || (t->op != OP_PERMUTE && t->op != OP_TRANSPOSE) || t->ndim != 4 || t->type != TENSOR_TYPE_F32) return false;
            return t->op_params[0] == 1 && t->op_params[1] == 0 && t->op_params[2] == 2 && t->op_params[3] == 3 &&
                   t->src[0] && t->src[0]->type == TENSOR_TYPE_F32 && t->src[0]->ndim == 4 && !t->view_src;
        };

        // (1) the layout bridges around fused attention nodes (ComputeGraphHelper.cpp:456-458, 483): a permutation
        // {1,0,2,3} that feeds only the attention node, or is the only reader of its result, is not executed; the
        // attention kernel reads / writes that layout itself.  All three inputs fuse together or not at all.
        if (fuse_attention_bridges_) {
            for (Tensor* n : *graph) {
                if (!n || n->op != OP_FLASH_ATTN_EXT || !node_supported(n)) continue;
                Plan b;
                b.bridges_in = true;
                for (int s = 0; s < 3; ++s) {
                    const Tensor* pq = n->src[s];
                    b.bridges_in = b.bridges_in && is_bridge(pq) && uses[pq] == 1 && before(pq, n);
                }
                // a tensor that feeds two of the three slots (self-attention on one projection) has uses == 2: not fused
                Tensor* user = uses[n] == 1 ? single_user[n] : nullptr;
                if (user && is_bridge(user) && user->src[0] == n && before(n, user)) b.bridge_out = user;
                if (!b.bridges_in && !b.bridge_out) continue;
                plans[n] = b;
                if (b.bridges_in) for (int s = 0; s < 3; ++s) skipped.insert(n->src[s]);
                if (b.bridge_out) skipped.insert(b.bridge_out);
            }
        }

        // (2) the reference's default attention chain (src/modules/Attention.cpp:264-281) as one fused launch
        if (fuse_attention_chain_) {
            for (Tensor* n : *graph) {
                if (!n || n->op != OP_OUT_PROD || n->type != TENSOR_TYPE_F32 || n->ndim != 4) continue;
                Tensor* attn_t = n->src[0];
                Tensor* v_t = n->src[1];
                if (!is_bridge(attn_t) || !is_bridge(v_t) || !private_to(attn_t, n) || !private_to(v_t, n)) continue;
                Tensor* attn = attn_t->src[0];
                if (!attn || attn->op != OP_SOFT_MAX || !private_to(attn, attn_t)) continue;
                Tensor* x = attn->src[0];
                Tensor* bias = nullptr;
                Tensor* added = nullptr;
                if (x && x->op == OP_ADD) {
                    if (!private_to(x, attn) || !x->src[0] || !x->src[1] || x->src[1]->numel() != x->numel() ||
                        x->src[1]->type != TENSOR_TYPE_F32) continue;
                    added = x;
                    bias = x->src[1];
                    x = x->src[0];
                }
                if (!x || x->op != OP_SCALE || !private_to(x, added ? added : attn)) continue;
                Tensor* scores = x->src[0];
                if (!scores || scores->op != OP_OUT_PROD || !private_to(scores, x)) continue;
                Tensor* k = scores->src[0];
                Tensor* q = scores->src[1];
                Tensor* v = v_t->src[0];
                const auto plain4 = [](const Tensor* t) { return t && t->type == TENSOR_TYPE_F32 && t->ndim == 4; };
                if (!plain4(k) || !plain4(q) || !plain4(v)) continue;
                const int64_t L = q->dims[0], D = q->dims[1];
                bool same = true;
                for (int d = 0; d < 4; ++d) same = same && k->dims[d] == q->dims[d] && v->dims[d] == q->dims[d];
                if (!same || D <= 0 || D > 64 || (D % 4) != 0) continue;           // the fused kernel's own range
                if (n->numel() != q->numel() || scores->numel() != L * L * q->dims[2] * q->dims[3]) continue;
                Plan c;
                c.chain = true;
                c.q = q; c.k = k; c.v = v; c.bias = bias;
                c.scale = x->param_f32(0);
                plans[n] = c;
                for (const Tensor* t : {static_cast<const Tensor*>(attn_t), static_cast<const Tensor*>(v_t),
                                        static_cast<const Tensor*>(attn), static_cast<const Tensor*>(added),
                                        static_cast<const Tensor*>(x), static_cast<const Tensor*>(scores)})
                    if (t) skipped.insert(t);
            }
        }

        // (3) ReLU in front of a quantized matmul (src/modules/Attention.cpp:1097-1104; in evaluation the dropout
        // between them is the identity, src/ops/Dropout.cpp:87-91): the matmul's quantizer applies it
        if (fuse_relu_into_q8_) {
            for (Tensor* n : *graph) {
                if (!n || n->op != OP_MUL_MAT || !node_supported(n) || !n->src[0] || !n->src[1]) continue;
                const bool q0 = is_quantized_type(n->src[0]->type), q1 = is_quantized_type(n->src[1]->type);
                if (q0 == q1) continue;
                const int slot = q0 ? 1 : 0;
                const Tensor* reader = n;
                Tensor* t = n->src[slot];
                // through whole views: same element count, no offset, nobody else looking
                for (int guard = 0; guard < 16 && t && (t->op == OP_VIEW || t->op == OP_RESHAPE); ++guard) {
                    Tensor* from = t->view_src ? t->view_src : t->src[0];
                    if (!from || (t->flag & TENSOR_FLAG_OUTPUT) || uses[t] != 1 || t->view_offs != 0 || from->numel() != t->numel() ||
                        !before(t, reader)) { t = nullptr; break; }
                    reader = t;
                    t = from;
                }
                if (!t || t->op != OP_UNARY || t->op_params[0] != UNARY_OP_RELU || !private_to(t, reader)) continue;
                if (!t->src[0] || t->src[0]->type != TENSOR_TYPE_F32 || t->src[0]->numel() != t->numel()) continue;
                Plan& r = plans[n];
                r.relu_slot = slot;
                r.relu = t;
                skipped.insert(t);
            }
        }

        // (4) the 1/sqrt(D) behind the attention logits (src/modules/Attention.cpp:264-270)
        if (fuse_scale_into_out_prod_) {
            for (Tensor* n : *graph) {
                if (!n || n->op != OP_SCALE || skipped.count(n) || !node_supported(n)) continue;
                Tensor* p = n->src[0];
                if (!p || p->op != OP_OUT_PROD || !node_supported(p) || !private_to(p, n) || p->numel() != n->numel()) continue;
                plans[n].out_prod = p;
                skipped.insert(p);
            }
        }

        // (5) the bias add in front of the attention softmax (src/modules/Attention.cpp:271-276)
        if (fuse_add_into_soft_max_) {
            for (Tensor* n : *graph) {
                if (!n || n->op != OP_SOFT_MAX || skipped.count(n) || !node_supported(n)) continue;
                Tensor* x = n->src[0];
                if (!x || x->op != OP_ADD || !node_supported(x) || !private_to(x, n) || x->numel() != n->numel()) continue;
                const Tensor* full = x->src[0];
                const Tensor* bias = x->src[1];
                const int64_t row = n->dims[0];
                if (!full || !bias || full->type != TENSOR_TYPE_F32 || bias->type != TENSOR_TYPE_F32 || full->numel() != x->numel() ||
                    row <= 0 || bias->numel() <= 0 || bias->numel() % row != 0 || (x->numel() / row) % (bias->numel() / row) != 0) continue;
                plans[n].added = x;
                skipped.insert(x);
            }
        }

        // (6) the two permutation copies in front of the second contraction of the attention chain
        // (src/modules/Attention.cpp:277-281)
        if (fuse_permutes_into_out_prod_) {
            for (Tensor* n : *graph) {
                if (!n || n->op != OP_OUT_PROD || n->type != TENSOR_TYPE_F32 || n->ndim != 4 || skipped.count(n) || !node_supported(n)) continue;
                const auto planned = plans.find(n);
                if (planned != plans.end() && planned->second.chain) continue;
                Tensor* p0 = n->src[0];
                Tensor* p1 = n->src[1];
                if (p0 == p1 || !is_bridge(p0) || !is_bridge(p1) || !private_to(p0, n) || !private_to(p1, n)) continue;
                if (p0->src[0]->numel() != p0->numel() || p1->src[0]->numel() != p1->numel()) continue;
                plans[n].transposed = true;
                skipped.insert(p0);
                skipped.insert(p1);
            }
        }

        // (7) the two matrix transpositions in front of a LinearLayer's weight gradient,
        // mul_mat(mat_transpose(grad), mat_transpose(x)) (src/core/ComputeGraph.cpp:733-738; mat_transpose is a
        // permutation copy of dims[0] and dims[1], src/core/ComputeGraphHelper.cpp:375-382)
        if (fuse_permutes_into_mul_mat_) {
            const auto is_mat_t = [](const Tensor* t) {
                if (!t || (t->op != OP_PERMUTE && t->op != OP_TRANSPOSE) || t->ndim < 2 || t->type != TENSOR_TYPE_F32 || t->view_src) return false;
                const Tensor* s = t->src[0];
                if (!s || s->type != TENSOR_TYPE_F32 || s->ndim != t->ndim || s->numel() != t->numel()) return false;
                for (int d = 2; d < t->ndim; ++d) if (t->op_params[d] != d || t->dims[d] != 1) return false;       // one matrix
                return t->op_params[0] == 1 && t->op_params[1] == 0 && s->dims[0] == t->dims[1] && s->dims[1] == t->dims[0];
            };
            for (Tensor* n : *graph) {
                if (!n || n->op != OP_MUL_MAT || n->type != TENSOR_TYPE_F32 || n->src[2] || skipped.count(n) || !node_supported(n)) continue;
                Tensor* p0 = n->src[0];
                Tensor* p1 = n->src[1];
                if (p0 == p1 || !is_mat_t(p0) || !is_mat_t(p1) || !private_to(p0, n) || !private_to(p1, n)) continue;
                plans[n].transposed = true;
                skipped.insert(p0);
                skipped.insert(p1);
            }
        }
        nodes_fused_away_ = skipped.size();
    }

    // the arithmetic this backend's f32 contractions were configured with, for the length of this call
    struct ArithmeticScope {
        int before = -1;
        explicit ArithmeticScope(int mode) { if (mode == 0 || mode == 1) before = ppml_hip_set_f32_arithmetic(mode); }
        ~ArithmeticScope() { if (before >= 0) ppml_hip_set_f32_arithmetic(before); }
    } arithmetic(f32_arithmetic_);

    HostShadows shadows;                                // restored and freed on every way out of this function
    host_shadows_made_ = 0;
    int index = -1;
    for (Tensor* node : *graph) {
        ++index;
        if (!node) return fail(Status::NOT_SUPPORTED, "null node " + std::to_string(index));
        if (node->op == OP_NONE || node->op == OP_VIEW || node->op == OP_RESHAPE) continue;
        if (skipped.count(node)) continue;

        // no other backend to fall back to: an unsupported node ends the graph instead of being skipped
        if (!supports_op(node))
            return fail(Status::NOT_SUPPORTED, "op " + std::to_string(node->op) + " (node " + std::to_string(index) + ") is not supported");

        // the node as it is executed: a copy with other sources / storage where the plan folded neighbours into it
        Tensor rewired;
        Tensor alias;                                   // a folded ReLU's input, seen through the matmul's own view of it
        Tensor* exec = node;
        Tensor* storage = node;
        attn_layout_ = 0;
        relu_in_quantizer_ = false;
        out_prod_scaled_ = false;
        out_prod_transposed_ = false;
        mul_mat_transposed_ = false;
        soft_max_bias_ = nullptr;
        const auto plan = plans.find(node);
        if (plan != plans.end()) {
            const Plan& pl = plan->second;
            rewired = *node;
            exec = &rewired;
            if (pl.bridges_in) {
                for (int s = 0; s < 3; ++s) rewired.src[s] = node->src[s]->src[0];
                attn_layout_ |= 1;
            }
            if (pl.bridge_out) {
                storage = pl.bridge_out;
                attn_layout_ |= 2;
            }
            if (pl.relu) {
                resolve_views(pl.relu);                 // binds the ReLU's own source if it is a view
                Tensor* in = pl.relu->src[0];
                if (!skip_alloc_) shadows.cover(in);
                alias = *node->src[pl.relu_slot];
                alias.op = OP_NONE;
                alias.view_src = nullptr;
                alias.view_offs = 0;
                alias.src[0] = nullptr;
                alias.data = in->data;
                alias.buffer = in->buffer;
                alias.buffer_offs = in->buffer_offs;
                rewired.src[pl.relu_slot] = &alias;
                relu_in_quantizer_ = true;
            }
            if (pl.out_prod) {
                rewired.op = OP_OUT_PROD;
                for (int s = 0; s < 10; ++s) rewired.src[s] = pl.out_prod->src[s];
                out_prod_scaled_ = true;
                out_prod_alpha_ = node->param_f32(0);
            }
            if (pl.added) {
                resolve_views(pl.added);                // binds the add's own sources if they are views
                rewired.src[0] = pl.added->src[0];
                rewired.src[1] = pl.added->src[1];      // (covered and checked with the other sources below)
                soft_max_bias_ = pl.added->src[1];
            }
            if (pl.transposed) {
                rewired.src[0] = node->src[0]->src[0];
                rewired.src[1] = node->src[1]->src[0];
                if (node->op == OP_MUL_MAT) mul_mat_transposed_ = true;
                else out_prod_transposed_ = true;
            }
            if (pl.chain) {
                // src/core/ComputeGraphHelper.cpp:450-484: Q, K, V, bias in src 0..3; scale, causal, eps, Br, Bc
                rewired.op = OP_FLASH_ATTN_EXT;
                for (int s = 0; s < 10; ++s) rewired.src[s] = nullptr;
                rewired.src[0] = pl.q; rewired.src[1] = pl.k; rewired.src[2] = pl.v; rewired.src[3] = pl.bias;
                for (int32_t& w : rewired.op_params) w = 0;
                rewired.set_param_f32(0, pl.scale);
                rewired.set_param_f32(2, 1e-9f);        // kernel_softmax's 1 / (sum + 1e-9), CPUKernels.cpp:1463
                rewired.op_params[4] = 64;
                attn_layout_ = 3;                       // inputs [L, D, h, B] as they are, result [L, D, h, B]
            }
        }
        resolve_views(exec);
        if (!skip_alloc_) {
            // under a scheduler the copies across backends are nodes of the graph; here nobody else makes them
            for (Tensor* src : exec->src) shadows.cover(src);
            host_shadows_made_ = shadows.count();
        }

        // single-backend mode: outputs nobody allocated get their own device buffer -- the node itself
        // and the second output the fused attention node carries in src[4] (its LSE buffer)
        // (the backward nodes of the triangle multiplication and of outer-product-mean carry both of their
        // outputs in src[3] and src[4]; the attention backward carries dQ, dK, dV in src[7..9] and uses its own
        // storage for dbias only when op_params[5] asks for it)
        const bool two_outputs = node->op == OP_TRI_MUL_BACK || node->op == OP_OUTER_PROD_MEAN_BACK;
        const bool attn_back = node->op == OP_FLASH_ATTN_BACK;
        Tensor* outputs[5] = {attn_back && node->op_params[5] == 0 ? nullptr : storage,
                              node->op == OP_FLASH_ATTN_EXT || two_outputs ? node->src[4] : nullptr,
                              two_outputs ? node->src[3] : nullptr, nullptr, nullptr};
        if (attn_back) { outputs[1] = node->src[7]; outputs[2] = node->src[8]; outputs[3] = node->src[9]; }
        for (Tensor* out : outputs) {
            if (!out || skip_alloc_ || out->data) continue;
            const size_t need = out->nbytes();
            auto buf = std::make_unique<Buffer>(buffer_type(), need);
            if (!buf->data()) return fail(Status::ALLOC_FAILED, "cannot allocate " + std::to_string(need) + " bytes for node " + std::to_string(index));
            out->data = buf->data();
            out->buffer = buf.get();
            out->buffer_offs = 0;
            owned_.push_back(std::move(buf));
        }
        if (exec != node) {                             // the copy was taken before its storage was settled
            rewired.data = storage->data;
            rewired.buffer = storage->buffer;
            rewired.buffer_offs = storage->buffer_offs;
        }

        if (!(attn_back && node->op_params[5] == 0) && !device_pointer_ok(exec))
            return fail(Status::NOT_SUPPORTED, "node " + std::to_string(index) + ": output is not device memory inside its buffer");
        for (int j = 0; j < 10; ++j) {
            if (exec->src[j] && !device_pointer_ok(exec->src[j]))
                return fail(Status::NOT_SUPPORTED, "node " + std::to_string(index) + ": src" + std::to_string(j) +
                                                    " is not device memory inside its buffer");
        }

        const Status st = dispatch_node(exec);
        attn_layout_ = 0;
        relu_in_quantizer_ = false;
        out_prod_scaled_ = false;
        out_prod_transposed_ = false;
        mul_mat_transposed_ = false;
        soft_max_bias_ = nullptr;
        if (st != Status::SUCCESS) return st;
        const hipError_t e = hipGetLastError();
        if (e != hipSuccess)
            return fail(Status::ABORTED, "launch failed at op " + std::to_string(node->op) + " (node " +
                                         std::to_string(index) + "): " + hipGetErrorString(e));
    }
    return Status::SUCCESS;
}

Status HipBackend::pack_weight(Tensor* w) {
    if (!w || !w->data) return fail(Status::NOT_SUPPORTED, "pack_weight: unbound tensor");
    if (w->type == TENSOR_TYPE_Q8_0M) return Status::SUCCESS;
    if (!is_quantized_type(w->type) || !w->quant_shape_valid())
        return fail(Status::NOT_SUPPORTED, "pack_weight: not a Q8 weight with K a multiple of 32");
    if (hipSetDevice(device_) != hipSuccess) return fail(Status::ABORTED, "cannot select device");
    const int64_t K = w->dims[0], M = w->numel() / K;
    const int wtype = w->type == TENSOR_TYPE_Q8_1 ? PPML_WTYPE_Q8_1 : w->type == TENSOR_TYPE_Q8_0R ? PPML_WTYPE_Q8_0R : PPML_WTYPE_Q8_0;
    const size_t need = q8_weight_packed_bytes_hip(static_cast<int>(M), static_cast<int>(K));
    auto buf = std::make_unique<Buffer>(buffer_type(), need);
    if (!buf->data()) return fail(Status::ALLOC_FAILED, "pack_weight: cannot allocate " + std::to_string(need) + " bytes");
    const int rc = q8_weight_pack_hip(w->data, wtype, static_cast<int>(M), static_cast<int>(K), buf->data(), nullptr);
    if (rc != 0) return fail(status_of_rc(rc), std::string("pack_weight: ") + ppml_hip_last_error());
    if (hipDeviceSynchronize() != hipSuccess) return fail(Status::ABORTED, "pack_weight: device error");
    w->data = buf->data();
    w->buffer = buf.get();
    w->buffer_offs = 0;
    w->type = TENSOR_TYPE_Q8_0M;
    owned_.push_back(std::move(buf));
    return Status::SUCCESS;
}

}  // namespace ppmlhip

// ------------------------------------------------------------------------------------------------
// C ABI of ppml_hip_backend.h
using namespace ppmlhip;

struct ppml_hip_backend {
    HipBackend impl;
    explicit ppml_hip_backend(int device) : impl(device) {}
};
struct ppml_hip_tensor {
    Tensor t;
    std::unique_ptr<Buffer> own;
};

extern "C" {

ppml_hip_backend* ppml_hip_backend_create(int device) {
    auto* b = new (std::nothrow) ppml_hip_backend(device);
    if (b && !b->impl.last_error().empty()) {   // no gfx950 device: the backend has no other path
        delete b;
        return nullptr;
    }
    return b;
}
void ppml_hip_backend_destroy(ppml_hip_backend* b) { delete b; }
const char* ppml_hip_backend_name(const ppml_hip_backend* b) { return b ? b->impl.get_name() : ""; }
const char* ppml_hip_backend_last_error(const ppml_hip_backend* b) { return b ? b->impl.last_error().c_str() : "null backend"; }
int ppml_hip_backend_priority(const ppml_hip_backend* b) { return b ? b->impl.priority() : 0; }
void ppml_hip_backend_synchronize(ppml_hip_backend* b) {
    if (b) b->impl.synchronize();
}

ppml_hip_tensor* ppml_hip_tensor_create(int op, int type, int ndim, const int64_t* dims) {
    if (ndim < 0 || ndim > 4 || (ndim > 0 && !dims)) return nullptr;
    auto* t = new (std::nothrow) ppml_hip_tensor();
    if (!t) return nullptr;
    t->t.op = op;
    t->t.type = type;
    t->t.ndim = ndim;
    for (int i = 0; i < ndim; ++i) t->t.dims[i] = dims[i];
    return t;
}
void ppml_hip_tensor_destroy(ppml_hip_tensor* t) { delete t; }
void ppml_hip_tensor_set_src(ppml_hip_tensor* t, int slot, ppml_hip_tensor* src) {
    if (t && slot >= 0 && slot < 10) t->t.src[slot] = src ? &src->t : nullptr;
}
void ppml_hip_tensor_set_data(ppml_hip_tensor* t, void* device_ptr) {
    if (!t) return;
    t->own.reset();
    t->t.data = device_ptr;
    t->t.buffer = nullptr;
    t->t.buffer_offs = 0;
}
void ppml_hip_tensor_set_view(ppml_hip_tensor* t, ppml_hip_tensor* view_src, size_t byte_offset) {
    if (!t) return;
    t->t.view_src = view_src ? &view_src->t : nullptr;
    t->t.view_offs = byte_offset;
}
void ppml_hip_tensor_set_param(ppml_hip_tensor* t, int index, float value) {
    if (t && index >= 0 && index < 16) t->t.set_param_f32(index, value);
}
void ppml_hip_tensor_set_param_i32(ppml_hip_tensor* t, int index, int value) {
    if (t && index >= 0 && index < 16) t->t.op_params[index] = value;
}
void ppml_hip_tensor_set_flag(ppml_hip_tensor* t, int flag) {
    if (t) t->t.flag = flag;
}
size_t ppml_hip_tensor_nbytes(const ppml_hip_tensor* t) { return t ? t->t.nbytes() : 0; }
int ppml_hip_tensor_type(const ppml_hip_tensor* t) { return t ? t->t.type : -1; }

int ppml_hip_tensor_upload(ppml_hip_backend* b, ppml_hip_tensor* t, const void* host, size_t nbytes) {
    if (!b || !t || !host) return static_cast<int>(Status::NOT_SUPPORTED);
    if (nbytes != t->t.nbytes()) return static_cast<int>(Status::NOT_SUPPORTED);
    if (!t->own || t->own->size() < nbytes) {
        t->own = std::make_unique<Buffer>(b->impl.buffer_type(), nbytes);
        if (!t->own->data()) {
            t->own.reset();
            return static_cast<int>(Status::ALLOC_FAILED);
        }
    }
    t->t.data = t->own->data();
    t->t.buffer = t->own.get();
    t->t.buffer_offs = 0;
    return t->own->set_tensor(&t->t, host, 0, nbytes) ? 0 : static_cast<int>(Status::ABORTED);
}
int ppml_hip_tensor_download(ppml_hip_backend* b, const ppml_hip_tensor* t, void* host, size_t nbytes) {
    if (!b || !t || !host || !t->t.data || nbytes > t->t.nbytes()) return static_cast<int>(Status::NOT_SUPPORTED);
    b->impl.synchronize();
    if (t->t.buffer) return t->t.buffer->get_tensor(&t->t, host, 0, nbytes) ? 0 : static_cast<int>(Status::ABORTED);
    return hipMemcpy(host, t->t.data, nbytes, hipMemcpyDeviceToHost) == hipSuccess ? 0 : static_cast<int>(Status::ABORTED);
}

int ppml_hip_backend_supports_op(const ppml_hip_backend* b, const ppml_hip_tensor* node) {
    (void)b;
    return node && node_supported(&node->t) ? 1 : 0;
}
int ppml_hip_backend_graph_compute(ppml_hip_backend* b, ppml_hip_tensor** nodes, int n) {
    if (!b || (n > 0 && !nodes)) return static_cast<int>(Status::NOT_SUPPORTED);
    ComputeGraph g;
    g.reserve(n);
    for (int i = 0; i < n; ++i) g.push_back(nodes[i] ? &nodes[i]->t : nullptr);
    return static_cast<int>(b->impl.graph_compute(&g));
}
int ppml_hip_backend_pack_weight(ppml_hip_backend* b, ppml_hip_tensor* weight) {
    if (!b || !weight) return static_cast<int>(Status::NOT_SUPPORTED);
    return static_cast<int>(b->impl.pack_weight(&weight->t));
}
void ppml_hip_backend_set_q8_1_activations(ppml_hip_backend* b, int on) {
    if (b) b->impl.set_q8_1_activations(on != 0);
}
void ppml_hip_backend_set_fuse_attention_bridges(ppml_hip_backend* b, int on) {
    if (b) b->impl.set_fuse_attention_bridges(on != 0);
}
void ppml_hip_backend_set_fuse_relu_into_q8(ppml_hip_backend* b, int on) {
    if (b) b->impl.set_fuse_relu_into_q8(on != 0);
}
void ppml_hip_backend_set_fuse_scale_into_out_prod(ppml_hip_backend* b, int on) {
    if (b) b->impl.set_fuse_scale_into_out_prod(on != 0);
}
void ppml_hip_backend_set_fuse_add_into_soft_max(ppml_hip_backend* b, int on) {
    if (b) b->impl.set_fuse_add_into_soft_max(on != 0);
}
void ppml_hip_backend_set_fuse_permutes_into_mul_mat(ppml_hip_backend* b, int on) {
    if (b) b->impl.set_fuse_permutes_into_mul_mat(on != 0);
}
void ppml_hip_backend_set_fuse_permutes_into_out_prod(ppml_hip_backend* b, int on) {
    if (b) b->impl.set_fuse_permutes_into_out_prod(on != 0);
}
void ppml_hip_backend_set_fuse_attention_chain(ppml_hip_backend* b, int on) {
    if (b) b->impl.set_fuse_attention_chain(on != 0);
}
int ppml_hip_backend_nodes_fused_away(const ppml_hip_backend* b) {
    return b ? static_cast<int>(b->impl.nodes_fused_away()) : 0;
}
void ppml_hip_backend_set_skip_alloc(ppml_hip_backend* b, int on) {
    if (b) b->impl.set_skip_alloc(on != 0);
}
void ppml_hip_backend_set_f32_arithmetic(ppml_hip_backend* b, int mode) {
    if (b) b->impl.set_f32_arithmetic(mode);
}
int ppml_hip_backend_host_shadows_made(const ppml_hip_backend* b) {
    return b ? static_cast<int>(b->impl.host_shadows_made()) : 0;
}

}  // extern "C"
