// Load-time side of the int8 path, host code only: the rule that picks the weights to quantize and the
// checkpoint file that carries them (declared in include/ppml_hip_weights.h).
//
// Reference behaviour restated here (paths relative to the reference tree):
//   src/model/PPML.cpp:4431-4456   ppml_int8_bigop_default_list, ppml_int8_bigop_selected
//   src/model/PPML.cpp:4481-4488   shape rule of quantize_big_weight_matrices
//   src/model/GGUF.cpp:31-74       FNV-1a layout fingerprint (its offset basis is 1469598103934665603,
//                                  one digit short of the usual FNV basis; files carry hashes made with it)
//   src/model/GGUF.cpp:134-191     layout: header 24 bytes, metadata, tensor infos, data from the next
//                                  multiple of 32, every tensor padded to 32; offsets are file offsets
//   src/model/GGUF.cpp:194-316     save_gguf      src/model/GGUF.cpp:318-470   load_gguf
// Beyond the reference (which writes F32 only and refuses quantized parameters, GGUF.cpp:203-213): a tensor of
// ggml type 8 (Q8_0) occupies numel / 32 blocks of 34 bytes.
#include "common.hpp"

#include <cstring>
#include <fstream>
#include <map>
#include <exception>
#include <memory>
#include <string>
#include <vector>

#include "../../include/ppml_hip_weights.h"

struct ppml_gguf_file {
    std::ifstream in;
    struct Info {
        std::string name;
        std::vector<uint64_t> dims;
        uint32_t type = 0;
        uint64_t offset = 0, nbytes = 0;
    };
    std::vector<Info> tensors;
    std::map<std::string, float> floats;
    std::map<std::string, std::string> strings;
    uint64_t file_size = 0;
};

namespace ppmlhip {
namespace {

constexpr uint32_t GGUF_MAGIC = 0x46554747u;           // "GGUF"
constexpr uint32_t GGUF_VERSION = 3;
constexpr uint64_t GGUF_ALIGN = 32;
constexpr uint64_t FNV_OFFSET_BASIS = 1469598103934665603ULL;   // the reference's constant (GGUF.cpp:34)
constexpr uint64_t FNV_PRIME = 1099511628211ULL;

enum ValueType : uint32_t { VT_UINT8 = 0, VT_INT8, VT_UINT16, VT_INT16, VT_UINT32, VT_INT32, VT_FLOAT32, VT_BOOL,
                            VT_STRING, VT_ARRAY, VT_UINT64, VT_INT64, VT_FLOAT64 };

uint64_t align_up(uint64_t n, uint64_t a) { return (n + a - 1) / a * a; }

struct Fnv {
    uint64_t h = FNV_OFFSET_BASIS;
    void byte(uint8_t b) { h ^= b; h *= FNV_PRIME; }
    void u32(uint32_t v) { for (int b = 0; b < 4; ++b) byte(static_cast<uint8_t>(v >> (8 * b))); }
    void u64(uint64_t v) { for (int b = 0; b < 8; ++b) byte(static_cast<uint8_t>(v >> (8 * b))); }
    void str(const std::string& s) { for (char c : s) byte(static_cast<uint8_t>(c)); }
};

std::string param_name(const char* const* names, size_t i) {
    if (names && names[i] && names[i][0]) return names[i];
    return "tensor_" + std::to_string(i);
}

uint64_t layout_hash(size_t n, const char* const* names, const uint32_t* ndims, const uint64_t* dims) {
    Fnv f;
    size_t at = 0;
    for (size_t i = 0; i < n; ++i) {
        f.str(param_name(names, i));
        f.u32(0xFF);                                   // keeps names from running into each other
        f.u32(ndims[i]);
        for (uint32_t d = 0; d < ndims[i]; ++d) f.u64(dims[at + d]);
        f.u32(0xFE);
        at += ndims[i];
    }
    return f.h;
}

std::string hex64(uint64_t v) {
    char buf[17];
    std::snprintf(buf, sizeof buf, "%016llx", static_cast<unsigned long long>(v));
    return buf;
}

// bytes of a tensor of `numel` elements, 0 if the type is unknown or the count does not fit whole blocks
uint64_t tensor_bytes(uint32_t type, uint64_t numel) {
    if (type == PPML_GGUF_TYPE_F32) return numel * 4;
    if (type == PPML_GGUF_TYPE_Q8_0) return numel % QK == 0 ? numel / QK * Q8_0_BYTES : 0;
    return 0;
}

struct Writer {
    std::ofstream& os;
    uint64_t pos = 0;
    void raw(const void* p, size_t n) { os.write(static_cast<const char*>(p), static_cast<std::streamsize>(n)); pos += n; }
    void u32(uint32_t v) { raw(&v, 4); }
    void u64(uint64_t v) { raw(&v, 8); }
    void f32(float v) { raw(&v, 4); }
    void str(const std::string& s) { u64(s.size()); raw(s.data(), s.size()); }
    void pad_to(uint64_t target) { static const char zeros[32] = {0}; while (pos < target) raw(zeros, static_cast<size_t>(target - pos < 32 ? target - pos : 32)); }
};

}  // namespace
}  // namespace ppmlhip

using namespace ppmlhip;

extern "C" const char* ppml_int8_bigop_default_list(void) {
    return "attention.msa_row.,attention.msa_col.,attention.pair_row.,attention.pair_col.,"
           "msa2pair_left_proj,msa2pair_right_proj,msa2pair_out_proj,pair2pair_gate_proj";
}

extern "C" int ppml_int8_bigop_selected(const char* name, const char* env_list) {
    if (!name || !env_list || env_list[0] == '\0') return 0;
    std::string list(env_list);
    if (list == "0" || list == "off") return 0;
    if (list == "1" || list == "on" || list == "all") list = ppml_int8_bigop_default_list();
    const std::string nm(name);
    size_t pos = 0;
    while (pos <= list.size()) {
        const size_t comma = list.find(',', pos);
        std::string tok = list.substr(pos, comma == std::string::npos ? std::string::npos : comma - pos);
        while (!tok.empty() && (tok.back() == ' ' || tok.back() == '\t')) tok.pop_back();
        while (!tok.empty() && (tok.front() == ' ' || tok.front() == '\t')) tok.erase(tok.begin());
        if (!tok.empty() && nm.find(tok) != std::string::npos) return 1;
        if (comma == std::string::npos) break;
        pos = comma + 1;
    }
    return 0;
}

extern "C" int ppml_int8_bigop_shape_ok(uint32_t ndim, const uint64_t* dims) {
    if (ndim != 2 || !dims) return 0;
    return dims[0] % QK == 0 && (dims[0] * dims[1]) % QK == 0 ? 1 : 0;
}

extern "C" uint64_t ppml_gguf_layout_hash(size_t n, const char* const* names, const uint32_t* ndims, const uint64_t* dims) {
    if (n > 0 && (!ndims || !dims)) return 0;
    return layout_hash(n, names, ndims, dims);
}

extern "C" int ppml_gguf_save(const char* path, const ppml_gguf_tensor* tensors, size_t n_params, size_t n_extra,
                              const char* const* float_keys, const float* float_values, size_t n_float,
                              const char* const* string_keys, const char* const* string_values, size_t n_string) {
    const size_t n_all = n_params + n_extra;
    if (!path || (n_all > 0 && !tensors) || (n_float > 0 && (!float_keys || !float_values)) ||
        (n_string > 0 && (!string_keys || !string_values))) {
        set_error("ppml_gguf_save: bad arguments");
        return RC_BAD_ARGS;
    }
    // names, sizes, fingerprint
    std::vector<std::string> names(n_all);
    std::vector<uint64_t> bytes(n_all);
    std::vector<uint32_t> ndims;
    std::vector<uint64_t> dims;
    for (size_t i = 0; i < n_all; ++i) {
        const ppml_gguf_tensor& t = tensors[i];
        if (t.ndim < 1 || t.ndim > 4 || !t.data) { set_error("ppml_gguf_save: tensor %zu has no data or %u dimensions", i, t.ndim); return RC_BAD_ARGS; }
        if (i >= n_params && (t.ndim != 1 || t.type != PPML_GGUF_TYPE_F32 || !t.name || !t.name[0])) {
            set_error("ppml_gguf_save: extra tensor %zu must be a named 1-D F32 tensor", i);
            return RC_BAD_ARGS;
        }
        uint64_t numel = 1;
        for (uint32_t d = 0; d < t.ndim; ++d) numel *= t.dims[d];
        bytes[i] = tensor_bytes(t.type, numel);
        if (bytes[i] == 0 || (t.type == PPML_GGUF_TYPE_Q8_0 && t.dims[0] % QK != 0)) {
            set_error("ppml_gguf_save: tensor %zu: type %u with %llu elements (innermost %llu) cannot be stored",
                      i, t.type, static_cast<unsigned long long>(numel), static_cast<unsigned long long>(t.dims[0]));
            return RC_BAD_ARGS;
        }
        if (i < n_params) {
            names[i] = (t.name && t.name[0]) ? std::string(t.name) : "tensor_" + std::to_string(i);
            ndims.push_back(t.ndim);
            for (uint32_t d = 0; d < t.ndim; ++d) dims.push_back(t.dims[d]);
        } else {
            names[i] = t.name;
        }
    }
    std::vector<const char*> hash_names(n_params);
    for (size_t i = 0; i < n_params; ++i) hash_names[i] = names[i].c_str();
    const std::string hash_hex = hex64(layout_hash(n_params, hash_names.data(), ndims.data(), dims.data()));

    std::vector<std::pair<std::string, std::string>> strings;
    strings.emplace_back("layout_hash", hash_hex);
    for (size_t i = 0; i < n_string; ++i) strings.emplace_back(string_keys[i] ? string_keys[i] : "", string_values[i] ? string_values[i] : "");

    // layout: sizes of the three front sections, then the data offsets
    uint64_t front = 4 + 4 + 8 + 8;
    for (size_t i = 0; i < n_float; ++i) front += 8 + std::strlen(float_keys[i] ? float_keys[i] : "") + 4 + 4;
    for (const auto& kv : strings) front += 8 + kv.first.size() + 4 + 8 + kv.second.size();
    for (size_t i = 0; i < n_all; ++i) front += 8 + names[i].size() + 4 + static_cast<uint64_t>(tensors[i].ndim) * 8 + 4 + 8;
    const uint64_t data_start = align_up(front, GGUF_ALIGN);
    std::vector<uint64_t> offsets(n_all);
    uint64_t cur = data_start;
    for (size_t i = 0; i < n_all; ++i) {
        offsets[i] = cur;
        cur = align_up(cur + bytes[i], GGUF_ALIGN);
    }

    std::ofstream ofs(path, std::ios::binary);
    if (!ofs) { set_error("ppml_gguf_save: cannot open %s", path); return RC_BAD_ARGS; }
    Writer w{ofs};
    w.u32(GGUF_MAGIC);
    w.u32(GGUF_VERSION);
    w.u64(n_all);
    w.u64(n_float + strings.size());
    for (size_t i = 0; i < n_float; ++i) {
        w.str(float_keys[i] ? float_keys[i] : "");
        w.u32(VT_FLOAT32);
        w.f32(float_values[i]);
    }
    for (const auto& kv : strings) {
        w.str(kv.first);
        w.u32(VT_STRING);
        w.str(kv.second);
    }
    for (size_t i = 0; i < n_all; ++i) {
        w.str(names[i]);
        w.u32(tensors[i].ndim);
        for (uint32_t d = 0; d < tensors[i].ndim; ++d) w.u64(tensors[i].dims[d]);
        w.u32(tensors[i].type);
        w.u64(offsets[i]);
    }
    w.pad_to(data_start);
    for (size_t i = 0; i < n_all; ++i) {
        w.raw(tensors[i].data, static_cast<size_t>(bytes[i]));
        w.pad_to(align_up(w.pos, GGUF_ALIGN));
    }
    ofs.close();
    if (!ofs) { set_error("ppml_gguf_save: writing %s failed", path); return RC_BAD_ARGS; }
    return RC_OK;
}

static ppml_gguf_file* gguf_open_checked(const char* path);

// No exception may leave an extern "C" function: a damaged file that asks for more memory than there is
// ends in a null handle and a message like every other refusal.
extern "C" ppml_gguf_file* ppml_gguf_open(const char* path) {
    try {
        return gguf_open_checked(path);
    } catch (const std::exception& e) {
        set_error("ppml_gguf_open: %s: %s", path ? path : "(null)", e.what());
        return nullptr;
    }
}

static ppml_gguf_file* gguf_open_checked(const char* path) {
    if (!path) { set_error("ppml_gguf_open: no path"); return nullptr; }
    std::unique_ptr<ppml_gguf_file> owner(new (std::nothrow) ppml_gguf_file);
    ppml_gguf_file* f = owner.get();                   // released to the caller on success only
    if (!f) { set_error("ppml_gguf_open: out of memory"); return nullptr; }
    const auto fail = [&](const char* why) -> ppml_gguf_file* {
        set_error("ppml_gguf_open: %s: %s", path, why);
        return nullptr;
    };
    f->in.open(path, std::ios::binary);
    if (!f->in) return fail("cannot open");
    f->in.seekg(0, std::ios::end);
    f->file_size = static_cast<uint64_t>(f->in.tellg());
    f->in.seekg(0, std::ios::beg);
    std::ifstream& in = f->in;
    const auto r32 = [&] { uint32_t v = 0; in.read(reinterpret_cast<char*>(&v), 4); return v; };
    const auto r64 = [&] { uint64_t v = 0; in.read(reinterpret_cast<char*>(&v), 8); return v; };
    bool bad_string = false;
    const auto rstr = [&] {
        const uint64_t len = r64();
        if (!in || len > f->file_size) { bad_string = true; return std::string(); }
        std::string s(static_cast<size_t>(len), '\0');
        in.read(&s[0], static_cast<std::streamsize>(len));
        return s;
    };
    if (r32() != GGUF_MAGIC) return fail("Not a GGUF file");
    if (r32() != GGUF_VERSION) return fail("Wrong version");
    const uint64_t tensor_count = r64(), kv_count = r64();
    // a tensor info takes at least 24 bytes (name length, rank, type, offset), a metadata entry at least 13:
    // counts a file of this size cannot hold are refused before anything is sized by them
    if (!in || tensor_count > f->file_size / 24 || kv_count > f->file_size / 13) return fail("truncated header");
    for (uint64_t i = 0; i < kv_count; ++i) {
        const std::string key = rstr();
        const uint32_t vtype = r32();
        switch (vtype) {
            case VT_UINT8: case VT_INT8: case VT_BOOL: in.seekg(1, std::ios::cur); break;
            case VT_UINT16: case VT_INT16: in.seekg(2, std::ios::cur); break;
            case VT_FLOAT32: { float v = 0; in.read(reinterpret_cast<char*>(&v), 4); f->floats[key] = v; break; }
            case VT_UINT32: case VT_INT32: f->floats[key] = static_cast<float>(r32()); break;
            case VT_UINT64: case VT_INT64: f->floats[key] = static_cast<float>(r64()); break;
            case VT_FLOAT64: { double v = 0; in.read(reinterpret_cast<char*>(&v), 8); f->floats[key] = static_cast<float>(v); break; }
            case VT_STRING: f->strings[key] = rstr(); break;
            case VT_ARRAY: {
                (void)r32();
                const uint64_t alen = r64();
                if (alen > f->file_size) return fail("truncated metadata");
                in.seekg(static_cast<std::streamoff>(alen * 4), std::ios::cur);   // taken as 4-byte elements, as the reference does
                break;
            }
            default: return fail("unknown metadata type");
        }
        if (!in || bad_string) return fail("truncated metadata");
    }
    f->tensors.resize(static_cast<size_t>(tensor_count));
    for (auto& t : f->tensors) {
        t.name = rstr();
        const uint32_t nd = r32();
        if (!in || bad_string || nd > 4) return fail("bad tensor info");
        t.dims.resize(nd);
        uint64_t numel = 1;
        bool wrapped = false;
        for (uint32_t d = 0; d < nd; ++d) {
            t.dims[d] = r64();
            wrapped = __builtin_mul_overflow(numel, t.dims[d], &numel) || wrapped;
        }
        if (wrapped) return fail("bad tensor info");   // a wrapped element count would pass for a small tensor
        t.type = r32();
        t.offset = r64();
        t.nbytes = tensor_bytes(t.type, numel);
        if (!in) return fail("truncated tensor infos");
    }
    return owner.release();
}

extern "C" void ppml_gguf_close(ppml_gguf_file* f) { delete f; }

extern "C" size_t ppml_gguf_tensor_count(const ppml_gguf_file* f) { return f ? f->tensors.size() : 0; }

extern "C" int ppml_gguf_tensor_info(const ppml_gguf_file* f, size_t i, const char** name, uint32_t* ndim, uint64_t dims[4],
                                     uint32_t* type, uint64_t* offset, uint64_t* nbytes) {
    if (!f || i >= f->tensors.size()) { set_error("ppml_gguf_tensor_info: no tensor %zu", i); return RC_BAD_ARGS; }
    const auto& t = f->tensors[i];
    if (name) *name = t.name.c_str();
    if (ndim) *ndim = static_cast<uint32_t>(t.dims.size());
    if (dims) for (size_t d = 0; d < 4; ++d) dims[d] = d < t.dims.size() ? t.dims[d] : 1;
    if (type) *type = t.type;
    if (offset) *offset = t.offset;
    if (nbytes) *nbytes = t.nbytes;
    return RC_OK;
}

extern "C" int64_t ppml_gguf_find_tensor(const ppml_gguf_file* f, const char* name) {
    if (!f || !name) return -1;
    for (size_t i = 0; i < f->tensors.size(); ++i)
        if (f->tensors[i].name == name) return static_cast<int64_t>(i);
    return -1;
}

extern "C" int ppml_gguf_read_tensor(ppml_gguf_file* f, size_t i, void* dst, size_t capacity) {
    if (!f || !dst || i >= f->tensors.size()) { set_error("ppml_gguf_read_tensor: bad arguments"); return RC_BAD_ARGS; }
    const auto& t = f->tensors[i];
    if (t.nbytes == 0) { set_error("ppml_gguf_read_tensor: tensor %s has type %u, which this library does not read", t.name.c_str(), t.type); return RC_BAD_ARGS; }
    if (capacity < t.nbytes) { set_error("ppml_gguf_read_tensor: %zu bytes given, %llu needed", capacity, static_cast<unsigned long long>(t.nbytes)); return RC_BAD_ARGS; }
    if (t.offset > f->file_size || t.nbytes > f->file_size - t.offset) { set_error("ppml_gguf_read_tensor: tensor %s lies outside the file", t.name.c_str()); return RC_BAD_ARGS; }
    f->in.clear();
    f->in.seekg(static_cast<std::streamoff>(t.offset), std::ios::beg);
    f->in.read(static_cast<char*>(dst), static_cast<std::streamsize>(t.nbytes));
    if (!f->in) { set_error("ppml_gguf_read_tensor: short read of tensor %s", t.name.c_str()); return RC_BAD_ARGS; }
    return RC_OK;
}

extern "C" int ppml_gguf_meta_float(const ppml_gguf_file* f, const char* key, float* value) {
    if (!f || !key) return 1;
    const auto it = f->floats.find(key);
    if (it == f->floats.end()) return 1;
    if (value) *value = it->second;
    return 0;
}

extern "C" const char* ppml_gguf_meta_string(const ppml_gguf_file* f, const char* key) {
    if (!f || !key) return nullptr;
    const auto it = f->strings.find(key);
    return it == f->strings.end() ? nullptr : it->second.c_str();
}

extern "C" int ppml_gguf_check_layout(const ppml_gguf_file* f, size_t n, const char* const* names, const uint32_t* ndims,
                                      const uint64_t* dims) {
    if (!f || (n > 0 && (!ndims || !dims))) { set_error("ppml_gguf_check_layout: bad arguments"); return RC_BAD_ARGS; }
    if (f->tensors.size() < n) {
        set_error("Tensor count mismatch: file=%zu params=%zu", f->tensors.size(), n);
        return RC_BAD_ARGS;
    }
    size_t at = 0;
    for (size_t i = 0; i < n; ++i) {
        const auto& t = f->tensors[i];
        if (t.dims.size() != ndims[i]) { set_error("Dimension count mismatch for tensor %zu", i); return RC_BAD_ARGS; }
        for (uint32_t d = 0; d < ndims[i]; ++d)
            if (t.dims[d] != dims[at + d]) { set_error("Shape mismatch for tensor %zu dim[%u]", i, d); return RC_BAD_ARGS; }
        at += ndims[i];
    }
    const auto saved = f->strings.find("layout_hash");
    if (saved == f->strings.end() || saved->second.empty()) return RC_OK;
    std::vector<const char*> file_names(n);
    for (size_t i = 0; i < n; ++i) file_names[i] = f->tensors[i].name.c_str();
    // with the model's own names the fingerprint also catches parameters that changed places but kept their shapes
    const std::string cur = hex64(layout_hash(n, names ? names : file_names.data(), ndims, dims));
    if (cur != saved->second) {
        set_error("Layout mismatch: file=%s current=%s (parameter collection order/shape/name changed vs. model definition)",
                  saved->second.c_str(), cur.c_str());
        return RC_BAD_ARGS;
    }
    return RC_OK;
}
