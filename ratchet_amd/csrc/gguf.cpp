// GGUF container reader: header, metadata, tensor directory (host only), and the
// tensor -> device path that ends in this library's layouts.
//
// Follows crates/ratchet-loader/src/gguf/gguf.rs:408-479 (Header::read), :164-180
// (read_string), :330-377 (Value::read), :63-106 (TensorInfo) and :118-142
// (ratchet_from_gguf); type tables from crates/ratchet-loader/src/lib.rs:62-140.
// RT_HOST_ONLY leaves out the one function that talks to the device, so that the parser can be built
// by a host compiler alone (the sanitizer build of the test suite does).
#ifndef RT_HOST_ONLY
#include <hip/hip_runtime.h>
#endif

#include <cstring>
#include <stdexcept>
#include <string>
#include <unordered_map>
#include <vector>

#ifndef RT_HOST_ONLY
#include "device_common.h"
#endif
#include "spec.h"

namespace {

struct Value {
    int32_t type = 0, elem_type = 0;
    uint64_t u64 = 0;
    int64_t i64 = 0;
    double f64 = 0;
    std::string str;
    std::vector<Value> arr;
};

struct TensorInfo {
    std::string name;
    int32_t ggml_dtype = 0;
    std::vector<int64_t> shape;
    uint64_t offset = 0, size_in_bytes = 0;
};

struct Unsupported : std::runtime_error {
    using std::runtime_error::runtime_error;
};

// Bounds-checked little-endian cursor over the image.
struct Cursor {
    const uint8_t *p;
    uint64_t size, pos = 0;
    void need(uint64_t n) const {
        if (n > size - pos) throw std::runtime_error("gguf: image truncated at byte " + std::to_string(pos));
    }
    template <typename T> T get() {
        need(sizeof(T));
        T v;
        std::memcpy(&v, p + pos, sizeof(T));
        pos += sizeof(T);
        return v;
    }
    // 32-bit in version 1, 64-bit from version 2 on (gguf.rs:166-171)
    uint64_t len(uint32_t version) { return version == 1 ? get<uint32_t>() : get<uint64_t>(); }
    std::string str(uint32_t version) {
        const uint64_t n = len(version);
        need(n);
        std::string s((const char *)p + pos, (size_t)n);
        pos += n;
        while (!s.empty() && s.back() == '\0') s.pop_back(); // gguf.rs:176-178
        return s;
    }
};

uint64_t type_size(int32_t t) {
    switch (t) { // sizeof of the block structs, k_quants.rs
    case RT_GGML_F32: return 4;
    case RT_GGML_F16: return 2;
    case RT_GGML_Q4_0: return 18;
    case RT_GGML_Q4_1: return 20;
    case RT_GGML_Q5_0: return 22;
    case RT_GGML_Q5_1: return 24;
    case RT_GGML_Q8_0: return 34;
    case RT_GGML_Q8_1: return 36;
    case RT_GGML_Q2K: return 84;
    case RT_GGML_Q3K: return 110;
    case RT_GGML_Q4K: return 144;
    case RT_GGML_Q5K: return 176;
    case RT_GGML_Q6K: return 210;
    case RT_GGML_Q8K: return 292;
    default: return 0;
    }
}

uint64_t block_numel(int32_t t) {
    switch (t) {
    case RT_GGML_F32:
    case RT_GGML_F16: return 1;
    case RT_GGML_Q4_0:
    case RT_GGML_Q4_1:
    case RT_GGML_Q5_0:
    case RT_GGML_Q5_1:
    case RT_GGML_Q8_0:
    case RT_GGML_Q8_1: return 32;
    case RT_GGML_Q2K:
    case RT_GGML_Q3K:
    case RT_GGML_Q4K:
    case RT_GGML_Q5K:
    case RT_GGML_Q6K:
    case RT_GGML_Q8K: return 256;
    default: return 0;
    }
}

Value read_value(Cursor &c, int32_t type, uint32_t version, int depth) {
    Value v;
    v.type = type;
    switch (type) {
    case RT_GGUF_U8: v.u64 = c.get<uint8_t>(); break;
    case RT_GGUF_I8: v.i64 = c.get<int8_t>(); break;
    case RT_GGUF_U16: v.u64 = c.get<uint16_t>(); break;
    case RT_GGUF_I16: v.i64 = c.get<int16_t>(); break;
    case RT_GGUF_U32: v.u64 = c.get<uint32_t>(); break;
    case RT_GGUF_I32: v.i64 = c.get<int32_t>(); break;
    case RT_GGUF_U64: v.u64 = c.get<uint64_t>(); break;
    case RT_GGUF_I64: v.i64 = c.get<int64_t>(); break;
    case RT_GGUF_F32: v.f64 = c.get<float>(); break;
    case RT_GGUF_F64: v.f64 = c.get<double>(); break;
    case RT_GGUF_BOOL: {
        const uint8_t b = c.get<uint8_t>();
        if (b > 1) throw std::runtime_error("gguf: unexpected bool value " + std::to_string(b)); // gguf.rs:349-353
        v.u64 = b;
        break;
    }
    case RT_GGUF_STRING: v.str = c.str(version); break;
    case RT_GGUF_ARRAY: {
        if (depth > 8) throw std::runtime_error("gguf: arrays nested too deeply");
        v.elem_type = (int32_t)c.get<uint32_t>();
        if (v.elem_type < 0 || v.elem_type > RT_GGUF_F64)
            throw Unsupported("gguf: unrecognized value-type " + std::to_string(v.elem_type));
        const uint64_t n = c.len(version);
        if (n > c.size - c.pos) throw std::runtime_error("gguf: array longer than the image"); // every element takes >= 1 byte
        v.arr.reserve((size_t)n);
        for (uint64_t i = 0; i < n; i++) v.arr.push_back(read_value(c, v.elem_type, version, depth + 1));
        break;
    }
    default: throw Unsupported("gguf: unrecognized value-type " + std::to_string(type));
    }
    return v;
}

void export_value(const Value &v, rt_gguf_value *out) {
    out->type = v.type;
    out->elem_type = v.elem_type;
    out->count = v.type == RT_GGUF_ARRAY ? v.arr.size() : (v.type == RT_GGUF_STRING ? v.str.size() : 1);
    out->u64 = v.u64;
    out->i64 = v.i64;
    out->f64 = v.f64;
    out->str = v.type == RT_GGUF_STRING ? v.str.c_str() : nullptr;
}

} // namespace

struct rt_gguf {
    uint32_t version = 0;
    std::vector<std::pair<std::string, Value>> metadata; // file order
    std::vector<TensorInfo> tensors;                     // file order
    std::unordered_map<std::string, size_t> meta_index, tensor_index; // name -> last occurrence
    uint64_t tensor_data_offset = 0;
    mutable std::string error;
};

extern "C" {

uint64_t rt_ggml_type_size(int32_t t) { return type_size(t); }
uint64_t rt_ggml_block_numel(int32_t t) { return block_numel(t); }

rt_status rt_gguf_parse(const void *image, uint64_t size, rt_gguf **out) {
    if (!out) return RT_ERR_INVALID_ARG;
    *out = nullptr;
    if (!image) return RT_ERR_INVALID_ARG;
    rt_gguf *g = nullptr;
    try {
        g = new rt_gguf();
        Cursor c{(const uint8_t *)image, size};
        const uint32_t magic = c.get<uint32_t>();
        if (magic != 0x46554747u && magic != 0x47475546u) throw Unsupported("gguf: unknown magic"); // gguf.rs:24-27
        g->version = c.get<uint32_t>();
        if (g->version < 1 || g->version > 3)
            throw Unsupported("gguf: unsupported version " + std::to_string(g->version)); // gguf.rs:45-50
        const uint64_t n_tensors = c.len(g->version), n_kv = c.len(g->version);
        if (n_kv > size || n_tensors > size) throw std::runtime_error("gguf: counts larger than the image");
        for (uint64_t i = 0; i < n_kv; i++) {
            std::string key = c.str(g->version);
            const int32_t type = (int32_t)c.get<uint32_t>();
            Value v = read_value(c, type, g->version, 0);
            g->meta_index[key] = g->metadata.size();
            g->metadata.emplace_back(std::move(key), std::move(v));
        }
        for (uint64_t i = 0; i < n_tensors; i++) {
            TensorInfo ti;
            ti.name = c.str(g->version);
            const uint32_t nd = c.get<uint32_t>();
            if (nd > RT_MAX_RANK) throw Unsupported("gguf: tensor rank " + std::to_string(nd) + " exceeds " + std::to_string(RT_MAX_RANK));
            ti.shape.resize(nd);
            for (uint32_t d = 0; d < nd; d++) ti.shape[d] = (int64_t)c.len(g->version);
            // the file lists the innermost dimension first (gguf.rs:450)
            for (uint32_t d = 0; d < nd / 2; d++) std::swap(ti.shape[d], ti.shape[nd - 1 - d]);
            ti.ggml_dtype = (int32_t)c.get<uint32_t>();
            if (type_size(ti.ggml_dtype) == 0)
                throw Unsupported("gguf: invalid data type " + std::to_string(ti.ggml_dtype)); // lib.rs:79
            ti.offset = c.get<uint64_t>();
            uint64_t numel = 1;
            for (int64_t d : ti.shape) {
                if (d < 0 || (d > 0 && numel > UINT64_MAX / (uint64_t)d)) throw std::runtime_error("gguf: tensor extent overflows");
                numel *= (uint64_t)d;
            }
            ti.size_in_bytes = numel / block_numel(ti.ggml_dtype) * type_size(ti.ggml_dtype); // gguf.rs:93-98
            g->tensor_index[ti.name] = g->tensors.size();
            g->tensors.push_back(std::move(ti));
        }
        // gguf.rs:464-473: general.alignment of a (non-negative) 8/16/32-bit integer type, else 32
        uint64_t alignment = 32;
        auto it = g->meta_index.find("general.alignment");
        if (it != g->meta_index.end()) {
            const Value &v = g->metadata[it->second].second;
            if (v.type == RT_GGUF_U8 || v.type == RT_GGUF_U16 || v.type == RT_GGUF_U32) alignment = v.u64;
            else if ((v.type == RT_GGUF_I8 || v.type == RT_GGUF_I16 || v.type == RT_GGUF_I32) && v.i64 >= 0)
                alignment = (uint64_t)v.i64;
        }
        if (alignment == 0) throw std::runtime_error("gguf: general.alignment is zero");
        g->tensor_data_offset = (c.pos + alignment - 1) / alignment * alignment;
        *out = g;
        return RT_OK;
    } catch (const Unsupported &) {
        delete g;
        return RT_ERR_UNSUPPORTED;
    } catch (const std::bad_alloc &) {
        delete g;
        return RT_ERR_OOM;
    } catch (...) {
        delete g;
        return RT_ERR_INVALID_ARG;
    }
}

void rt_gguf_free(rt_gguf *g) { delete g; }
const char *rt_gguf_error(const rt_gguf *g) { return g ? g->error.c_str() : ""; }
uint32_t rt_gguf_version(const rt_gguf *g) { return g ? g->version : 0; }
uint64_t rt_gguf_tensor_count(const rt_gguf *g) { return g ? g->tensors.size() : 0; }
uint64_t rt_gguf_metadata_count(const rt_gguf *g) { return g ? g->metadata.size() : 0; }
uint64_t rt_gguf_tensor_data_offset(const rt_gguf *g) { return g ? g->tensor_data_offset : 0; }

rt_status rt_gguf_tensor_info_at(const rt_gguf *g, uint64_t index, rt_gguf_tensor_info *info) {
    if (!g || !info || index >= g->tensors.size()) return RT_ERR_INVALID_ARG;
    const TensorInfo &ti = g->tensors[index];
    *info = rt_gguf_tensor_info{};
    info->name = ti.name.c_str();
    info->ggml_dtype = ti.ggml_dtype;
    info->rank = (int32_t)ti.shape.size();
    for (size_t d = 0; d < ti.shape.size(); d++) info->shape[d] = ti.shape[d];
    info->offset = ti.offset;
    info->size_in_bytes = ti.size_in_bytes;
    return RT_OK;
}

rt_status rt_gguf_find_tensor(const rt_gguf *g, const char *name, uint64_t *index) {
    if (!g || !name || !index) return RT_ERR_INVALID_ARG;
    auto it = g->tensor_index.find(name);
    if (it == g->tensor_index.end()) {
        g->error = std::string("cannot find tensor info for ") + name; // gguf.rs:491
        return RT_ERR_INVALID_ARG;
    }
    *index = it->second;
    return RT_OK;
}

rt_status rt_gguf_metadata_key_at(const rt_gguf *g, uint64_t index, const char **key) {
    if (!g || !key || index >= g->metadata.size()) return RT_ERR_INVALID_ARG;
    *key = g->metadata[index].first.c_str();
    return RT_OK;
}

rt_status rt_gguf_metadata_get(const rt_gguf *g, const char *key, rt_gguf_value *value) {
    if (!g || !key || !value) return RT_ERR_INVALID_ARG;
    auto it = g->meta_index.find(key);
    if (it == g->meta_index.end()) {
        g->error = std::string("missing key ") + key; // gguf.rs:151-153
        return RT_ERR_INVALID_ARG;
    }
    export_value(g->metadata[it->second].second, value);
    return RT_OK;
}

rt_status rt_gguf_metadata_array_get(const rt_gguf *g, const char *key, uint64_t i, rt_gguf_value *value) {
    if (!g || !key || !value) return RT_ERR_INVALID_ARG;
    auto it = g->meta_index.find(key);
    if (it == g->meta_index.end()) {
        g->error = std::string("missing key ") + key;
        return RT_ERR_INVALID_ARG;
    }
    const Value &v = g->metadata[it->second].second;
    if (v.type != RT_GGUF_ARRAY || i >= v.arr.size()) {
        g->error = std::string("not an array or index out of range: ") + key; // Value::to_vec, gguf.rs:314-319
        return RT_ERR_INVALID_ARG;
    }
    export_value(v.arr[i], value);
    return RT_OK;
}

} // extern "C"

namespace rt {

// TensorInfo::byte_range (gguf.rs:100-105) against an image of `size` bytes: where tensor `index` begins, or why
// it cannot lie in the image.  Offsets and sizes come from the file and are not trusted: neither sum may wrap.
rt_status gguf_tensor_range(const rt_gguf *g, uint64_t size, uint64_t index, uint64_t *begin, uint64_t *numel_out,
                            std::string &why) {
    if (index >= g->tensors.size()) return why = "tensor index out of range", RT_ERR_INVALID_ARG;
    const TensorInfo &ti = g->tensors[index];
    uint64_t numel = 1;
    for (int64_t d : ti.shape) numel *= (uint64_t)d;
    const uint64_t bn = block_numel(ti.ggml_dtype);
    if (numel % bn != 0) // gguf.rs:72-76
        return why = "the number of elements " + std::to_string(numel) + " is not divisible by the block size " + std::to_string(bn),
               RT_ERR_INVALID_SHAPE;
    if (g->tensor_data_offset > size || ti.offset > size - g->tensor_data_offset)
        return why = "tensor data lies outside the image", RT_ERR_INVALID_ARG;
    const uint64_t b = g->tensor_data_offset + ti.offset;
    if (ti.size_in_bytes > size - b) return why = "tensor data lies outside the image", RT_ERR_INVALID_ARG;
    *begin = b, *numel_out = numel;
    return RT_OK;
}

#ifndef RT_HOST_ONLY
// Host image -> device tensor in this library's layout.  Returns a message on failure.
rt_status gguf_load_tensor(const rt_gguf *g, const void *image, uint64_t size, uint64_t index, int32_t dst_dtype,
                           void *staging, void *dst, hipStream_t stream, std::string &why, hipError_t &herr) {
    herr = hipSuccess;
    uint64_t begin = 0, numel = 0;
    const rt_status rs = gguf_tensor_range(g, size, index, &begin, &numel, why);
    if (rs != RT_OK) return rs;
    const TensorInfo &ti = g->tensors[index];
    const uint8_t *src = (const uint8_t *)image + begin;
    if (numel == 0) return RT_OK;
    if (!dst) return why = "null destination", RT_ERR_INVALID_ARG;
    const bool plain = (ti.ggml_dtype == RT_GGML_F32 && dst_dtype == RT_F32) || (ti.ggml_dtype == RT_GGML_F16 && dst_dtype == RT_F16) ||
                       (ti.ggml_dtype == RT_GGML_Q4K && dst_dtype == RT_Q4_K);
    if (plain) {
        herr = hipMemcpyAsync(dst, src, ti.size_in_bytes, hipMemcpyHostToDevice, stream);
        return herr == hipSuccess ? RT_OK : (why = "tensor upload", RT_ERR_HIP);
    }
    if (ti.ggml_dtype == RT_GGML_Q8_0 && (dst_dtype == RT_Q8_0H || dst_dtype == RT_Q8_0F)) {
        if (!staging) return why = "Q8_0 tensors need a staging buffer of size_in_bytes", RT_ERR_INVALID_ARG;
        if (((uintptr_t)staging & 1u) || ((uintptr_t)dst & 15u)) return why = "misaligned buffer", RT_ERR_INVALID_ARG;
        herr = hipMemcpyAsync(staging, src, ti.size_in_bytes, hipMemcpyHostToDevice, stream);
        if (herr != hipSuccess) return why = "tensor upload", RT_ERR_HIP;
        herr = launch_transcode_gguf_q8_0(staging, numel / 32, dst_dtype, dst, stream);
        return herr == hipSuccess ? RT_OK : (why = "transcode launch", RT_ERR_HIP);
    }
    return why = "unsupported ggml dtype " + std::to_string(ti.ggml_dtype) + " for destination dtype " + std::to_string(dst_dtype), // gguf.rs:140
           RT_ERR_UNSUPPORTED;
}
#endif

} // namespace rt
