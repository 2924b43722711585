// GGUF container: header, metadata and tensor directory (gguf::GgufFile, reference
// src/gguf.rs:403-561), so that a .gguf can be mapped and its block tensors handed to
// pg_gguf_upload without materialising f32 (the reference's load_tensor_f32 +
// load_transposed_weight, src/gguf.rs:485-517, src/models/llama/model.rs:243-257).
// Host code only; the tensor loaders call the device kernels of pg_gguf.hip.
//
// Unlike the reference's reader, which indexes the byte slice unchecked and panics on a
// short file, every read here is bounds-checked and a malformed file is PG_EINVAL.
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <map>
#include <new>

#include <exception>
#include <new>
#include "pg_internal.h"

namespace {

constexpr uint32_t GGUF_MAGIC = 0x46554747u;  // "GGUF"  src/gguf.rs:10

struct MetaValue {
    uint32_t type = 0;                 // GGUF value type 0..12  src/gguf.rs:253-279
    uint64_t u = 0;                    // integers and bool
    double f = 0.0;                    // floats
    std::string s;                     // strings
    uint32_t arr_type = 0;             // arrays: element type and elements
    std::vector<MetaValue> arr;
};

struct TensorInfo {
    std::string name;
    int ggml_type = 0;
    std::vector<uint64_t> shape;  // GGUF order: innermost dimension first
    uint64_t data_offset = 0;     // relative to the data section
};

struct Reader {
    const uint8_t *p;
    size_t len, pos = 0;
    bool ok = true;
    bool need(size_t n) {
        if (!ok || n > len - pos) { ok = false; return false; }
        return true;
    }
    template <class T> T rd() {
        T v{};
        if (need(sizeof(T))) { memcpy(&v, p + pos, sizeof(T)); pos += sizeof(T); }
        return v;
    }
    std::string str() {
        const uint64_t n = rd<uint64_t>();
        if (!ok || n > len - pos) { ok = false; return std::string(); }
        std::string s(reinterpret_cast<const char *>(p + pos), (size_t)n);
        pos += (size_t)n;
        return s;
    }
    MetaValue value(uint32_t t, int depth) {
        MetaValue v;
        v.type = t;
        switch (t) {
            case 0: v.u = rd<uint8_t>(); break;
            case 1: v.u = (uint64_t)(int64_t)rd<int8_t>(); break;
            case 2: v.u = rd<uint16_t>(); break;
            case 3: v.u = (uint64_t)(int64_t)rd<int16_t>(); break;
            case 4: v.u = rd<uint32_t>(); break;
            case 5: v.u = (uint64_t)(int64_t)rd<int32_t>(); break;
            case 6: v.f = rd<float>(); break;
            case 7: v.u = rd<uint8_t>() != 0; break;
            case 8: v.s = str(); break;
            case 9: {
                v.arr_type = rd<uint32_t>();
                const uint64_t n = rd<uint64_t>();
                if (depth > 4 || n > len - pos) { ok = false; break; }  // every element takes >= 1 byte
                // (no reserve of n: a forged count would ask for ~100 bytes per claimed element; growth
                // by push_back is bounded by what the file can really hold)
                for (uint64_t i = 0; ok && i < n; ++i) v.arr.push_back(value(v.arr_type, depth + 1));
                break;
            }
            case 10: v.u = rd<uint64_t>(); break;
            case 11: v.u = (uint64_t)rd<int64_t>(); break;
            case 12: v.f = rd<double>(); break;
            default: ok = false; break;  // the reference panics: unknown GGUF metadata value type
        }
        return v;
    }
};

// GgmlType::block_size / block_bytes  src/gguf.rs:36-56
bool type_geometry(int t, size_t *elems, size_t *bytes) {
    switch (t) {
        case 0: *elems = 1; *bytes = 4; return true;                     // F32
        case 1: *elems = 1; *bytes = 2; return true;                     // F16
        case PG_GGML_Q4_0: *elems = 32; *bytes = 18; return true;
        case PG_GGML_Q4_1: *elems = 32; *bytes = 20; return true;
        case PG_GGML_Q8_0: *elems = 32; *bytes = 34; return true;
        default: return false;
    }
}

}  // namespace

struct pg_gguf_file {
    const uint8_t *data = nullptr;
    size_t len = 0;
    void *map = nullptr;  // non-null when this object owns an mmap of the file
    size_t map_len = 0;
    uint32_t version = 0;
    uint64_t data_start = 0;
    std::map<std::string, MetaValue> metadata;
    std::vector<TensorInfo> tensors;          // in file order
    std::map<std::string, size_t> by_name;
};

static pg_status parse_into(pg_gguf_file *f) {
    Reader r{f->data, f->len};
    const uint32_t magic = r.rd<uint32_t>();
    if (!r.ok || magic != GGUF_MAGIC)
        return pg_fail(PG_EINVAL, "invalid GGUF magic: 0x%08X, expected 0x%08X", magic, GGUF_MAGIC);  // src/gguf.rs:415-420
    f->version = r.rd<uint32_t>();
    if (!r.ok || f->version < 2 || f->version > 3)
        return pg_fail(PG_EINVAL, "unsupported GGUF version: %u", f->version);  // src/gguf.rs:423-428
    const uint64_t n_tensors = r.rd<uint64_t>(), n_kv = r.rd<uint64_t>();
    if (!r.ok || n_tensors > f->len || n_kv > f->len) return pg_fail(PG_EINVAL, "GGUF header is truncated or corrupt");
    for (uint64_t i = 0; i < n_kv; ++i) {
        std::string key = r.str();
        const uint32_t vtype = r.rd<uint32_t>();
        MetaValue v = r.value(vtype, 0);
        if (!r.ok) return pg_fail(PG_EINVAL, "GGUF metadata entry %llu is truncated or has an unknown type", (unsigned long long)i);
        f->metadata[key] = std::move(v);  // a repeated key keeps the last value, as HashMap::insert does
    }
    for (uint64_t i = 0; i < n_tensors; ++i) {
        TensorInfo t;
        t.name = r.str();
        const uint32_t n_dims = r.rd<uint32_t>();
        if (!r.ok || n_dims > 8) return pg_fail(PG_EINVAL, "GGUF tensor entry %llu is truncated or corrupt", (unsigned long long)i);
        for (uint32_t d = 0; d < n_dims; ++d) t.shape.push_back(r.rd<uint64_t>());
        const uint32_t dtype = r.rd<uint32_t>();
        t.data_offset = r.rd<uint64_t>();
        if (!r.ok) return pg_fail(PG_EINVAL, "GGUF tensor entry %llu is truncated", (unsigned long long)i);
        size_t be, bb;
        if (!type_geometry((int)dtype, &be, &bb))
            return pg_fail(PG_EUNSUPPORTED, "unsupported GGML type %u for tensor '%s'", dtype, t.name.c_str());  // src/gguf.rs:453-455
        t.ggml_type = (int)dtype;
        f->by_name[t.name] = f->tensors.size();
        f->tensors.push_back(std::move(t));
    }
    // data section: next multiple of general.alignment (default 32) after the header  src/gguf.rs:469-475
    uint64_t align = 32;
    auto it = f->metadata.find("general.alignment");
    if (it != f->metadata.end()) {
        const uint32_t ty = it->second.type;
        if (ty == 4 || ty == 5 || ty == 10 || ty == 11) align = (uint32_t)it->second.u;  // MetadataValue::as_u32  src/gguf.rs:77-85
    }
    if (align == 0) return pg_fail(PG_EINVAL, "GGUF general.alignment is 0");
    f->data_start = (r.pos + align - 1) / align * align;
    return PG_OK;
}

PG_API pg_status pg_gguf_file_parse(const void *data, size_t len, pg_gguf_file **out) {
    PG_CHECK_ARG(out != nullptr, "pg_gguf_file_parse: out is null");
    *out = nullptr;
    PG_CHECK_ARG(data != nullptr || len == 0, "pg_gguf_file_parse: null data");
    pg_gguf_file *f = new (std::nothrow) pg_gguf_file();
    if (!f) return pg_fail(PG_ENOMEM, "host allocation failed");
    f->data = static_cast<const uint8_t *>(data);
    f->len = len;
    pg_status st;
    try {  // the containers can throw (bad_alloc, length_error): nothing may unwind across the ABI
        st = parse_into(f);
    } catch (const std::bad_alloc &) {
        st = pg_fail(PG_ENOMEM, "out of host memory while parsing the GGUF header");
    } catch (const std::exception &e) {
        st = pg_fail(PG_EINVAL, "GGUF header is corrupt (%s)", e.what());
    }
    if (st != PG_OK) { delete f; return st; }
    *out = f;
    return PG_OK;
}

PG_API pg_status pg_gguf_file_open(const char *path, pg_gguf_file **out) {
    PG_CHECK_ARG(out != nullptr && path != nullptr, "pg_gguf_file_open: null argument");
    *out = nullptr;
    const int fd = open(path, O_RDONLY);
    if (fd < 0) return pg_fail(PG_EINVAL, "cannot open '%s'", path);
    struct stat sb;
    if (fstat(fd, &sb) != 0 || sb.st_size <= 0) { close(fd); return pg_fail(PG_EINVAL, "cannot stat '%s' or it is empty", path); }
    void *m = mmap(nullptr, (size_t)sb.st_size, PROT_READ, MAP_PRIVATE, fd, 0);
    close(fd);
    if (m == MAP_FAILED) return pg_fail(PG_ENOMEM, "mmap of '%s' (%lld bytes) failed", path, (long long)sb.st_size);
    const pg_status st = pg_gguf_file_parse(m, (size_t)sb.st_size, out);
    if (st != PG_OK) { munmap(m, (size_t)sb.st_size); return st; }
    (*out)->map = m;
    (*out)->map_len = (size_t)sb.st_size;
    return PG_OK;
}

PG_API void pg_gguf_file_close(pg_gguf_file *f) {
    if (!f) return;
    if (f->map) munmap(f->map, f->map_len);
    delete f;
}

PG_API pg_status pg_gguf_file_counts(const pg_gguf_file *f, size_t *n_tensors, size_t *n_metadata, uint32_t *version,
                                     uint64_t *data_start) {
    PG_CHECK_ARG(f != nullptr, "pg_gguf_file_counts: null file");
    if (n_tensors) *n_tensors = f->tensors.size();
    if (n_metadata) *n_metadata = f->metadata.size();
    if (version) *version = f->version;
    if (data_start) *data_start = f->data_start;
    return PG_OK;
}

static const TensorInfo *find_tensor(const pg_gguf_file *f, const char *name) {
    if (!f || !name) return nullptr;
    auto it = f->by_name.find(name);
    return it == f->by_name.end() ? nullptr : &f->tensors[it->second];
}

// Element count and byte size with the reference's checks (GgufTensor::num_elements / data_size).
static pg_status tensor_extent(const pg_gguf_file *f, const TensorInfo &t, size_t *n_elems, size_t *n_bytes, const uint8_t **ptr) {
    size_t be = 1, bb = 1;
    (void)type_geometry(t.ggml_type, &be, &bb);
    unsigned __int128 n = 1;
    // no tensor holds more elements than 32 per byte of the file (Q4_0 packs 32 into 18 bytes): a
    // larger count is corrupt, and bounding it here keeps every product below in range
    const unsigned __int128 max_elems = (unsigned __int128)f->len * 32 + 32;
    for (uint64_t d : t.shape) { n *= d; if (n > max_elems) return pg_fail(PG_EINVAL, "tensor '%s' is larger than the file", t.name.c_str()); }
    const size_t ne = (size_t)n;
    PG_CHECK_ARG(ne % be == 0, "tensor elements %zu not divisible by block size %zu", ne, be);  // src/gguf.rs:160
    const size_t nbytes = ne / be * bb;
    PG_CHECK_ARG(f->data_start <= f->len && t.data_offset <= f->len - f->data_start &&
                     nbytes <= f->len - f->data_start - t.data_offset,
                 "tensor '%s' extends past the end of the file", t.name.c_str());
    if (n_elems) *n_elems = ne;
    if (n_bytes) *n_bytes = nbytes;
    if (ptr) *ptr = f->data + f->data_start + t.data_offset;
    return PG_OK;
}

PG_API pg_status pg_gguf_file_tensor_name(const pg_gguf_file *f, size_t index, const char **name) {
    PG_CHECK_ARG(f != nullptr && name != nullptr, "pg_gguf_file_tensor_name: null argument");
    PG_CHECK_ARG(index < f->tensors.size(), "pg_gguf_file_tensor_name: index %zu of %zu", index, f->tensors.size());
    *name = f->tensors[index].name.c_str();
    return PG_OK;
}

PG_API pg_status pg_gguf_file_tensor_info(const pg_gguf_file *f, const char *name, int *ggml_type, size_t *n_dims,
                                          uint64_t *shape, size_t shape_cap, uint64_t *data_offset,
                                          size_t *data_size, const void **data) {
    const TensorInfo *t = find_tensor(f, name);
    if (!t) return pg_fail(PG_EINVAL, "tensor '%s' not found in GGUF file", name ? name : "(null)");  // src/gguf.rs:487-489
    if (ggml_type) *ggml_type = t->ggml_type;
    if (n_dims) *n_dims = t->shape.size();
    if (shape)
        for (size_t i = 0; i < t->shape.size() && i < shape_cap; ++i) shape[i] = t->shape[i];
    if (data_offset) *data_offset = t->data_offset;
    if (data_size || data) {
        size_t nb = 0;
        const uint8_t *p = nullptr;
        PG_TRY(tensor_extent(f, *t, nullptr, &nb, &p));
        if (data_size) *data_size = nb;
        if (data) *data = p;
    }
    return PG_OK;
}

static const MetaValue *find_meta(const pg_gguf_file *f, const char *key) {
    if (!f || !key) return nullptr;
    auto it = f->metadata.find(key);
    return it == f->metadata.end() ? nullptr : &it->second;
}

PG_API pg_status pg_gguf_file_get_u32(const pg_gguf_file *f, const char *key, uint32_t *value, int *found) {
    PG_CHECK_ARG(f && key && value && found, "pg_gguf_file_get_u32: null argument");
    const MetaValue *v = find_meta(f, key);
    // MetadataValue::as_u32  src/gguf.rs:77-85: Uint32, Int32, Uint64, Int64 only
    *found = v && (v->type == 4 || v->type == 5 || v->type == 10 || v->type == 11);
    if (*found) *value = (uint32_t)v->u;
    return PG_OK;
}

PG_API pg_status pg_gguf_file_get_f32(const pg_gguf_file *f, const char *key, float *value, int *found) {
    PG_CHECK_ARG(f && key && value && found, "pg_gguf_file_get_f32: null argument");
    const MetaValue *v = find_meta(f, key);
    *found = v && (v->type == 6 || v->type == 12);  // MetadataValue::as_f32  src/gguf.rs:87-93
    if (*found) *value = (float)v->f;
    return PG_OK;
}

PG_API pg_status pg_gguf_file_get_str(const pg_gguf_file *f, const char *key, const char **value, size_t *len) {
    PG_CHECK_ARG(f && key && value, "pg_gguf_file_get_str: null argument");
    const MetaValue *v = find_meta(f, key);
    *value = (v && v->type == 8) ? v->s.c_str() : nullptr;  // MetadataValue::as_str  src/gguf.rs:95-100
    if (len) *len = *value ? v->s.size() : 0;
    return PG_OK;
}

PG_API pg_status pg_gguf_file_get_array(const pg_gguf_file *f, const char *key, uint32_t *elem_type, size_t *count) {
    PG_CHECK_ARG(f && key && count, "pg_gguf_file_get_array: null argument");
    const MetaValue *v = find_meta(f, key);
    const bool is_arr = v && v->type == 9;
    *count = is_arr ? v->arr.size() : (size_t)-1;
    if (elem_type) *elem_type = is_arr ? v->arr_type : 0;
    return PG_OK;
}

PG_API pg_status pg_gguf_file_get_array_str(const pg_gguf_file *f, const char *key, size_t index, const char **value) {
    PG_CHECK_ARG(f && key && value, "pg_gguf_file_get_array_str: null argument");
    const MetaValue *v = find_meta(f, key);
    *value = (v && v->type == 9 && index < v->arr.size() && v->arr[index].type == 8) ? v->arr[index].s.c_str() : nullptr;
    return PG_OK;
}

PG_API pg_status pg_gguf_file_get_array_f64(const pg_gguf_file *f, const char *key, double *values, size_t cap) {
    PG_CHECK_ARG(f && key && (values || cap == 0), "pg_gguf_file_get_array_f64: null argument");
    const MetaValue *v = find_meta(f, key);
    PG_CHECK_ARG(v && v->type == 9, "pg_gguf_file_get_array_f64: '%s' is not an array", key);
    for (size_t i = 0; i < v->arr.size() && i < cap; ++i) {
        const MetaValue &e = v->arr[i];
        PG_CHECK_ARG(e.type != 8 && e.type != 9, "pg_gguf_file_get_array_f64: '%s' holds non-numeric elements", key);
        const bool is_signed = e.type == 1 || e.type == 3 || e.type == 5 || e.type == 11;
        values[i] = (e.type == 6 || e.type == 12) ? e.f : (is_signed ? (double)(int64_t)e.u : (double)e.u);
    }
    return PG_OK;
}

// GgufFile::load_tensor_f32  src/gguf.rs:485-517: any supported type -> f32, element order as stored.
PG_API pg_status pg_gguf_file_load_tensor_f32(pg_ctx *ctx, const pg_gguf_file *f, const char *name, float *out,
                                              size_t out_cap) {
    const TensorInfo *t = find_tensor(f, name);
    if (!t) return pg_fail(PG_EINVAL, "tensor '%s' not found in GGUF file", name ? name : "(null)");
    size_t ne = 0, nb = 0;
    const uint8_t *p = nullptr;
    PG_TRY(tensor_extent(f, *t, &ne, &nb, &p));
    PG_CHECK_ARG(out != nullptr || ne == 0, "pg_gguf_file_load_tensor_f32: null output");
    PG_CHECK_ARG(out_cap >= ne, "pg_gguf_file_load_tensor_f32: output holds %zu of %zu elements", out_cap, ne);
    switch (t->ggml_type) {
        case 0: memcpy(out, p, ne * sizeof(float)); return PG_OK;  // little-endian host
        case 1: {
            // the file offset of an F16 tensor need not be 2-byte aligned in memory
            std::vector<uint16_t> tmp(ne);
            memcpy(tmp.data(), p, ne * 2);
            return pg_f16_to_f32(ctx, tmp.data(), ne, out);
        }
        case PG_GGML_Q8_0: return pg_dequant_q8_0(ctx, p, ne, out);
        case PG_GGML_Q4_0: return pg_dequant_q4_0(ctx, p, ne, out);
        default: return pg_dequant_q4_1(ctx, p, ne, out);
    }
}

// Keep a 2-D Q4_0 / Q8_0 tensor quantised on the device.  GGUF shape [in, out] (innermost
// first) is Peregrine's [out, in] (GgufFile::tensor_shape, src/gguf.rs:551-556): n_out =
// shape[1], k_in = shape[0]; a 1-D tensor is one output row (as load_tensor_q8 treats it,
// src/gguf.rs:530-534).
PG_API pg_status pg_gguf_file_upload_tensor(pg_ctx *ctx, const pg_gguf_file *f, const char *name, pg_gguf_tensor **out) {
    PG_CHECK_ARG(out != nullptr, "pg_gguf_file_upload_tensor: out is null");
    *out = nullptr;
    const TensorInfo *t = find_tensor(f, name);
    if (!t) return pg_fail(PG_EINVAL, "tensor '%s' not found in GGUF file", name ? name : "(null)");
    PG_CHECK_ARG(t->shape.size() == 1 || t->shape.size() == 2, "expected 1D or 2D tensor for '%s', got %zu dimensions",
                 t->name.c_str(), t->shape.size());
    const uint8_t *p = nullptr;
    PG_TRY(tensor_extent(f, *t, nullptr, nullptr, &p));
    const size_t k_in = (size_t)t->shape[0], n_out = t->shape.size() == 2 ? (size_t)t->shape[1] : 1;
    return pg_gguf_upload(ctx, p, t->ggml_type, n_out, k_in, out);
}
