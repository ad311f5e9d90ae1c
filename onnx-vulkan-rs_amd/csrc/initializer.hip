// ONNX initializers -> raw little-endian bytes: the data format in front of the prepack calls.
//
// Host code only. It restates what the reference's frontend does with a weight before any kernel sees
// it (crates/onnx-vulkan-frontend/src/convert.rs:51-113 for the walk over a model's initializers,
// :247-300 for the three storage forms of a TensorProto, :311-384 for weights kept in a file beside
// the model), on the protobuf wire format directly: there is no protobuf library behind this file, a
// TensorProto is a handful of varints and length-delimited fields.
//
//   storage forms (mutually exclusive, in this order of precedence):
//     data_location == EXTERNAL   the bytes [offset, offset + length) of <base_dir>/<location>
//     raw_data                    already the layout wanted
//     typed repeated fields       float_data / double_data / int64_data / uint64_data / int32_data; ONNX packs
//                                 every narrow dtype into int32_data, so the width written comes from
//                                 data_type, never from the field the values arrived in
#include <cerrno>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <exception>
#include <string>
#include <utility>
#include <vector>

#include "../../include/hipcompute.h"

namespace {

thread_local std::string g_host_error;

int host_fail(int code, const char *fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    g_host_error = buf;
    return code;
}

// TensorProto.DataType
enum : int32_t {
    DT_FLOAT = 1, DT_UINT8 = 2, DT_INT8 = 3, DT_UINT16 = 4, DT_INT16 = 5, DT_INT32 = 6, DT_INT64 = 7, DT_BOOL = 9, DT_FLOAT16 = 10,
    DT_DOUBLE = 11, DT_UINT32 = 12, DT_UINT64 = 13, DT_BFLOAT16 = 16,
};

struct Span {
    const uint8_t *p = nullptr;
    size_t n = 0;
};

// One pass over the fields of a message. next() returns false at the end or on a malformed field (bad() tells which).
struct Reader {
    const uint8_t *p, *end;
    bool broken = false;
    uint32_t field = 0, wire = 0;
    uint64_t value = 0;  // varint, or the little-endian bits of a fixed32 / fixed64
    Span bytes;          // length-delimited payload

    Reader(const void *data, size_t n) : p(static_cast<const uint8_t *>(data)), end(p + n) {}
    explicit Reader(Span s) : p(s.p), end(s.p + s.n) {}

    bool varint(uint64_t *out) {
        uint64_t v = 0;
        for (int shift = 0; shift < 64; shift += 7) {
            if (p >= end) return false;
            const uint8_t c = *p++;
            v |= (uint64_t)(c & 0x7f) << shift;
            if (c < 0x80) {
                *out = v;
                return true;
            }
        }
        return false;  // more than ten bytes
    }
    bool next() {
        if (broken || p >= end) return false;
        uint64_t key;
        if (!varint(&key) || (key >> 3) == 0 || (key >> 3) > 0x1fffffff) return !(broken = true);
        field = (uint32_t)(key >> 3), wire = (uint32_t)(key & 7);
        switch (wire) {
            case 0: return varint(&value) || !(broken = true);
            case 1:
                if (end - p < 8) return !(broken = true);
                memcpy(&value, p, 8), p += 8;
                return true;
            case 2: {
                uint64_t n;
                if (!varint(&n) || n > (uint64_t)(end - p)) return !(broken = true);
                bytes = Span{p, (size_t)n}, p += n;
                return true;
            }
            case 5: {
                if (end - p < 4) return !(broken = true);
                uint32_t v;
                memcpy(&v, p, 4), p += 4, value = v;
                return true;
            }
            default: return !(broken = true);  // groups are not part of ONNX
        }
    }
    bool bad() const { return broken; }
};

// a repeated scalar field arrives packed (one length-delimited run) or one element per key
template <typename Push>
bool each_varint(const Reader &r, Push push) {
    if (r.wire == 0) return push(r.value), true;
    if (r.wire != 2) return false;
    Reader run(r.bytes);
    uint64_t v;
    while (run.p < run.end) {
        if (!run.varint(&v)) return false;
        push(v);
    }
    return true;
}
template <typename Push>
bool each_fixed(const Reader &r, unsigned width, Push push) {  // width 4 or 8
    if (r.wire == (width == 4 ? 5u : 1u)) return push(r.value), true;
    if (r.wire != 2 || r.bytes.n % width != 0) return false;
    for (size_t i = 0; i < r.bytes.n; i += width) {
        uint64_t v = 0;
        memcpy(&v, r.bytes.p + i, width);
        push(v);
    }
    return true;
}

void put_le(std::vector<uint8_t> &out, uint64_t v, unsigned width) {
    for (unsigned i = 0; i < width; i++) out.push_back((uint8_t)(v >> (8 * i)));
}

struct Tensor {
    std::string name, location;
    std::vector<int64_t> dims;
    int32_t data_type = 0;
    bool external = false, has_offset = false, has_length = false;
    uint64_t offset = 0, length = 0;
    Span raw;
    std::vector<uint64_t> f32, f64, i32, i64, u64;  // typed fields, as bit patterns / sign-extended varints
};

int parse_number(const std::string &tensor, const char *key, const std::string &text, uint64_t *out) {
    if (text.empty()) return host_fail(HIPC_ERR_INVALID, "tensor '%s': '%s' = '' not numeric", tensor.c_str(), key);
    uint64_t v = 0;
    for (char c : text) {
        if (c < '0' || c > '9' || v > (UINT64_MAX - 9) / 10) return host_fail(HIPC_ERR_INVALID, "tensor '%s': '%s' = '%s' not numeric", tensor.c_str(), key, text.c_str());
        v = v * 10 + (uint64_t)(c - '0');
    }
    *out = v;
    return HIPC_OK;
}

int parse_tensor(const void *data, size_t len, Tensor *t) {
    Reader r(data, len);
    std::vector<std::pair<std::string, std::string>> entries;
    while (r.next()) {
        bool ok = true;
        switch (r.field) {
            case 1: ok = each_varint(r, [&](uint64_t v) { t->dims.push_back((int64_t)v); }); break;
            case 2: ok = r.wire == 0, t->data_type = (int32_t)r.value; break;
            case 4: ok = each_fixed(r, 4, [&](uint64_t v) { t->f32.push_back(v); }); break;
            case 5: ok = each_varint(r, [&](uint64_t v) { t->i32.push_back(v); }); break;
            case 7: ok = each_varint(r, [&](uint64_t v) { t->i64.push_back(v); }); break;
            case 8: ok = r.wire == 2, t->name.assign(reinterpret_cast<const char *>(r.bytes.p), r.wire == 2 ? r.bytes.n : 0); break;
            case 9: ok = r.wire == 2, t->raw = r.bytes; break;
            case 10: ok = each_fixed(r, 8, [&](uint64_t v) { t->f64.push_back(v); }); break;
            case 11: ok = each_varint(r, [&](uint64_t v) { t->u64.push_back(v); }); break;
            case 13: {  // StringStringEntryProto { key = 1, value = 2 }
                if (!(ok = r.wire == 2)) break;
                Reader e(r.bytes);
                std::string key, value;
                while (e.next()) {
                    if (e.wire != 2) continue;
                    if (e.field == 1) key.assign(reinterpret_cast<const char *>(e.bytes.p), e.bytes.n);
                    if (e.field == 2) value.assign(reinterpret_cast<const char *>(e.bytes.p), e.bytes.n);
                }
                ok = !e.bad();
                entries.emplace_back(key, value);
                break;
            }
            case 14: ok = r.wire == 0, t->external = r.value == 1; break;
            default: break;  // segment, string_data, doc_string, metadata: nothing the payload depends on
        }
        if (!ok) return host_fail(HIPC_ERR_INVALID, "TensorProto decode: field %u has wire type %u", r.field, r.wire);
    }
    if (r.bad()) return host_fail(HIPC_ERR_INVALID, "TensorProto decode: truncated or malformed field");
    for (const auto &kv : entries) {  // the first entry of a key counts
        int rc = HIPC_OK;
        if (kv.first == "location" && t->location.empty()) t->location = kv.second;
        if (kv.first == "offset" && !t->has_offset) rc = parse_number(t->name, "offset", kv.second, &t->offset), t->has_offset = true;
        if (kv.first == "length" && !t->has_length) rc = parse_number(t->name, "length", kv.second, &t->length), t->has_length = true;
        if (rc != HIPC_OK) return rc;
    }
    return HIPC_OK;
}

// A path made of ordinary components only: relative, no "." or "..", so that it cannot leave the model's directory.
bool plain_relative(const std::string &path) {
    if (path.empty() || path[0] == '/') return false;
    size_t i = 0;
    bool any = false;
    while (i < path.size()) {
        size_t j = path.find('/', i);
        if (j == std::string::npos) j = path.size();
        const std::string part = path.substr(i, j - i);
        if (part == "." || part == "..") return false;
        if (!part.empty()) any = true;  // repeated separators are not components
        i = j + 1;
    }
    return any;
}

int read_external(const Tensor &t, const char *base_dir, std::vector<uint8_t> *out, size_t *bytes, bool want_data) {
    const char *name = t.name.c_str();
    if (t.location.empty()) return host_fail(HIPC_ERR_INVALID, "tensor '%s': missing 'location' key", name);
    if (!plain_relative(t.location)) return host_fail(HIPC_ERR_INVALID, "tensor '%s': external path '%s' not relative", name, t.location.c_str());
    if (!base_dir) return host_fail(HIPC_ERR_INVALID, "tensor '%s': weights in '%s', but the model directory is not known", name, t.location.c_str());
    const std::string path = std::string(base_dir) + "/" + t.location;
    FILE *f = fopen(path.c_str(), "rb");
    if (!f) return host_fail(HIPC_ERR_INVALID, "opening %s: %s", path.c_str(), strerror(errno));
    // the tensor's slice only: every initializer of a model points into the same file
    int rc = HIPC_OK;
    if (fseeko(f, 0, SEEK_END) != 0) rc = host_fail(HIPC_ERR_INVALID, "stat %s: %s", path.c_str(), strerror(errno));
    const uint64_t file_len = rc == HIPC_OK ? (uint64_t)ftello(f) : 0;
    const uint64_t offset = t.has_offset ? t.offset : 0;
    const uint64_t length = t.has_length ? t.length : (file_len > offset ? file_len - offset : 0);
    if (rc == HIPC_OK && offset + length < offset) rc = host_fail(HIPC_ERR_INVALID, "tensor '%s': offset+length overflow", name);
    if (rc == HIPC_OK && offset + length > file_len)
        rc = host_fail(HIPC_ERR_INVALID, "tensor '%s': requested bytes %llu..%llu of a file of %llu", name, (unsigned long long)offset,
                       (unsigned long long)(offset + length), (unsigned long long)file_len);
    *bytes = (size_t)length;
    if (rc == HIPC_OK && want_data) {
        out->resize((size_t)length);
        if (fseeko(f, (off_t)offset, SEEK_SET) != 0)
            rc = host_fail(HIPC_ERR_INVALID, "seeking %s to %llu: %s", path.c_str(), (unsigned long long)offset, strerror(errno));
        else if (length && fread(out->data(), 1, (size_t)length, f) != (size_t)length)
            rc = host_fail(HIPC_ERR_INVALID, "reading %llu bytes of %s at %llu", (unsigned long long)length, path.c_str(), (unsigned long long)offset);
    }
    fclose(f);
    return rc;
}

// the typed fields, narrowed to the width data_type says
int typed_payload(const Tensor &t, std::vector<uint8_t> *out) {
    switch (t.data_type) {
        case DT_FLOAT: for (uint64_t v : t.f32) put_le(*out, v, 4); return HIPC_OK;
        case DT_DOUBLE: for (uint64_t v : t.f64) put_le(*out, v, 8); return HIPC_OK;
        case DT_INT64: for (uint64_t v : t.i64) put_le(*out, v, 8); return HIPC_OK;
        case DT_UINT64: for (uint64_t v : t.u64) put_le(*out, v, 8); return HIPC_OK;
        case DT_UINT32: for (uint64_t v : t.u64) put_le(*out, v, 4); return HIPC_OK;
        case DT_INT32: for (uint64_t v : t.i32) put_le(*out, v, 4); return HIPC_OK;
        case DT_INT16: case DT_UINT16: case DT_FLOAT16: case DT_BFLOAT16: for (uint64_t v : t.i32) put_le(*out, v, 2); return HIPC_OK;
        case DT_INT8: case DT_UINT8: case DT_BOOL: for (uint64_t v : t.i32) put_le(*out, v, 1); return HIPC_OK;
        default: return host_fail(HIPC_ERR_UNSUPPORTED, "tensor '%s': dtype %d without a readable data field", t.name.c_str(), t.data_type);
    }
}

}  // namespace

extern "C" {

const char *hipc_host_error(void) { return g_host_error.c_str(); }

int hipc_initializer_read(const void *tensor, size_t len, const char *base_dir, hipc_initializer_info *info, void *data, size_t data_cap) {
    if (!tensor || !info) return host_fail(HIPC_ERR_INVALID, "hipc_initializer_read: null pointer");
    try {
        Tensor t;
        int rc = parse_tensor(tensor, len, &t);
        if (rc != HIPC_OK) return rc;
        if (t.dims.size() > HIPC_INITIALIZER_MAX_DIMS) return host_fail(HIPC_ERR_UNSUPPORTED, "tensor '%s': %zu dimensions", t.name.c_str(), t.dims.size());
        if (t.name.size() >= sizeof info->name) return host_fail(HIPC_ERR_UNSUPPORTED, "tensor name of %zu bytes", t.name.size());
        memset(info, 0, sizeof *info);
        info->data_type = t.data_type, info->n_dims = (int32_t)t.dims.size();
        for (size_t i = 0; i < t.dims.size(); i++) info->dims[i] = t.dims[i];
        memcpy(info->name, t.name.data(), t.name.size());
        std::vector<uint8_t> payload;
        const uint8_t *src = nullptr;
        if (t.external) {
            if ((rc = read_external(t, base_dir, &payload, &info->bytes, data != nullptr)) != HIPC_OK) return rc;
            src = payload.data();
        } else if (t.raw.n != 0) {
            info->bytes = t.raw.n, src = t.raw.p;
        } else {
            if ((rc = typed_payload(t, &payload)) != HIPC_OK) return rc;
            info->bytes = payload.size(), src = payload.data();
        }
        if (data) {
            if (data_cap < info->bytes) return host_fail(HIPC_ERR_INVALID, "tensor '%s': %zu bytes into a buffer of %zu", info->name, info->bytes, data_cap);
            if (info->bytes) memcpy(data, src, info->bytes);
        }
        return HIPC_OK;
    } catch (const std::exception &e) {
        return host_fail(HIPC_ERR_BACKEND, "hipc_initializer_read: %s", e.what());
    }
}

int hipc_model_initializers(const void *model, size_t len, size_t *offsets, size_t *sizes, int64_t cap, int64_t *count) {
    if (!model || !count) return host_fail(HIPC_ERR_INVALID, "hipc_model_initializers: null pointer");
    const uint8_t *base = static_cast<const uint8_t *>(model);
    Reader m(model, len);
    Span graph;
    bool have_graph = false;
    while (m.next())
        if (m.field == 7 && m.wire == 2) graph = m.bytes, have_graph = true;  // the last occurrence of a singular field counts
    if (m.bad()) return host_fail(HIPC_ERR_INVALID, "ModelProto decode: truncated or malformed field");
    if (!have_graph) return host_fail(HIPC_ERR_INVALID, "no graph in the model");
    Reader g(graph);
    int64_t n = 0, sparse = 0;
    while (g.next()) {
        if (g.wire != 2) continue;
        if (g.field == 15) sparse++;
        if (g.field != 5) continue;
        if (n < cap && offsets && sizes) offsets[n] = (size_t)(g.bytes.p - base), sizes[n] = g.bytes.n;
        n++;
    }
    if (g.bad()) return host_fail(HIPC_ERR_INVALID, "GraphProto decode: truncated or malformed field");
    if (sparse) return host_fail(HIPC_ERR_UNSUPPORTED, "%lld sparse initializers", (long long)sparse);
    *count = n;
    return HIPC_OK;
}

}  // extern "C"
