// C ABI, part 3: the GGUF container (gguf/format.zig, gguf/tensor_types.zig,
// gguf/tensor_catalog.zig) and the path from a file on disk to resident device
// weights (models/tensor_store.zig:370-392, :450-468 feeding insertWeightFromLoaded).
// Host code only.
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cstring>
#include <new>
#include <string>
#include <vector>

#include "antfly_hip_qmatmul.h"
#include "api_internal.h"

namespace {

constexpr uint64_t kDefaultAlignment = 32;  // format.zig:19

// gguf/tensor_types.zig:17-56 (ids), :160-219 (block geometry)
struct TypeRow {
    uint32_t raw;
    const char* name;
    uint32_t values_per_block;  // 0: not a block format handled by the generic rule
    uint32_t bytes_per_block;
    bool quantized;
};
constexpr TypeRow kTypes[] = {
    {0, "F32", 32, 128, false},    {1, "F16", 32, 64, false},     {2, "Q4_0", 32, 18, true},
    {3, "Q4_1", 32, 20, true},     {6, "Q5_0", 32, 22, true},     {7, "Q5_1", 32, 24, true},
    {8, "Q8_0", 32, 34, true},     {9, "Q8_1", 32, 36, true},     {10, "Q2_K", 256, 84, true},
    {11, "Q3_K", 256, 110, true},  {12, "Q4_K", 256, 144, true},  {13, "Q5_K", 256, 176, true},
    {14, "Q6_K", 256, 210, true},  {15, "Q8_K", 256, 292, true},  {16, "IQ2_XXS", 256, 66, true},
    {17, "IQ2_XS", 256, 74, true}, {18, "IQ3_XXS", 256, 98, true}, {19, "IQ1_S", 256, 50, true},
    {20, "IQ4_NL", 32, 18, true},  {21, "IQ3_S", 256, 110, true}, {22, "IQ2_S", 256, 82, true},
    {23, "IQ4_XS", 256, 136, true}, {24, "I8", 32, 32, false},    {25, "I16", 32, 64, false},
    {26, "I32", 32, 128, false},   {27, "I64", 32, 256, false},   {28, "F64", 32, 256, false},
    {29, "IQ1_M", 256, 56, true},  {30, "BF16", 32, 64, false},   {34, "TQ1_0", 256, 54, true},
    {35, "TQ2_0", 256, 66, true},  {36, "I2_S", 128, 32, true},   {37, "I8_S", 1, 1, true},
    {38, "TL1", 1, 1, true},       {39, "MXFP4", 32, 17, true},   {40, "NVFP4", 64, 36, true},
    {41, "Q1_0", 128, 18, true},
};

const TypeRow* find_type(uint32_t raw) {
    for (const TypeRow& t : kTypes)
        if (t.raw == raw) return &t;
    return nullptr;
}

bool mul_u64(uint64_t a, uint64_t b, uint64_t* out) { return !__builtin_mul_overflow(a, b, out); }

uint64_t align_forward(uint64_t value, uint64_t alignment) {  // format.zig:268-273
    if (alignment == 0 || alignment == 1) return value;
    const uint64_t rem = value % alignment;
    return rem == 0 ? value : value + (alignment - rem);
}

// tensor_types.byteLen, :238-260; 0 = unknown type or overflow.  `bitnet` selects the
// BitNet dialect, where raw type 39 is TL2 (:262-280) instead of MXFP4.
uint64_t byte_len(uint32_t raw, bool bitnet, const uint64_t* dims, size_t n) {
    uint64_t total = 1;
    for (size_t i = 0; i < n; ++i)
        if (!mul_u64(total, dims[i], &total)) return 0;
    if (bitnet && raw == 39) {  // TL2, :262-278: a 256-column dense prefix (4 bits per pair) + 5 bits per ternary triple
        if (n < 2 || dims[0] < 256) return 0;
        uint64_t rows = 1, a, b;
        for (size_t i = 1; i < n; ++i)
            if (!mul_u64(rows, dims[i], &rows)) return 0;
        if (!mul_u64(dims[0] - 256, rows, &a) || !mul_u64(256, rows, &b)) return 0;
        const uint64_t unaligned = a / 3 * 5 / 8 + b / 2 * 4 / 8;
        return align_forward(unaligned, 32) + 32;
    }
    const TypeRow* t = find_type(raw);
    if (!t) return 0;
    uint64_t r = 0;
    switch (raw) {
        case 0: return mul_u64(total, 4, &r) ? r : 0;
        case 1: case 30: case 25: return mul_u64(total, 2, &r) ? r : 0;
        case 24: case 37: return total;
        case 26: return mul_u64(total, 4, &r) ? r : 0;
        case 27: case 28: return mul_u64(total, 8, &r) ? r : 0;
        case 36: case 38: return (total + 3) / 4 + 32;  // I2_S, TL1
        default: break;
    }
    const uint64_t blocks = total / t->values_per_block + (total % t->values_per_block != 0);
    return mul_u64(blocks, t->bytes_per_block, &r) ? r : 0;
}

struct Metadata {
    std::string key;
    uint32_t value_type = 0;
    uint32_t element_type = 0;  // arrays
    uint64_t count = 0;         // arrays
    uint64_t u = 0;
    int64_t i = 0;
    double f = 0.0;
    std::string str;
};

struct TensorInfo {
    std::string name;
    std::vector<uint64_t> dimensions;
    uint32_t raw_type = 0;
    uint64_t offset = 0;
    uint64_t data_offset = 0;
};

struct Cursor {  // format.zig:275-298
    const uint8_t* bytes;
    size_t len;
    uint64_t pos = 0;

    afhip_status read_bytes(size_t count, const uint8_t** out) {
        if (pos > len || count > len - pos) return AFHIP_ERR_GGUF_UNEXPECTED_EOF;
        *out = bytes + pos;
        pos += count;
        return AFHIP_OK;
    }
    template <typename T>
    afhip_status read_int(T* out) {  // little-endian, as the host is
        const uint8_t* p;
        if (afhip_status s = read_bytes(sizeof(T), &p); s != AFHIP_OK) return s;
        std::memcpy(out, p, sizeof(T));
        return AFHIP_OK;
    }
    afhip_status read_string(std::string* out) {
        uint64_t n;
        if (afhip_status s = read_int(&n); s != AFHIP_OK) return s;
        if (n > len) return AFHIP_ERR_GGUF_UNEXPECTED_EOF;
        const uint8_t* p;
        if (afhip_status s = read_bytes(static_cast<size_t>(n), &p); s != AFHIP_OK) return s;
        out->assign(reinterpret_cast<const char*>(p), static_cast<size_t>(n));
        return AFHIP_OK;
    }
};

enum : uint32_t { kU8, kI8, kU16, kI16, kU32, kI32, kF32, kBool, kString, kArray, kU64, kI64, kF64 };  // format.zig:27-41

// One value of `type`; scalars land in `m` (arrays call this per element with a scratch entry).
afhip_status parse_value(Cursor& c, uint32_t type, Metadata* m, bool in_array) {
    switch (type) {
        case kU8: { uint8_t v; if (afhip_status s = c.read_int(&v); s != AFHIP_OK) return s; m->u = v; m->i = v; m->f = v; return AFHIP_OK; }
        case kI8: { int8_t v; if (afhip_status s = c.read_int(&v); s != AFHIP_OK) return s; m->i = v; m->u = static_cast<uint64_t>(static_cast<int64_t>(v)); m->f = v; return AFHIP_OK; }
        case kU16: { uint16_t v; if (afhip_status s = c.read_int(&v); s != AFHIP_OK) return s; m->u = v; m->i = v; m->f = v; return AFHIP_OK; }
        case kI16: { int16_t v; if (afhip_status s = c.read_int(&v); s != AFHIP_OK) return s; m->i = v; m->u = static_cast<uint64_t>(static_cast<int64_t>(v)); m->f = v; return AFHIP_OK; }
        case kU32: { uint32_t v; if (afhip_status s = c.read_int(&v); s != AFHIP_OK) return s; m->u = v; m->i = v; m->f = v; return AFHIP_OK; }
        case kI32: { int32_t v; if (afhip_status s = c.read_int(&v); s != AFHIP_OK) return s; m->i = v; m->u = static_cast<uint64_t>(static_cast<int64_t>(v)); m->f = v; return AFHIP_OK; }
        case kF32: { float v; if (afhip_status s = c.read_int(&v); s != AFHIP_OK) return s; m->f = v; return AFHIP_OK; }
        case kBool: { uint8_t v; if (afhip_status s = c.read_int(&v); s != AFHIP_OK) return s; m->u = v != 0; m->i = v != 0; return AFHIP_OK; }
        case kString: return c.read_string(&m->str);
        case kU64: { uint64_t v; if (afhip_status s = c.read_int(&v); s != AFHIP_OK) return s; m->u = v; m->i = static_cast<int64_t>(v); m->f = static_cast<double>(v); return AFHIP_OK; }
        case kI64: { int64_t v; if (afhip_status s = c.read_int(&v); s != AFHIP_OK) return s; m->i = v; m->u = static_cast<uint64_t>(v); m->f = static_cast<double>(v); return AFHIP_OK; }
        case kF64: { double v; if (afhip_status s = c.read_int(&v); s != AFHIP_OK) return s; m->f = v; return AFHIP_OK; }
        case kArray: {
            if (in_array) return AFHIP_ERR_GGUF_NESTED_ARRAY;
            uint32_t elem;
            if (afhip_status s = c.read_int(&elem); s != AFHIP_OK) return s;
            if (elem > kF64) return AFHIP_ERR_GGUF_UNSUPPORTED_METADATA;
            if (elem == kArray) return AFHIP_ERR_GGUF_NESTED_ARRAY;
            uint64_t count;
            if (afhip_status s = c.read_int(&count); s != AFHIP_OK) return s;
            m->element_type = elem;
            m->count = count;
            Metadata scratch;  // the elements are walked (bounds, strings) but not kept
            for (uint64_t i = 0; i < count; ++i)
                if (afhip_status s = parse_value(c, elem, &scratch, true); s != AFHIP_OK) return s;
            return AFHIP_OK;
        }
        default: return AFHIP_ERR_GGUF_UNSUPPORTED_METADATA;
    }
}

}  // namespace

struct afhip_gguf {
    const uint8_t* bytes = nullptr;
    size_t len = 0;
    void* mapping = nullptr;  // non-null: this object owns an mmap of `len` bytes
    uint32_t version = 0;
    uint64_t tensor_count = 0, metadata_count = 0;
    uint64_t alignment = kDefaultAlignment;
    uint64_t data_region_offset = 0;
    bool bitnet = false;
    std::vector<Metadata> metadata;
    std::vector<TensorInfo> tensors;
};

namespace {

afhip_status parse_into(afhip_gguf* g) {  // format.parse, :113-161
    Cursor c{g->bytes, g->len};
    const uint8_t* magic;
    if (afhip_status s = c.read_bytes(4, &magic); s != AFHIP_OK) return s;
    if (std::memcmp(magic, "GGUF", 4) != 0) return AFHIP_ERR_GGUF_INVALID_MAGIC;
    if (afhip_status s = c.read_int(&g->version); s != AFHIP_OK) return s;
    if (afhip_status s = c.read_int(&g->tensor_count); s != AFHIP_OK) return s;
    if (afhip_status s = c.read_int(&g->metadata_count); s != AFHIP_OK) return s;
    // every entry takes at least 12 bytes (key length + type), every tensor 24: counts beyond that are truncated files
    if (g->metadata_count > g->len / 12 || g->tensor_count > g->len / 24) return AFHIP_ERR_GGUF_UNEXPECTED_EOF;

    g->metadata.reserve(static_cast<size_t>(g->metadata_count));
    for (uint64_t i = 0; i < g->metadata_count; ++i) {
        Metadata m;
        if (afhip_status s = c.read_string(&m.key); s != AFHIP_OK) return s;
        if (afhip_status s = c.read_int(&m.value_type); s != AFHIP_OK) return s;
        if (m.value_type > kF64) return AFHIP_ERR_GGUF_UNSUPPORTED_METADATA;
        if (afhip_status s = parse_value(c, m.value_type, &m, false); s != AFHIP_OK) return s;
        g->metadata.push_back(std::move(m));
    }
    for (const Metadata& m : g->metadata) {  // readAlignment :236-247, tensorDialectFromMetadata :224-234 (first match decides)
        if (m.key == "general.alignment") {
            if (m.value_type == kU32 || m.value_type == kU64) g->alignment = m.u;
            break;
        }
    }
    for (const Metadata& m : g->metadata) {
        if (m.key == "general.architecture") {
            g->bitnet = m.value_type == kString && (m.str == "bitnet-b1.58" || m.str == "bitnet");
            break;
        }
    }

    g->tensors.reserve(static_cast<size_t>(g->tensor_count));
    for (uint64_t i = 0; i < g->tensor_count; ++i) {
        TensorInfo t;
        if (afhip_status s = c.read_string(&t.name); s != AFHIP_OK) return s;
        uint32_t n_dims;
        if (afhip_status s = c.read_int(&n_dims); s != AFHIP_OK) return s;
        if (n_dims > g->len / 8) return AFHIP_ERR_GGUF_UNEXPECTED_EOF;
        t.dimensions.resize(n_dims);
        for (uint32_t d = 0; d < n_dims; ++d)
            if (afhip_status s = c.read_int(&t.dimensions[d]); s != AFHIP_OK) return s;
        if (afhip_status s = c.read_int(&t.raw_type); s != AFHIP_OK) return s;
        if (afhip_status s = c.read_int(&t.offset); s != AFHIP_OK) return s;
        g->tensors.push_back(std::move(t));
    }
    // file-supplied alignment and offsets: sums that wrap 64 bits would pass the bounds check in
    // afhip_gguf_tensor_data with the wrong bytes, so they are refused here
    const uint64_t aligned = align_forward(c.pos, g->alignment);
    if (aligned < c.pos) return AFHIP_ERR_GGUF_UNEXPECTED_EOF;
    g->data_region_offset = aligned;
    for (TensorInfo& t : g->tensors)
        if (__builtin_add_overflow(g->data_region_offset, t.offset, &t.data_offset)) return AFHIP_ERR_GGUF_UNEXPECTED_EOF;
    return AFHIP_OK;
}

void fill_tensor_info(const afhip_gguf* g, const TensorInfo& t, afhip_gguf_tensor_info* out) {
    std::memset(out, 0, sizeof(*out));
    out->name = t.name.c_str();
    out->name_len = t.name.size();
    out->n_dimensions = static_cast<uint32_t>(t.dimensions.size());
    for (size_t i = 0; i < t.dimensions.size() && i < AFHIP_GGUF_MAX_DIMS; ++i) out->dimensions[i] = t.dimensions[i];
    out->tensor_type = t.raw_type;
    const TypeRow* row = find_type(t.raw_type);
    const bool tl2 = g->bitnet && t.raw_type == 39;
    out->type_name = tl2 ? "TL2" : (row ? row->name : "UNKNOWN");
    out->is_quantized = tl2 || !row || row->quantized;  // isQuantized: unknown types count as quantized
    out->offset = t.offset;
    out->data_offset = t.data_offset;
    out->byte_len = byte_len(t.raw_type, g->bitnet, t.dimensions.data(), t.dimensions.size());
}

void fill_metadata(const Metadata& m, afhip_gguf_metadata* out) {
    std::memset(out, 0, sizeof(*out));
    out->key = m.key.c_str();
    out->key_len = m.key.size();
    out->value_type = m.value_type;
    out->element_type = m.element_type;
    out->count = m.count;
    out->u64 = m.u;
    out->i64 = m.i;
    out->f64 = m.f;
    out->str = m.str.c_str();
    out->str_len = m.str.size();
}

const TensorInfo* find_tensor(const afhip_gguf* g, const char* name) {  // Catalog.find, tensor_catalog.zig:26-31
    for (const TensorInfo& t : g->tensors)
        if (t.name == name) return &t;
    return nullptr;
}

}  // namespace

extern "C" {

afhip_status afhip_gguf_parse(const void* bytes, size_t len, afhip_gguf** out) {
    if (!out || (!bytes && len != 0)) return AFHIP_ERR_INVALID_ARGUMENT;
    *out = nullptr;
    afhip_gguf* g = new (std::nothrow) afhip_gguf();
    if (!g) return AFHIP_ERR_OUT_OF_MEMORY;
    g->bytes = static_cast<const uint8_t*>(bytes);
    g->len = len;
    const afhip_status s = parse_into(g);
    if (s != AFHIP_OK) {
        delete g;
        return s;
    }
    *out = g;
    return AFHIP_OK;
}

afhip_status afhip_gguf_open(const char* path, afhip_gguf** out) {
    if (!path || !out) return AFHIP_ERR_INVALID_ARGUMENT;
    *out = nullptr;
    const int fd = ::open(path, O_RDONLY | O_CLOEXEC);
    if (fd < 0) return AFHIP_ERR_IO;
    struct stat st;
    if (::fstat(fd, &st) != 0 || st.st_size <= 0) {
        ::close(fd);
        return st.st_size == 0 ? AFHIP_ERR_GGUF_UNEXPECTED_EOF : AFHIP_ERR_IO;
    }
    const size_t len = static_cast<size_t>(st.st_size);
    void* map = ::mmap(nullptr, len, PROT_READ, MAP_PRIVATE, fd, 0);  // weights are read in place, never copied on the host
    ::close(fd);
    if (map == MAP_FAILED) return AFHIP_ERR_IO;
    afhip_gguf* g = new (std::nothrow) afhip_gguf();
    if (!g) {
        ::munmap(map, len);
        return AFHIP_ERR_OUT_OF_MEMORY;
    }
    g->bytes = static_cast<const uint8_t*>(map);
    g->len = len;
    g->mapping = map;
    const afhip_status s = parse_into(g);
    if (s != AFHIP_OK) {
        afhip_gguf_close(g);
        return s;
    }
    *out = g;
    return AFHIP_OK;
}

void afhip_gguf_close(afhip_gguf* g) {
    if (!g) return;
    if (g->mapping) ::munmap(g->mapping, g->len);
    delete g;
}

afhip_status afhip_gguf_get_summary(const afhip_gguf* g, afhip_gguf_summary* out) {
    if (!g || !out) return AFHIP_ERR_INVALID_ARGUMENT;
    out->version = g->version;
    out->tensor_count = g->tensor_count;
    out->metadata_count = g->metadata_count;
    out->alignment = g->alignment;
    out->data_region_offset = g->data_region_offset;
    out->file_len = g->len;
    return AFHIP_OK;
}

afhip_status afhip_gguf_tensor_at(const afhip_gguf* g, size_t index, afhip_gguf_tensor_info* out) {
    if (!g || !out) return AFHIP_ERR_INVALID_ARGUMENT;
    if (index >= g->tensors.size()) return AFHIP_ERR_TENSOR_NOT_FOUND;
    fill_tensor_info(g, g->tensors[index], out);
    return AFHIP_OK;
}

afhip_status afhip_gguf_find_tensor(const afhip_gguf* g, const char* name, afhip_gguf_tensor_info* out) {
    if (!g || !name || !out) return AFHIP_ERR_INVALID_ARGUMENT;
    const TensorInfo* t = find_tensor(g, name);
    if (!t) return AFHIP_ERR_TENSOR_NOT_FOUND;
    fill_tensor_info(g, *t, out);
    return AFHIP_OK;
}

afhip_status afhip_gguf_metadata_at(const afhip_gguf* g, size_t index, afhip_gguf_metadata* out) {
    if (!g || !out) return AFHIP_ERR_INVALID_ARGUMENT;
    if (index >= g->metadata.size()) return AFHIP_ERR_TENSOR_NOT_FOUND;
    fill_metadata(g->metadata[index], out);
    return AFHIP_OK;
}

afhip_status afhip_gguf_find_metadata(const afhip_gguf* g, const char* key, afhip_gguf_metadata* out) {
    if (!g || !key || !out) return AFHIP_ERR_INVALID_ARGUMENT;
    for (const Metadata& m : g->metadata) {
        if (m.key == key) {
            fill_metadata(m, out);
            return AFHIP_OK;
        }
    }
    return AFHIP_ERR_TENSOR_NOT_FOUND;
}

uint64_t afhip_gguf_tensor_byte_len(uint32_t tensor_type, int bitnet_dialect, const uint64_t* dimensions,
                                    size_t n_dimensions) {
    if (!dimensions && n_dimensions != 0) return 0;
    return byte_len(tensor_type, bitnet_dialect != 0, dimensions, n_dimensions);
}

afhip_status afhip_gguf_tensor_data(const afhip_gguf* g, const afhip_gguf_tensor_info* info, const void** data,
                                    size_t* len) {
    if (!g || !info || !data || !len) return AFHIP_ERR_INVALID_ARGUMENT;
    *data = nullptr;
    *len = 0;
    if (info->byte_len == 0) return AFHIP_ERR_UNSUPPORTED_TENSOR_TYPE;  // byteLen == null, tensor_store.zig:371
    if (info->data_offset > g->len || info->byte_len > g->len - info->data_offset) return AFHIP_ERR_GGUF_UNEXPECTED_EOF;
    *data = g->bytes + info->data_offset;
    *len = static_cast<size_t>(info->byte_len);
    return AFHIP_OK;
}

// ---- file -> resident device weight

afhip_status afhip_compute_insert_weight_from_gguf(afhip_compute* self, const afhip_gguf* g, const char* tensor_name,
                                                   const char* key, int keep_raw_layout) {
    if (!self || !g || !tensor_name) return AFHIP_ERR_INVALID_ARGUMENT;
    const TensorInfo* t = find_tensor(g, tensor_name);
    if (!t) return AFHIP_ERR_TENSOR_NOT_FOUND;
    afhip_gguf_tensor_info info;
    fill_tensor_info(g, *t, &info);
    const void* data;
    size_t len;
    if (afhip_status s = afhip_gguf_tensor_data(g, &info, &data, &len); s != AFHIP_OK) return s;
    // normalizedShapeFromDims, tensor_store.zig:654-658: GGUF lists the fastest dimension first
    if (t->dimensions.empty() || t->dimensions.size() > AFHIP_GGUF_MAX_DIMS) return AFHIP_ERR_INVALID_SHAPE;
    int64_t shape[AFHIP_GGUF_MAX_DIMS];
    const size_t rank = t->dimensions.size();
    for (size_t i = 0; i < rank; ++i) {
        if (t->dimensions[rank - 1 - i] > static_cast<uint64_t>(INT64_MAX)) return AFHIP_ERR_INVALID_SHAPE;
        shape[i] = static_cast<int64_t>(t->dimensions[rank - 1 - i]);
    }
    const char* name = key ? key : tensor_name;
    if (t->raw_type == AFHIP_TYPE_F32) {
        if (reinterpret_cast<uintptr_t>(data) % 4 != 0) return AFHIP_ERR_INVALID_STATE;
        return afhip_compute_insert_weight_f32(self, name, static_cast<const float*>(data), shape, rank);
    }
    if (t->raw_type != AFHIP_TYPE_Q4_0 && t->raw_type != AFHIP_TYPE_Q8_0 && t->raw_type != AFHIP_TYPE_Q4_K)
        return AFHIP_ERR_UNSUPPORTED_TENSOR_TYPE;
    return afhip_compute_insert_weight_from_loaded(self, name, static_cast<int>(t->raw_type), data, len, shape, rank,
                                                   keep_raw_layout);
}

afhip_status afhip_compute_load_gguf(afhip_compute* self, const afhip_gguf* g, int keep_raw_layout, size_t* loaded,
                                     size_t* skipped) {
    if (!self || !g) return AFHIP_ERR_INVALID_ARGUMENT;
    size_t n_loaded = 0, n_skipped = 0;
    for (const TensorInfo& t : g->tensors) {
        const bool supported = t.raw_type == AFHIP_TYPE_F32 || t.raw_type == AFHIP_TYPE_Q4_0 || t.raw_type == AFHIP_TYPE_Q8_0 ||
                               t.raw_type == AFHIP_TYPE_Q4_K;
        if (!supported) {
            ++n_skipped;
            continue;
        }
        const afhip_status s = afhip_compute_insert_weight_from_gguf(self, g, t.name.c_str(), nullptr, keep_raw_layout);
        if (s != AFHIP_OK) return s;
        ++n_loaded;
    }
    if (loaded) *loaded = n_loaded;
    if (skipped) *skipped = n_skipped;
    return AFHIP_OK;
}

}  // extern "C"
