// GGUF v3 reader (declarations and purpose: gguf_q8.hpp).
//
// Container, little endian:
//   "GGUF", u32 version, u64 tensor count, u64 metadata count,
//   metadata entries  { text key, u32 type, value },
//   tensor entries    { text name, u32 rank, u64 dims[rank], u32 ggml type, u64 offset },
//   zero padding up to a multiple of general.alignment (32 if absent), tensor data.
//   text = u64 length + bytes; array value = u32 element type, u64 count, elements.
//
// The reader is a single forward pass over the read-only mapping.  Everything it needs to know
// about a metadata type comes from one table (width and how to widen it), so scalars, and the
// elements of arrays that are only skipped, share one code path; nested arrays are walked with an
// explicit stack of outstanding element counts rather than by recursion.  Tensors are found by
// name through a sorted index.
#include "gguf_q8.hpp"

#include <algorithm>
#include <cerrno>
#include <cstring>
#include <stdexcept>

#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

namespace qw3 {
namespace {

[[noreturn]] void reject(const std::string &what) { throw std::runtime_error("GGUF: " + what); }

// ---- the mapped file as a bounds-checked byte range ----------------------------------------
struct Bytes {
    const uint8_t *base = nullptr;
    uint64_t size = 0;
    uint64_t at = 0;   // read position of the forward pass

    const uint8_t *claim(uint64_t n, const char *what) {
        if (n > size - at) reject(std::string("file ends inside ") + what);
        const uint8_t *p = base + at;
        at += n;
        return p;
    }
    uint64_t word(unsigned width, const char *what) {   // unsigned little-endian integer of 1..8 bytes
        const uint8_t *p = claim(width, what);
        uint64_t v = 0;
        for (unsigned i = 0; i < width; ++i) v |= static_cast<uint64_t>(p[i]) << (8 * i);
        return v;
    }
    std::string text(const char *what) {
        const uint64_t n = word(8, what);
        if (n > (1ull << 30)) reject(std::string("text of ") + std::to_string(n) + " bytes in " + what);
        const uint8_t *p = claim(n, what);
        return std::string(reinterpret_cast<const char *>(p), static_cast<size_t>(n));
    }
};

// ---- metadata types, one row per GgufValueType -------------------------------------------------
enum class Widen : uint8_t { Unsigned, Signed, Real, Flag, Text, List };
struct TypeRow {
    uint8_t width;   // bytes of a scalar; 0 for text and arrays
    Widen widen;
};
constexpr TypeRow kTypes[] = {
    {1, Widen::Unsigned}, {1, Widen::Signed}, {2, Widen::Unsigned}, {2, Widen::Signed},   // u8 i8 u16 i16
    {4, Widen::Unsigned}, {4, Widen::Signed}, {4, Widen::Real},     {1, Widen::Flag},     // u32 i32 f32 bool
    {0, Widen::Text},     {0, Widen::List},   {8, Widen::Unsigned}, {8, Widen::Signed},   // string array u64 i64
    {8, Widen::Real},                                                                     // f64
};
constexpr uint32_t kTypeCount = sizeof(kTypes) / sizeof(kTypes[0]);

const TypeRow &type_row(uint32_t id) {
    if (id >= kTypeCount) reject("metadata type " + std::to_string(id) + " is not known");
    return kTypes[id];
}

void put_scalar(GgufValue &v, const TypeRow &row, uint64_t raw) {
    const unsigned bits = 8u * row.width;
    switch (row.widen) {
        case Widen::Unsigned: v.unsigned_value = raw; break;
        case Widen::Signed:   // sign-extend from `bits`
            v.signed_value = bits == 64 ? static_cast<int64_t>(raw)
                                        : static_cast<int64_t>(raw << (64 - bits)) >> (64 - bits);
            break;
        case Widen::Real:
            if (row.width == 4) {
                const uint32_t r32 = static_cast<uint32_t>(raw);
                float f;
                std::memcpy(&f, &r32, 4);
                v.float_value = f;
            } else {
                std::memcpy(&v.float_value, &raw, 8);
            }
            break;
        case Widen::Flag: v.bool_value = raw != 0; break;
        default: break;
    }
}

// An array value.  Arrays of text are kept; arrays of scalars are stepped over in one move;
// arrays of arrays are stepped over element by element with a stack of (element type, elements
// left) frames.  The value records the outermost count.
void read_array(Bytes &in, GgufValue &v) {
    struct Frame { uint32_t elem; uint64_t left; };
    std::vector<Frame> open;
    auto enter = [&](bool outermost) {
        Frame f;
        f.elem = static_cast<uint32_t>(in.word(4, "an array header"));
        f.left = in.word(8, "an array header");
        const TypeRow &row = type_row(f.elem);
        if (outermost) v.unsigned_value = f.left;
        if (row.widen == Widen::Text) {
            if (outermost) v.string_array.reserve(static_cast<size_t>(std::min<uint64_t>(f.left, 1u << 20)));
            for (uint64_t i = 0; i < f.left; ++i) {
                std::string s = in.text("an array of text");
                if (outermost) v.string_array.push_back(std::move(s));
            }
        } else if (row.widen == Widen::List) {
            open.push_back(f);
        } else {
            if (f.left > UINT64_MAX / row.width) reject("array of " + std::to_string(f.left) + " elements overflows");
            (void)in.claim(f.left * row.width, "an array");
        }
    };
    enter(true);
    while (!open.empty()) {
        if (open.back().left == 0) {
            open.pop_back();
            continue;
        }
        --open.back().left;
        enter(false);
    }
}

GgufValue read_value(Bytes &in, uint32_t type_id) {
    const TypeRow &row = type_row(type_id);
    GgufValue v;
    v.type = static_cast<GgufValueType>(type_id);
    if (row.widen == Widen::Text) v.string_value = in.text("a metadata value");
    else if (row.widen == Widen::List) read_array(in, v);
    else put_scalar(v, row, in.word(row.width, "a metadata value"));
    return v;
}

uint64_t product(uint64_t a, uint64_t b) {
    uint64_t r;
    if (__builtin_mul_overflow(a, b, &r)) reject("tensor size overflows 64 bits");
    return r;
}

// ---- ggml tensor types this reader can size: {id, elements per block, bytes per block, name} ----
struct GgmlType { uint32_t id; uint32_t per_block; uint32_t block_bytes; const char *name; };
constexpr GgmlType kGgml[] = {
    {0, 1, 4, "F32"}, {1, 1, 2, "F16"}, {8, 32, 34, "Q8_0"}, {9, 32, 36, "Q8_1"}, {24, 1, 1, "I8"},
    {25, 1, 2, "I16"}, {26, 1, 4, "I32"}, {27, 1, 8, "I64"}, {28, 1, 8, "F64"}, {30, 1, 2, "BF16"},
};

const GgmlType *ggml_type(uint32_t id) {
    for (const GgmlType &t : kGgml)
        if (t.id == id) return &t;
    return nullptr;
}

}  // namespace

struct GgufFile::Impl {
    std::string path;
    int fd = -1;
    void *map = MAP_FAILED;
    uint64_t size = 0;
    uint32_t version = 0;
    uint32_t alignment = 32;
    uint64_t data_offset = 0;
    std::unordered_map<std::string, GgufValue> metadata;
    std::vector<GgufTensorInfo> tensors;
    std::vector<uint32_t> by_name;   // tensor indices ordered by name

    void map_file();
    void parse();
    ~Impl() {
        if (map != MAP_FAILED) munmap(map, static_cast<size_t>(size));
        if (fd >= 0) close(fd);
    }
};

void GgufFile::Impl::map_file() {
    fd = open(path.c_str(), O_RDONLY | O_CLOEXEC);
    if (fd < 0) reject("cannot open " + path + " (" + std::strerror(errno) + ")");
    struct stat st{};
    if (fstat(fd, &st) != 0) reject("cannot stat " + path + " (" + std::strerror(errno) + ")");
    if (st.st_size <= 0) reject(path + " is empty");
    size = static_cast<uint64_t>(st.st_size);
    map = mmap(nullptr, static_cast<size_t>(size), PROT_READ, MAP_PRIVATE, fd, 0);
    if (map == MAP_FAILED) reject("cannot map " + path + " (" + std::strerror(errno) + ")");
}

void GgufFile::Impl::parse() {
    Bytes in{static_cast<const uint8_t *>(map), size, 0};
    if (std::memcmp(in.claim(4, "the header"), "GGUF", 4) != 0) reject(path + " does not start with the GGUF magic");
    version = static_cast<uint32_t>(in.word(4, "the header"));
    if (version != 3) reject("version " + std::to_string(version) + " is not supported (only 3 is)");
    const uint64_t n_tensors = in.word(8, "the header"), n_meta = in.word(8, "the header");

    for (uint64_t i = 0; i < n_meta; ++i) {
        std::string key = in.text("a metadata key");
        const uint32_t type_id = static_cast<uint32_t>(in.word(4, "a metadata entry"));
        metadata[std::move(key)] = read_value(in, type_id);
    }
    if (const auto a = metadata.find("general.alignment"); a != metadata.end()) {
        const uint64_t want = a->second.unsigned_value;
        if (want >= 1 && want <= (1u << 30)) alignment = static_cast<uint32_t>(want);
    }

    for (uint64_t i = 0; i < n_tensors; ++i) {
        GgufTensorInfo t;
        t.name = in.text("a tensor name");
        const uint64_t rank = in.word(4, "a tensor entry");
        if (rank > 8) reject("tensor " + t.name + " has rank " + std::to_string(rank) + " (at most 8)");
        t.dims.resize(static_cast<size_t>(rank));
        t.elements = 1;
        for (uint64_t &d : t.dims) {
            d = in.word(8, "a tensor entry");
            t.elements = product(t.elements, d);
        }
        t.type = static_cast<uint32_t>(in.word(4, "a tensor entry"));
        t.rel_offset = in.word(8, "a tensor entry");
        t.bytes = gguf_tensor_type_size(t.type, t.elements);
        tensors.push_back(std::move(t));
    }
    data_offset = (in.at + alignment - 1) / alignment * alignment;
    for (GgufTensorInfo &t : tensors) {
        if (__builtin_add_overflow(data_offset, t.rel_offset, &t.abs_offset) || t.abs_offset > size ||
            t.bytes > size - t.abs_offset)
            reject("tensor " + t.name + " lies outside the file");
    }
    by_name.resize(tensors.size());
    for (uint32_t i = 0; i < by_name.size(); ++i) by_name[i] = i;
    std::stable_sort(by_name.begin(), by_name.end(),
                     [&](uint32_t a, uint32_t b) { return tensors[a].name < tensors[b].name; });
}

GgufFile::GgufFile(const std::string &path) : impl_(new Impl) {
    impl_->path = path;
    impl_->map_file();
    impl_->parse();
}

GgufFile::~GgufFile() = default;

const std::string &GgufFile::path() const { return impl_->path; }
uint64_t GgufFile::size() const { return impl_->size; }
const uint8_t *GgufFile::data() const { return static_cast<const uint8_t *>(impl_->map); }
uint32_t GgufFile::version() const { return impl_->version; }
uint32_t GgufFile::alignment() const { return impl_->alignment; }
uint64_t GgufFile::tensor_data_offset() const { return impl_->data_offset; }
const std::unordered_map<std::string, GgufValue> &GgufFile::metadata() const { return impl_->metadata; }
const std::vector<GgufTensorInfo> &GgufFile::tensors() const { return impl_->tensors; }

// first tensor of that name in file order
const GgufTensorInfo *GgufFile::find_tensor(const std::string &name) const {
    const auto &t = impl_->tensors;
    const auto &idx = impl_->by_name;
    const auto it = std::lower_bound(idx.begin(), idx.end(), name,
                                     [&](uint32_t i, const std::string &n) { return t[i].name < n; });
    return it != idx.end() && t[*it].name == name ? &t[*it] : nullptr;
}

std::string gguf_tensor_type_name(uint32_t type) {
    const GgmlType *t = ggml_type(type);
    // the names the loader prints; integer types are sized but have no name of their own there
    if (t != nullptr && (type == 0 || type == 1 || type == 8 || type == 30)) return t->name;
    return "type" + std::to_string(type);
}

uint64_t gguf_tensor_type_size(uint32_t type, uint64_t elements) {
    const GgmlType *t = ggml_type(type);
    if (t == nullptr) return 0;   // a quantization this reader does not size
    if (elements % t->per_block != 0)
        reject(std::to_string(elements) + " elements of " + t->name + " do not fill whole blocks of " +
               std::to_string(t->per_block));
    return product(elements / t->per_block, t->block_bytes);
}

uint64_t gguf_tensor_rows(const GgufTensorInfo &t) {
    uint64_t rows = 1;
    for (size_t i = 1; i < t.dims.size(); ++i) rows *= t.dims[i];
    return rows;
}

uint64_t gguf_tensor_cols(const GgufTensorInfo &t) { return t.dims.empty() ? 1 : t.dims.front(); }

std::unique_ptr<DeviceWeight> gguf_upload_q8_0(HipQ8Backend &backend, const GgufFile &file, const std::string &name) {
    const GgufTensorInfo *t = file.find_tensor(name);
    if (t == nullptr || t->type != 8) return nullptr;
    return backend.weight_q8_0(file.data() + t->abs_offset, gguf_tensor_rows(*t), gguf_tensor_cols(*t), name.c_str());
}

}  // namespace qw3
