// See gguf_q8.hpp.  Container layout (GGUF v3, little endian):
//   u32 magic "GGUF", u32 version, u64 tensor_count, u64 kv_count,
//   kv_count x { string key, u32 type, value },
//   tensor_count x { string name, u32 n_dims, u64 dims[n_dims], u32 type, u64 offset },
//   padding to `general.alignment` (32 unless the metadata says otherwise), tensor data.
// A string is a u64 length followed by the bytes; an array is u32 element type, u64 count, elements.
#include "gguf_q8.hpp"

#include <cerrno>
#include <cstring>
#include <stdexcept>

#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

namespace qw3 {
namespace {

constexpr uint32_t kMagic = 0x46554747u;   // "GGUF"
constexpr uint64_t kMaxString = 1ull << 30;

class Cursor {
public:
    Cursor(const uint8_t *p, uint64_t n) : p_(p), n_(n) {}
    uint64_t pos() const { return at_; }
    void need(uint64_t bytes) const {
        if (bytes > n_ - at_) throw std::runtime_error("truncated GGUF file");
    }
    template <class T>
    T scalar() {
        need(sizeof(T));
        T v;
        std::memcpy(&v, p_ + at_, sizeof(T));
        at_ += sizeof(T);
        return v;
    }
    std::string string() {
        const uint64_t len = scalar<uint64_t>();
        if (len > kMaxString) throw std::runtime_error("GGUF string is too large");
        need(len);
        std::string s(reinterpret_cast<const char *>(p_ + at_), static_cast<size_t>(len));
        at_ += len;
        return s;
    }
    void skip(uint64_t bytes) {
        need(bytes);
        at_ += bytes;
    }

private:
    const uint8_t *p_;
    uint64_t n_;
    uint64_t at_ = 0;
};

uint64_t scalar_size(GgufValueType t) {
    switch (t) {
        case GgufValueType::Uint8: case GgufValueType::Int8: case GgufValueType::Bool: return 1;
        case GgufValueType::Uint16: case GgufValueType::Int16: return 2;
        case GgufValueType::Uint32: case GgufValueType::Int32: case GgufValueType::Float32: return 4;
        case GgufValueType::Uint64: case GgufValueType::Int64: case GgufValueType::Float64: return 8;
        default: return 0;
    }
}

GgufValue read_value(Cursor &c, GgufValueType type) {
    GgufValue v;
    v.type = type;
    switch (type) {
        case GgufValueType::Uint8: v.unsigned_value = c.scalar<uint8_t>(); break;
        case GgufValueType::Int8: v.signed_value = c.scalar<int8_t>(); break;
        case GgufValueType::Uint16: v.unsigned_value = c.scalar<uint16_t>(); break;
        case GgufValueType::Int16: v.signed_value = c.scalar<int16_t>(); break;
        case GgufValueType::Uint32: v.unsigned_value = c.scalar<uint32_t>(); break;
        case GgufValueType::Int32: v.signed_value = c.scalar<int32_t>(); break;
        case GgufValueType::Uint64: v.unsigned_value = c.scalar<uint64_t>(); break;
        case GgufValueType::Int64: v.signed_value = c.scalar<int64_t>(); break;
        case GgufValueType::Float32: v.float_value = c.scalar<float>(); break;
        case GgufValueType::Float64: v.float_value = c.scalar<double>(); break;
        case GgufValueType::Bool: v.bool_value = c.scalar<uint8_t>() != 0; break;
        case GgufValueType::String: v.string_value = c.string(); break;
        case GgufValueType::Array: {
            const auto elem = static_cast<GgufValueType>(c.scalar<uint32_t>());
            const uint64_t count = c.scalar<uint64_t>();
            if (elem == GgufValueType::String) {
                v.string_array.reserve(static_cast<size_t>(count < (1u << 20) ? count : (1u << 20)));
                for (uint64_t i = 0; i < count; ++i) v.string_array.push_back(c.string());
            } else if (elem == GgufValueType::Array) {
                for (uint64_t i = 0; i < count; ++i) (void)read_value(c, GgufValueType::Array);
            } else {
                const uint64_t each = scalar_size(elem);
                if (each == 0) throw std::runtime_error("unknown GGUF metadata type");
                if (count > UINT64_MAX / each) throw std::runtime_error("GGUF array size overflow");
                c.skip(count * each);
            }
            v.unsigned_value = count;
            break;
        }
        default: throw std::runtime_error("unknown GGUF metadata type");
    }
    return v;
}

uint64_t mul_checked(uint64_t a, uint64_t b) {
    if (a != 0 && b > UINT64_MAX / a) throw std::runtime_error("GGUF tensor size overflow");
    return a * b;
}

uint64_t round_up(uint64_t v, uint64_t to) { return to == 0 ? v : (v + to - 1) / to * to; }

}  // namespace

struct GgufFile::Impl {
    std::string path;
    int fd = -1;
    const uint8_t *map = nullptr;
    uint64_t size = 0;
    uint32_t version = 0;
    uint32_t alignment = 32;
    uint64_t data_offset = 0;
    std::unordered_map<std::string, GgufValue> metadata;
    std::vector<GgufTensorInfo> tensors;
    std::unordered_map<std::string, size_t> by_name;
    ~Impl() {
        if (map) munmap(const_cast<uint8_t *>(map), static_cast<size_t>(size));
        if (fd >= 0) close(fd);
    }
};

GgufFile::GgufFile(const std::string &path) : impl_(new Impl) {
    Impl &m = *impl_;
    m.path = path;
    m.fd = open(path.c_str(), O_RDONLY);
    if (m.fd < 0) throw std::runtime_error("failed to open GGUF: " + path + ": " + std::strerror(errno));
    struct stat st{};
    if (fstat(m.fd, &st) != 0) throw std::runtime_error("failed to stat GGUF: " + path + ": " + std::strerror(errno));
    if (st.st_size <= 0) throw std::runtime_error("empty GGUF: " + path);
    m.size = static_cast<uint64_t>(st.st_size);
    void *p = mmap(nullptr, static_cast<size_t>(m.size), PROT_READ, MAP_PRIVATE, m.fd, 0);
    if (p == MAP_FAILED) throw std::runtime_error("failed to mmap GGUF: " + path + ": " + std::strerror(errno));
    m.map = static_cast<const uint8_t *>(p);

    Cursor c(m.map, m.size);
    if (c.scalar<uint32_t>() != kMagic) throw std::runtime_error("not a GGUF file: " + path);
    m.version = c.scalar<uint32_t>();
    if (m.version != 3) throw std::runtime_error("only GGUF v3 is supported");
    const uint64_t n_tensors = c.scalar<uint64_t>();
    const uint64_t n_kv = c.scalar<uint64_t>();
    for (uint64_t i = 0; i < n_kv; ++i) {
        std::string key = c.string();
        const auto type = static_cast<GgufValueType>(c.scalar<uint32_t>());
        m.metadata[std::move(key)] = read_value(c, type);
    }
    if (const auto it = m.metadata.find("general.alignment"); it != m.metadata.end()) {
        const uint64_t a = it->second.unsigned_value;
        if (a != 0 && a <= (1u << 30)) m.alignment = static_cast<uint32_t>(a);
    }
    for (uint64_t i = 0; i < n_tensors; ++i) {
        GgufTensorInfo t;
        t.name = c.string();
        const uint32_t rank = c.scalar<uint32_t>();
        if (rank > 8) throw std::runtime_error("unsupported GGUF tensor rank");
        t.elements = 1;
        for (uint32_t d = 0; d < rank; ++d) {
            t.dims.push_back(c.scalar<uint64_t>());
            t.elements = mul_checked(t.elements, t.dims.back());
        }
        t.type = c.scalar<uint32_t>();
        t.rel_offset = c.scalar<uint64_t>();
        t.bytes = gguf_tensor_type_size(t.type, t.elements);
        m.by_name.emplace(t.name, m.tensors.size());
        m.tensors.push_back(std::move(t));
    }
    m.data_offset = round_up(c.pos(), m.alignment);
    for (GgufTensorInfo &t : m.tensors) {
        t.abs_offset = m.data_offset + t.rel_offset;
        if (t.abs_offset > m.size || t.bytes > m.size - t.abs_offset)
            throw std::runtime_error("GGUF tensor points outside file: " + t.name);
    }
}

GgufFile::~GgufFile() = default;

const std::string &GgufFile::path() const { return impl_->path; }
uint64_t GgufFile::size() const { return impl_->size; }
const uint8_t *GgufFile::data() const { return impl_->map; }
uint32_t GgufFile::version() const { return impl_->version; }
uint32_t GgufFile::alignment() const { return impl_->alignment; }
uint64_t GgufFile::tensor_data_offset() const { return impl_->data_offset; }
const std::unordered_map<std::string, GgufValue> &GgufFile::metadata() const { return impl_->metadata; }
const std::vector<GgufTensorInfo> &GgufFile::tensors() const { return impl_->tensors; }

const GgufTensorInfo *GgufFile::find_tensor(const std::string &name) const {
    const auto it = impl_->by_name.find(name);
    return it == impl_->by_name.end() ? nullptr : &impl_->tensors[it->second];
}

std::string gguf_tensor_type_name(uint32_t type) {
    switch (type) {
        case 0: return "F32";
        case 1: return "F16";
        case 8: return "Q8_0";
        case 30: return "BF16";
        default: return "type" + std::to_string(type);
    }
}

uint64_t gguf_tensor_type_size(uint32_t type, uint64_t elements) {
    auto blocks = [&](uint64_t per_block, uint64_t block_bytes) {
        if (elements % per_block != 0)
            throw std::runtime_error("quantized GGUF tensor elements are not block aligned");
        return mul_checked(elements / per_block, block_bytes);
    };
    switch (type) {
        case 0: return mul_checked(elements, 4);    // F32
        case 1: return mul_checked(elements, 2);    // F16
        case 8: return blocks(32, 34);              // Q8_0: fp16 scale + 32 int8
        case 9: return blocks(32, 36);              // Q8_1
        case 24: return elements;                   // I8
        case 25: return mul_checked(elements, 2);   // I16
        case 26: return mul_checked(elements, 4);   // I32
        case 27: return mul_checked(elements, 8);   // I64
        case 28: return mul_checked(elements, 8);   // F64
        case 30: return mul_checked(elements, 2);   // BF16
        default: return 0;                          // other quantized types: not sized here
    }
}

uint64_t gguf_tensor_rows(const GgufTensorInfo &t) {
    uint64_t rows = 1;
    for (size_t i = 1; i < t.dims.size(); ++i) rows *= t.dims[i];
    return rows;
}

uint64_t gguf_tensor_cols(const GgufTensorInfo &t) { return t.dims.empty() ? 1 : t.dims[0]; }

std::unique_ptr<DeviceWeight> gguf_upload_q8_0(HipQ8Backend &backend, const GgufFile &file, const std::string &name) {
    const GgufTensorInfo *t = file.find_tensor(name);
    if (t == nullptr || t->type != 8) return nullptr;
    return backend.weight_q8_0(file.data() + t->abs_offset, gguf_tensor_rows(*t), gguf_tensor_cols(*t), name.c_str());
}

}  // namespace qw3
