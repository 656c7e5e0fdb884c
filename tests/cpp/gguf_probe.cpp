// Test driver (no GPU): opens a GGUF file with qw3::GgufFile and prints what it parsed, one
// record per line, for tests/test_gguf_reader.py to compare with what it wrote.
//   header <version> <alignment> <tensor_data_offset> <n_tensors> <n_metadata>
//   kv <key> <type> <value>
//   tensor <name> <type> <type_name> <rows> <cols> <rel_offset> <abs_offset> <bytes> <fnv1a64 of the data>
// A parse error prints "error <message>" and exits with status 2.
#include <cinttypes>
#include <cstdio>
#include <exception>

#include "gguf_q8.hpp"

int main(int argc, char **argv) {
    if (argc != 2) {
        std::fprintf(stderr, "usage: gguf_probe <file.gguf>\n");
        return 1;
    }
    try {
        const qw3::GgufFile f(argv[1]);
        std::printf("header %u %u %" PRIu64 " %zu %zu\n", f.version(), f.alignment(), f.tensor_data_offset(),
                    f.tensors().size(), f.metadata().size());
        for (const auto &kv : f.metadata()) {
            const qw3::GgufValue &v = kv.second;
            std::printf("kv %s %u ", kv.first.c_str(), static_cast<unsigned>(v.type));
            switch (v.type) {
                case qw3::GgufValueType::String: std::printf("%s\n", v.string_value.c_str()); break;
                case qw3::GgufValueType::Float32:
                case qw3::GgufValueType::Float64: std::printf("%.9g\n", v.float_value); break;
                case qw3::GgufValueType::Bool: std::printf("%d\n", v.bool_value ? 1 : 0); break;
                case qw3::GgufValueType::Int8:
                case qw3::GgufValueType::Int16:
                case qw3::GgufValueType::Int32:
                case qw3::GgufValueType::Int64: std::printf("%" PRId64 "\n", v.signed_value); break;
                case qw3::GgufValueType::Array:
                    std::printf("%" PRIu64, v.unsigned_value);
                    for (const auto &s : v.string_array) std::printf(" %s", s.c_str());
                    std::printf("\n");
                    break;
                default: std::printf("%" PRIu64 "\n", v.unsigned_value); break;
            }
        }
        for (const auto &t : f.tensors()) {
            uint64_t h = 1469598103934665603ull;
            for (uint64_t i = 0; i < t.bytes; ++i) h = (h ^ f.data()[t.abs_offset + i]) * 1099511628211ull;
            std::printf("tensor %s %u %s %" PRIu64 " %" PRIu64 " %" PRIu64 " %" PRIu64 " %" PRIu64 " %016" PRIx64 "\n",
                        t.name.c_str(), t.type, qw3::gguf_tensor_type_name(t.type).c_str(), qw3::gguf_tensor_rows(t),
                        qw3::gguf_tensor_cols(t), t.rel_offset, t.abs_offset, t.bytes, h);
        }
    } catch (const std::exception &e) {
        std::printf("error %s\n", e.what());
        return 2;
    }
    return 0;
}
