// GGUF v3 reader: header parsing with the reference's validation, limits and messages
// (crates/runtime/src/gguf.rs:682-957), positioned tensor reads (:959-994) and the upload of a
// tensor's bytes into device memory. Host code; the only HIP calls are the copies of the upload.
#pragma once

#include <cstdint>
#include <string>
#include <vector>

namespace et {
namespace gguf {

// Outcome categories of GgufParseError (gguf.rs:80-105).
enum class Failure { kNone, kInvalid, kIo, kCancelled };

struct Error {
    Failure kind = Failure::kNone;
    std::string message;  // with the "gguf: " prefix of the reference's Display
};

// GGUF metadata value type codes 0..12 (gguf.rs:617-650); 9 = array.
struct Value {
    uint32_t type = 0;
    uint32_t element_type = 0;         // arrays only
    std::vector<uint64_t> integers;    // unsigned and bool payloads (zero-extended)
    std::vector<int64_t> signed_integers;
    std::vector<double> reals;         // f32 widened exactly, f64
    std::vector<std::string> strings;
    uint64_t length() const;
};

struct Entry {
    std::string key;
    Value value;
};

struct Tensor {
    std::string name;
    uint32_t format;                       // GGML type code: 0 F32, 2 Q4_0, 8 Q8_0, 10..14 Q2_K..Q6_K
    std::vector<uint64_t> logical_shape;   // row-major
    std::vector<uint64_t> physical_shape;  // F32: = logical; quantized: [rows, encoded_row_bytes]
    uint64_t data_offset = 0;              // absolute, validated against the file and the other tensors
    uint64_t byte_len = 0;
};

struct File {
    int fd = -1;
    uint64_t file_len = 0;
    std::string architecture;
    std::vector<Entry> metadata;  // file order
    std::vector<Tensor> tensors;  // file order
    void* staging[2] = {nullptr, nullptr};  // pinned buffers of the upload, allocated on first use
    ~File();
};

// parse_gguf (gguf.rs:682-957). On failure returns nullptr and fills *error.
File* open(const char* path, const volatile int32_t* cancel, Error* error);
// read_gguf_tensor_into (gguf.rs:959-994): exactly tensor.byte_len bytes into host memory.
bool read_tensor(const File& file, const Tensor& tensor, void* destination, uint64_t destination_bytes,
                 const volatile int32_t* cancel, Error* error);
// The same bytes into device memory through two pinned staging buffers; returns when they are there.
bool upload_tensor(File& file, const Tensor& tensor, void* device_destination, uint64_t destination_bytes,
                   void* stream, const volatile int32_t* cancel, Error* error);

}  // namespace gguf
}  // namespace et
