#include "gguf.h"

#include <fcntl.h>
#include <hip/hip_runtime_api.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <cerrno>
#include <cstring>
#include <unordered_set>

namespace et {
namespace gguf {
namespace {

// gguf.rs:63-76
constexpr uint32_t kVersion = 3;
constexpr uint32_t kQuantizationVersion = 2;
constexpr uint64_t kDefaultAlignment = 32;
constexpr uint64_t kSafeInteger = 9007199254740991ull;
constexpr uint64_t kReadChunkBytes = 8ull * 1024 * 1024;
constexpr uint64_t kHeaderReadChunkBytes = 64ull * 1024;
constexpr uint64_t kMaxHeaderBytes = 64ull * 1024 * 1024;
constexpr uint64_t kMaxMetadataCount = 4096;
constexpr uint64_t kMaxTensorCount = 65536;
constexpr uint64_t kMaxMetadataKeyBytes = 65535;
constexpr uint64_t kMaxTensorNameBytes = 64;
constexpr uint64_t kMaxMetadataStringBytes = 16ull * 1024 * 1024;
constexpr uint64_t kMaxMetadataArrayElements = 1048576;

struct Stop {  // thrown inside this file only, caught in open()
    Failure kind;
    std::string message;
};

[[noreturn]] void invalid(const std::string& message) { throw Stop{Failure::kInvalid, message}; }
[[noreturn]] void io_failed(const std::string& message) { throw Stop{Failure::kIo, message}; }

// Rust's {:?} of a str: quotes and backslashes escaped, NUL, tab, CR and LF by name, the other
// control characters (C0, DEL, C1) as \u{hex}; everything else as it is. The text is valid UTF-8.
std::string quoted(const std::string& text) {
    static const char* digits = "0123456789abcdef";
    const auto hex = [&](uint32_t code) {
        std::string out = "\\u{";
        bool started = false;
        for (int shift = 28; shift >= 0; shift -= 4) {
            const uint32_t nibble = (code >> shift) & 0xf;
            if (nibble != 0 || started || shift == 0) {
                out += digits[nibble];
                started = true;
            }
        }
        return out + "}";
    };
    std::string out = "\"";
    for (size_t i = 0; i < text.size(); i++) {
        const unsigned char c = static_cast<unsigned char>(text[i]);
        if (c == '"' || c == '\\') {
            out += '\\';
            out += static_cast<char>(c);
        } else if (c == 0) {
            out += "\\0";
        } else if (c == '\n') {
            out += "\\n";
        } else if (c == '\t') {
            out += "\\t";
        } else if (c == '\r') {
            out += "\\r";
        } else if (c < 0x20 || c == 0x7f) {
            out += hex(c);
        } else if (c == 0xc2 && i + 1 < text.size() && static_cast<unsigned char>(text[i + 1]) < 0xa0) {
            out += hex(static_cast<unsigned char>(text[i + 1]));  // U+0080..U+009F
            i++;
        } else {
            out += static_cast<char>(c);
        }
    }
    return out + "\"";
}

bool valid_utf8(const std::string& s) {
    size_t i = 0;
    const auto* p = reinterpret_cast<const unsigned char*>(s.data());
    while (i < s.size()) {
        const unsigned char c = p[i];
        size_t extra;
        uint32_t code;
        if (c < 0x80) { extra = 0; code = c; }
        else if ((c & 0xe0) == 0xc0) { extra = 1; code = c & 0x1f; }
        else if ((c & 0xf0) == 0xe0) { extra = 2; code = c & 0x0f; }
        else if ((c & 0xf8) == 0xf0) { extra = 3; code = c & 0x07; }
        else return false;
        if (i + extra >= s.size() && extra != 0) return false;
        for (size_t k = 1; k <= extra; k++) {
            if (i + k >= s.size() || (p[i + k] & 0xc0) != 0x80) return false;
            code = (code << 6) | (p[i + k] & 0x3f);
        }
        if ((extra == 1 && code < 0x80) || (extra == 2 && code < 0x800) || (extra == 3 && code < 0x10000) ||
            code > 0x10ffff || (code >= 0xd800 && code <= 0xdfff))
            return false;
        i += extra + 1;
    }
    return true;
}

// HeaderReader (gguf.rs:356-507): a bounds-checked sequential cursor over the header.
struct Reader {
    int fd;
    uint64_t file_len;
    uint64_t position = 0;
    const volatile int32_t* cancel;
    // read-ahead window: the header is a long run of small fields
    std::vector<char> window;
    uint64_t window_start = 0;

    void check_cancelled() const {
        if (cancel != nullptr && *cancel != 0) throw Stop{Failure::kCancelled, ""};
    }
    void read_exact(void* output, uint64_t length) {
        check_cancelled();
        if (position + length < position) invalid("header position overflows");
        const uint64_t end = position + length;
        if (end > file_len) invalid("unexpected end of file in header");
        if (end > kMaxHeaderBytes)
            invalid("header exceeds the " + std::to_string(kMaxHeaderBytes) + "-byte resource limit");
        auto* out = static_cast<char*>(output);
        uint64_t done = 0;
        while (done < length) {
            if (position < window_start || position >= window_start + window.size()) {
                check_cancelled();  // once per chunk of header I/O
                fill_window();
            }
            const uint64_t at = position - window_start;
            const uint64_t chunk = std::min<uint64_t>(window.size() - at, length - done);
            std::memcpy(out + done, window.data() + at, chunk);
            done += chunk;
            position += chunk;
        }
    }
    void fill_window() {
        const uint64_t want = std::min(kHeaderReadChunkBytes, file_len - position);  // > 0: the caller checked
        window.resize(want);
        window_start = position;
        uint64_t got = 0;
        while (got < want) {
            const ssize_t n = pread(fd, window.data() + got, want - got, static_cast<off_t>(position + got));
            if (n < 0) {
                if (errno == EINTR) continue;
                window.clear();
                io_failed(std::strerror(errno));
            }
            if (n == 0) {
                window.clear();
                io_failed("failed to fill whole buffer");
            }
            got += static_cast<uint64_t>(n);
        }
    }
    template <class T>
    T read() {
        T value;
        read_exact(&value, sizeof value);  // little-endian host
        return value;
    }
    bool read_bool() {
        const uint8_t value = read<uint8_t>();
        if (value > 1) invalid("invalid boolean metadata byte " + std::to_string(value));
        return value == 1;
    }
    // count (gguf.rs:463-486): against the hard maximum and the bytes that remain, before allocating
    uint64_t count(uint64_t value, const char* what, uint64_t minimum_bytes, uint64_t maximum) const {
        if (value > maximum)
            invalid(std::string(what) + " count " + std::to_string(value) + " exceeds the resource limit " +
                    std::to_string(maximum));
        const uint64_t bound = std::min(file_len, kMaxHeaderBytes);
        const uint64_t remaining = bound > position ? bound - position : 0;
        if (minimum_bytes > 0 && value > remaining / minimum_bytes)
            invalid(std::string(what) + " count " + std::to_string(value) + " exceeds the remaining file");
        return value;
    }
    std::string read_string(const char* what, uint64_t maximum) {
        const uint64_t byte_len = read<uint64_t>();
        const uint64_t length = count(byte_len, what, 1, maximum);
        std::string text(length, '\0');
        read_exact(text.data(), length);
        if (!valid_utf8(text)) invalid(std::string(what) + " is not valid UTF-8");
        return text;
    }
};

uint64_t checked_u64(uint64_t value, const char* what) {
    if (value > kSafeInteger)
        invalid(std::string(what) + " value " + std::to_string(value) + " is outside the JavaScript safe integer range");
    return value;
}
int64_t checked_i64(int64_t value, const char* what) {
    if (value < -static_cast<int64_t>(kSafeInteger) || value > static_cast<int64_t>(kSafeInteger))
        invalid(std::string(what) + " value " + std::to_string(value) + " is outside the JavaScript safe integer range");
    return value;
}

void read_scalar(Reader& reader, uint32_t type, Value* value, const char* what_u64, const char* what_i64,
                 const char* what_string) {
    switch (type) {
        case 0: value->integers.push_back(reader.read<uint8_t>()); break;
        case 1: value->signed_integers.push_back(reader.read<int8_t>()); break;
        case 2: value->integers.push_back(reader.read<uint16_t>()); break;
        case 3: value->signed_integers.push_back(reader.read<int16_t>()); break;
        case 4: value->integers.push_back(reader.read<uint32_t>()); break;
        case 5: value->signed_integers.push_back(reader.read<int32_t>()); break;
        case 6: value->reals.push_back(static_cast<double>(reader.read<float>())); break;
        case 7: value->integers.push_back(reader.read_bool() ? 1 : 0); break;
        case 8: value->strings.push_back(reader.read_string(what_string, kMaxMetadataStringBytes)); break;
        case 10: value->integers.push_back(checked_u64(reader.read<uint64_t>(), what_u64)); break;
        case 11: value->signed_integers.push_back(checked_i64(reader.read<int64_t>(), what_i64)); break;
        case 12: value->reals.push_back(reader.read<double>()); break;
        default: break;
    }
}

// read_array (gguf.rs:537-615)
void read_array(Reader& reader, Value* value) {
    const uint32_t element_type = reader.read<uint32_t>();
    if (element_type == 9) invalid("nested metadata arrays are not supported by this parser");
    const uint64_t raw_count = reader.read<uint64_t>();
    uint64_t minimum_bytes;
    switch (element_type) {
        case 0: case 1: case 7: minimum_bytes = 1; break;
        case 2: case 3: minimum_bytes = 2; break;
        case 4: case 5: case 6: minimum_bytes = 4; break;
        case 8: case 10: case 11: case 12: minimum_bytes = 8; break;
        default: invalid("unsupported metadata array element type " + std::to_string(element_type));
    }
    const uint64_t count = reader.count(raw_count, "metadata array", minimum_bytes, kMaxMetadataArrayElements);
    value->element_type = element_type;
    for (uint64_t i = 0; i < count; i++)
        read_scalar(reader, element_type, value, "metadata u64 array", "metadata i64 array", "metadata array string");
}

// read_metadata_value (gguf.rs:617-650)
void read_value(Reader& reader, uint32_t type, Value* value) {
    value->type = type;
    if (type == 9) return read_array(reader, value);
    if (type > 12) invalid("unsupported metadata value type " + std::to_string(type));
    read_scalar(reader, type, value, "metadata u64", "metadata i64", "metadata string");
}

struct Format {
    const char* name;
    uint64_t block_values, block_bytes;  // 0: dense f32
};

// GgufTensorFormat::from_code (gguf.rs:278-292) plus the two legacy block formats this library
// also contracts (GGML type codes 2 and 8).
Format format_of(uint32_t code) {
    switch (code) {
        case 0: return {"F32", 0, 0};
        case 2: return {"Q4_0", 32, 18};
        case 8: return {"Q8_0", 32, 34};
        case 10: return {"Q2_K", 256, 84};
        case 11: return {"Q3_K", 256, 110};
        case 12: return {"Q4_K", 256, 144};
        case 13: return {"Q5_K", 256, 176};
        case 14: return {"Q6_K", 256, 210};
        default: invalid("unsupported GGML tensor type code " + std::to_string(code));
    }
}

uint64_t checked_mul(uint64_t a, uint64_t b, const std::string& overflow_message) {
    if (a != 0 && b > UINT64_MAX / a) invalid(overflow_message);
    return a * b;
}

const Entry* find(const std::vector<Entry>& metadata, const char* key) {
    for (const Entry& entry : metadata)
        if (entry.key == key) return &entry;
    return nullptr;
}

struct RawTensor {
    std::string name;
    std::vector<uint64_t> dimensions;  // least-major first, as stored
    uint32_t format;
    uint64_t relative_offset;
};

void parse(Reader& reader, File* file) {
    char magic[4];
    reader.read_exact(magic, 4);
    if (std::memcmp(magic, "GGUF", 4) != 0) invalid("invalid magic");
    const uint32_t version = reader.read<uint32_t>();
    if (version != kVersion)
        invalid("unsupported version " + std::to_string(version) + "; expected version " + std::to_string(kVersion));
    const uint64_t raw_tensor_count = reader.read<uint64_t>();
    const uint64_t raw_metadata_count = reader.read<uint64_t>();
    const uint64_t metadata_count = reader.count(raw_metadata_count, "metadata", 13, kMaxMetadataCount);
    const uint64_t tensor_count = reader.count(raw_tensor_count, "tensor", 32, kMaxTensorCount);

    std::unordered_set<std::string> keys;
    file->metadata.reserve(metadata_count);
    for (uint64_t i = 0; i < metadata_count; i++) {
        Entry entry;
        entry.key = reader.read_string("metadata key", kMaxMetadataKeyBytes);
        if (entry.key.empty()) invalid("metadata key must not be empty");
        if (!keys.insert(entry.key).second) invalid("duplicate metadata key " + quoted(entry.key));
        const uint32_t type = reader.read<uint32_t>();
        read_value(reader, type, &entry.value);
        file->metadata.push_back(std::move(entry));
    }

    const Entry* architecture = find(file->metadata, "general.architecture");
    if (architecture == nullptr) invalid("missing general.architecture metadata");
    if (architecture->value.type != 8) invalid("general.architecture metadata must be a string");
    if (architecture->value.strings[0].empty()) invalid("general.architecture metadata must not be empty");
    file->architecture = architecture->value.strings[0];

    uint64_t alignment = kDefaultAlignment;
    if (const Entry* entry = find(file->metadata, "general.alignment")) {
        if (entry->value.type != 4) invalid("general.alignment metadata must be u32");
        alignment = entry->value.integers[0];
    }
    if (alignment == 0 || (alignment & (alignment - 1)) != 0)
        invalid("general.alignment must be a positive power of two, got " + std::to_string(alignment));

    std::vector<RawTensor> raw_tensors;
    raw_tensors.reserve(tensor_count);
    std::unordered_set<std::string> names;
    bool has_quantized = false;
    for (uint64_t i = 0; i < tensor_count; i++) {
        RawTensor raw;
        raw.name = reader.read_string("tensor name", kMaxTensorNameBytes);
        if (raw.name.empty()) invalid("tensor name must not be empty");
        if (!names.insert(raw.name).second) invalid("duplicate tensor name " + quoted(raw.name));
        const uint32_t rank = reader.read<uint32_t>();
        if (rank < 1 || rank > 4)
            invalid("tensor " + quoted(raw.name) + " rank must be in 1..=4, got " + std::to_string(rank));
        for (uint32_t d = 0; d < rank; d++) {
            const uint64_t dimension = reader.read<uint64_t>();
            if (dimension == 0 || dimension > kSafeInteger)
                invalid("tensor " + quoted(raw.name) + " has invalid dimension " + std::to_string(dimension));
            raw.dimensions.push_back(dimension);
        }
        raw.format = reader.read<uint32_t>();
        has_quantized |= format_of(raw.format).block_bytes != 0;
        raw.relative_offset = reader.read<uint64_t>();
        if (raw.relative_offset % alignment != 0)
            invalid("tensor " + quoted(raw.name) + " offset " + std::to_string(raw.relative_offset) +
                    " is not aligned to " + std::to_string(alignment));
        raw_tensors.push_back(std::move(raw));
    }

    if (has_quantized) {
        const Entry* entry = find(file->metadata, "general.quantization_version");
        if (entry == nullptr) invalid("missing general.quantization_version metadata for quantized tensors");
        if (entry->value.type != 4) invalid("general.quantization_version metadata must be u32");
        if (entry->value.integers[0] != kQuantizationVersion)
            invalid("unsupported general.quantization_version " + std::to_string(entry->value.integers[0]) +
                    "; expected " + std::to_string(kQuantizationVersion));
    }

    if (reader.position + (alignment - 1) < reader.position) invalid("aligned tensor-data offset overflows");
    const uint64_t data_start = (reader.position + (alignment - 1)) & ~(alignment - 1);
    if (data_start > reader.file_len) invalid("aligned tensor-data section starts beyond the file");

    file->tensors.reserve(tensor_count);
    for (RawTensor& raw : raw_tensors) {
        Tensor tensor;
        tensor.format = raw.format;
        tensor.logical_shape.assign(raw.dimensions.rbegin(), raw.dimensions.rend());
        const Format format = format_of(raw.format);
        if (format.block_bytes == 0) {
            uint64_t elements = 1;
            for (uint64_t d : tensor.logical_shape)
                elements = checked_mul(elements, d, "tensor " + quoted(raw.name) + " size overflows");
            tensor.byte_len = checked_mul(elements, 4, "tensor " + quoted(raw.name) + " byte length overflows");
            tensor.physical_shape = tensor.logical_shape;
        } else {
            const uint64_t columns = raw.dimensions[0];
            if (columns % format.block_values != 0)
                invalid("tensor " + quoted(raw.name) + " least-major dimension " + std::to_string(columns) +
                        " is not divisible by " + std::to_string(format.block_values) + " for " + format.name);
            uint64_t rows = 1;
            for (size_t d = 1; d < raw.dimensions.size(); d++)
                rows = checked_mul(rows, raw.dimensions[d], "tensor " + quoted(raw.name) + " row count size overflows");
            const uint64_t row_bytes = checked_mul(columns / format.block_values, format.block_bytes,
                                                   "tensor " + quoted(raw.name) + " encoded row length overflows");
            tensor.byte_len = checked_mul(rows, row_bytes, "tensor " + quoted(raw.name) + " byte length overflows");
            tensor.physical_shape = {rows, row_bytes};
        }
        if (data_start + raw.relative_offset < data_start) invalid("absolute tensor offset overflows");
        tensor.data_offset = data_start + raw.relative_offset;
        if (tensor.data_offset + tensor.byte_len < tensor.data_offset) invalid("tensor range end overflows");
        const uint64_t end = tensor.data_offset + tensor.byte_len;
        if (end > reader.file_len)
            invalid("tensor " + quoted(raw.name) + " range [" + std::to_string(tensor.data_offset) + ", " +
                    std::to_string(end) + ") exceeds file size " + std::to_string(reader.file_len));
        tensor.name = std::move(raw.name);
        file->tensors.push_back(std::move(tensor));
    }

    std::vector<const Tensor*> order;
    for (const Tensor& tensor : file->tensors) order.push_back(&tensor);
    std::sort(order.begin(), order.end(), [](const Tensor* a, const Tensor* b) {
        return a->data_offset != b->data_offset ? a->data_offset < b->data_offset : a < b;
    });
    for (size_t i = 1; i < order.size(); i++)
        if (order[i]->data_offset < order[i - 1]->data_offset + order[i - 1]->byte_len)
            invalid("tensor ranges for " + quoted(order[i - 1]->name) + " and " + quoted(order[i]->name) + " overlap");
    reader.check_cancelled();
}

void fill(Error* error, const Stop& stop) {
    error->kind = stop.kind;
    switch (stop.kind) {  // Display of GgufParseError, gguf.rs:99-107
        case Failure::kInvalid: error->message = "gguf: " + stop.message; break;
        case Failure::kIo: error->message = "gguf: I/O failed: " + stop.message; break;
        default: error->message = "gguf: operation aborted"; break;
    }
}

bool positioned_read(int fd, void* destination, uint64_t length, uint64_t offset, Error* error) {
    auto* out = static_cast<char*>(destination);
    uint64_t got = 0;
    while (got < length) {
        const ssize_t n = pread(fd, out + got, length - got, static_cast<off_t>(offset + got));
        if (n < 0 && errno == EINTR) continue;
        if (n <= 0) {
            fill(error, Stop{Failure::kIo, n < 0 ? std::strerror(errno) : "failed to fill whole buffer"});
            return false;
        }
        got += static_cast<uint64_t>(n);
    }
    return true;
}

bool size_matches(const Tensor& tensor, uint64_t destination_bytes, Error* error) {
    if (destination_bytes == tensor.byte_len) return true;
    fill(error, Stop{Failure::kInvalid, "tensor " + quoted(tensor.name) + " requires " + std::to_string(tensor.byte_len) +
                                            " destination bytes, got " + std::to_string(destination_bytes)});
    return false;
}

}  // namespace

uint64_t Value::length() const {
    return integers.size() + signed_integers.size() + reals.size() + strings.size();
}

File::~File() {
    for (void* buffer : staging)
        if (buffer != nullptr) (void)hipHostFree(buffer);
    if (fd >= 0) close(fd);
}

File* open(const char* path, const volatile int32_t* cancel, Error* error) {
    auto* file = new File();
    try {
        if (cancel != nullptr && *cancel != 0) throw Stop{Failure::kCancelled, ""};
        file->fd = ::open(path, O_RDONLY | O_CLOEXEC);
        if (file->fd < 0) io_failed(std::strerror(errno));
        struct stat info;
        if (fstat(file->fd, &info) != 0) io_failed(std::strerror(errno));
        file->file_len = static_cast<uint64_t>(info.st_size);
        if (cancel != nullptr && *cancel != 0) throw Stop{Failure::kCancelled, ""};
        Reader reader{file->fd, file->file_len, 0, cancel, {}, 0};
        parse(reader, file);
        return file;
    } catch (const Stop& stop) {
        fill(error, stop);
    } catch (const std::bad_alloc&) {
        fill(error, Stop{Failure::kInvalid, "header is too large"});
    }
    delete file;
    return nullptr;
}

bool read_tensor(const File& file, const Tensor& tensor, void* destination, uint64_t destination_bytes,
                 const volatile int32_t* cancel, Error* error) {
    if (!size_matches(tensor, destination_bytes, error)) return false;
    for (uint64_t done = 0; done < tensor.byte_len; done += kReadChunkBytes) {
        if (cancel != nullptr && *cancel != 0) {
            fill(error, Stop{Failure::kCancelled, ""});
            return false;
        }
        const uint64_t chunk = std::min(kReadChunkBytes, tensor.byte_len - done);
        if (!positioned_read(file.fd, static_cast<char*>(destination) + done, chunk, tensor.data_offset + done, error))
            return false;
    }
    if (cancel != nullptr && *cancel != 0) {
        fill(error, Stop{Failure::kCancelled, ""});
        return false;
    }
    return true;
}

bool upload_tensor(File& file, const Tensor& tensor, void* device_destination, uint64_t destination_bytes,
                   void* stream, const volatile int32_t* cancel, Error* error) {
    if (!size_matches(tensor, destination_bytes, error)) return false;
    const auto hip_failed = [&](hipError_t status) {
        fill(error, Stop{Failure::kIo, std::string("HIP error: ") + hipGetErrorString(status)});
        return false;
    };
    for (void*& buffer : file.staging)
        if (buffer == nullptr)
            if (hipError_t status = hipHostMalloc(&buffer, kReadChunkBytes, hipHostMallocDefault)) return hip_failed(status);
    auto* s = static_cast<hipStream_t>(stream);
    hipEvent_t copied[2] = {nullptr, nullptr};
    bool ok = true;
    uint64_t index = 0;
    for (uint64_t done = 0; ok && done < tensor.byte_len; done += kReadChunkBytes, index++) {
        if (cancel != nullptr && *cancel != 0) {
            fill(error, Stop{Failure::kCancelled, ""});
            ok = false;
            break;
        }
        const int slot = static_cast<int>(index & 1);
        // the copy that last used this buffer must have left it
        if (copied[slot] != nullptr) {
            if (hipError_t status = hipEventSynchronize(copied[slot])) { ok = hip_failed(status); break; }
        } else if (hipError_t status = hipEventCreateWithFlags(&copied[slot], hipEventDisableTiming)) {
            ok = hip_failed(status);
            break;
        }
        const uint64_t chunk = std::min(kReadChunkBytes, tensor.byte_len - done);
        if (!positioned_read(file.fd, file.staging[slot], chunk, tensor.data_offset + done, error)) { ok = false; break; }
        if (hipError_t status = hipMemcpyAsync(static_cast<char*>(device_destination) + done, file.staging[slot], chunk,
                                               hipMemcpyHostToDevice, s)) { ok = hip_failed(status); break; }
        if (hipError_t status = hipEventRecord(copied[slot], s)) { ok = hip_failed(status); break; }
    }
    // the staging buffers are reused by the next call: drain before returning, also after a failure
    const hipError_t drained = hipStreamSynchronize(s);
    for (hipEvent_t event : copied)
        if (event != nullptr) (void)hipEventDestroy(event);
    if (ok && drained != hipSuccess) ok = hip_failed(drained);
    return ok;
}

}  // namespace gguf
}  // namespace et
