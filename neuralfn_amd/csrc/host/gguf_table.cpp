// Tensor table of a GGUF version 3 file (include/nfn_mi355_gguf.h).
//
// Structure and checks follow the reference engine's loader
// (neuralfn/csrc/native_gpt2/resident_glimmer.cpp:976-1160): little-endian
// header (magic, version, tensor count, metadata count), metadata key/value
// pairs (skipped here by type), tensor infos (name, rank, dimensions, type,
// offset), zero padding to a multiple of 32, then the tensor bytes, contiguous
// in offset order with 32-byte alignment and nothing after the last one.
#include "../../../include/nfn_mi355_gguf.h"

#include <algorithm>
#include <cstring>
#include <exception>
#include <limits>
#include <string>
#include <unordered_map>
#include <vector>

#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

namespace {

enum Error : int {
    kOk = 0,
    kArgument = 1,
    kOpen = 2,
    kTruncated = 3,
    kMagic = 4,
    kVersion = 5,
    kMetadata = 6,
    kRank = 7,
    kDimension = 8,
    kEncoding = 9,
    kAlignment = 10,
    kDuplicate = 11,
    kPadding = 12,
    kExtent = 13,
    kLayout = 14,
    kNotFound = 15,
    kEmpty = 16,
};

constexpr std::uint64_t kAlignment32 = 32;
constexpr int kMaxArrayDepth = 4;

// metadata value types (neuralfn/native_gguf.py:60-72)
enum ValueType : std::uint32_t {
    kUint8 = 0, kInt8 = 1, kUint16 = 2, kInt16 = 3, kUint32 = 4, kInt32 = 5, kFloat32 = 6,
    kBool = 7, kString = 8, kArray = 9, kUint64 = 10, kInt64 = 11, kFloat64 = 12,
};

struct Layout {
    std::int64_t elements;
    std::int64_t bytes;
};

// ggml type id -> block layout (resident_glimmer.cpp:1137-1142; Q8_0 from
// vendor/llama_mmq_62bf73d/ggml/src/ggml-common.h:251-256)
bool layout_of(std::uint32_t type, Layout* layout) {
    switch (type) {
        case 0: *layout = {1, 4}; return true;       // F32
        case 30: *layout = {1, 2}; return true;      // BF16
        case 8: *layout = {32, 34}; return true;     // Q8_0
        case 12: *layout = {256, 144}; return true;  // Q4_K
        case 13: *layout = {256, 176}; return true;  // Q5_K
        case 14: *layout = {256, 210}; return true;  // Q6_K
        default: return false;
    }
}

class Cursor {
public:
    Cursor(const std::uint8_t* data, std::uint64_t size) : data_(data), size_(size) {}
    bool has(std::uint64_t count) const { return count <= size_ - offset_; }
    bool skip(std::uint64_t count) {
        if (!has(count)) return false;
        offset_ += count;
        return true;
    }
    template <typename T>
    bool read(T* value) {
        if (!has(sizeof(T))) return false;
        std::memcpy(value, data_ + offset_, sizeof(T));
        offset_ += sizeof(T);
        return true;
    }
    bool string(std::string* value) {
        std::uint64_t length = 0;
        if (!read(&length) || !has(length)) return false;
        value->assign(reinterpret_cast<const char*>(data_ + offset_), length);
        offset_ += length;
        return true;
    }
    std::uint64_t offset() const { return offset_; }
    const std::uint8_t* data() const { return data_; }

private:
    const std::uint8_t* data_;
    std::uint64_t size_;
    std::uint64_t offset_ = 0;
};

std::uint64_t scalar_bytes(std::uint32_t type) {
    switch (type) {
        case kUint8: case kInt8: case kBool: return 1;
        case kUint16: case kInt16: return 2;
        case kUint32: case kInt32: case kFloat32: return 4;
        case kUint64: case kInt64: case kFloat64: return 8;
        default: return 0;
    }
}

bool skip_value(Cursor* cursor, std::uint32_t type, int depth) {
    if (const std::uint64_t bytes = scalar_bytes(type)) return cursor->skip(bytes);
    if (type == kString) {
        std::uint64_t length = 0;
        return cursor->read(&length) && cursor->skip(length);
    }
    if (type != kArray || depth >= kMaxArrayDepth) return false;
    std::uint32_t element = 0;
    std::uint64_t count = 0;
    if (!cursor->read(&element) || !cursor->read(&count)) return false;
    if (const std::uint64_t bytes = scalar_bytes(element)) {
        return count <= std::numeric_limits<std::uint64_t>::max() / bytes && cursor->skip(count * bytes);
    }
    for (std::uint64_t index = 0; index < count; ++index) {
        if (!skip_value(cursor, element, depth + 1)) return false;
    }
    return true;
}

struct Tensor {
    std::string name;
    std::uint32_t encoding = 0;
    std::uint32_t rank = 0;
    std::int64_t rows = 0, cols = 0, row_stride = 0, nbytes = 0;
    std::uint64_t offset = 0;  // relative to the data section while parsing, then absolute
};

}  // namespace

struct NfnMi355GgufFileV1 {
    const std::uint8_t* data = nullptr;
    std::uint64_t size = 0;
    std::uint64_t metadata_count = 0;
    std::vector<Tensor> tensors;
    std::unordered_map<std::string, std::size_t> by_name;
};

namespace {

int parse(NfnMi355GgufFileV1* file) {
    Cursor cursor(file->data, file->size);
    if (!cursor.has(4)) return kTruncated;
    if (std::memcmp(file->data, "GGUF", 4) != 0) return kMagic;
    cursor.skip(4);
    std::uint32_t version = 0;
    std::uint64_t tensor_count = 0;
    if (!cursor.read(&version)) return kTruncated;
    if (version != 3) return kVersion;
    if (!cursor.read(&tensor_count) || !cursor.read(&file->metadata_count)) return kTruncated;
    if (tensor_count == 0) return kEmpty;
    // every entry takes bytes: a tensor info is at least 32 (name length, rank, one
    // dimension, encoding, offset), a metadata entry at least 13 (key length, type, one byte)
    if (tensor_count > file->size / 32 || file->metadata_count > file->size / 13) return kTruncated;

    for (std::uint64_t entry = 0; entry < file->metadata_count; ++entry) {
        std::string key;
        std::uint32_t type = 0;
        if (!cursor.string(&key) || !cursor.read(&type)) return kTruncated;
        if (type > kFloat64) return kMetadata;
        if (!skip_value(&cursor, type, 0)) return kMetadata;
    }

    file->tensors.reserve(static_cast<std::size_t>(tensor_count < 4096 ? tensor_count : 4096));
    for (std::uint64_t index = 0; index < tensor_count; ++index) {
        Tensor tensor;
        std::uint64_t dimensions[2] = {1, 1};
        if (!cursor.string(&tensor.name) || !cursor.read(&tensor.rank)) return kTruncated;
        if (tensor.rank < 1 || tensor.rank > 2) return kRank;
        for (std::uint32_t d = 0; d < tensor.rank; ++d) {
            if (!cursor.read(&dimensions[d])) return kTruncated;
            if (dimensions[d] == 0 ||
                dimensions[d] > static_cast<std::uint64_t>(std::numeric_limits<std::int64_t>::max())) {
                return kDimension;
            }
        }
        if (!cursor.read(&tensor.encoding) || !cursor.read(&tensor.offset)) return kTruncated;
        Layout layout;
        if (!layout_of(tensor.encoding, &layout)) return kEncoding;
        tensor.cols = static_cast<std::int64_t>(dimensions[0]);
        tensor.rows = static_cast<std::int64_t>(dimensions[1]);
        if (tensor.cols % layout.elements != 0) return kDimension;
        if (tensor.offset % kAlignment32 != 0) return kAlignment;
        const std::int64_t blocks = tensor.cols / layout.elements;
        if (blocks > std::numeric_limits<std::int64_t>::max() / layout.bytes) return kDimension;
        tensor.row_stride = blocks * layout.bytes;
        if (tensor.rows > std::numeric_limits<std::int64_t>::max() / tensor.row_stride) return kDimension;
        tensor.nbytes = tensor.rows * tensor.row_stride;
        if (!file->by_name.emplace(tensor.name, file->tensors.size()).second) return kDuplicate;
        file->tensors.push_back(std::move(tensor));
    }

    const std::uint64_t header_end = cursor.offset();
    const std::uint64_t data_offset = (header_end + kAlignment32 - 1) / kAlignment32 * kAlignment32;
    if (data_offset > file->size) return kTruncated;
    for (std::uint64_t index = header_end; index < data_offset; ++index) {
        if (file->data[index] != 0) return kPadding;
    }

    // extents: inside the file, contiguous in offset order, nothing after the last
    const std::uint64_t data_size = file->size - data_offset;
    std::vector<const Tensor*> ordered;
    ordered.reserve(file->tensors.size());
    for (const Tensor& tensor : file->tensors) {
        if (tensor.offset > data_size ||
            static_cast<std::uint64_t>(tensor.nbytes) > data_size - tensor.offset) {
            return kExtent;
        }
        ordered.push_back(&tensor);
    }
    std::sort(ordered.begin(), ordered.end(),
              [](const Tensor* left, const Tensor* right) { return left->offset < right->offset; });
    std::uint64_t expected = 0;
    for (const Tensor* tensor : ordered) {
        if (tensor->offset != expected) return kLayout;
        const std::uint64_t end = tensor->offset + static_cast<std::uint64_t>(tensor->nbytes);
        expected = (end + kAlignment32 - 1) / kAlignment32 * kAlignment32;
    }
    const Tensor* last = ordered.back();
    if (last->offset + static_cast<std::uint64_t>(last->nbytes) != data_size) return kLayout;

    for (Tensor& tensor : file->tensors) tensor.offset += data_offset;
    return kOk;
}

void fill(const Tensor& tensor, NfnMi355GgufTensorV1* out) {
    out->name = tensor.name.c_str();
    out->encoding = tensor.encoding;
    out->rank = tensor.rank;
    out->rows = tensor.rows;
    out->cols = tensor.cols;
    out->row_stride_bytes = tensor.row_stride;
    out->nbytes = tensor.nbytes;
    out->file_offset = tensor.offset;
}

}  // namespace

extern "C" {

int nfn_mi355_gguf_open_v1(const char* path, NfnMi355GgufFileV1** file) {
    if (path == nullptr || file == nullptr) return kArgument;
    *file = nullptr;
    const int descriptor = ::open(path, O_RDONLY | O_CLOEXEC);
    if (descriptor < 0) return kOpen;
    struct stat status {};
    if (::fstat(descriptor, &status) != 0 || !S_ISREG(status.st_mode) || status.st_size <= 0) {
        ::close(descriptor);
        return kOpen;
    }
    void* mapping = ::mmap(nullptr, static_cast<std::size_t>(status.st_size), PROT_READ, MAP_PRIVATE,
                           descriptor, 0);
    ::close(descriptor);
    if (mapping == MAP_FAILED) return kOpen;
    auto* handle = new NfnMi355GgufFileV1();
    handle->data = static_cast<const std::uint8_t*>(mapping);
    handle->size = static_cast<std::uint64_t>(status.st_size);
    int code = kArgument;
    try {
        code = parse(handle);
    } catch (const std::exception&) {  // allocation failure or the like: no exception leaves this call
        code = kTruncated;
    }
    if (code != kOk) {
        nfn_mi355_gguf_close_v1(handle);
        return code;
    }
    *file = handle;
    return kOk;
}

void nfn_mi355_gguf_close_v1(NfnMi355GgufFileV1* file) {
    if (file == nullptr) return;
    if (file->data != nullptr) {
        ::munmap(const_cast<std::uint8_t*>(file->data), static_cast<std::size_t>(file->size));
    }
    delete file;
}

int64_t nfn_mi355_gguf_tensor_count_v1(const NfnMi355GgufFileV1* file) {
    return file == nullptr ? 0 : static_cast<int64_t>(file->tensors.size());
}

int64_t nfn_mi355_gguf_metadata_count_v1(const NfnMi355GgufFileV1* file) {
    return file == nullptr ? 0 : static_cast<int64_t>(file->metadata_count);
}

int nfn_mi355_gguf_tensor_v1(const NfnMi355GgufFileV1* file, int64_t index,
                             NfnMi355GgufTensorV1* tensor) {
    if (file == nullptr || tensor == nullptr || index < 0 ||
        index >= static_cast<int64_t>(file->tensors.size())) {
        return kArgument;
    }
    fill(file->tensors[static_cast<std::size_t>(index)], tensor);
    return kOk;
}

int nfn_mi355_gguf_find_v1(const NfnMi355GgufFileV1* file, const char* name,
                           NfnMi355GgufTensorV1* tensor) {
    if (file == nullptr || name == nullptr || tensor == nullptr) return kArgument;
    const auto found = file->by_name.find(name);
    if (found == file->by_name.end()) return kNotFound;
    fill(file->tensors[found->second], tensor);
    return kOk;
}

const uint8_t* nfn_mi355_gguf_data_v1(const NfnMi355GgufFileV1* file, uint64_t* size) {
    if (file == nullptr) return nullptr;
    if (size != nullptr) *size = file->size;
    return file->data;
}

const char* nfn_mi355_gguf_error_string(int code) {
    switch (code) {
        case kOk: return "ok";
        case kArgument: return "invalid argument";
        case kOpen: return "cannot open or map the file";
        case kTruncated: return "the file ends inside the header";
        case kMagic: return "not a GGUF file";
        case kVersion: return "GGUF version is not 3";
        case kMetadata: return "malformed metadata value";
        case kRank: return "tensor rank is not 1 or 2";
        case kDimension: return "tensor dimension is zero, too large or not a multiple of the block";
        case kEncoding: return "tensor encoding has no packed-weight layout";
        case kAlignment: return "tensor offset is not a multiple of 32";
        case kDuplicate: return "duplicate tensor name";
        case kPadding: return "header padding is not zero";
        case kExtent: return "tensor exceeds the file";
        case kLayout: return "tensor data is not contiguous, or bytes trail the last tensor";
        case kNotFound: return "no tensor of that name";
        case kEmpty: return "the file holds no tensors";
        default: return "unknown error";
    }
}

}  // extern "C"
