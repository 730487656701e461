/* Tensor table of a GGUF version 3 file, as the packed-weight entry points need
 * it: for every tensor its name, encoding, [rows, cols] geometry, row stride and
 * the place of its bytes in the file.  Host-side, no GPU involved: the caller
 * copies (or maps) the bytes to the device and fills an
 * NfnNativeTilePackedWeightDescriptorV1 from the fields below.
 *
 * What it replaces: the structural part of the reference engine's loader
 * (neuralfn/csrc/native_gpt2/resident_glimmer.cpp:976-1160) and of its Python
 * reader (neuralfn/native_gguf.py:34-99, 1560-1600).  The checks are the
 * reference's: magic "GGUF", version 3, rank 1 or 2, known encodings, columns a
 * multiple of the encoding's block, tensor offsets multiples of 32, zero header
 * padding, tensor extents contiguous in offset order with 32-byte alignment, no
 * trailing bytes.  The reference's allowlists of one model's tensor names,
 * shapes and metadata values are not part of this reader.
 *
 * Every function returns 0 on success and a positive code otherwise;
 * nfn_mi355_gguf_error_string() names the code.
 */
#ifndef NFN_MI355_GGUF_H
#define NFN_MI355_GGUF_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct NfnMi355GgufFileV1 NfnMi355GgufFileV1;

typedef struct NfnMi355GgufTensorV1 {
    const char* name;          /* owned by the file handle */
    uint32_t encoding;         /* ggml type id = NFN_NATIVE_TILE_PACKED_WEIGHT_ENCODING_* */
    uint32_t rank;             /* 1 or 2 */
    int64_t rows;              /* ne[1], or 1 for rank 1 */
    int64_t cols;              /* ne[0] */
    int64_t row_stride_bytes;  /* cols / block elements * block bytes */
    int64_t nbytes;            /* rows * row_stride_bytes */
    uint64_t file_offset;      /* of the first byte, from the start of the file */
} NfnMi355GgufTensorV1;

/* Maps `path` read-only, parses and validates the header and the tensor table
 * (resident_glimmer.cpp:976-1160).  The handle owns the mapping. */
int nfn_mi355_gguf_open_v1(const char* path, NfnMi355GgufFileV1** file);
void nfn_mi355_gguf_close_v1(NfnMi355GgufFileV1* file);

int64_t nfn_mi355_gguf_tensor_count_v1(const NfnMi355GgufFileV1* file);
int64_t nfn_mi355_gguf_metadata_count_v1(const NfnMi355GgufFileV1* file);
/* Tensor `index` in file order. */
int nfn_mi355_gguf_tensor_v1(const NfnMi355GgufFileV1* file, int64_t index,
                             NfnMi355GgufTensorV1* tensor);
/* Tensor by name (the engine looks its layers up this way,
 * resident_glimmer.cpp:1186-1210). */
int nfn_mi355_gguf_find_v1(const NfnMi355GgufFileV1* file, const char* name,
                           NfnMi355GgufTensorV1* tensor);
/* First byte of the mapped file and its size: tensor bytes are at
 * data + file_offset for as long as the handle is open. */
const uint8_t* nfn_mi355_gguf_data_v1(const NfnMi355GgufFileV1* file, uint64_t* size);

const char* nfn_mi355_gguf_error_string(int code);

#ifdef __cplusplus
}
#endif

#endif /* NFN_MI355_GGUF_H */
