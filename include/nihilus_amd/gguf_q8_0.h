/*
 * gguf_q8_0.h -- reading a GGUF model file and placing its Q8_0 tensors on the GPU, C ABI.
 *
 * Stands for the reference's model loader on the GPU path: gguf header and metadata
 * (infra/model_parser.hpp:635-671), tensor records (:855-880), data-section placement (:895-940) and the
 * host-to-device copy of every tensor into the arena (:130-160, memory_transfer::host_to_device), with the one
 * difference that a Q8_0 weight can land directly in the tiled device layout the mat-mul kernels read
 * (q8_0_abi.h).  Paths of the reference are relative to include/nihilus-incl/.
 *
 * The file is memory-mapped read-only; nothing is copied on the host.  Same status convention as q8_0_abi.h.
 */
#ifndef NIHILUS_AMD_GGUF_Q8_0_H
#define NIHILUS_AMD_GGUF_Q8_0_H

#include <stdint.h>

#include "q8_0_abi.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef struct nh_gguf nh_gguf; /* an open, parsed file */

/* ggml tensor types as stored in the file (the reference's data_types, common/data_types.hpp / type_traits.hpp:38-61) */
enum nh_ggml_type { NH_GGML_F32 = 0, NH_GGML_F16 = 1, NH_GGML_Q8_0 = 8, NH_GGML_I8 = 24, NH_GGML_I16 = 25, NH_GGML_I32 = 26, NH_GGML_I64 = 27, NH_GGML_F64 = 28, NH_GGML_BF16 = 30 };

typedef struct nh_gguf_tensor_info {
	const char* name; /* NUL-terminated, owned by the handle */
	uint32_t n_dims; /* <= 4 (model_parser.hpp:862-866) */
	uint32_t ggml_type;
	uint64_t dims[4]; /* ggml order, dims[0] fastest (= K of a weight matrix, dims[1] = rows); unused dims are 1 */
	uint64_t offset; /* as stored: relative to the data section */
	uint64_t file_offset; /* absolute position of the first byte in the file */
	uint64_t byte_size; /* type_traits<...>::total_byte_size; 0 if the type's size is not known to this loader */
	int32_t layer; /* N of "blk.N." (model_parser.hpp:830-852), -1 for tensors outside the blocks */
	int32_t reserved;
} nh_gguf_tensor_info;

/* Bytes of a tensor of `ggml_type` with these dims (block types: dims[0] must be a multiple of the block size).
 * Negative status on a bad shape, 0 for a type this loader has no size for. */
int64_t nh_ggml_tensor_bytes(uint32_t ggml_type, const uint64_t* dims, uint32_t n_dims);

/* Opens and parses `path`.  Checks: magic "GGUF" (model_parser.hpp:638-642), version 2 or 3, tensor count <= 100000
 * and metadata count <= 10000 (:647-657), n_dims <= 4 and dim <= 2^32 (:862-875), every tensor inside the file.
 * NH_ERR_IO: cannot open/map; NH_ERR_FORMAT: not a GGUF file this loader accepts. */
int nh_gguf_open(const char* path, nh_gguf** out);
void nh_gguf_close(nh_gguf* file);

int64_t nh_gguf_tensor_count(const nh_gguf* file);
int64_t nh_gguf_metadata_count(const nh_gguf* file);
uint64_t nh_gguf_alignment(const nh_gguf* file); /* general.alignment, 32 if absent */
uint64_t nh_gguf_data_offset(const nh_gguf* file); /* where the data section starts */
uint32_t nh_gguf_version(const nh_gguf* file);

int nh_gguf_tensor_at(const nh_gguf* file, int64_t index, nh_gguf_tensor_info* out); /* file order */
int nh_gguf_find_tensor(const nh_gguf* file, const char* name, nh_gguf_tensor_info* out); /* NH_ERR_NOT_FOUND */
const void* nh_gguf_tensor_data(const nh_gguf* file, const nh_gguf_tensor_info* info); /* host pointer into the mapping */

/* Metadata lookups by key.  Integers of any stored width (and bools) widen to 64 bits; floats to double.
 * NH_ERR_NOT_FOUND if the key is absent, NH_ERR_ARGUMENT if it holds another kind of value. */
int nh_gguf_metadata_u64(const nh_gguf* file, const char* key, uint64_t* out);
int nh_gguf_metadata_i64(const nh_gguf* file, const char* key, int64_t* out);
int nh_gguf_metadata_f64(const nh_gguf* file, const char* key, double* out);
/* string value: pointer into the mapping (not NUL-terminated) and its length */
int nh_gguf_metadata_string(const nh_gguf* file, const char* key, const char** out, uint64_t* length);
/* array value: element type (a gguf metadata value type, 0..12), count, and a pointer to the first element as stored */
int nh_gguf_metadata_array(const nh_gguf* file, const char* key, uint32_t* element_type, uint64_t* count, const void** first);

/* Copies one tensor to the GPU.  Q8_0 tensors only for tiled = 1: the blocks go to `device_staging` (>= byte_size
 * bytes, device memory, 16-byte aligned) and nh_q8_0_tile writes `device_dst` (nh_q8_0_tiled_bytes(dims[1], dims[0])
 * bytes); needs dims[0] % 128 == 0.  tiled = 0: the tensor's bytes as stored go straight to `device_dst`, any type,
 * no staging.  Asynchronous on `stream` after the host-to-device copy has been queued. */
int nh_gguf_upload_tensor(const nh_gguf* file, const nh_gguf_tensor_info* info, void* device_dst, int tiled, void* device_staging, int64_t staging_bytes, void* stream);

#ifdef __cplusplus
}
#endif

#endif
