// GGUF reader + tensor upload behind include/nihilus_amd/gguf_q8_0.h.  Host code only.
//
// File layout (GGUF v2/v3, little-endian): "GGUF" u32 version, u64 tensor count, u64 metadata count; metadata pairs
// (string key, u32 value type, value); tensor records (string name, u32 n_dims, u64 dims[n_dims], u32 type, u64 offset);
// padding to general.alignment (default 32); tensor data.  The reference walks the same records
// (infra/model_parser.hpp:635-671, :855-880) and places tensor data by offset (:922-937).
#include <nihilus_amd/gguf_q8_0.h>

#include <hip/hip_runtime_api.h>

#include <cstring>
#include <fcntl.h>
#include <string>
#include <string_view>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>
#include <unordered_map>
#include <vector>

namespace {

enum value_type : uint32_t { T_U8, T_I8, T_U16, T_I16, T_U32, T_I32, T_F32, T_BOOL, T_STRING, T_ARRAY, T_U64, T_I64, T_F64, T_COUNT };

constexpr uint64_t scalar_size(uint32_t t) {
	switch (t) {
		case T_U8:
		case T_I8:
		case T_BOOL:
			return 1;
		case T_U16:
		case T_I16:
			return 2;
		case T_U32:
		case T_I32:
		case T_F32:
			return 4;
		case T_U64:
		case T_I64:
		case T_F64:
			return 8;
		default:
			return 0;
	}
}

struct metadata_value {
	uint32_t type		  = T_COUNT;
	uint32_t element_type = T_COUNT; // arrays
	uint64_t count		  = 0; // arrays: elements; strings: bytes
	const uint8_t* data	  = nullptr; // scalars: the value; strings: first byte; arrays: first element as stored
};

struct cursor {
	const uint8_t* base;
	uint64_t size;
	uint64_t pos = 0;
	bool ok		 = true;

	bool has(uint64_t n) const {
		return ok && n <= size - pos;
	}
	template<typename T> T read() {
		T v{};
		if (!has(sizeof(T))) {
			ok = false;
			return v;
		}
		std::memcpy(&v, base + pos, sizeof(T));
		pos += sizeof(T);
		return v;
	}
	std::string_view read_string() {
		const uint64_t n = read<uint64_t>();
		if (!has(n)) {
			ok = false;
			return {};
		}
		std::string_view s(reinterpret_cast<const char*>(base + pos), n);
		pos += n;
		return s;
	}
	void skip(uint64_t n) {
		if (!has(n)) {
			ok = false;
			return;
		}
		pos += n;
	}
};

// bytes per block and values per block of the types this loader can size
bool type_geometry(uint32_t t, uint64_t* block_bytes, uint64_t* block_values) {
	switch (t) {
		case NH_GGML_F32:
		case NH_GGML_I32:
			*block_bytes = 4, *block_values = 1;
			return true;
		case NH_GGML_F16:
		case NH_GGML_BF16:
		case NH_GGML_I16:
			*block_bytes = 2, *block_values = 1;
			return true;
		case NH_GGML_I8:
			*block_bytes = 1, *block_values = 1;
			return true;
		case NH_GGML_I64:
		case NH_GGML_F64:
			*block_bytes = 8, *block_values = 1;
			return true;
		case NH_GGML_Q8_0:
			*block_bytes = NH_Q8_0_BLOCK_BYTES, *block_values = NH_Q8_0_QK;
			return true;
		case 2: // Q4_0
			*block_bytes = 18, *block_values = 32;
			return true;
		case 3: // Q4_1
			*block_bytes = 20, *block_values = 32;
			return true;
		case 6: // Q5_0
			*block_bytes = 22, *block_values = 32;
			return true;
		case 7: // Q5_1
			*block_bytes = 24, *block_values = 32;
			return true;
		default:
			return false;
	}
}

int layer_of(std::string_view name) {
	if (name.size() > 4 && name.substr(0, 4) == "blk.") {
		int n	 = 0;
		size_t i = 4;
		for (; i < name.size() && name[i] >= '0' && name[i] <= '9'; ++i) {
			n = n * 10 + (name[i] - '0');
		}
		if (i > 4 && i < name.size() && name[i] == '.') {
			return n;
		}
	}
	return -1;
}

template<typename T> T load(const uint8_t* p) {
	T v;
	std::memcpy(&v, p, sizeof(T));
	return v;
}

} // namespace

struct nh_gguf {
	int fd				= -1;
	const uint8_t* base = nullptr;
	uint64_t size		= 0;
	uint32_t version	= 0;
	uint64_t alignment	= 32;
	uint64_t data_start = 0;
	std::vector<std::string> names; // NUL-terminated copies for the C side
	std::vector<nh_gguf_tensor_info> tensors;
	std::unordered_map<std::string, size_t> tensor_index;
	std::unordered_map<std::string, metadata_value> metadata;
};

extern "C" {

int64_t nh_ggml_tensor_bytes(uint32_t ggml_type, const uint64_t* dims, uint32_t n_dims) {
	if (!dims || n_dims == 0 || n_dims > 4) {
		return NH_ERR_SHAPE;
	}
	uint64_t bb = 0, bv = 0;
	if (!type_geometry(ggml_type, &bb, &bv)) {
		return 0;
	}
	if (dims[0] % bv != 0) {
		return NH_ERR_SHAPE;
	}
	uint64_t total = dims[0] / bv * bb;
	for (uint32_t i = 1; i < n_dims; ++i) {
		if (dims[i] != 0 && total > (uint64_t(1) << 62) / dims[i]) {
			return NH_ERR_TOO_LARGE;
		}
		total *= dims[i];
	}
	return static_cast<int64_t>(total);
}

void nh_gguf_close(nh_gguf* f) {
	if (!f) {
		return;
	}
	if (f->base) {
		munmap(const_cast<uint8_t*>(f->base), f->size);
	}
	if (f->fd >= 0) {
		close(f->fd);
	}
	delete f;
}

int nh_gguf_open(const char* path, nh_gguf** out) {
	if (!path || !out) {
		return NH_ERR_NULL_POINTER;
	}
	*out	   = nullptr;
	nh_gguf* f = new nh_gguf;
	auto fail  = [&](int status) {
		 nh_gguf_close(f);
		 return status;
	};
	f->fd = open(path, O_RDONLY | O_CLOEXEC);
	if (f->fd < 0) {
		return fail(NH_ERR_IO);
	}
	struct stat st {};
	if (fstat(f->fd, &st) != 0 || st.st_size < 24) {
		return fail(st.st_size < 24 ? NH_ERR_FORMAT : NH_ERR_IO);
	}
	f->size	   = static_cast<uint64_t>(st.st_size);
	void* base = mmap(nullptr, f->size, PROT_READ, MAP_PRIVATE, f->fd, 0);
	if (base == MAP_FAILED) {
		return fail(NH_ERR_IO);
	}
	f->base = static_cast<const uint8_t*>(base);

	cursor c{ f->base, f->size };
	if (c.read<uint32_t>() != 0x46554747u) { // "GGUF"
		return fail(NH_ERR_FORMAT);
	}
	f->version = c.read<uint32_t>();
	if (f->version != 2 && f->version != 3) {
		return fail(NH_ERR_FORMAT);
	}
	const uint64_t n_tensors  = c.read<uint64_t>();
	const uint64_t n_metadata = c.read<uint64_t>();
	if (n_tensors > 100000 || n_metadata > 10000) { // the reference's sanity limits
		return fail(NH_ERR_FORMAT);
	}

	for (uint64_t i = 0; i < n_metadata && c.ok; ++i) {
		const std::string_view key = c.read_string();
		metadata_value v;
		v.type = c.read<uint32_t>();
		if (!c.ok || v.type >= T_COUNT) {
			return fail(NH_ERR_FORMAT);
		}
		if (v.type == T_STRING) {
			const std::string_view s = c.read_string();
			v.data					 = reinterpret_cast<const uint8_t*>(s.data());
			v.count					 = s.size();
		} else if (v.type == T_ARRAY) {
			v.element_type = c.read<uint32_t>();
			v.count		   = c.read<uint64_t>();
			v.data		   = f->base + c.pos;
			if (!c.ok || v.element_type >= T_COUNT || v.element_type == T_ARRAY) {
				return fail(NH_ERR_FORMAT); // nested arrays do not occur in model files
			}
			if (v.element_type == T_STRING) {
				for (uint64_t e = 0; e < v.count && c.ok; ++e) {
					c.read_string();
				}
			} else {
				const uint64_t es = scalar_size(v.element_type);
				if (v.count > (f->size - c.pos) / es) {
					return fail(NH_ERR_FORMAT);
				}
				c.skip(v.count * es);
			}
		} else {
			v.data = f->base + c.pos;
			c.skip(scalar_size(v.type));
		}
		if (!c.ok) {
			return fail(NH_ERR_FORMAT);
		}
		f->metadata.emplace(std::string(key), v);
	}
	if (!c.ok) {
		return fail(NH_ERR_FORMAT);
	}
	{
		auto it = f->metadata.find("general.alignment");
		if (it != f->metadata.end() && it->second.type == T_U32) {
			uint32_t a = 0;
			std::memcpy(&a, it->second.data, 4);
			if (a == 0 || (a & (a - 1)) != 0) {
				return fail(NH_ERR_FORMAT);
			}
			f->alignment = a;
		}
	}

	f->names.reserve(n_tensors);
	f->tensors.reserve(n_tensors);
	for (uint64_t i = 0; i < n_tensors; ++i) {
		const std::string_view name = c.read_string();
		nh_gguf_tensor_info t{};
		t.n_dims = c.read<uint32_t>();
		if (!c.ok || t.n_dims == 0 || t.n_dims > 4) {
			return fail(NH_ERR_FORMAT);
		}
		for (uint32_t d = 0; d < 4; ++d) {
			t.dims[d] = d < t.n_dims ? c.read<uint64_t>() : 1;
			if (t.dims[d] > (uint64_t(1) << 32)) {
				return fail(NH_ERR_FORMAT);
			}
		}
		t.ggml_type = c.read<uint32_t>();
		t.offset	= c.read<uint64_t>();
		if (!c.ok) {
			return fail(NH_ERR_FORMAT);
		}
		const int64_t bytes = nh_ggml_tensor_bytes(t.ggml_type, t.dims, t.n_dims);
		if (bytes < 0) {
			return fail(NH_ERR_FORMAT);
		}
		t.byte_size = static_cast<uint64_t>(bytes);
		t.layer		= layer_of(name);
		f->names.emplace_back(name);
		f->tensors.push_back(t);
	}
	f->data_start = (c.pos + f->alignment - 1) / f->alignment * f->alignment;
	if (f->data_start > f->size && n_tensors > 0) {
		return fail(NH_ERR_FORMAT);
	}
	for (size_t i = 0; i < f->tensors.size(); ++i) {
		nh_gguf_tensor_info& t = f->tensors[i];
		t.name				   = f->names[i].c_str();
		// checked before the addition: an offset close to 2^64 would wrap to a small file offset that passes the range checks below
		if (t.offset > f->size - f->data_start) {
			return fail(NH_ERR_FORMAT);
		}
		t.file_offset = f->data_start + t.offset;
		if (t.offset % f->alignment != 0 || t.file_offset > f->size || t.byte_size > f->size - t.file_offset) {
			return fail(NH_ERR_FORMAT);
		}
		if (!f->tensor_index.emplace(f->names[i], i).second) {
			return fail(NH_ERR_FORMAT); // duplicate tensor name
		}
	}
	*out = f;
	return NH_OK;
}

int64_t nh_gguf_tensor_count(const nh_gguf* f) {
	return f ? static_cast<int64_t>(f->tensors.size()) : NH_ERR_NULL_POINTER;
}
int64_t nh_gguf_metadata_count(const nh_gguf* f) {
	return f ? static_cast<int64_t>(f->metadata.size()) : NH_ERR_NULL_POINTER;
}
uint64_t nh_gguf_alignment(const nh_gguf* f) {
	return f ? f->alignment : 0;
}
uint64_t nh_gguf_data_offset(const nh_gguf* f) {
	return f ? f->data_start : 0;
}
uint32_t nh_gguf_version(const nh_gguf* f) {
	return f ? f->version : 0;
}

int nh_gguf_tensor_at(const nh_gguf* f, int64_t index, nh_gguf_tensor_info* out) {
	if (!f || !out) {
		return NH_ERR_NULL_POINTER;
	}
	if (index < 0 || index >= static_cast<int64_t>(f->tensors.size())) {
		return NH_ERR_NOT_FOUND;
	}
	*out = f->tensors[static_cast<size_t>(index)];
	return NH_OK;
}

int nh_gguf_find_tensor(const nh_gguf* f, const char* name, nh_gguf_tensor_info* out) {
	if (!f || !name || !out) {
		return NH_ERR_NULL_POINTER;
	}
	const auto it = f->tensor_index.find(name);
	if (it == f->tensor_index.end()) {
		return NH_ERR_NOT_FOUND;
	}
	*out = f->tensors[it->second];
	return NH_OK;
}

const void* nh_gguf_tensor_data(const nh_gguf* f, const nh_gguf_tensor_info* info) {
	if (!f || !info || info->file_offset > f->size || info->byte_size > f->size - info->file_offset) {
		return nullptr;
	}
	return f->base + info->file_offset;
}

static int find_value(const nh_gguf* f, const char* key, const metadata_value** v) {
	if (!f || !key) {
		return NH_ERR_NULL_POINTER;
	}
	const auto it = f->metadata.find(key);
	if (it == f->metadata.end()) {
		return NH_ERR_NOT_FOUND;
	}
	*v = &it->second;
	return NH_OK;
}

int nh_gguf_metadata_i64(const nh_gguf* f, const char* key, int64_t* out) {
	const metadata_value* v = nullptr;
	if (const int rc = find_value(f, key, &v); rc != NH_OK) {
		return rc;
	}
	if (!out) {
		return NH_ERR_NULL_POINTER;
	}
	switch (v->type) {
		case T_U8:
		case T_BOOL:
			*out = load<uint8_t>(v->data);
			return NH_OK;
		case T_I8:
			*out = load<int8_t>(v->data);
			return NH_OK;
		case T_U16:
			*out = load<uint16_t>(v->data);
			return NH_OK;
		case T_I16:
			*out = load<int16_t>(v->data);
			return NH_OK;
		case T_U32:
			*out = load<uint32_t>(v->data);
			return NH_OK;
		case T_I32:
			*out = load<int32_t>(v->data);
			return NH_OK;
		case T_U64:
			*out = static_cast<int64_t>(load<uint64_t>(v->data));
			return NH_OK;
		case T_I64:
			*out = load<int64_t>(v->data);
			return NH_OK;
		default:
			return NH_ERR_ARGUMENT;
	}
}

int nh_gguf_metadata_u64(const nh_gguf* f, const char* key, uint64_t* out) {
	int64_t v	 = 0;
	const int rc = nh_gguf_metadata_i64(f, key, &v);
	if (rc == NH_OK) {
		if (!out) {
			return NH_ERR_NULL_POINTER;
		}
		*out = static_cast<uint64_t>(v);
	}
	return rc;
}

int nh_gguf_metadata_f64(const nh_gguf* f, const char* key, double* out) {
	const metadata_value* v = nullptr;
	if (const int rc = find_value(f, key, &v); rc != NH_OK) {
		return rc;
	}
	if (!out) {
		return NH_ERR_NULL_POINTER;
	}
	if (v->type == T_F32) {
		*out = load<float>(v->data);
		return NH_OK;
	}
	if (v->type == T_F64) {
		*out = load<double>(v->data);
		return NH_OK;
	}
	return NH_ERR_ARGUMENT;
}

int nh_gguf_metadata_string(const nh_gguf* f, const char* key, const char** out, uint64_t* length) {
	const metadata_value* v = nullptr;
	if (const int rc = find_value(f, key, &v); rc != NH_OK) {
		return rc;
	}
	if (!out || !length) {
		return NH_ERR_NULL_POINTER;
	}
	if (v->type != T_STRING) {
		return NH_ERR_ARGUMENT;
	}
	*out	= reinterpret_cast<const char*>(v->data);
	*length = v->count;
	return NH_OK;
}

int nh_gguf_metadata_array(const nh_gguf* f, const char* key, uint32_t* element_type, uint64_t* count, const void** first) {
	const metadata_value* v = nullptr;
	if (const int rc = find_value(f, key, &v); rc != NH_OK) {
		return rc;
	}
	if (!element_type || !count || !first) {
		return NH_ERR_NULL_POINTER;
	}
	if (v->type != T_ARRAY) {
		return NH_ERR_ARGUMENT;
	}
	*element_type = v->element_type;
	*count		  = v->count;
	*first		  = v->data;
	return NH_OK;
}

int nh_gguf_upload_tensor(const nh_gguf* f, const nh_gguf_tensor_info* info, void* device_dst, int tiled, void* device_staging, int64_t staging_bytes, void* stream) {
	if (!f || !info || !device_dst) {
		return NH_ERR_NULL_POINTER;
	}
	const void* src = nh_gguf_tensor_data(f, info);
	if (!src || info->byte_size == 0) {
		return NH_ERR_ARGUMENT; // not a tensor of this file, or a type without a known size
	}
	// the caller owns this copy of the record and may have edited it: the byte count must still be the one its type and dims give,
	// or the tile kernel would read past the staging slice
	if (info->n_dims == 0 || info->n_dims > 4 || nh_ggml_tensor_bytes(info->ggml_type, info->dims, info->n_dims) != static_cast<int64_t>(info->byte_size)) {
		return NH_ERR_ARGUMENT;
	}
	hipStream_t s = static_cast<hipStream_t>(stream);
	if (!tiled) {
		const hipError_t e = hipMemcpyAsync(device_dst, src, info->byte_size, hipMemcpyHostToDevice, s);
		return e == hipSuccess ? NH_OK : static_cast<int>(e);
	}
	if (info->ggml_type != NH_GGML_Q8_0 || info->n_dims > 2) {
		return NH_ERR_ARGUMENT;
	}
	if (info->dims[0] % 128 != 0) {
		return NH_ERR_SHAPE;
	}
	if (!device_staging) {
		return NH_ERR_NULL_POINTER;
	}
	if (staging_bytes < 0 || static_cast<uint64_t>(staging_bytes) < info->byte_size || device_staging == device_dst) {
		return NH_ERR_ARGUMENT;
	}
	const hipError_t e = hipMemcpyAsync(device_staging, src, info->byte_size, hipMemcpyHostToDevice, s);
	if (e != hipSuccess) {
		return static_cast<int>(e);
	}
	return nh_q8_0_tile(device_staging, device_dst, static_cast<int64_t>(info->dims[1]), static_cast<int64_t>(info->dims[0]), stream);
}

} // extern "C"
