// Mutates a valid GGUF file (truncations, byte and bit flips, overwritten 32- and 64-bit fields, sizes near the end of the file) and runs
// every query of the reader on each mutant; built with AddressSanitizer and UBSan, CPU only.  Usage: fuzz_gguf <file> <mutants> <seed> <scratch path>
#include <nihilus_amd/gguf_q8_0.h>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <vector>
static std::vector<unsigned char> slurp(const char* p) { FILE* f = fopen(p, "rb"); std::vector<unsigned char> b; unsigned char t[4096]; size_t n; while ((n = fread(t, 1, sizeof t, f)) > 0) b.insert(b.end(), t, t + n); fclose(f); return b; }
int main(int argc, char** argv) {
	const std::vector<unsigned char> base = slurp(argv[1]);
	const int iters = argc > 2 ? atoi(argv[2]) : 1000;
	std::mt19937_64 rng(argc > 3 ? atoi(argv[3]) : 1);
	const char* keys[] = { "general.architecture", "general.alignment", "llama.block_count", "llama.attention.layer_norm_rms_epsilon", "llama.context_length", "some.negative", "some.flag", "some.double", "tokenizer.ggml.tokens", "tokenizer.ggml.token_type", "missing" };
	long opened = 0;
	// the header and directory end well before the tensor data: mutate mostly there
	const size_t head = base.size() < 1024 ? base.size() : 1024;
	for (int it = 0; it < iters; ++it) {
		std::vector<unsigned char> b = base;
		const int kind = rng() % 7;
		if (kind == 0) b.resize(rng() % (b.size() + 1));
		else if (kind == 1) for (int j = 0, n = 1 + rng() % 4; j < n; ++j) b[rng() % head] = static_cast<unsigned char>(rng());
		else if (kind == 2) { const size_t at = rng() % (head - 8); const unsigned long long v = (rng() % 4 == 0) ? ~0ull >> (rng() % 64) : rng(); memcpy(&b[at], &v, 8); }
		else if (kind == 3) { const size_t at = rng() % (head - 4); const unsigned v = static_cast<unsigned>(rng() % 64); memcpy(&b[at], &v, 4); }
		else if (kind == 4) { b[rng() % head] ^= 1u << (rng() % 8); b.resize(head + rng() % (b.size() - head + 1)); }
		else if (kind == 5) { const size_t at = rng() % (head - 8); const unsigned long long v = b.size() + (rng() % 64) - 32; memcpy(&b[at], &v, 8); }
		else { const size_t at = rng() % (head - 8); const unsigned long long v = 0ull - 32ull * (1 + rng() % 64); memcpy(&b[at], &v, 8); } // just below 2^64: an offset that wraps when added to the data start
		const char* tmp = argc > 4 ? argv[4] : "/tmp/nh_fuzz.gguf";
		FILE* f = fopen(tmp, "wb"); fwrite(b.data(), 1, b.size(), f); fclose(f);
		nh_gguf* g = nullptr;
		if (nh_gguf_open(tmp, &g) != 0 || !g) continue;
		++opened;
		const int64_t nt = nh_gguf_tensor_count(g);
		(void)nh_gguf_metadata_count(g); (void)nh_gguf_alignment(g); (void)nh_gguf_data_offset(g); (void)nh_gguf_version(g);
		unsigned long long sink = 0;
		for (int64_t i = -1; i <= nt; ++i) {
			nh_gguf_tensor_info ti;
			if (nh_gguf_tensor_at(g, i, &ti) == 0) {
				nh_gguf_tensor_info tj;
				sink += strlen(ti.name) + (nh_gguf_find_tensor(g, ti.name, &tj) == 0);
				if (ti.file_offset < nh_gguf_data_offset(g)) { printf("iter %d: tensor %s starts before the data section (%llu < %llu)\n", it, ti.name, (unsigned long long)ti.file_offset, (unsigned long long)nh_gguf_data_offset(g)); return 1; }
				if (ti.file_offset + ti.byte_size > b.size()) { printf("iter %d: tensor %s past the end of the file (%llu + %llu > %zu)\n", it, ti.name, (unsigned long long)ti.file_offset, (unsigned long long)ti.byte_size, b.size()); return 1; }
			}
		}
		for (const char* k : keys) {
			int64_t i64; uint64_t u64, len, cnt; double f64; const char* s; uint32_t et; const void* first;
			(void)nh_gguf_metadata_i64(g, k, &i64); (void)nh_gguf_metadata_u64(g, k, &u64); (void)nh_gguf_metadata_f64(g, k, &f64);
			if (nh_gguf_metadata_string(g, k, &s, &len) == 0) for (uint64_t j = 0; j < len; ++j) sink += static_cast<unsigned char>(s[j]);
			if (nh_gguf_metadata_array(g, k, &et, &cnt, &first) == 0 && first && cnt) sink += *static_cast<const unsigned char*>(first);
		}
		nh_gguf_close(g);
		if (sink == 42) puts("");
	}
	printf("%d mutants, %ld opened\n", iters, opened);
	return 0;
}
