#include "gguf_common.h"
extern "C" int gguf_mmq(const void*, const void*, int, void*, void*, int, int64_t, int64_t, int64_t, gguf_stream_t) { return GGUF_ERR_TYPE; }
extern "C" int gguf_moe_mmq(const void*, int, void*, const void*, int64_t, const int32_t*, const int32_t*, const int32_t*, int64_t, void*, int, int64_t, int64_t, int64_t, int64_t, gguf_stream_t) { return GGUF_ERR_TYPE; }
extern "C" int gguf_moe_vec(const void*, int, void*, const void*, const int32_t*, void*, int, int64_t, int64_t, int64_t, int64_t, gguf_stream_t) { return GGUF_ERR_TYPE; }
extern "C" int gguf_moe_block_size(int) { return 0; }
