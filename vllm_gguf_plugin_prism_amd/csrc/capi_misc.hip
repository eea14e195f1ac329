// Entry points of the C ABI that launch nothing.
#include "gguf_common.h"

extern "C" const char* gguf_hip_version(void) { return "gguf_hip 0.1 (gfx950)"; }
extern "C" int gguf_block_elems(int type) { return gguf::block_elems(type); }
extern "C" int gguf_block_bytes(int type) { return gguf::block_bytes(type); }
