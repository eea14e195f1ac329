// gguf_mmq for callers that cannot allocate: the activation workspace (quantized rows and the fp32 partial tiles of
// a K split) is a fixed array in device memory that the library owns, so the caller passes inputs and outputs only.
#include <atomic>

#include "gguf_common.h"

namespace gguf {
int mmq_linear_impl(const void* W, int64_t w_row_pitch_bytes, const void* x, int xdtype, void* q8_workspace, void* Y,
                    int64_t y_row_pitch, const void* bias, int type, int64_t N, int64_t K, int64_t M, int engine,
                    int64_t workspace_bytes, int64_t rows_bytes, gguf_stream_t stream);
}

namespace {

constexpr int64_t kScratchBytes = 32ll << 20;
// One copy per GPU the library's code object is loaded on, held until the process ends.  Its name is a host-side
// stand-in, not a device address: host code only ever uses the address hipGetSymbolAddress returns for the current
// device.
static __device__ __align__(256) unsigned char scratch[kScratchBytes];
constexpr int kMaxDevices = 64;
std::atomic<void*> g_scratch_ptr[kMaxDevices];

int scratch_for_current_device(void** out) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return GGUF_ERR_LAUNCH;
  void* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (!p) {
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) return GGUF_ERR_LAUNCH;
    g_scratch_ptr[dev].store(p, std::memory_order_release);   // every thread that races here stores the same address
  }
  *out = p;
  return GGUF_OK;
}

}  // namespace

extern "C" int64_t gguf_mmq_static_capacity(void) {
  void* p = nullptr;
  return scratch_for_current_device(&p) == GGUF_OK ? kScratchBytes : 0;
}

extern "C" int gguf_mmq_static(const void* W, const void* x, int xdtype, void* Y, int type, int64_t N, int64_t K, int64_t M,
                               gguf_stream_t stream) {
  const int qk = gguf::block_elems(type);
  if (qk == 0) return GGUF_ERR_TYPE;
  if (K <= 0 || K % qk != 0 || M < 0 || N < 0 || M > 0x7FFFFFF0LL) return GGUF_ERR_SHAPE;
  const int64_t rows_bytes = (M * gguf::q8_row_bytes(K) + 255) / 256 * 256;
  if (rows_bytes > kScratchBytes) return GGUF_ERR_WORKSPACE;
  void* ws = nullptr;
  const int rc = scratch_for_current_device(&ws);
  if (rc != GGUF_OK) return rc;
  return gguf::mmq_linear_impl(W, K / qk * gguf::block_bytes(type), x, xdtype, ws, Y, N, nullptr, type, N, K, M, GGUF_MMQ_AUTO,
                               kScratchBytes, rows_bytes, stream);
}
