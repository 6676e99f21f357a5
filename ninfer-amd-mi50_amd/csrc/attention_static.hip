// Decode attention with its workspace in a fixed device array: see no_alloc.h.
#include "no_alloc.h"
#include <mutex>

using namespace ninfer;

namespace {

constexpr long long kScratchFloats = 4ll << 20;   // 16 MiB
static __device__ __align__(256) float scratch[kScratchFloats];

constexpr int kMaxDevices = 64;
float* g_scratch_ptr[kMaxDevices] = {};   // the array's address on each device, once looked up
std::mutex g_mutex;

// The address of `scratch` on the current device. In host code the array's name is only a
// handle for this lookup, not a device address: kernels get the pointer found here.
int scratch_on_current_device(float** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return set_error(-2, "decode_attention_static: no current device: %s", hipGetErrorString(e));
  if (dev < 0 || dev >= kMaxDevices)
    return set_error(-2, "decode_attention_static: device %d is beyond the %d this library counts", dev, kMaxDevices);
  std::lock_guard<std::mutex> lock(g_mutex);
  if (!g_scratch_ptr[dev]) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p)
      return set_error(-2, "decode_attention_static: cannot find the workspace on device %d: %s", dev, hipGetErrorString(e));
    g_scratch_ptr[dev] = (float*)p;
  }
  *out = g_scratch_ptr[dev];
  return 0;
}

}  // namespace

extern "C" int ninfer_decode_attention_static_init() {
  float* p;
  return scratch_on_current_device(&p);
}

extern "C" long long ninfer_decode_attention_static_max_floats() { return kScratchFloats; }

extern "C" int ninfer_decode_attention_static(const AttnArgs* args, hipStream_t stream) {
  if (int rc = attention_check(*args)) return rc;
  AttnArgs a = *args;
  NINFER_REQUIRE(a.max_qlen == 1 && a.T == a.S, "decode_attention_static: single-token rows only "
                 "(%d rows of %d requests, longest %d)", a.T, a.S, a.max_qlen);
  NINFER_REQUIRE(a.dtype == kBF16, "decode_attention_static: bf16 only");
  const long long need = attention_decode_workspace_floats(a.T, a.Hq, a.D, a.max_kv_len);
  NINFER_REQUIRE(need <= kScratchFloats, "decode_attention_static: %d rows of %d heads over %d keys "
                 "need %lld floats of workspace; the fixed one holds %lld", a.T, a.Hq, a.max_kv_len,
                 need, kScratchFloats);
  float* ws = nullptr;
  if (int rc = scratch_on_current_device(&ws)) return rc;
  a.workspace = ws;
  a.workspace_floats = kScratchFloats;
  NINFER_REQUIRE(attention_decode_takes(a), "decode_attention_static: the split-context kernels do "
                 "not take heads of %d with pages of %d (row stride %d)", a.D, a.page_size, a.q_stride);
  return attention_decode(a, stream);
}
