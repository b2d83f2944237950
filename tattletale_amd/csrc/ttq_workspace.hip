// Device workspaces the library keeps for the paths that need one, one per (slot, device, stream): launches
// on one stream run in order and can share a buffer; launches on different streams may overlap and get their
// own.  Grown on demand (by at least a factor of two; outgrown buffers stay allocated, because launches in
// flight and captured graphs may still name them) and kept until the process ends.  Also here: the activation-type conversion that lets
// fp16 and fp32 activations use the bf16 matrix-core GEMM.
#include "ttq_device.h"
#include "ttq_internal.h"

#include <mutex>
#include <unordered_map>

namespace ttq {

namespace {
struct Buf { void* p; size_t bytes; };
std::mutex g_mutex;
std::unordered_map<uint64_t, Buf> g_bufs;
}  // namespace

hipError_t stream_workspace(int slot, hipStream_t s, size_t bytes, void** out, bool zeroed) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  const uint64_t key = ((uint64_t)(uint32_t)slot << 56) ^ ((uint64_t)(uint32_t)dev << 48) ^ (uint64_t)reinterpret_cast<uintptr_t>(s);
  std::lock_guard<std::mutex> lock(g_mutex);
  Buf& b = g_bufs[key];
  if (b.bytes < bytes) {
    // A buffer that has become too small is kept, not freed: launches still in flight on the stream use it, and
    // so does every HIP graph that was captured while it was current.  Growing by at least a factor of two
    // bounds what the retired buffers hold to the size of the current one.
    const size_t want = bytes > 2 * b.bytes ? bytes : 2 * b.bytes;
    size_t got = want;
    void* p = nullptr;
    e = hipMalloc(&p, want);
    if (e != hipSuccess && want > bytes) {        // no room for the spare half
      (void)hipGetLastError();
      got = bytes;
      e = hipMalloc(&p, bytes);
    }
    if (e != hipSuccess) return e;
    if (zeroed) {
      // ordered before every launch that will use the buffer: they are all on this stream
      e = hipMemsetAsync(p, 0, got, s);
      if (e != hipSuccess) {
        (void)hipFree(p);
        return e;
      }
    }
    b.p = p;
    b.bytes = got;
  }
  *out = b.p;
  return hipSuccess;
}

// 8 values per thread, rounded to bf16 (nearest even)
template <typename XT>
__global__ void __launch_bounds__(256) to_bf16_kernel(const XT* __restrict__ x, uint16_t* __restrict__ out, int64_t n8) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n8) return;
  float v[8];
#pragma unroll
  for (int k = 0; k < 8; k++) v[k] = XElem<XT>::load(x, 8 * i + k);
  uint4 o;
  o.x = pack_bf16x2(v[0], v[1]);
  o.y = pack_bf16x2(v[2], v[3]);
  o.z = pack_bf16x2(v[4], v[5]);
  o.w = pack_bf16x2(v[6], v[7]);
  *reinterpret_cast<uint4*>(out + 8 * i) = o;
}

hipError_t launch_to_bf16(const void* x, int x_dtype, uint16_t* out, int64_t n, hipStream_t s) {
  if (n == 0) return hipSuccess;
  if (n % 8) return hipErrorInvalidValue;
  const int64_t n8 = n / 8;
  const dim3 grid((unsigned)((n8 + 255) / 256)), block(256);
  if (x_dtype == kF32) hipLaunchKernelGGL(to_bf16_kernel<float>, grid, block, 0, s, static_cast<const float*>(x), out, n8);
  else if (x_dtype == kF16) hipLaunchKernelGGL(to_bf16_kernel<f16_tag>, grid, block, 0, s, static_cast<const f16_tag*>(x), out, n8);
  else return hipErrorInvalidValue;
  return hipGetLastError();
}

}  // namespace ttq
