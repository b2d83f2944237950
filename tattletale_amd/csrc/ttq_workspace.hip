// Device workspaces for the paths that need one (partial sums of split launches and their arrival counters, the
// trellis GEMV's hand-off words, bf16 / rotated copies of the activations).
//
// Caller-owned (the ttq_*_ws entry points): the caller's buffer is bound to the calling thread for the duration of
// one call and every request is served from it; nothing is allocated, so the call can be captured into a HIP graph
// the first time it runs.  Layout: [0, 64 KiB) arrival counters, then the trellis hand-off words with their control
// words, then the scratch of the call, handed out front to back.  The first two regions rely on what earlier calls
// left there (counters back at zero, a generation count): the caller clears the buffer once, before its first use.
//
// Library-owned (the entry points without a workspace argument): one buffer per (slot, device, stream) -- launches
// on one stream run in order and can share a buffer, launches on different streams may overlap and get their own --
// grown on demand (by at least a factor of two; outgrown buffers stay allocated, because launches in flight and
// captured graphs may still name them) and kept until ttq_release_workspaces or the end of the process.

#include "ttq_device.h"
#include "ttq_internal.h"

#include <mutex>
#include <unordered_map>
#include <vector>

namespace ttq {

namespace {
struct Buf { void* p; size_t bytes; };
struct Owned { Buf cur; std::vector<void*> retired; };
std::mutex g_mutex;
std::unordered_map<uint64_t, Owned> g_bufs;

struct CallerWs { uint8_t* base; size_t bytes, bump; bool too_small; };
thread_local CallerWs* t_caller = nullptr;

constexpr size_t kCwCounterBytes = 64 * 1024;
size_t round256(size_t v) { return (v + 255) & ~(size_t)255; }
}  // namespace

size_t caller_workspace_header_bytes() {
  return kCwCounterBytes + round256((size_t)exl3_workspace_words() * sizeof(unsigned long long));
}

CallerWsScope::CallerWsScope(void* ws, size_t bytes) {
  static_assert(sizeof(CallerWs) <= sizeof(state_), "state_ holds a CallerWs");
  CallerWs* c = reinterpret_cast<CallerWs*>(state_);
  c->base = static_cast<uint8_t*>(ws);
  c->bytes = bytes;
  c->bump = caller_workspace_header_bytes();
  c->too_small = false;
  t_caller = c;
}
CallerWsScope::~CallerWsScope() { t_caller = nullptr; }
bool CallerWsScope::too_small() const { return reinterpret_cast<const CallerWs*>(state_)->too_small; }

bool caller_workspace_region(int region, size_t bytes, void** out, hipError_t* err) {
  CallerWs* c = t_caller;
  if (!c) return false;
  size_t off = 0;
  if (region == kCwCounters) {
    if (bytes > kCwCounterBytes) c->too_small = true;
  } else if (region == kCwExl3Words) {
    off = kCwCounterBytes;
    if (bytes > caller_workspace_header_bytes() - kCwCounterBytes) c->too_small = true;
  } else {
    off = c->bump;
    c->bump = off + round256(bytes);
  }
  if (!c->base || off + bytes > c->bytes) c->too_small = true;
  *out = c->too_small ? nullptr : c->base + off;
  *err = c->too_small ? hipErrorOutOfMemory : hipSuccess;
  return true;
}

hipError_t stream_workspace(int slot, hipStream_t s, size_t bytes, void** out, bool zeroed) {
  hipError_t e = hipSuccess;
  if (caller_workspace_region(slot == kWsGemmCounters ? kCwCounters : kCwScratch, bytes, out, &e)) return e;
  int dev = 0;
  e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  const uint64_t key = ((uint64_t)(uint32_t)slot << 56) ^ ((uint64_t)(uint32_t)dev << 48) ^ (uint64_t)reinterpret_cast<uintptr_t>(s);
  std::lock_guard<std::mutex> lock(g_mutex);
  Owned& o = g_bufs[key];
  Buf& b = o.cur;
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
    if (b.p) o.retired.push_back(b.p);
    b.p = p;
    b.bytes = got;
  }
  *out = b.p;
  return hipSuccess;
}

hipError_t release_stream_workspaces() {
  hipError_t first = exl3_release_workspaces();
  std::lock_guard<std::mutex> lock(g_mutex);
  for (auto& kv : g_bufs) {
    kv.second.retired.push_back(kv.second.cur.p);
    for (void* p : kv.second.retired) {
      if (!p) continue;
      const hipError_t e = hipFree(p);
      if (e != hipSuccess && first == hipSuccess) first = e;
    }
  }
  g_bufs.clear();
  return first;
}

}  // namespace ttq
