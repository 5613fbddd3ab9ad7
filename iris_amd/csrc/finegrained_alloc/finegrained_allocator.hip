// Fine-grained allocator plug-in for torch.cuda.memory.CUDAPluggableAllocator.
//
// Same two C symbols and the same behaviour as the reference plug-in
// (csrc/finegrained_alloc/finegrained_allocator.hip:28-55): allocate with
// hipExtMallocWithFlags(hipDeviceMallocFinegrained) on the requested device,
// restore the caller's device, ignore the stream; on any HIP error report to
// stderr and terminate (there is no error channel in this ABI).
// LOG_FINEGRAINED_ALLOCATOR in the environment turns on per-call logging.
#include <hip/hip_runtime.h>
#include <sys/types.h>

#include <cstdio>
#include <cstdlib>

namespace {

void check(hipError_t err, int line) {
  if (err == hipSuccess) return;
  std::fprintf(stderr, "[finegrained_allocator] Hip error: %s at line %d\n", hipGetErrorString(err), line);
  std::exit(EXIT_FAILURE);
}
#define FG_CHECK(expr) check((expr), __LINE__)

bool logging() { return std::getenv("LOG_FINEGRAINED_ALLOCATOR") != nullptr; }

// Runs `fn` with `device` current and puts the previous device back.
class DeviceScope {
 public:
  explicit DeviceScope(int device) {
    FG_CHECK(hipGetDevice(&prev_));
    FG_CHECK(hipSetDevice(device));
  }
  ~DeviceScope() { FG_CHECK(hipSetDevice(prev_)); }

 private:
  int prev_ = 0;
};

}  // namespace

extern "C" void* finegrained_hipMalloc(ssize_t size, int device, void* /*stream*/) {
  void* ptr = nullptr;
  {
    DeviceScope scope(device);
    FG_CHECK(hipExtMallocWithFlags(&ptr, static_cast<size_t>(size), hipDeviceMallocFinegrained));
  }
  if (logging())
    std::printf("[finegrained_allocator] Allocation: ptr=%p, size=%zd bytes, device=%d\n", ptr, size, device);
  return ptr;
}

extern "C" void finegrained_hipFree(void* ptr, ssize_t size, int device, void* /*stream*/) {
  if (logging())
    std::printf("[finegrained_allocator] Deallocation: ptr=%p, size=%zd bytes, device=%d\n", ptr, size, device);
  DeviceScope scope(device);
  FG_CHECK(hipFree(ptr));
}
