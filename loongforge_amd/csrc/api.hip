// Error state + version of the C ABI.
#include "dsa_common.h"
#include <string.h>

static thread_local char g_err[512] = "";

void dsa_set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

extern "C" int dsa_version(void) { return 1; }
extern "C" const char* dsa_last_error(void) { return g_err; }

#include <mutex>
#include <vector>
namespace {
struct Reserved { const void* fn; int dev; size_t bytes; };
std::mutex g_reserved_mutex;
std::vector<Reserved> g_reserved;
}  // namespace

hipError_t dsa_reserve_lds(const void* fn, size_t bytes) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess) dev = -1;
  std::lock_guard<std::mutex> lock(g_reserved_mutex);
  for (Reserved& r : g_reserved)
    if (r.fn == fn && r.dev == dev) {
      if (r.bytes >= bytes) return hipSuccess;
      const hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
      if (e == hipSuccess) r.bytes = bytes;
      return e;
    }
  const hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
  if (e == hipSuccess) g_reserved.push_back({fn, dev, bytes});
  return e;
}
