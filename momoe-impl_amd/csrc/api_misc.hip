// Version and status strings of the C ABI.
#include <atomic>

#include "common.hpp"

namespace momoe {
namespace {
std::atomic<unsigned long long*> g_clock_trace{nullptr};
}
unsigned long long* clock_trace_buffer() { return g_clock_trace.load(std::memory_order_relaxed); }
}  // namespace momoe

extern "C" int momoe_abi_version(void) { return 2; }

extern "C" const char* momoe_status_string(int status) {
  switch (status) {
    case MOMOE_OK: return "ok";
    case MOMOE_ERR_BAD_ARG: return "bad argument (null/misaligned pointer or non-positive size)";
    case MOMOE_ERR_UNSUPPORTED: return "unsupported shape";
    case MOMOE_ERR_LAUNCH: return "kernel launch failed";
    default: return "unknown status";
  }
}

extern "C" int momoe_set_clock_trace(unsigned long long* ticks2) {
  momoe::g_clock_trace.store(ticks2, std::memory_order_relaxed);
  return MOMOE_OK;
}
