// Host-side plumbing of libsmr_gfx950: error text, spin timeout, version.
#include <atomic>
#include <cstdio>
#include <cstring>

#include "smr_internal.hpp"

namespace smr {

static thread_local char g_err[256] = "";
// wall_clock64() ticks at a constant 100 MHz on gfx9-family parts.
static constexpr uint64_t kTicksPerUs = 100;
static std::atomic<int64_t> g_spin_timeout_us{2000000};

void set_last_error(const char* msg) {
  std::strncpy(g_err, msg ? msg : "", sizeof(g_err) - 1);
  g_err[sizeof(g_err) - 1] = 0;
}

int fail(int code, const char* msg) {
  set_last_error(msg);
  return code;
}

int check_hip(hipError_t e, const char* what) {
  if (e == hipSuccess) return 0;
  char buf[256];
  std::snprintf(buf, sizeof(buf), "%s: %s", what, hipGetErrorString(e));
  set_last_error(buf);
  return (int)e;
}

static std::atomic<uint64_t*> g_trace{nullptr};
static std::atomic<int64_t> g_trace_words{0};

uint64_t* trace_buffer(int64_t min_words) {
  uint64_t* p = g_trace.load(std::memory_order_relaxed);
  return (p != nullptr && g_trace_words.load(std::memory_order_relaxed) >= min_words) ? p : nullptr;
}

uint64_t spin_limit_ticks() {
  int64_t us = g_spin_timeout_us.load(std::memory_order_relaxed);
  return us <= 0 ? 0 : (uint64_t)us * kTicksPerUs;
}

}  // namespace smr

extern "C" {

int smr_version(void) { return SMR_VERSION; }

const char* smr_last_error_string(void) { return smr::g_err; }

int smr_set_spin_timeout_us(int64_t us) {
  if (us < 0) return smr::fail(SMR_E_INVALID, "smr_set_spin_timeout_us: negative timeout");
  smr::g_spin_timeout_us.store(us, std::memory_order_relaxed);
  return 0;
}

int smr_set_trace_buffer(uint64_t* trace_dev, int64_t words) {
  if (words < 0 || (trace_dev == nullptr) != (words == 0))
    return smr::fail(SMR_E_INVALID, "smr_set_trace_buffer: pointer and size must both be set or both be zero");
  smr::g_trace.store(trace_dev, std::memory_order_relaxed);
  smr::g_trace_words.store(words, std::memory_order_relaxed);
  return 0;
}

int64_t smr_get_spin_timeout_us(void) {
  return smr::g_spin_timeout_us.load(std::memory_order_relaxed);
}

}  // extern "C"
