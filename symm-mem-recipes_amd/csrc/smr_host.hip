// Host-side plumbing of libsmr_gfx950: error text, spin timeout, version.
#include <atomic>
#include <cstdio>
#include <cstring>

#include "smr_device.hpp"

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

int64_t smr_get_spin_timeout_us(void) {
  return smr::g_spin_timeout_us.load(std::memory_order_relaxed);
}

}  // extern "C"
