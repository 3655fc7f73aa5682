// Only for builds with -DCP4_DEBUG_PHASES (never the shipped library): where the
// in-kernel time stamps of such a build go.  The one place in the sources that
// takes a device address from the environment: CP4_DBG_PTR holds, in decimal, the
// address of a caller-allocated device buffer of 64-bit words; unset, the stamps
// are off.
#ifndef CP4_DEBUG_H
#define CP4_DEBUG_H
#ifndef CP4_DEBUG_PHASES
#error "cp4_debug.h is for -DCP4_DEBUG_PHASES builds only"
#endif
#include <cstdlib>

namespace cp4 {
inline long long* debug_stamp_buffer() {
  const char* e = getenv("CP4_DBG_PTR");
  return e ? reinterpret_cast<long long*>(strtoull(e, nullptr, 10)) : nullptr;
}
// CP4_FWD_PHASES=<n>: the phase-by-phase strip kernel stops after phase n (timing
// the phases one by one).
inline int debug_phase_limit(int all) {
  const char* e = getenv("CP4_FWD_PHASES");
  return e ? atoi(e) : all;
}
}  // namespace cp4
#endif
