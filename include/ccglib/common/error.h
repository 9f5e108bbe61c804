// Turns a C ABI status into the exception the ccglib classes throw.
#ifndef CCGLIB_COMMON_ERROR_H_
#define CCGLIB_COMMON_ERROR_H_
#include <stdexcept>

#include <ccglib_amd.h>

namespace ccglib::detail {
inline void check(int status) {
  if (status != CCGLIB_OK) throw std::runtime_error(ccglib_last_error());
}
// HIP device handles are ordinals; the C ABI takes the ordinal.
inline int ordinal(int device) { return device; }
}  // namespace ccglib::detail
#endif  // CCGLIB_COMMON_ERROR_H_
