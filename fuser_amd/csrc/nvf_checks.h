// NVF_CHECK / NVF_CHECK_EQ / NVF_THROW for the host layer.  With the reference's csrc/exceptions.h on the include path
// (nvf_cutlass.h then defines NVF_HIP_REFERENCE_EXCEPTIONS) these are the reference's own macros, which throw its
// nvfError with source location and backtrace; otherwise they are defined here with the same message shape
// (csrc/exceptions.h:200-245: "Expected <cond> . <message>") and throw the stand-in class of nvf_cutlass.h.
#pragma once

#include "nvf_cutlass.h"

#ifndef NVF_HIP_REFERENCE_EXCEPTIONS
#include <sstream>

namespace nvfuser {
namespace checks_detail {
template <typename... Args>
std::string concat(const Args&... args) {
  std::ostringstream os;
  (void)std::initializer_list<int>{((os << args), 0)...};
  return os.str();
}
}  // namespace checks_detail
}  // namespace nvfuser

#define NVF_CHECK(cond, ...)                                                                                       \
  do {                                                                                                             \
    if (!(cond)) throw ::nvfuser::nvfError(::nvfuser::checks_detail::concat("Expected " #cond " . ", ##__VA_ARGS__)); \
  } while (0)
#define NVF_CHECK_EQ(lhs, rhs, ...)                                                                                 \
  do {                                                                                                              \
    if (!((lhs) == (rhs)))                                                                                          \
      throw ::nvfuser::nvfError(                                                                                    \
          ::nvfuser::checks_detail::concat("Expected " #lhs " == " #rhs " . Found ", (lhs), " vs ", (rhs), ". ", ##__VA_ARGS__)); \
  } while (0)
#define NVF_THROW(...) throw ::nvfuser::nvfError(::nvfuser::checks_detail::concat(__VA_ARGS__))
#endif
