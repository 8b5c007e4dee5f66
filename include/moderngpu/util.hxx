// mgpu for AMD CDNA4: printf into a std::string (used by device_prop_string).
#pragma once
#include "types.hxx"
#include <cstdarg>
#include <cstdio>
#include <string>
#include <vector>

BEGIN_MGPU_NAMESPACE

namespace detail {

inline std::string stringprintf(const char* format, ...) {
  va_list args;
  va_start(args, format);
  int len = vsnprintf(nullptr, 0, format, args);
  va_end(args);
  if(len <= 0) return std::string();

  std::vector<char> buffer(len + 1);
  va_start(args, format);
  vsnprintf(buffer.data(), buffer.size(), format, args);
  va_end(args);
  return std::string(buffer.data(), len);
}

} // namespace detail

END_MGPU_NAMESPACE
