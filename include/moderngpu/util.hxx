// mgpu for AMD CDNA4: formatted text into a std::string, for the device
// description that standard_context_t prints (the helper has the name it has
// in src/moderngpu/util.hxx:11).
#pragma once
#include <cstdio>
#include <string>
#include "types.hxx"

BEGIN_MGPU_NAMESPACE
namespace detail {

// snprintf twice: once for the length, once into a string of that length.
template<typename... args_t>
std::string stringprintf(const char* format, args_t... args) {
  int length = std::snprintf(nullptr, 0, format, args...);
  std::string text(length > 0 ? length : 0, '\0');
  if(length > 0)
    std::snprintf(&text[0], (size_t)length + 1, format, args...);
  return text;
}

} // namespace detail
END_MGPU_NAMESPACE
