// mgpu for AMD CDNA4: host<->device copies and mem_t factories
// (interface after src/moderngpu/memory.hxx:12-129; returns hipError_t).
#pragma once

#include <vector>
#include <cstring>
#include "transform.hxx"
#include "context.hxx"

BEGIN_MGPU_NAMESPACE

namespace detail {
template<typename type_t>
hipError_t copy_n(type_t* dest, const type_t* source, size_t count,
  hipMemcpyKind kind) {
  return count ?
    hipMemcpy(dest, source, sizeof(type_t) * count, kind) : hipSuccess;
}
} // namespace detail

////////////////////////////////////////////////////////////////////////////////
// Raw-pointer copies.

template<typename type_t>
hipError_t htoh(type_t* dest, const type_t* source, size_t count) {
  if(count) memcpy(dest, source, sizeof(type_t) * count);
  return hipSuccess;
}
template<typename type_t>
hipError_t dtoh(type_t* dest, const type_t* source, size_t count) {
  return detail::copy_n(dest, source, count, hipMemcpyDeviceToHost);
}
template<typename type_t>
hipError_t htod(type_t* dest, const type_t* source, size_t count) {
  return detail::copy_n(dest, source, count, hipMemcpyHostToDevice);
}
template<typename type_t>
hipError_t dtod(type_t* dest, const type_t* source, size_t count) {
  return detail::copy_n(dest, source, count, hipMemcpyDeviceToDevice);
}
template<typename type_t>
hipError_t dtoh(std::vector<type_t>& dest, const type_t* source,
  size_t count) {
  dest.resize(count);
  return dtoh(dest.data(), source, count);
}
template<typename type_t>
hipError_t htod(type_t* dest, const std::vector<type_t>& source) {
  return htod(dest, source.data(), source.size());
}

////////////////////////////////////////////////////////////////////////////////
// mem_t factories.

template<typename type_t>
mem_t<type_t> to_mem(const std::vector<type_t>& data, context_t& context) {
  mem_t<type_t> mem(data.size(), context);
  hipError_t result = htod(mem.data(), data);
  if(hipSuccess != result) throw cuda_exception_t(result);
  return mem;
}

template<typename type_t>
std::vector<type_t> from_mem(const mem_t<type_t>& mem) {
  std::vector<type_t> host;
  hipError_t result = dtoh(host, mem.data(), mem.size());
  if(hipSuccess != result) throw cuda_exception_t(result);
  return host;
}

template<typename type_t, typename func_t>
mem_t<type_t> fill_function(func_t f, size_t count, context_t& context) {
  mem_t<type_t> mem(count, context);
  type_t* p = mem.data();
  transform([=]MGPU_DEVICE(int index) { p[index] = f(index); },
    count, context);
  return mem;
}

template<typename type_t>
mem_t<type_t> fill(type_t value, size_t count, context_t& context) {
  mem_t<type_t> mem(count, context);
  type_t* p = mem.data();
  transform([=]MGPU_DEVICE(int index) { p[index] = value; }, count, context);
  return mem;
}

template<typename it_t>
auto copy_to_mem(it_t input, size_t count, context_t& context) ->
  mem_t<typename std::iterator_traits<it_t>::value_type> {
  typedef typename std::iterator_traits<it_t>::value_type type_t;
  mem_t<type_t> mem(count, context);
  type_t* p = mem.data();
  transform([=]MGPU_DEVICE(int index) { p[index] = input[index]; },
    count, context);
  return mem;
}

inline std::mt19937& get_mt19937() {
  static std::mt19937 mt19937;
  return mt19937;
}

// count uniform ints in [a, b], optionally sorted, on the device.
inline mem_t<int> fill_random(int a, int b, size_t count, bool sorted,
  context_t& context) {
  std::uniform_int_distribution<int> d(a, b);
  std::vector<int> data(count);
  for(int& i : data) i = d(get_mt19937());
  if(sorted) std::sort(data.begin(), data.end());
  return to_mem(data, context);
}

END_MGPU_NAMESPACE
