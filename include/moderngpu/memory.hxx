// mgpu for AMD CDNA4: copies between host and device memory and the mem_t
// factories the tests and demos build their inputs with.  Function names and
// argument orders after src/moderngpu/memory.hxx:12-129; the copies return a
// hipError_t, the factories throw cuda_exception_t.
#pragma once

#include <cstring>
#include <vector>
#include "transform.hxx"
#include "context.hxx"

BEGIN_MGPU_NAMESPACE

namespace detail {

// count elements, blocking; nothing is issued for an empty copy.
template<hipMemcpyKind kind, typename type_t>
hipError_t copy_elements(type_t* dest, const type_t* source, size_t count) {
  if(!count) return hipSuccess;
  return hipMemcpy(dest, source, sizeof(type_t) * count, kind);
}

inline void throw_on_error(hipError_t status) {
  if(hipSuccess != status) throw cuda_exception_t(status);
}

// The same copy issued on the context's stream and waited for.  Memory that
// comes from a context may be a recycled block (standard_context_t keeps
// released blocks) that kernels queued earlier on the context's stream still
// use; a copy on the null stream is not ordered behind a non-blocking stream,
// a copy on the context's stream is.
template<hipMemcpyKind kind, typename type_t>
hipError_t copy_elements(type_t* dest, const type_t* source, size_t count,
  context_t& context) {
  if(!count) return hipSuccess;
  hipStream_t stream = context.stream();
  hipError_t result = hipMemcpyAsync(dest, source, sizeof(type_t) * count,
    kind, stream);
  if(hipSuccess != result) return result;
  return hipStreamSynchronize(stream);
}

// A mem_t of count elements, element i set to value_at(i) by a kernel.
template<typename type_t, typename value_at_t>
mem_t<type_t> mem_from_function(value_at_t value_at, size_t count,
  context_t& context) {
  mem_t<type_t> mem(count, context);
  type_t* data = mem.data();
  transform([=]MGPU_DEVICE(int i) { data[i] = value_at(i); }, count, context);
  return mem;
}

} // namespace detail

////////////////////////////////////////////////////////////////////////////////
// Copies through raw pointers, named source-to-destination.

template<typename type_t>
hipError_t htoh(type_t* dest, const type_t* source, size_t count) {
  return detail::copy_elements<hipMemcpyHostToHost>(dest, source, count);
}
template<typename type_t>
hipError_t dtoh(type_t* dest, const type_t* source, size_t count) {
  return detail::copy_elements<hipMemcpyDeviceToHost>(dest, source, count);
}
template<typename type_t>
hipError_t htod(type_t* dest, const type_t* source, size_t count) {
  return detail::copy_elements<hipMemcpyHostToDevice>(dest, source, count);
}
template<typename type_t>
hipError_t dtod(type_t* dest, const type_t* source, size_t count) {
  return detail::copy_elements<hipMemcpyDeviceToDevice>(dest, source, count);
}

// The host side as a std::vector; a destination vector is resized to count.
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

// The same copies on a context's stream, waited for: the forms to use with
// memory that came from that context when its stream does not synchronise with
// the null stream (hipStreamNonBlocking) -- the block may be a recycled one
// that kernels queued earlier on the stream still use, and only a copy on the
// same stream is ordered behind them.  (No counterpart in the CUDA library,
// whose contexts return blocks with a cudaFree that waits for the device.)
template<typename type_t>
hipError_t dtoh(type_t* dest, const type_t* source, size_t count,
  context_t& context) {
  return detail::copy_elements<hipMemcpyDeviceToHost>(dest, source, count,
    context);
}
template<typename type_t>
hipError_t htod(type_t* dest, const type_t* source, size_t count,
  context_t& context) {
  return detail::copy_elements<hipMemcpyHostToDevice>(dest, source, count,
    context);
}
template<typename type_t>
hipError_t dtod(type_t* dest, const type_t* source, size_t count,
  context_t& context) {
  return detail::copy_elements<hipMemcpyDeviceToDevice>(dest, source, count,
    context);
}
template<typename type_t>
hipError_t dtoh(std::vector<type_t>& dest, const type_t* source,
  size_t count, context_t& context) {
  dest.resize(count);
  return dtoh(dest.data(), source, count, context);
}
template<typename type_t>
hipError_t htod(type_t* dest, const std::vector<type_t>& source,
  context_t& context) {
  return htod(dest, source.data(), source.size(), context);
}

////////////////////////////////////////////////////////////////////////////////
// mem_t factories.

// A device copy of a host vector, and back.
// Both copies run on the context's stream (see detail::copy_elements).
template<typename type_t>
mem_t<type_t> to_mem(const std::vector<type_t>& data, context_t& context) {
  mem_t<type_t> mem(data.size(), context);
  detail::throw_on_error(detail::copy_elements<hipMemcpyHostToDevice>(
    mem.data(), data.data(), data.size(), context));
  return mem;
}
template<typename type_t>
std::vector<type_t> from_mem(const mem_t<type_t>& mem) {
  std::vector<type_t> host(mem.size());
  detail::throw_on_error(detail::copy_elements<hipMemcpyDeviceToHost>(
    host.data(), mem.data(), mem.size(), mem.context()));
  return host;
}

// Element i is f(i).
template<typename type_t, typename func_t>
mem_t<type_t> fill_function(func_t f, size_t count, context_t& context) {
  return detail::mem_from_function<type_t>(f, count, context);
}

// Every element is value.
template<typename type_t>
mem_t<type_t> fill(type_t value, size_t count, context_t& context) {
  return detail::mem_from_function<type_t>(
    [=]MGPU_DEVICE(int) { return value; }, count, context);
}

// Element i is input[i], for any device-readable iterator.
template<typename it_t>
auto copy_to_mem(it_t input, size_t count, context_t& context) {
  typedef typename std::iterator_traits<it_t>::value_type type_t;
  return detail::mem_from_function<type_t>(
    [=]MGPU_DEVICE(int i) { return (type_t)input[i]; }, count, context);
}

// The generator the random fills draw from: one per process, default seeded,
// so a test's inputs are the same on every run.
inline std::mt19937& get_mt19937() {
  static std::mt19937 generator;
  return generator;
}

// count integers uniform in [a, b], ascending if sorted, as device memory.
inline mem_t<int> fill_random(int a, int b, size_t count, bool sorted,
  context_t& context) {
  std::vector<int> host(count);
  std::uniform_int_distribution<int> draw(a, b);
  std::generate(host.begin(), host.end(),
    [&] { return draw(get_mt19937()); });
  if(sorted) std::sort(host.begin(), host.end());
  return to_mem(host, context);
}

END_MGPU_NAMESPACE
