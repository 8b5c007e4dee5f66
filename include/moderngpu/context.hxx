// mgpu for AMD CDNA4: the context object every algorithm takes -- device
// properties, the stream all work is enqueued on, the temporary allocator and
// a timer.  Interface after src/moderngpu/context.hxx:12-225, on HIP types.
//
// Difference that matters for speed: the reference's standard_context_t calls
// cudaMalloc/cudaFree for every temporary, and cudaFree synchronises the
// device.  segreduce needs 3+ temporaries per call and its kernels run for
// tens of microseconds, so here standard_context_t keeps freed device blocks
// in a size-keyed cache and hands them out again.  Reuse is ordered by the
// context's single stream: a block released by one mgpu call can only be
// touched by work enqueued later on that same stream.
#pragma once

#include <vector>
#include <map>
#include <unordered_map>
#include <memory>
#include <cassert>
#include <exception>
#include <string>
#include <cstring>
#include "util.hxx"
#include "launch_params.hxx"

BEGIN_MGPU_NAMESPACE

enum memory_space_t {
  memory_space_device = 0,
  memory_space_host = 1
};

inline std::string device_prop_string(const hipDeviceProp_t& prop) {
  int ordinal = 0;
  hipError_t result = hipGetDevice(&ordinal);
  if(hipSuccess != result) throw cuda_exception_t(result);

  size_t free_mem = 0, total_mem = 0;
  result = hipMemGetInfo(&free_mem, &total_mem);
  if(hipSuccess != result) throw cuda_exception_t(result);

  // HBM is double data rate: bytes/s = clock * 2 * bus width / 8.
  double bandwidth = (prop.memoryClockRate * 1000.0) *
    (prop.memoryBusWidth / 8 * 2) / 1.0e9;

  return detail::stringprintf(
    "%s (%s) : %8.3lf Mhz   (Ordinal %d)\n"
    "%d CUs enabled, wavefront %d, %d KB LDS per workgroup.\n"
    "FreeMem: %6dMB   TotalMem: %6dMB   %2d-bit pointers.\n"
    "Mem Clock: %8.3lf Mhz x %d bits   (%5.1lf GB/s)\n"
    "L2: %d KB   ECC %s\n\n",
    prop.name, prop.gcnArchName, prop.clockRate / 1000.0, ordinal,
    prop.multiProcessorCount, prop.warpSize,
    (int)(prop.sharedMemPerBlock / 1024),
    (int)(free_mem >> 20), (int)(total_mem >> 20), (int)(8 * sizeof(int*)),
    prop.memoryClockRate / 1000.0, prop.memoryBusWidth, bandwidth,
    prop.l2CacheSize / 1024, prop.ECCEnabled ? "Enabled" : "Disabled");
}

////////////////////////////////////////////////////////////////////////////////
// context_t: derive from it to supply a stream or a custom allocator.

struct context_t {
  context_t() = default;
  virtual ~context_t() = default;

  // Not copyable: algorithms hold it by reference.
  context_t(const context_t& rhs) = delete;
  context_t& operator=(const context_t& rhs) = delete;

  virtual const hipDeviceProp_t& props() const = 0;
  virtual int ptx_version() const = 0;
  virtual hipStream_t stream() = 0;

  virtual void* alloc(size_t size, memory_space_t space) = 0;
  virtual void free(void* p, memory_space_t space) = 0;

  // Waits for the context's stream (the whole device for stream 0).
  virtual void synchronize() = 0;

  virtual hipEvent_t event() = 0;
  virtual void timer_begin() = 0;
  virtual double timer_end() = 0;
};

////////////////////////////////////////////////////////////////////////////////
// standard_context_t

class standard_context_t : public context_t {
protected:
  hipDeviceProp_t _props;
  int _ptx_version;
  hipStream_t _stream;

  hipEvent_t _timer[2];
  hipEvent_t _event;

  // Cache of released device blocks, keyed by capacity.  A block handed out
  // again may still be in use by kernels queued earlier on this context's
  // stream, so whoever gets it has to touch it through that stream only:
  // the library's kernels do, and so do to_mem(), from_mem() and
  // mem_t::clone() and the htod()/dtoh()/dtod() overloads that take the
  // context.  The raw-pointer copies without a context run on the null
  // stream, which a stream created with hipStreamNonBlocking does not wait
  // for: pass the context, or call synchronize() first, when the context has
  // such a stream.
  std::multimap<size_t, void*> _free_blocks;
  std::unordered_map<void*, size_t> _live_blocks;
  size_t _cached_bytes;
  size_t _cache_limit;

  // Small pinned host blocks (the words that totals travel back in) are
  // kept too: hipHostMalloc and hipHostFree cost far more than the kernels
  // between them.
  enum { host_block_max = 1 << 16, host_cache_limit = 1 << 20 };
  std::multimap<size_t, void*> _free_host_blocks;
  std::unordered_map<void*, size_t> _live_host_blocks;
  size_t _cached_host_bytes;

  static void check(hipError_t result) {
    if(hipSuccess != result) throw cuda_exception_t(result);
  }

  void init() {
    int ordinal = 0;
    check(hipGetDevice(&ordinal));
    check(hipGetDeviceProperties(&_props, ordinal));
    _ptx_version = arch_version_gfx950;
    if(0 != strncmp(_props.gcnArchName, "gfx950", 6))
      fprintf(stderr, "mgpu: kernels are tuned and built for gfx950; device "
        "reports %s\n", _props.gcnArchName);

    check(hipEventCreate(&_timer[0]));
    check(hipEventCreate(&_timer[1]));
    check(hipEventCreate(&_event));
    _cached_bytes = 0;
    _cached_host_bytes = 0;
    // Keep at most 1/8 of device memory parked in the cache.
    _cache_limit = _props.totalGlobalMem / 8;
  }

  static size_t round_size(size_t size) {
    // 256-byte granules up to 1 MB, then 1/8-octave steps, so that calls
    // with slightly different tile counts share blocks.
    if(size <= (1u << 20)) return (size + 255) & ~(size_t)255;
    size_t step = (size_t)1 << (63 - __builtin_clzll(size) - 3);
    return (size + step - 1) & ~(step - 1);
  }

public:
  standard_context_t(bool print_prop = true, hipStream_t stream_ = 0) :
    context_t(), _stream(stream_) {
    init();
    if(print_prop)
      printf("%s\n", device_prop_string(_props).c_str());
  }

  ~standard_context_t() {
    release_cache();
    (void)hipEventDestroy(_timer[0]);
    (void)hipEventDestroy(_timer[1]);
    (void)hipEventDestroy(_event);
  }

  virtual const hipDeviceProp_t& props() const { return _props; }
  virtual int ptx_version() const { return _ptx_version; }
  virtual hipStream_t stream() { return _stream; }

  // Returns every cached block to the driver (waits for the stream first).
  void release_cache() {
    if(_free_blocks.empty() && _free_host_blocks.empty()) return;
    (void)hipStreamSynchronize(_stream);
    for(auto& kv : _free_blocks) (void)hipFree(kv.second);
    _free_blocks.clear();
    _cached_bytes = 0;
    for(auto& kv : _free_host_blocks) (void)hipHostFree(kv.second);
    _free_host_blocks.clear();
    _cached_host_bytes = 0;
  }

  virtual void* alloc(size_t size, memory_space_t space) {
    void* p = nullptr;
    if(!size) return p;
    if(memory_space_host == space) {
      if(size > host_block_max) {
        check(hipHostMalloc(&p, size, hipHostMallocDefault));
        return p;
      }
      size_t host_capacity = (size + 255) & ~(size_t)255;
      auto found = _free_host_blocks.lower_bound(host_capacity);
      if(found != _free_host_blocks.end()) {
        p = found->second;
        host_capacity = found->first;
        _cached_host_bytes -= host_capacity;
        _free_host_blocks.erase(found);
      } else
        check(hipHostMalloc(&p, host_capacity, hipHostMallocDefault));
      _live_host_blocks[p] = host_capacity;
      return p;
    }
    size_t capacity = round_size(size);
    auto it = _free_blocks.lower_bound(capacity);
    if(it != _free_blocks.end() && it->first <= capacity + capacity / 4) {
      p = it->second;
      capacity = it->first;
      _cached_bytes -= capacity;
      _free_blocks.erase(it);
    } else {
      hipError_t result = hipMalloc(&p, capacity);
      if(hipSuccess != result) {
        // Out of memory with blocks parked in the cache: drop them, retry.
        (void)hipGetLastError();
        release_cache();
        check(hipMalloc(&p, capacity));
      }
    }
    _live_blocks[p] = capacity;
    return p;
  }

  virtual void free(void* p, memory_space_t space) {
    if(!p) return;
    if(memory_space_host == space) {
      auto host = _live_host_blocks.find(p);
      if(host == _live_host_blocks.end()) {
        check(hipHostFree(p));
        return;
      }
      size_t host_capacity = host->second;
      _live_host_blocks.erase(host);
      if(_cached_host_bytes + host_capacity > host_cache_limit)
        check(hipHostFree(p));
      else {
        _free_host_blocks.emplace(host_capacity, p);
        _cached_host_bytes += host_capacity;
      }
      return;
    }
    auto it = _live_blocks.find(p);
    if(it == _live_blocks.end()) {
      check(hipFree(p));     // not ours (allocated before a cache reset)
      return;
    }
    size_t capacity = it->second;
    _live_blocks.erase(it);
    if(_cached_bytes + capacity > _cache_limit) {
      check(hipFree(p));     // synchronises, like the reference always does
    } else {
      _free_blocks.emplace(capacity, p);
      _cached_bytes += capacity;
    }
  }

  virtual void synchronize() {
    check(_stream ? hipStreamSynchronize(_stream) : hipDeviceSynchronize());
  }

  virtual hipEvent_t event() { return _event; }

  virtual void timer_begin() {
    check(hipEventRecord(_timer[0], _stream));
  }
  // Seconds since timer_begin, measured on the context's stream.
  virtual double timer_end() {
    check(hipEventRecord(_timer[1], _stream));
    check(hipEventSynchronize(_timer[1]));
    float ms = 0;
    check(hipEventElapsedTime(&ms, _timer[0], _timer[1]));
    return ms / 1.0e3;
  }
};

////////////////////////////////////////////////////////////////////////////////
// mem_t: move-only owner of a device or pinned-host array allocated through
// a context.

template<typename type_t>
class mem_t {
  context_t* _context;
  type_t* _pointer;
  size_t _size;
  memory_space_t _space;

public:
  void swap(mem_t& rhs) {
    std::swap(_context, rhs._context);
    std::swap(_pointer, rhs._pointer);
    std::swap(_size, rhs._size);
    std::swap(_space, rhs._space);
  }

  mem_t() : _context(nullptr), _pointer(nullptr), _size(0),
    _space(memory_space_device) { }
  mem_t& operator=(const mem_t& rhs) = delete;
  mem_t(const mem_t& rhs) = delete;

  mem_t(size_t size, context_t& context,
    memory_space_t space = memory_space_device) :
    _context(&context), _pointer(nullptr), _size(size), _space(space) {
    _pointer = (type_t*)context.alloc(sizeof(type_t) * size, space);
  }

  mem_t(mem_t&& rhs) : mem_t() { swap(rhs); }
  mem_t& operator=(mem_t&& rhs) {
    swap(rhs);
    return *this;
  }

  ~mem_t() {
    if(_context && _pointer) _context->free(_pointer, _space);
    _pointer = nullptr;
    _size = 0;
  }

  context_t& context() const { return *_context; }
  size_t size() const { return _size; }
  type_t* data() const { return _pointer; }
  memory_space_t space() const { return _space; }

  // Deep copy in the same memory space, made on the context's stream and
  // waited for: either block may be one that kernels queued earlier on that
  // stream still use.
  mem_t clone() {
    mem_t cloned(size(), context(), space());
    if(size()) {
      hipStream_t stream = context().stream();
      hipError_t result = hipMemcpyAsync(cloned.data(), data(),
        sizeof(type_t) * size(), memory_space_device == space() ?
          hipMemcpyDeviceToDevice : hipMemcpyHostToHost, stream);
      if(hipSuccess == result) result = hipStreamSynchronize(stream);
      if(hipSuccess != result) throw cuda_exception_t(result);
    }
    return cloned;
  }
};

END_MGPU_NAMESPACE
