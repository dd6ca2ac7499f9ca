// Shared by every device library: element types, conversions, wave and block
// reductions, and the error channel of the C entry points.
//
// Every entry point is `extern "C" int gb_*(...)`: it checks on the host that the
// operand shapes fit what the kernel and its grid assume, launches on the given
// stream and returns 0, or returns 1 after leaving a message for gb_last_error().
#pragma once
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <string>
#include <type_traits>
#include <utility>

namespace gb {

typedef __bf16 bf16;
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int kWave = 64;

// dtype codes shared with the Python side
enum : int { kF32 = 0, kBF16 = 1 };

// Key pages.  The block of one (page, kv head) holds the head's dimensions in pieces of key_piece(hd) elements
// (8 for every head size that is a multiple of 8), and of each piece the page's slots side by side:
// [hd / piece][slot in page][piece].  Lanes that take neighbouring keys for an MFMA operand then read
// neighbouring addresses, which the memory pipeline takes three times as fast as neighbours a whole key apart.
__host__ __device__ __forceinline__ int key_piece(int hd) { return hd % 8 == 0 ? 8 : hd % 4 == 0 ? 4 : hd % 2 == 0 ? 2 : 1; }
// offset of dimension d of the key in `slot` inside its (page, kv head) block
__device__ __forceinline__ int key_offset(int slot, int d, int page_size, int piece) {
  return ((d / piece) * page_size + slot) * piece + d % piece;
}

__device__ __forceinline__ float to_f(float v) { return v; }
__device__ __forceinline__ float to_f(bf16 v) { return (float)v; }
template <typename T> __device__ __forceinline__ T from_f(float v);
template <> __device__ __forceinline__ float from_f<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16 from_f<bf16>(float v) { return (bf16)v; }  // round to nearest even

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, kWave));
  return v;
}

// Sum over a block of up to 1024 threads; `scratch` holds at least 17 floats.  Every thread
// gets the result.  The order of additions is fixed by the thread layout alone.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int waves = (blockDim.x + kWave - 1) / kWave;
  v = wave_sum(v);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  if (threadIdx.x == 0) {
    float t = 0.f;
    for (int w = 0; w < waves; ++w) t += scratch[w];
    scratch[16] = t;
  }
  __syncthreads();
  return scratch[16];
}
__device__ __forceinline__ float block_max(float v, float* scratch) {
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int waves = (blockDim.x + kWave - 1) / kWave;
  v = wave_max(v);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  if (threadIdx.x == 0) {
    float t = scratch[0];
    for (int w = 1; w < waves; ++w) t = fmaxf(t, scratch[w]);
    scratch[16] = t;
  }
  __syncthreads();
  return scratch[16];
}

inline std::string& last_error() {
  static thread_local std::string msg;
  return msg;
}

inline int fail(const char* fmt, ...) {
  char buf[512];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof buf, fmt, ap);
  va_end(ap);
  last_error() = buf;
  return 1;
}

inline int launched(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail("%s: launch failed: %s", what, hipGetErrorString(e));
  return 0;
}

}  // namespace gb

#define GB_REQUIRE(cond, ...) \
  do {                        \
    if (!(cond)) return gb::fail(__VA_ARGS__); \
  } while (0)

// A launch can be recorded as its entry point and its arguments and made again later, with other operands in
// the places of some pointers, without a walk through the bindings.  Recorded arguments lie in 64-bit slots:
// integers sign-extended, the bits of a float in the low half, pointers as they are.  GB_TAPED(entry) gives an
// entry point `<entry>_taped(slots)` that unpacks the slots by the entry point's own parameter types and calls it.
namespace gb {
template <class T> inline T from_slot(unsigned long long v) {
  if constexpr (std::is_pointer_v<T>) {
    return reinterpret_cast<T>(static_cast<uintptr_t>(v));
  } else if constexpr (std::is_floating_point_v<T>) {
    // a slot carries the 32 bits of a float: a parameter of more precision would be cut to float without a word
    static_assert(std::is_same_v<T, float>, "a taped entry point takes its floating-point parameters as float");
    const uint32_t bits = static_cast<uint32_t>(v);
    float f;
    std::memcpy(&f, &bits, sizeof f);
    return static_cast<T>(f);
  } else {
    return static_cast<T>(static_cast<long long>(v));
  }
}
template <class... A, std::size_t... I>
inline int call_slots(int (*f)(A...), const unsigned long long* slots, std::index_sequence<I...>) {
  return f(from_slot<A>(slots[I])...);
}
template <class... A> inline int call_slots(int (*f)(A...), const unsigned long long* slots) {
  return call_slots(f, slots, std::index_sequence_for<A...>{});
}
}  // namespace gb

#define GB_TAPED(entry) \
  extern "C" int entry##_taped(const unsigned long long* slots) { return gb::call_slots(&entry, slots); }

#define GB_DEFINE_LAST_ERROR \
  extern "C" const char* gb_last_error() { return gb::last_error().c_str(); }
