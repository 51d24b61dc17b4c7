// Shared device helpers for the gfx950 MoBA kernels.
#pragma once
#include <cstdlib>
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace moba {

typedef __bf16 bf16;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef _Float16 f16;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(4))) _Float16 f16x4;
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

// Element types of q, k, v: every kernel is a template over one of these and names the
// types elem, elem2, elem4, elem8 inside its body (MOBA_ELEM_TYPES).
struct Bf16 {
  typedef bf16 elem;
  typedef bf16x2 elem2;
  typedef bf16x4 elem4;
  typedef bf16x8 elem8;
};
struct F16 {
  typedef f16 elem;
  typedef f16x2 elem2;
  typedef f16x4 elem4;
  typedef f16x8 elem8;
};
#define MOBA_ELEM_TYPES(E)                              \
  using elem [[maybe_unused]] = typename E::elem;       \
  using elem2 [[maybe_unused]] = typename E::elem2;     \
  using elem4 [[maybe_unused]] = typename E::elem4;     \
  using elem8 [[maybe_unused]] = typename E::elem8;
enum : int { MOBA_DTYPE_BF16 = 0, MOBA_DTYPE_F16 = 1 };

constexpr int kHeadDim = 128;  // the MFMA kernels are specialised for D = 128

// error codes returned by every extern "C" entry point
enum : int {
  MOBA_OK = 0,
  MOBA_ERR_ARG = -1,        // bad argument (null pointer, unsupported size, misalignment)
  MOBA_ERR_UNSUPPORTED = -2,
  MOBA_ERR_LAUNCH = -3,     // hipGetLastError() after a launch
  MOBA_ERR_LIMIT = -4,      // size beyond a stated limit
};

// S^T = K Q^T style product of one 32x32 tile, contraction depth 16:
// lane l supplies A[l%32][8*(l/32)..+7] and B[8*(l/32)..+7][l%32]; the result
// element e of lane l is C[8*(e/4) + 4*(l/32) + e%4][l%32].
__device__ __forceinline__ f32x16 mfma32(bf16x8 a, bf16x8 b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ f32x16 mfma32(f16x8 a, f16x8 b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
}

// The same product with the result in ordinary vector registers and the operands in accumulation
// registers, for a kernel that needs the accumulation registers at all: there the compiler gives every
// builtin MFMA the accumulation-register form, and a result that vector instructions consume is then
// copied out one register at a time.  `first` (a constant once loops are unrolled) starts from zero
// instead of from d.
// The compiler does not see a matrix instruction here and inserts no wait states after it: the caller
// keeps every other access to d at least two later matrix instructions away (they queue behind this
// one), chained accumulations into the same d excepted, which the hardware orders itself.
__device__ __forceinline__ void mfma32_into_vgprs(f32x16& d, bf16x8 a, bf16x8 b, bool first) {
  if (first) asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=v"(d) : "a"(a), "a"(b));
  else                 asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(d) : "a"(a), "a"(b));
}
__device__ __forceinline__ void mfma32_into_vgprs(f32x16& d, f16x8 a, f16x8 b, bool first) {
  if (first) asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, 0" : "=v"(d) : "a"(a), "a"(b));
  else                 asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(d) : "a"(a), "a"(b));
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }

// two floats rounded (to nearest even) to the element type, packed into 32 bits
template <class E>
__device__ __forceinline__ uint32_t pack2(float lo, float hi) {
  typename E::elem2 p;
  p[0] = (typename E::elem)lo;
  p[1] = (typename E::elem)hi;
  return __builtin_bit_cast(uint32_t, p);
}

// A fresh copy of a piece of the running kernel's argument block, read where this is called.  A kernel
// that needs some arguments only now and then (table pointers at a tile switch) reads them again there
// instead of holding them in scalar registers all through its inner loop.  `offset` is the byte offset
// of the piece inside the kernel's (single, by-value) parameter.
template <class T>
__device__ __forceinline__ T kernarg_now(int offset) {
  typedef __attribute__((address_space(4))) const char* kernarg_ptr;
  kernarg_ptr kp = (kernarg_ptr)__builtin_amdgcn_kernarg_segment_ptr();
  asm volatile("" : "+s"(kp));  // not the pointer the compiler knows: the loads stay where they are written
  // read through a pointer of the piece's own type: with the alignment known the loads are scalar loads
  // (a byte-wise copy makes them vector loads, which queue behind every vector load and copy in flight)
#if defined(__HIP_DEVICE_COMPILE__)
  return *reinterpret_cast<__attribute__((address_space(4))) const T*>(kp + offset);
#else
  return T();  // (the host pass only parses device code)
#endif
}

// Load from a table that no kernel writes while this one runs, at an address that is the same in every lane:
// read through the constant address space, so that the compiler may use a scalar load (its own counter, not
// queued behind the vector loads and copies in flight).
template <class T>
__device__ __forceinline__ T table_load(const T* p) {
  const uint64_t a = (uint64_t)(uintptr_t)p;  // made uniform explicitly: a scalar load whatever the compiler can prove
  // (the builtin returns a signed int: through uint32_t, or the low half would be sign-extended over the high one)
  const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)a);
  const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(a >> 32));
  const uint64_t ua = ((uint64_t)hi << 32) | lo;
#if defined(__HIP_DEVICE_COMPILE__)
  return *reinterpret_cast<__attribute__((address_space(4))) const T*>(ua);
#else
  return T();  // (the host pass only parses device code)
#endif
}

// Result of the launches of one entry point: an error that was already pending on the calling thread when the
// entry point began is neither reported nor cleared; an error the entry point's own launches raised is reported
// and cleared.
struct LaunchCheck {
  hipError_t before = hipPeekAtLastError();
  int result() const {
    const hipError_t after = hipPeekAtLastError();
    if (after == hipSuccess || after == before) return MOBA_OK;
    (void)hipGetLastError();
    return MOBA_ERR_LAUNCH;
  }
};

// Dynamic LDS above 64 KiB must be allowed per kernel, and the allowance belongs to the current
// device: `done` (one array per kernel) remembers the devices it was given on.
constexpr int kMaxDevices = 64;
inline bool allow_dynamic_lds(const void* kernel, int bytes, bool (&done)[kMaxDevices]) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0) return false;
  if (dev < kMaxDevices && done[dev]) return true;
  if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes) != hipSuccess) return false;
  if (dev < kMaxDevices) done[dev] = true;
  return true;
}

// compute units of the current device (0 on error), asked once per device
inline int compute_units() {
  static int count[kMaxDevices];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0) return 0;
  if (dev < kMaxDevices && count[dev] > 0) return count[dev];
  int n = 0;
  if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) return 0;
  if (dev < kMaxDevices) count[dev] = n;
  return n;
}

// Diagnostic: the environment variable MOBA_RESIDENT_CUS (read once) makes the kernels whose workgroups stay
// resident and draw tiles from queues occupy only that many compute units' worth of workgroups.  With part of
// the chip idle the rest runs at a higher clock: this is how the power-limited clock under full load is told
// apart from the kernels' own efficiency.  Results do not depend on it.
inline int resident_compute_units() {
  static int limit = -1;
  if (limit < 0) {
    const char* e = getenv("MOBA_RESIDENT_CUS");
    limit = e ? atoi(e) : 0;
    if (limit < 0) limit = 0;
  }
  const int cus = compute_units();
  return (limit > 0 && limit < cus) ? limit : cus;
}

// largest i in [0, n) with a[i] <= x, for ascending a with a[0] <= x
__device__ __forceinline__ int upper_row(const int* __restrict__ a, int n, int x) {
  int lo = 0, hi = n;  // invariant: a[lo] <= x, a[hi] > x (hi == n means +inf)
  while (hi - lo > 1) {
    int mid = (lo + hi) >> 1;
    if (a[mid] <= x) lo = mid; else hi = mid;
  }
  return lo;
}

}  // namespace moba
