// Device-side element conversions shared by the kernels.
#ifndef poplibs_amd_device_types_hpp
#define poplibs_amd_device_types_hpp
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mxk {

/// OCP 8-bit float -> fp32 in software.  E4M3FN: bias 7, S.1111.111 is NaN, no
/// infinities.  E5M2: bias 15, IEEE-like infinities / NaNs.  Every finite code
/// is exactly representable in fp32 (and in fp16).
__device__ __forceinline__ float decodeFp8(uint32_t code, int format) {
  const uint32_t sign = (code & 0x80u) << 24;
  uint32_t bits;
  if (format == 1) { // E4M3FN
    const uint32_t e = (code >> 3) & 0xfu, m = code & 7u;
    if (e == 0xfu && m == 7u)
      bits = 0x7fc00000u;
    else if (e == 0u)
      return __uint_as_float(sign | __float_as_uint(float(m) * 0x1p-9f));
    else
      bits = ((e + 120u) << 23) | (m << 20); // 127 - 7 = 120
  } else { // E5M2
    const uint32_t e = (code >> 2) & 0x1fu, m = code & 3u;
    if (e == 0x1fu)
      bits = m ? 0x7fc00000u : 0x7f800000u;
    else if (e == 0u)
      return __uint_as_float(sign | __float_as_uint(float(m) * 0x1p-16f));
    else
      bits = ((e + 112u) << 23) | (m << 21); // 127 - 15 = 112
  }
  return __uint_as_float(sign | bits);
}

template <class T> struct Load;
template <> struct Load<float> {
  static __device__ __forceinline__ float at(const float *p, size_t i, int) {
    return p[i];
  }
};
template <> struct Load<__half> {
  static __device__ __forceinline__ float at(const __half *p, size_t i, int) {
    return __half2float(p[i]);
  }
};
template <> struct Load<uint8_t> {
  static __device__ __forceinline__ float at(const uint8_t *p, size_t i,
                                             int format) {
    return decodeFp8(p[i], format);
  }
};

/// Two fp32 sums rounded to half, to nearest even, as fp32 values: the empty
/// asm keeps the compiler from folding the multiply-add that produced a sum
/// into the conversion (v_fma_mixlo_f16 rounds once, from the exact result),
/// which it does for some of a kernel's sums and not for others.  Every
/// vector-ALU kernel rounds through here, so that a layer's output does not
/// depend on which of them ran it - and is the fp32 partial cast to half that
/// the reference's partialsType float produces.
__device__ __forceinline__ __half2 roundPairToHalf(float a, float b) {
  asm("" : "+v"(a), "+v"(b));
  return __floats2half2_rn(a, b);
}

/// fp32 -> output element, round to nearest even.
__device__ __forceinline__ void storeOut(float *p, size_t i, float v) {
  p[i] = v;
}
__device__ __forceinline__ void storeOut(__half *p, size_t i, float v) {
  asm("" : "+v"(v)); // (as in roundPairToHalf)
  p[i] = __float2half_rn(v);
}

/// Division of a 31-bit number by a launch constant: one multiply-high and a
/// shift (round-up method: mul = ceil(2^(31 + s) / d), s = ceil(log2 d)).
struct FastDiv {
  uint32_t mul, shift, one; // one: all bits set when the divisor is 1
  __device__ __forceinline__ uint32_t operator()(uint32_t n) const {
    // a select written with bit operations: no branch, whatever the compiler
    // knows about `one`
    const uint32_t q = __umulhi(n, mul) >> shift;
    return q ^ ((q ^ n) & one);
  }
};

inline FastDiv makeFastDiv(uint32_t d) {
  if (d <= 1)
    return {0, 0, 0xffffffffu};
  uint32_t s = 0;
  while ((1ull << s) < d)
    ++s;
  const uint64_t m = ((1ull << (31 + s)) + d - 1) / d;
  return {uint32_t(m), s - 1, 0};
}

/// Four consecutive outputs as one vector store; p is aligned to the vector.
__device__ __forceinline__ void storeOut4(float *p, const float (&v)[4]) {
  *reinterpret_cast<float4 *>(p) = float4{v[0], v[1], v[2], v[3]};
}
__device__ __forceinline__ void storeOut4(__half *p, const float (&v)[4]) {
  union {
    __half2 h[2];
    uint2 u;
  } pack;
  pack.h[0] = roundPairToHalf(v[0], v[1]);
  pack.h[1] = roundPairToHalf(v[2], v[3]);
  *reinterpret_cast<uint2 *>(p) = pack.u;
}

} // namespace mxk
#endif
