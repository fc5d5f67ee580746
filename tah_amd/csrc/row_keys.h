// bf16 logits as order-preserving 16-bit keys: shared by the kernels that search a vocabulary row by value.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>

namespace tah {

typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4;
typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
typedef short i16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2e __attribute__((ext_vector_type(2)));

// bf16 bits -> unsigned key with the same order as the values (negative values reversed below the positive ones)
__device__ __forceinline__ uint32_t order_key(uint32_t bits) { return (bits & 0x8000u) ? (~bits & 0xffffu) : (bits | 0x8000u); }
// the same for the two bf16 halves of a dword at once: bits ^ 0xffff where negative, bits ^ 0x8000 where not
__device__ __forceinline__ uint32_t order_keys2(uint32_t w) {
    const i16x2 fifteen = {15, 15};
    const i16x2 neg = __builtin_bit_cast(i16x2, w) >> fifteen;  // 0xffff per negative half
    return w ^ (__builtin_bit_cast(uint32_t, neg) | 0x80008000u);
}
__device__ __forceinline__ float key_value(uint32_t key) {
    const uint32_t bits = (key & 0x8000u) ? (key & 0x7fffu) : (~key & 0xffffu);
    return __uint_as_float(bits << 16);
}

// x rounded to bfloat16 (nearest even), as a float.  Through the packed conversion on purpose: a scalar
// cast to __bf16 and back may be evaluated in excess precision, i.e. not round at all.
__device__ __forceinline__ float round_bf16(float x) {
    const f32x2 v = {x, 0.f};
    return __uint_as_float(__builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2e)) << 16);
}

}  // namespace tah
