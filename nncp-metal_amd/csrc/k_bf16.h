// float -> bf16 rounding shared by every kernel that writes bf16 operand copies (the
// product loaders, the cast kernel, the producers' shadow stores, the optimiser): round to
// nearest even through the hardware conversion (v_cvt_pk_bf16_f32), so that a value rounded
// by its producer and the same value rounded by a later cast are the same 16 bits.
#ifndef NCHIP_K_BF16_H
#define NCHIP_K_BF16_H

#include <stdint.h>

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float floatx2_t __attribute__((ext_vector_type(2)));

__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi)
{
    floatx2_t f = { lo, hi };
    bf16x2_t h = __builtin_convertvector(f, bf16x2_t);
    return __builtin_bit_cast(uint32_t, h);
}

__device__ __forceinline__ uint16_t f32_to_bf16_rne(float f)
{
    return (uint16_t)(pack_bf16(f, 0.0f) & 0xffffu);
}

#endif
