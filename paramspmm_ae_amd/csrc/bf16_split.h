// An fp32 number as the exact sum of three bf16 numbers (8 + 8 + 8 significant bits), for the layer products that run
// on the bf16 matrix cores: x w = the sum of nine term products, of which the six with at least 16 significant bits
// between them carry the product to 2^-23 of |x||w|.
#pragma once

typedef __bf16 psp_bf16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 psp_bf16x8 __attribute__((ext_vector_type(8)));
typedef unsigned int psp_u32x4 __attribute__((ext_vector_type(4)));
typedef float psp_mfma_acc4 __attribute__((ext_vector_type(4)));

// two floats -> their three bf16 terms, packed in pairs (low half = first float); v_cvt_pk_bf16_f32 rounds to nearest even
__device__ __forceinline__ void psp_split3(float a, float b, unsigned &hi, unsigned &mid, unsigned &lo)
{
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    f32x2 v = {a, b};
    hi = __builtin_bit_cast(unsigned, __builtin_convertvector(v, psp_bf16x2));
    v[0] = a - __uint_as_float(hi << 16);
    v[1] = b - __uint_as_float(hi & 0xffff0000u);
    mid = __builtin_bit_cast(unsigned, __builtin_convertvector(v, psp_bf16x2));
    v[0] -= __uint_as_float(mid << 16);
    v[1] -= __uint_as_float(mid & 0xffff0000u);
    lo = __builtin_bit_cast(unsigned, __builtin_convertvector(v, psp_bf16x2));
}
