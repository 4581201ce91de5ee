// Device-side helpers shared by the gfx950 MoE kernels: bf16 packing, e2m1 / e4m3
// decode, wavefront reductions.  gfx950 only; wavefront size 64.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace moe {

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t h) { return __uint_as_float(h << 16); }
__device__ __forceinline__ float bf16_lo(uint32_t pair) { return __uint_as_float(pair << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t pair) { return __uint_as_float(pair & 0xffff0000u); }

// Two fp32 -> packed bf16 pair, round to nearest even (one v_cvt_pk_bf16_f32).
__device__ __forceinline__ uint32_t pack_bf16_rne(float lo, float hi) {
    bf16x2_t r;
    r[0] = (__bf16)lo;
    r[1] = (__bf16)hi;
    return __builtin_bit_cast(uint32_t, r);
}

// Exact e2m1 decode of the two nibbles of byte `SEL` of `word` to fp32 (low nibble
// first).  The hardware convert is used with scale 1.0: it honours only the
// exponent of its scale operand, so the block scale is applied afterwards with
// an ordinary fp32 multiply.  Code 8 yields -0.0.
template <int SEL>
__device__ __forceinline__ f32x2_t e2m1_pair_to_f32(uint32_t word) {
    return __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(word, 1.0f, SEL);
}

// RNE_bf16(e2m1(code) * scale) for the two nibbles of byte SEL, packed.
template <int SEL>
__device__ __forceinline__ uint32_t e2m1_pair_scaled_bf16(uint32_t word, float scale) {
    f32x2_t v = e2m1_pair_to_f32<SEL>(word);
    return pack_bf16_rne(v[0] * scale, v[1] * scale);
}

// Two e4m3 codes decoded the way the reference does it (no NaN: 0x7F / 0xFF give +-480), returned
// as value / 256.  `pair` holds the codes in bytes 0 and 2, bytes 1 and 3 zero.  code << 7 with
// the sign moved from bit 14 to bit 15 is an fp16 worth 2^-8 of the e4m3 value, subnormals
// included (preCastFP8Weight, grouped_gemm/op_kernel/antiquant_impl.h:87-129, does the same);
// fp16 -> fp32 is exact, so callers fold the 2^8 into their scale and round once.
__device__ __forceinline__ uint32_t e4m3_ref_pair_over_256_fp16(uint32_t pair) {
    uint32_t h = pair << 7;
    h += h & 0x40004000u;
    return h;   // two fp16
}
__device__ __forceinline__ f32x2_t e4m3_ref_pair_over_256(uint32_t pair) {
    typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
    const half2_t v = __builtin_bit_cast(half2_t, e4m3_ref_pair_over_256_fp16(pair));
    return f32x2_t{(float)v[0], (float)v[1]};
}

// fp32(low / high fp16 of h2) * s in one instruction (v_fma_mix_f32 converts the fp16 operand on the way
// in; the product is rounded to fp32 once, exactly as a conversion followed by a multiply).  The addend
// is -0.0 so that the sign of a zero product survives.
__device__ __forceinline__ float fp16_lo_times(uint32_t h2, float s, float neg_zero) {
    float r;
    asm("v_fma_mix_f32 %0, %1, %2, %3 op_sel_hi:[1,0,0]" : "=v"(r) : "v"(h2), "v"(s), "v"(neg_zero));
    return r;
}
__device__ __forceinline__ float fp16_hi_times(uint32_t h2, float s, float neg_zero) {
    float r;
    asm("v_fma_mix_f32 %0, %1, %2, %3 op_sel:[1,0,0] op_sel_hi:[1,0,0]" : "=v"(r) : "v"(h2), "v"(s), "v"(neg_zero));
    return r;
}

__device__ __forceinline__ float wave_reduce_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

}  // namespace moe
