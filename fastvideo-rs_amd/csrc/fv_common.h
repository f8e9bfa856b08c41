// Shared device helpers for the gfx950 (CDNA4, wave64) SDPA kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace fv {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(8))) short s16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(8))) float f32x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;
typedef __attribute__((ext_vector_type(2))) unsigned int u32x2;

typedef __attribute__((address_space(3))) unsigned char lds_u8;

#define FV_DEV __device__ __forceinline__

FV_DEV float neg_inf() { return __builtin_bit_cast(float, 0xff800000u); }

// 16-byte LDS read / write.
FV_DEV bf16x8 lds_read_b128(const lds_u8* p) {
    return *reinterpret_cast<const __attribute__((address_space(3))) bf16x8*>(p);
}
FV_DEV void lds_write_b128(lds_u8* p, u32x4 v) {
    *reinterpret_cast<__attribute__((address_space(3))) u32x4*>(p) = v;
}

// ds_read_b64_tr_b16: within each block of 16 lanes the 16 x (4 x b16) values
// are read as a 4-row x 16-column matrix (row r supplied by lanes 4r..4r+3,
// 4 consecutive columns each) and lane i receives column i, rows 0..3. It
// turns a row-major [key][d] tile into the k-contiguous MFMA operand without
// a register transpose.
FV_DEV s16x4 lds_read_tr16_b64(const lds_u8* p) {
    return __builtin_amdgcn_ds_read_tr16_b64_v4i16(
        (__attribute__((address_space(3))) s16x4*)(p));
}

// v_mfma_f32_32x32x16_bf16: A 32x16 (lane l: row l%32, k 8*(l/32)..+7),
// B 16x32 (lane l: column l%32, k 8*(l/32)..+7), C 32x32 (lane l, reg i:
// column l%32, row 8*(i/4) + 4*(l/32) + i%4).
FV_DEV f32x16 mfma32(bf16x8 a, bf16x8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}

// max / sum over the pair of lanes {l, l ^ 32}, result in both.
FV_DEV float pair_max(float x) {
    const unsigned u = __builtin_bit_cast(unsigned, x);
    auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return __builtin_fmaxf(__builtin_bit_cast(float, (unsigned)r[0]),
                           __builtin_bit_cast(float, (unsigned)r[1]));
}
FV_DEV float pair_sum(float x) {
    const unsigned u = __builtin_bit_cast(unsigned, x);
    auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return __builtin_bit_cast(float, (unsigned)r[0]) + __builtin_bit_cast(float, (unsigned)r[1]);
}

// A store through a pointer whose address space the compiler no longer knows (a kernel argument that went
// through an `asm` pin, an address built from one) is emitted as a FLAT store, which also takes an LDS issue
// slot and counts against the LDS counter. This names the address space.
template <class T>
FV_DEV void global_store(void* p, T v) {
    *(__attribute__((address_space(1))) T*)p = v;
}

FV_DEV float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// f32 -> bf16 bits, round to nearest even, NaN quiet, overflow to inf: the
// rounding of the reference's fv_bf16_rne (kernels/core.cu:6-15).
FV_DEV unsigned short bf16_rne_bits(float x) {
    unsigned int u = __builtin_bit_cast(unsigned int, x);
    if ((u & 0x7F800000u) == 0x7F800000u) {
        unsigned int h = u >> 16;
        if (u & 0x007FFFFFu) h |= 0x0040u;
        return (unsigned short)h;
    }
    u += 0x7FFFu + ((u >> 16) & 1u);
    return (unsigned short)(u >> 16);
}
FV_DEV float bf16_bits_to_f32(unsigned short b) {
    return __builtin_bit_cast(float, ((unsigned int)b) << 16);
}

}  // namespace fv
