// Shared device helpers for the gfx950 kernels of libfieldfare_moe_hip.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

namespace ffmoe {

constexpr int kGroup = 64;     // MLX-affine group size (Infrastructure/ModelIO/Quantization.swift:2)
constexpr int kWave = 64;      // CDNA wavefront
constexpr int kTileRows = 16;  // weight rows per arena tile = MFMA 16x16x32 column block
constexpr int kTileBytes = 1024;   // one arena tile: 64 lanes x 16 B (two 16-row x 64-k nibble blocks)
constexpr int kTileScaleBytes = 128;  // 16 rows x 4 bf16 (scale/bias of the two blocks)

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

__device__ __forceinline__ float bf16_to_f32(uint16_t b) { return __uint_as_float((uint32_t)b << 16); }
__device__ __forceinline__ float bf16lo_to_f32(uint32_t pair) { return __uint_as_float(pair << 16); }
__device__ __forceinline__ float bf16hi_to_f32(uint32_t pair) { return __uint_as_float(pair & 0xFFFF0000u); }

// Round-to-nearest-even fp32 -> bf16 on the gfx950 converter (v_cvt_pk_bf16_f32). For every non-NaN
// input the bits equal the integer recipe of Quantization.bf16Bits
// (Infrastructure/ModelIO/Quantization.swift:9-15): add 0x7FFF + lsb, keep the high half.
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint16_t f32_to_bf16(float x) { return __builtin_bit_cast(uint16_t, (__bf16)x); }
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
    bf16x2 v;
    v[0] = (__bf16)lo;
    v[1] = (__bf16)hi;
    return __builtin_bit_cast(uint32_t, v);
}

// gelu_pytorch_tanh, Metal/MoE/moe.metal:40-47 (clamp kept: it guards the exponential at large magnitudes),
// through 0.5 (1 + tanh z) = 1 / (1 + exp(-2 z)) on the hardware exp2 and reciprocal:
// about ten instructions instead of a tanhf call, relative error ~1e-6 (the result is rounded to bf16).
__device__ __forceinline__ float gelu_tanh_fast(float x) {
    const float x3 = x * x * x;
    float inner = 0.7978845608028654f * (x + 0.044715f * x3);
    inner = fminf(fmaxf(inner, -20.0f), 20.0f);
    return x * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-2.8853900817779268f * inner));
}

// Arena nibble order inside one dword: nibble position m (m = 0..3) holds element 2m of the lane's
// eight k-slots and position m + 4 holds element 2m + 1, so that ((w >> 4m) & 0x000F000F) is the
// 16-bit pair (element 2m, element 2m + 1) with no cross-lane or cross-register shuffling.
//
// dequant8_bf16: the eight nibbles as bf16(fma(q, scale, bias)) - the reference's 16-bit tile weight
// (Metal/Prefill/prefill.metal:581-590 with half replaced by bfloat as Metal/TensorCore/tensorops.metal:267).
// q * scale is exact in fp32 (4-bit x 8-bit significands), so fma and mul-then-add agree.
__device__ __forceinline__ uint4 dequant8_bf16(uint32_t w, float scale, float bias) {
    // even nibbles / odd nibbles as bytes; the empty asm keeps the two masks as written so that each
    // byte converts with one v_cvt_f32_ubyteN instead of a bit-field extract plus a convert
    uint32_t lo = w & 0x0F0F0F0Fu, hi = (w >> 4) & 0x0F0F0F0Fu;
    asm("" : "+v"(lo), "+v"(hi));
    uint4 r;
    r.x = pack_bf16x2(__builtin_fmaf((float)(lo & 0xFFu), scale, bias), __builtin_fmaf((float)((lo >> 16) & 0xFFu), scale, bias));
    r.y = pack_bf16x2(__builtin_fmaf((float)(hi & 0xFFu), scale, bias), __builtin_fmaf((float)((hi >> 16) & 0xFFu), scale, bias));
    r.z = pack_bf16x2(__builtin_fmaf((float)((lo >> 8) & 0xFFu), scale, bias), __builtin_fmaf((float)(lo >> 24), scale, bias));
    r.w = pack_bf16x2(__builtin_fmaf((float)((hi >> 8) & 0xFFu), scale, bias), __builtin_fmaf((float)(hi >> 24), scale, bias));
    return r;
}

__device__ __forceinline__ f32x4 mfma16(bf16x8 a, bf16x8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}

// The two 16-bit activation types a context can run in (FFMOE_BF16, FFMOE_FP16): conversions, the offset
// form of an INT4 weight for the streaming kernels and the matrix instruction that goes with it.
// FP16 is the reference's text-path type (Metal/MoE/moe.metal:69,389,555). Offset form: 1024 + q is exact in
// FP16 (ulp 1 at 1024) as 128 + q is in bf16, and 0x6400 | q needs no shift either.
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

template <bool F16> struct Act;
template <> struct Act<false> {
    static constexpr uint32_t kOffsetBits = 0x43004300u, kOnesBits = 0x3F803F80u;
    static constexpr float kOffset = 128.0f;
    static __device__ __forceinline__ float lo(uint32_t pair) { return bf16lo_to_f32(pair); }
    static __device__ __forceinline__ float hi(uint32_t pair) { return bf16hi_to_f32(pair); }
    static __device__ __forceinline__ float widen(uint16_t b) { return bf16_to_f32(b); }
    static __device__ __forceinline__ uint16_t round(float x) { return f32_to_bf16(x); }
    static __device__ __forceinline__ uint32_t pack(float a, float b) { return pack_bf16x2(a, b); }
    static __device__ __forceinline__ f32x4 mfma(const uint4 &a, const uint4 &b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
};
template <> struct Act<true> {
    static constexpr uint32_t kOffsetBits = 0x64006400u, kOnesBits = 0x3C003C00u;
    static constexpr float kOffset = 1024.0f;
    static __device__ __forceinline__ float lo(uint32_t pair) { return (float)__builtin_bit_cast(_Float16, (uint16_t)(pair & 0xFFFFu)); }
    static __device__ __forceinline__ float hi(uint32_t pair) { return (float)__builtin_bit_cast(_Float16, (uint16_t)(pair >> 16)); }
    static __device__ __forceinline__ float widen(uint16_t b) { return (float)__builtin_bit_cast(_Float16, b); }
    static __device__ __forceinline__ uint16_t round(float x) { return __builtin_bit_cast(uint16_t, (_Float16)x); }
    static __device__ __forceinline__ uint32_t pack(float a, float b) {
        f16x2 v;
        v[0] = (_Float16)a;
        v[1] = (_Float16)b;
        return __builtin_bit_cast(uint32_t, v);
    }
    static __device__ __forceinline__ f32x4 mfma(const uint4 &a, const uint4 &b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    }
};

// The eight nibbles of a dword as 16-bit values offset + q in the activation type (128 + q as bf16: 0x4300 | q
// is exact, the bf16 ulp at 128 is 1). The matrix unit then accumulates sum (offset + q) x; the caller removes
// offset * sum x. One v_and_or_b32 per pair: gfx9 VOP3 takes no literals and one scalar operand, so the mask has
// to sit in a scalar register and the constant in a vector register. The empty asm statements only hide the two
// values' constness, which makes the compiler itself select v_and_or_b32 (it otherwise emits and + or).
template <bool F16>
__device__ __forceinline__ uint4 unpack8_offset(uint32_t w) {
    uint32_t mask = 0x000F000Fu, c = Act<F16>::kOffsetBits;
    asm("" : "+s"(mask));
    asm("" : "+v"(c));
    uint4 r;
    r.x = (w & mask) | c;
    r.y = ((w >> 4) & mask) | c;
    r.z = ((w >> 8) & mask) | c;
    r.w = ((w >> 12) & mask) | c;
    return r;
}

// Workgroup barrier that waits for this wave's LDS traffic only. __syncthreads() also drains every
// outstanding global load, which would serialise a register prefetch that is meant to stay in flight
// across the barrier; here the compiler's own counters still guard each prefetched register at its use.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// xor-butterfly sum across the 64 lanes (masks 32,16,8,4,2,1): every lane ends with the same value, and
// every addition has the operands v[i] and v[i ^ mask] - the order the CPU oracle restates. The partners
// come through register-to-register lane moves (gfx950 row swaps for 32 and 16, DPP rotations and quad
// permutations below that) at a few cycles a step; __shfl_xor goes through the LDS crossbar at more than
// a hundred, six times in a row on the critical path of every row reduction.
__device__ __forceinline__ float wave_butterfly_sum(float v) {
    auto dpp = [](float x, auto ctrl, auto banks, float old) {
        return __uint_as_float((uint32_t)__builtin_amdgcn_update_dpp((int)__float_as_uint(old), (int)__float_as_uint(x),
                                                                      decltype(ctrl)::value, 0xF, decltype(banks)::value, false));
    };
    using std::integral_constant;
    // 32: the swap leaves (lower half, lower half) and (upper half, upper half) in the two registers
    auto h = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = __uint_as_float(h[0]) + __uint_as_float(h[1]);
    // 16: the same with the odd rows of one register and the even rows of the other
    auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = __uint_as_float(r[0]) + __uint_as_float(r[1]);
    // 8: rotation by half a row
    v = v + dpp(v, integral_constant<int, 0x128>{}, integral_constant<int, 0xF>{}, v);
    // 4: lanes 0-3 and 8-11 of a row take from four lanes up (rotate right by 12), the others from four down
    float p = dpp(v, integral_constant<int, 0x12C>{}, integral_constant<int, 0x5>{}, v);
    p = dpp(v, integral_constant<int, 0x124>{}, integral_constant<int, 0xA>{}, p);
    v = v + p;
    // 2 and 1: permutations inside each quad
    v = v + dpp(v, integral_constant<int, 0x4E>{}, integral_constant<int, 0xF>{}, v);
    v = v + dpp(v, integral_constant<int, 0xB1>{}, integral_constant<int, 0xF>{}, v);
    return v;
}

// The same sums (same operands in every addition) through the LDS crossbar: for kernels that reduce many
// independent values per wave and have the vector ALU busy with other work, where throughput counts and the
// latency of a step does not.
__device__ __forceinline__ float wave_butterfly_sum_shuffle(float v) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) v = v + __shfl_xor(v, m, 64);
    return v;
}

}  // namespace ffmoe
