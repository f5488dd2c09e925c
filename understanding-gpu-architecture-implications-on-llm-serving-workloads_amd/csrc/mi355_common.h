// Shared device-side helpers for the gfx950 (MI355X, CDNA4) serving kernels.
//
// Everything here is written for wave64 and for the gfx950 instruction set only:
//   * v_mfma_f32_32x32x16_f16 / v_mfma_f32_16x16x32_f16 (fp16 in, fp32 accumulate)
//   * global_load_lds_dwordx4 / buffer_load_dwordx4 ... lds (16-byte global -> LDS copies that bypass the VGPRs)
//   * ds_read_b64_tr_b16 (LDS read that transposes a 4x16 block of 16-bit values)
//
// Register layouts (checked on hardware):
//   mfma 32x32x16: operand lane l holds 8 consecutive k (k = 8*(l/32) .. +7) of row/col l%32;
//                  accumulator element 4p+q of lane l is D[8p + 4*(l/32) + q][l%32].
//   mfma 16x16x32: operand lane l holds k = 8*(l/16) .. +7 of row/col l%16;
//                  accumulator element q of lane l is D[4*(l/16) + q][l%16].
//   ds_read_b64_tr_b16: inside each group of 16 lanes, input lane j supplies the four 16-bit values
//                  X[j/4][4*(j%4) .. +3] of a 4x16 block X; output lane i receives X[0..3][i].
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mi355 {

typedef _Float16 half_t;
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float float16v __attribute__((ext_vector_type(16)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef short short4v __attribute__((ext_vector_type(4)));
typedef int int4v __attribute__((ext_vector_type(4)));
typedef int int2v __attribute__((ext_vector_type(2)));

#define MI355_LDS __attribute__((address_space(3)))
#define MI355_GLOBAL __attribute__((address_space(1)))

// s_waitcnt immediates (gfx9 encoding): vmcnt = bits [3:0] and [15:14], expcnt [6:4], lgkmcnt [11:8].
__device__ __forceinline__ constexpr int waitcnt_imm(int vm, int lgkm) {
    return (vm & 0xF) | ((vm >> 4) << 14) | (0x7 << 4) | ((lgkm & 0xF) << 8);
}
template <int VM>
__device__ __forceinline__ void wait_vmcnt() {
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(VM, 0xF));
}
template <int LGKM>
__device__ __forceinline__ void wait_lgkmcnt() {
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(0x3F, LGKM));
}

// 16-byte global -> LDS copy (global_load_lds_dwordx4). Lane l of the wave writes LDS bytes
// [lds_wave_base + 16*l, +16); lds_wave_base must be wave-uniform (it travels in M0).
// Written as inline assembly on purpose: the compiler then does not treat the copy as an LDS store, so it
// does not put a full "s_waitcnt vmcnt(0)" in front of every later LDS read. The caller orders the copy
// against LDS reads itself: wait_vmcnt<N>() followed by a workgroup barrier before the data is read.
__device__ __forceinline__ void copy16_global_to_lds(const void* gptr, MI355_LDS void* lds_wave_base) {
    asm volatile(
        "s_mov_b32 m0, %1\n\t"
        "s_nop 0\n\t"
        "global_load_lds_dwordx4 %0, off"
        :
        : "v"(gptr), "s"((uint32_t)(uintptr_t)lds_wave_base)
        : "memory", "m0");
}

// The same copy with the address split into a wave-uniform 64-bit base (kept in scalar registers) and a 32-bit
// per-lane byte offset: per-tile address arithmetic then runs on the scalar unit and a lane needs one VALU add or none.
__device__ __forceinline__ void copy16_global_to_lds(const void* uniform_base, uint32_t lane_byte_offset,
                                                     MI355_LDS void* lds_wave_base) {
    asm volatile(
        "s_mov_b32 m0, %2\n\t"
        "s_nop 0\n\t"
        "global_load_lds_dwordx4 %0, %1"
        :
        : "v"(lane_byte_offset), "s"(uniform_base), "s"((uint32_t)(uintptr_t)lds_wave_base)
        : "memory", "m0");
}

// The same with the LDS destination as a scalar register plus a compile-time constant (one scalar instruction into M0).
// The instruction's own offset field is not used: the hardware adds it to the LDS address as well as to the global one.
template <int LDS_IMM>
__device__ __forceinline__ void copy16_global_to_lds_imm(const void* uniform_base, uint32_t lane_byte_offset, uint32_t lds_wave_base) {
    asm volatile(
        "s_add_u32 m0, %2, %3\n\t"
        "s_nop 0\n\t"
        "global_load_lds_dwordx4 %0, %1"
        :
        : "v"(lane_byte_offset), "s"(uniform_base), "s"(lds_wave_base), "n"(LDS_IMM)
        : "memory", "m0", "scc");
}

// Buffer resource (V#) over a whole address range: 48-bit base, no stride, no swizzle, the largest record count, raw
// 32-bit data format. The four words must sit in scalar registers, so every word is made wave-uniform explicitly.
__device__ __forceinline__ int4v make_buffer_resource(const void* base) {
    const uint64_t b = (uint64_t)(uintptr_t)base;
    int4v r;
    r[0] = __builtin_amdgcn_readfirstlane((int)(uint32_t)b);
    r[1] = __builtin_amdgcn_readfirstlane((int)(uint32_t)(b >> 32) & 0xffff);
    r[2] = __builtin_amdgcn_readfirstlane((int)0xffffffffu);
    r[3] = __builtin_amdgcn_readfirstlane(0x00020000);
    return r;
}

// The same 16-byte global -> LDS copy through a buffer resource: lane address = resource base + lane_byte_offset (one
// 32-bit VGPR) + uniform_byte_offset (a scalar register). A wave instruction that reads one address VGPR instead of a
// 64-bit pair takes about half as much issue time away from the MFMAs it runs beside, and all per-tile address
// arithmetic (advancing the base) runs on the scalar unit. The LDS destination is a scalar register plus a compile-time
// offset: one scalar instruction sets M0 (a destination that is a run-time value needs a second one to form it).
template <int IMM>
__device__ __forceinline__ void copy16_buffer_to_lds_at(int4v resource, uint32_t lane_byte_offset, uint32_t uniform_byte_offset,
                                                        uint32_t lds_wave_base) {
    asm volatile(
        "s_add_u32 m0, %3, %4\n\t"
        "s_nop 0\n\t"
        "buffer_load_dwordx4 %0, %1, %2 offen lds"
        :
        : "v"(lane_byte_offset), "s"(resource), "s"(uniform_byte_offset), "s"(lds_wave_base), "n"(IMM)
        : "memory", "m0", "scc");
}

// The two halves of the copy above for code that can place an unrelated instruction between them (M0 needs one wait
// state between the scalar write and the load that uses it; any instruction serves). Nothing else may write M0 in between:
// the compiler uses M0 only for instructions this library does not contain (LDS-direct and GWS operations, s_movrel).
template <int IMM>
__device__ __forceinline__ void set_m0_at(uint32_t lds_wave_base) {
    asm volatile("s_add_u32 m0, %0, %1" : : "s"(lds_wave_base), "n"(IMM) : "m0", "scc");
}
__device__ __forceinline__ void copy16_buffer_to_lds_m0(int4v resource, uint32_t lane_byte_offset, uint32_t uniform_byte_offset) {
    asm volatile("buffer_load_dwordx4 %0, %1, %2 offen lds" : : "v"(lane_byte_offset), "s"(resource), "s"(uniform_byte_offset) : "memory");
}

__device__ __forceinline__ half4 lds_read_tr16_b64(MI355_LDS const void* p) {
    short4v t = __builtin_amdgcn_ds_read_tr16_b64_v4i16((MI355_LDS short4v*)p);
    return __builtin_bit_cast(half4, t);
}

__device__ __forceinline__ half8 lds_read_b128(MI355_LDS const void* p) {
    return *(MI355_LDS const half8*)p;
}

__device__ __forceinline__ half8 concat(half4 lo, half4 hi) {
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
}

// Element types of the kernels. LDS traffic is type-blind (16-bit lanes); only the MFMA opcode and the
// float conversions differ. The register layouts of the bf16 MFMAs are those of their fp16 twins.
typedef __bf16 bf16_t;
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

template <typename T>
struct Elem;
template <>
struct Elem<half_t> {
    using v8 = half8;
    using v4 = half4;
    using v2 = half2v;
    static __device__ __forceinline__ v8 frag(half8 raw) { return raw; }
    static __device__ __forceinline__ float16v mfma32(v8 a, v8 b, float16v c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ float4v mfma16(v8 a, v8 b, float4v c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
    }
};
template <>
struct Elem<bf16_t> {
    using v8 = bf16x8;
    using v4 = bf16x4;
    using v2 = bf16x2;
    static __device__ __forceinline__ v8 frag(half8 raw) { return __builtin_bit_cast(bf16x8, raw); }
    static __device__ __forceinline__ float16v mfma32(v8 a, v8 b, float16v c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ float4v mfma16(v8 a, v8 b, float4v c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
    }
};

}  // namespace mi355
