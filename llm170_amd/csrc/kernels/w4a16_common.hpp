// Device helpers shared by the gfx950 W4A16 kernels.
//
// Tiled weight layout ("T16x128"), produced at upload from the operand format q u32 [n][k/8]:
//   a tile covers 16 output rows x 128 k and is 1 KiB, stored as 64 lanes x 16 B; tiles are ordered
//   [row_block = n/16][k_tile = k/128], so one row block's k range is one contiguous run.
//   lane l = g*16 + r (r = row in block, g = 0..3) owns dwords w = 0..3; dword w holds the eight weights
//   k = k_tile*128 + w*32 + g*8 + j, j = 0..7.  With this choice dword w of all 64 lanes is exactly the A operand
//   (16 rows x 32 k) of one v_mfma_f32_16x16x32_f16, and for group size 32 that MFMA stays inside one scale group.
//   Inside a dword the nibbles are interleaved: nibble position p holds j = PERM[p], PERM = {0,2,4,6,1,3,5,7}, so
//   that (dword & 0x000F000F) picks the pair (j=0, j=1) into the two f16 halves of one register, etc.
// Tiled scale layout: u16 [row_block][k/group][16 rows] (the 4 rows an MFMA result lane owns are 8 contiguous bytes).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef _Float16 h2_t __attribute__((ext_vector_type(2)));
typedef _Float16 h4_t __attribute__((ext_vector_type(4)));
typedef _Float16 h8_t __attribute__((ext_vector_type(8)));
typedef float f4_t __attribute__((ext_vector_type(4)));
typedef float f16_t __attribute__((ext_vector_type(16)));
typedef unsigned u2_t __attribute__((ext_vector_type(2)));
typedef unsigned u4_t __attribute__((ext_vector_type(4)));

#define W4_TILE_ROWS 16
#define W4_TILE_K 128

// nibble position p (bits 4p..4p+3) of a tiled dword holds element PERM[p]; element j sits at position POS[j]
__device__ __forceinline__ int w4_perm(int p) { return ((p & 3) << 1) | (p >> 2); }
__device__ __forceinline__ int w4_pos(int j) { return ((j & 1) << 2) | (j >> 1); }

// (w & mask) | bits in one VALU op.  The mask travels in an SGPR and the or-constant in a VGPR (one scalar operand
// per VOP3 instruction on this target); the compiler would otherwise emit v_and + v_or with literals.
__device__ __forceinline__ unsigned w4_and_or(unsigned w, unsigned mask, unsigned bits) {
    unsigned r;
    asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(w), "s"(mask), "v"(bits));
    return r;
}

// Eight weights of one tiled dword as exact f16 integers (nibble - 8), in element order j = 0..7.
// 0x6400 is f16 1024.0 (mantissa unit 1): or-ing a nibble into bits 0..3 gives 1024 + nibble exactly.
// 0x5400 is f16 64.0 (mantissa unit 1/16): or-ing a nibble into bits 4..7 gives 64 + nibble exactly.
// 9 VALU ops per dword: one shift, four and-or, four packed f16 adds.
__device__ __forceinline__ h8_t w4_deq8(unsigned w) {
    const h2_t off_lo = {(_Float16)-1032.0f, (_Float16)-1032.0f};
    const h2_t off_hi = {(_Float16)-72.0f, (_Float16)-72.0f};
    unsigned w1 = w >> 8;
    unsigned a0 = w4_and_or(w, 0x000F000Fu, 0x64006400u);
    unsigned a1 = w4_and_or(w, 0x00F000F0u, 0x54005400u);
    unsigned a2 = w4_and_or(w1, 0x000F000Fu, 0x64006400u);
    unsigned a3 = w4_and_or(w1, 0x00F000F0u, 0x54005400u);
    h2_t p0 = __builtin_bit_cast(h2_t, a0) + off_lo;
    h2_t p1 = __builtin_bit_cast(h2_t, a1) + off_hi;
    h2_t p2 = __builtin_bit_cast(h2_t, a2) + off_lo;
    h2_t p3 = __builtin_bit_cast(h2_t, a3) + off_hi;
    h8_t r;
    r[0] = p0[0]; r[1] = p0[1]; r[2] = p1[0]; r[3] = p1[1];
    r[4] = p2[0]; r[5] = p2[1]; r[6] = p3[0]; r[7] = p3[1];
    return r;
}

// Raw buffer descriptor over [base, base + bytes): loads whose byte offset falls outside return 0 and touch no
// memory, which gives branch-free predication of per-lane loads.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t w4_make_rsrc(const void* base, unsigned bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);
}
#define W4_OOB 0x80000000u  // a byte offset no buffer here reaches

// IEEE binary16 bits -> f32 by integer manipulation (subnormals normalised, Inf/NaN payload shifted), the routine
// the reference uses on both host and device (crates/core/src/quant/deq.rs:4-27).
__device__ __forceinline__ float w4_half_bits_to_f32(unsigned h) {
    unsigned sign = (h >> 15) & 1u, exp = (h >> 10) & 0x1fu, frac = h & 0x3ffu, bits;
    if (exp == 0) {
        if (frac == 0) {
            bits = sign << 31;
        } else {
            int sh = __builtin_clz(frac) - 21;  // shifts needed to bring the leading one to bit 10
            unsigned f = (frac << sh) & 0x3ffu;
            bits = (sign << 31) | ((unsigned)(127 - 15 + 1 - sh) << 23) | (f << 13);
        }
    } else if (exp == 0x1f) {
        bits = (sign << 31) | (0xffu << 23) | (frac << 13);
    } else {
        bits = (sign << 31) | ((exp + 112u) << 23) | (frac << 13);
    }
    return __builtin_bit_cast(float, bits);
}

template <bool SBF>
__device__ __forceinline__ float w4_scale_to_f32(unsigned bits16) {
    if (SBF) return __builtin_bit_cast(float, bits16 << 16);  // crates/core/src/quant/deq.rs:29-31
    return w4_half_bits_to_f32(bits16);
}

// Fast-path scale conversion: hardware cvt for f16 (identical to the integer routine for every finite value).
template <bool SBF>
__device__ __forceinline__ float w4_scale_fast(unsigned bits16) {
    if (SBF) return __builtin_bit_cast(float, bits16 << 16);
    return (float)__builtin_bit_cast(_Float16, (unsigned short)bits16);
}

// c + a * b as one fused multiply-add per element.  Written out because the kernels are compiled without floating-point
// contraction (a library routine such as expf must expand to the same instructions in every code object, so that a
// fused epilogue gives the bits of the separate kernel).
__device__ __forceinline__ f4_t w4_fma4(f4_t a, f4_t b, f4_t c) {
    f4_t r;
#pragma unroll
    for (int i = 0; i < 4; i++) r[i] = __builtin_fmaf(a[i], b[i], c[i]);
    return r;
}

// act(gate) * up in f32, the element-wise step between a gated FFN's projections: kind 0 = silu (assets/ew.cu:9-32,
// w4a16_moe_act_silu_f16), kind 1 = the tanh form of gelu (assets/ew.cu:34-57, w4a16_moe_act_gelu_f16,
// assets/moe.cu:1635-1647), in the reference's order of operations.  One definition for every kernel that applies it,
// so that fused epilogues give the bits of the separate kernel.  `kind` is uniform.
__device__ __forceinline__ float w4_act_mul(float g, float u, int kind) {
    if (kind == 1) {
        const float x3 = g * g * g;
        return (0.5f * g * (1.0f + tanhf(0.7978846f * (g + 0.044715f * x3)))) * u;
    }
    return (g / (1.0f + expf(-g))) * u;
}
