// Shared device helpers of the gfx950 W4A16 library: vector types, the int4 -> fp16
// conversion and the tiled weight layout.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "w4a16_internal.h"

namespace w4a16 {

typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float    float4_t __attribute__((ext_vector_type(4)));
typedef float    float16_t __attribute__((ext_vector_type(16)));

constexpr int kGroup = 128;  // quantisation group size == rows of one weight tile
constexpr int kTileN = 16;   // columns of one weight tile
constexpr int kWave  = 64;

// Layout of the repacked weights.  One tile = 16 columns x 128 rows = 1024 bytes, stored as
// 64 lanes x uint4.  Tile index = kt * (N/16) + nt: the column tiles of one group are
// contiguous, so waves on neighbouring columns stream neighbouring DRAM pages (measured: about
// 10 % more bandwidth on a 240 MB matrix than with the tiles of a column contiguous).
// Lane l = 16*b + c holds column
// 16*nt + c; its word j holds rows 128*kt + 32*j + 8*b + e (e = 0..7), row offset e in
// nibble kNibbleOfRow[e].  One word is therefore one B operand of v_mfma_f32_16x16x32_f16.
// Pack order along the rows is the AWQ order [0,2,4,6,1,3,5,7], which lets the unpack
// below produce rows (0,1), (2,3), (4,5), (6,7) as fp16 pairs with a single shift.
__device__ __host__ constexpr int row_of_nibble(int p)
{
    return (p & 3) * 2 + (p >> 2);  // [0,2,4,6,1,3,5,7]
}
__device__ __host__ constexpr int nibble_of_row(int e)
{
    return (e & 1) * 4 + (e >> 1);  // [0,4,1,5,2,6,3,7]
}

__device__ __forceinline__ half2_t as_half2(uint32_t u)
{
    return __builtin_bit_cast(half2_t, u);
}
__device__ __forceinline__ uint32_t as_u32(half2_t h)
{
    return __builtin_bit_cast(uint32_t, h);
}

// Mask and magic constants of the unpack, held in registers.  gfx9-family VOP3 encodings take
// no 32-bit literals, so (w & mask) | magic only becomes one v_and_or_b32 when both constants
// already live in registers; the empty asm statements keep the optimiser from folding them
// back into literals (which would cost a separate v_and_b32 and v_or_b32 per pair).
struct UnpackConsts {
    uint32_t mask_lo, mask_hi;    // SGPRs
    uint32_t magic_lo, magic_hi;  // VGPRs
    __device__ __forceinline__ UnpackConsts()
    {
        mask_lo  = 0x000f000fu;
        mask_hi  = 0x00f000f0u;
        magic_lo = 0x64006400u;
        magic_hi = 0x54005400u;
        asm volatile("" : "+s"(mask_lo), "+s"(mask_hi));
        asm volatile("" : "+v"(magic_lo), "+v"(magic_hi));
    }
};

// The four fp16 pairs of one weight word, still carrying their offsets:
//   v[0] = 1024 + rows (0,1), v[1] = 64 + rows (2,3), v[2] = 1024 + rows (4,5), v[3] = 64 + rows (6,7)
// 0x6400 is 1024.0 (ulp 1) so OR-ing a nibble into bits 0..3 adds it; 0x5400 is 64.0
// (ulp 1/16) so OR-ing a nibble into bits 4..7 adds it too.
__device__ __forceinline__ void unpack_offset(uint32_t w, uint32_t (&v)[4])
{
    const uint32_t w8 = w >> 8;
    v[0] = (w & 0x000f000fu) | 0x64006400u;
    v[1] = (w & 0x00f000f0u) | 0x54005400u;
    v[2] = (w8 & 0x000f000fu) | 0x64006400u;
    v[3] = (w8 & 0x00f000f0u) | 0x54005400u;
}
__device__ __forceinline__ void unpack_offset(uint32_t w, uint32_t (&v)[4], const UnpackConsts& k)
{
    const uint32_t w8 = w >> 8;
    v[0] = (w & k.mask_lo) | k.magic_lo;
    v[1] = (w & k.mask_hi) | k.magic_hi;
    v[2] = (w8 & k.mask_lo) | k.magic_lo;
    v[3] = (w8 & k.mask_hi) | k.magic_hi;
}

// One weight word -> eight fp16 weights, rows 0..7 in order: fp16_rn((q - z) * s), the reference's
// weight.  z1024 = (1024 + z) x2 and z64 = (64 + z) x2; both subtractions are exact.
__device__ __forceinline__ half8_t dequant_full(uint32_t w, half2_t z1024, half2_t z64, half2_t s,
                                                const UnpackConsts& k)
{
    uint32_t v[4];
    unpack_offset(w, v, k);
    const half2_t a = (as_half2(v[0]) - z1024) * s;
    const half2_t b = (as_half2(v[1]) - z64) * s;
    const half2_t c = (as_half2(v[2]) - z1024) * s;
    const half2_t d = (as_half2(v[3]) - z64) * s;
    half8_t r;
    r[0] = a[0]; r[1] = a[1]; r[2] = b[0]; r[3] = b[1];
    r[4] = c[0]; r[5] = c[1]; r[6] = d[0]; r[7] = d[1];
    return r;
}

// The reference multiplies (q - z) by the scale with flush-to-zero (mul.ftz.f16x2, common.h:229-230):
// a subnormal scale counts as zero, and that is the only case in which the flush acts, because a
// normal scale times a non-zero integer is never subnormal.  True if the scale of Q word `q` is normal.
__device__ __forceinline__ bool scale_is_normal(uint32_t q)
{
    return (q & 0x7c000000u) != 0;
}

// A Q entry is half2(64 + z, s) with bits 0x5400 | z << 4 in the low half.
__device__ __forceinline__ void split_q(uint32_t q, half2_t& z1024, half2_t& z64, half_t& s)
{
    const half2_t h = as_half2(q);
    z64             = half2_t{h[0], h[0]};
    const uint32_t zb = ((q >> 4) & 0xfu) | 0x6400u;
    z1024           = as_half2(zb | (zb << 16));
    s               = scale_is_normal(q) ? h[1] : (half_t)0.f;
}

// Measurement aid: the engine clock a kernel ran at.  One thread of a launch subtracts the core-clock counter and the
// constant-rate counter from clk[0] and clk[1] when it starts and adds them when it ends (clk[2] counts launches), so
// that nothing stays in a register in between; summed over launches, clk[0] / clk[1] x the constant rate is the
// clock.  clk == nullptr (every ordinary launch) records nothing.
__device__ __forceinline__ void clock_record_start(unsigned long long* clk, bool this_thread)
{
    if (clk != nullptr && this_thread) {
        atomicAdd(clk, 0ull - (unsigned long long)clock64());
        atomicAdd(clk + 1, 0ull - (unsigned long long)wall_clock64());
        // (the kernels that follow wait for their loads by count: nothing else may be in flight)
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
}
__device__ __forceinline__ void clock_record_stop(unsigned long long* clk, bool this_thread)
{
    if (clk != nullptr && this_thread) {
        atomicAdd(clk, (unsigned long long)clock64());
        atomicAdd(clk + 1, (unsigned long long)wall_clock64());
        atomicAdd(clk + 2, 1ull);
    }
}

}  // namespace w4a16
