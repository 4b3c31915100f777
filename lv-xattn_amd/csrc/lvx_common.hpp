// Shared device helpers for the gfx950 (CDNA4) kernels: vector types, the
// 32x32x16 bf16 MFMA wrapper with its operand/accumulator lane layout, bf16
// packing, and the register-level 4x8 transpose used when a tile has to be
// staged into LDS with its contraction index contiguous.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace lvx {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

constexpr int WAVE = 64;

// D = A(32x16) * B(16x32) + C on one wavefront.  With lane l, g = l / 32:
//   A operand: row i = l % 32, the 8 values are contraction slots (g, e), e = 0..7
//   B operand: col j = l % 32, the 8 values are contraction slots (g, e)
//   C/D      : col j = l % 32, register v holds row i = 8*(v/4) + 4*g + (v%4)
// Slot (g, e) of A multiplies slot (g, e) of B; which logical k a slot stands
// for is the caller's choice as long as both operands agree.
__device__ __forceinline__ f32x16 mfma32(bf16x8 a, bf16x8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}

// Row of accumulator register v for lane-half g (see above).
__device__ __forceinline__ int acc_row(int v, int g) { return 8 * (v >> 2) + 4 * g + (v & 3); }

// When an accumulator tile is fed back as a B operand (its 32 rows become the
// contraction index), registers 8*s .. 8*s+7 form k-step s and slot (g, e)
// stands for row 16*s + 8*(e/4) + 4*g + (e%4).  The other operand is staged in
// LDS with that row stored at column 16*s + 8*g + e, i.e. with bits 2 and 3 of
// the row index exchanged:
__device__ __forceinline__ int swap23(int r) {
    return (r & ~12) | ((r & 4) << 1) | ((r & 8) >> 1);
}

__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
    f32x2 x = {lo, hi};
    bf16x2 y = __builtin_convertvector(x, bf16x2);   // v_cvt_pk_bf16_f32, round-to-nearest-even
    return __builtin_bit_cast(uint32_t, y);
}
__device__ __forceinline__ float bf16_lo(uint32_t u) { return __uint_as_float(u << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t u) { return __uint_as_float(u & 0xffff0000u); }

__device__ __forceinline__ bf16x8 as_bf16x8(u32x4 u) { return __builtin_bit_cast(bf16x8, u); }

// The 16-bit element type of a kernel instance: packing, unpacking and the MFMA.  Operands
// travel as bf16x8 (8 x 16 bits) whatever the type; only these functions interpret them.
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2;
template <bool F16>
struct Elt;
template <>
struct Elt<false> {   // bf16
    static __device__ __forceinline__ uint32_t pack(float lo, float hi) { return pack_bf16(lo, hi); }
    static __device__ __forceinline__ float lo(uint32_t u) { return bf16_lo(u); }
    static __device__ __forceinline__ float hi(uint32_t u) { return bf16_hi(u); }
    static __device__ __forceinline__ f32x16 mfma(bf16x8 a, bf16x8 b, f32x16 c) { return mfma32(a, b, c); }
};
template <>
struct Elt<true> {    // fp16
    static __device__ __forceinline__ uint32_t pack(float lo, float hi) {
        f32x2 x = {lo, hi};
        f16x2 y = __builtin_convertvector(x, f16x2);   // round-to-nearest-even
        return __builtin_bit_cast(uint32_t, y);
    }
    static __device__ __forceinline__ float lo(uint32_t u) { return (float)__builtin_bit_cast(f16x2, u)[0]; }
    static __device__ __forceinline__ float hi(uint32_t u) { return (float)__builtin_bit_cast(f16x2, u)[1]; }
    static __device__ __forceinline__ f32x16 mfma(bf16x8 a, bf16x8 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    }
};

// 16-byte global load, zero when !ok.
__device__ __forceinline__ u32x4 ldg16(const void* p, bool ok) {
    u32x4 z = {0u, 0u, 0u, 0u};
    return ok ? *reinterpret_cast<const u32x4*>(p) : z;
}

// r[i] = 8 bf16 of source row i (columns c..c+7), i = 0..3.
// out[c] = the 4 values of column c (rows 0..3) packed as 4 bf16 = 8 bytes.
__device__ __forceinline__ void transpose_4x8(const u32x4 r[4], u32x2 out[8]) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        uint32_t a = r[0][j], b = r[1][j], c = r[2][j], d = r[3][j];
        out[2 * j][0] = (a & 0xffffu) | (b << 16);
        out[2 * j][1] = (c & 0xffffu) | (d << 16);
        out[2 * j + 1][0] = (a >> 16) | (b & 0xffff0000u);
        out[2 * j + 1][1] = (c >> 16) | (d & 0xffff0000u);
    }
}

typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef s16x4 __attribute__((address_space(3)))* lds_s16x4_ptr;

// ds_read_b64_tr_b16: every lane supplies the LDS address of an 8-byte word
// (4 x 16 bit).  Within each group of 16 lanes, lane i receives element (i & 3)
// of the words addressed by lanes (i >> 2), (i >> 2) + 4, + 8, + 12.  Pointing
// the lane quad q of a group at row k0 + q of a tile T[k][m] (m contiguous,
// lane q*4 + t at columns m0 + 4t .. 4t+3) hands lane i the four values
// T[k0 .. k0+3][m0 + i]: an MFMA operand whose contraction index runs down the
// rows of a tile stored with the OTHER index contiguous, with no transposed copy.
__device__ __forceinline__ u32x2 lds_read_tr16(const uint16_t* p) {
    s16x4 r = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)p);
    return __builtin_bit_cast(u32x2, r);
}

// Per-lane element offset into T[k][m] (row stride `stride`) for a transposing
// operand read of a 32(m) x 16(k) MFMA operand; the second half of the operand
// (slots e = 4..7) is `half_rows` rows further down.
//   natural order : slot (g, e) <-> k = 8g + e          -> half_rows = 4
//   permuted order: slot (g, e) <-> k = 8(e/4) + 4g + e%4 -> half_rows = 8
// (the permuted order is the one an accumulator tile has when it is fed back
// as the other operand).
__device__ __forceinline__ int tr_lane_offset(int lane, int stride, bool permuted) {
    const int r = (lane & 15) >> 2, t = lane & 3, u = (lane >> 4) & 1, g = lane >> 5;
    return ((permuted ? 4 * g : 8 * g) + r) * stride + 16 * u + 4 * t;
}

__device__ __forceinline__ bf16x8 lds_operand_tr(const uint16_t* p, int half_offset) {
    const u32x2 a = lds_read_tr16(p), b = lds_read_tr16(p + half_offset);
    const u32x4 u = {a[0], a[1], b[0], b[1]};
    return as_bf16x8(u);
}

// 64 lanes x 16 bytes from global memory to the 1 KiB of LDS at byte address
// lds_byte (wave-uniform); lane i lands at lds_byte + 16 i.  Counted by vmcnt.
__device__ __forceinline__ void dma16(const char* sbase, uint32_t voff, uint32_t lds_byte) {
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_byte), "v"(voff), "s"(sbase)
                 : "memory", "m0");
}
__device__ __forceinline__ void dma16_addr(const char* addr, uint32_t lds_byte) {
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds_byte), "v"(addr) : "memory", "m0");
}
// the same with 4 bytes per lane: lane i lands at lds_byte + 4 i
__device__ __forceinline__ void dma4(const char* sbase, uint32_t voff, uint32_t lds_byte) {
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dword %1, %2" ::"s"(lds_byte), "v"(voff), "s"(sbase)
                 : "memory", "m0");
}
__device__ __forceinline__ void dma4_addr(const char* addr, uint32_t lds_byte) {
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dword %1, off" ::"s"(lds_byte), "v"(addr) : "memory", "m0");
}
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}
__device__ __forceinline__ void wait_lds() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }
// Work-group barrier that orders LDS traffic only: this wave's LDS accesses are
// complete before it and (being a compiler memory barrier too) none moves across
// it, but vector-memory operations in flight - loads straight to LDS that are
// waited for separately, stores - are not waited for, as __syncthreads() would.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// Values that are the same in every lane, made so for the compiler too (an inline-asm operand in a
// scalar register must not look lane-dependent).
__device__ __forceinline__ uint32_t uniform32(uint32_t x) { return (uint32_t)__builtin_amdgcn_readfirstlane((int)x); }
__device__ __forceinline__ int uniform32(int x) { return __builtin_amdgcn_readfirstlane(x); }
__device__ __forceinline__ float uniform32(float x) { return __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(x))); }
__device__ __forceinline__ int64_t uniform64(int64_t x) {
    const uint32_t lo = uniform32((uint32_t)x), hi = uniform32((uint32_t)((uint64_t)x >> 32));
    return (int64_t)(((uint64_t)hi << 32) | lo);
}
template <typename T>
__device__ __forceinline__ const T* uniform_ptr(const T* x) { return reinterpret_cast<const T*>(uniform64((int64_t)(uintptr_t)x)); }

// max of three (one instruction; fmaxf chains cost an extra canonicalising
// v_max per MFMA result)
__device__ __forceinline__ float max3(float a, float b, float c) {
    float r;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}

// Work-groups are dealt to the 8 XCDs of an MI355X round-robin by linear id.  Remap so that
// each XCD receives one contiguous range of the work list: neighbours in the
// list (which share K/V or Q tiles) then share that XCD's L2.  A placement hint only: every id
// below `total` is produced exactly once whatever the hardware does with it, so a device with
// another XCD count computes the same results with less L2 sharing.
__device__ __forceinline__ int xcd_remap(int bid, int total) {
    constexpr int NX = 8;
    int per = (total + NX - 1) / NX;
    return (bid % NX) * per + bid / NX;      // caller drops ids >= total
}

}  // namespace lvx
