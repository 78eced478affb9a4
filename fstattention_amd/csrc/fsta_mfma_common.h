// Pieces shared by the matrix-core attention kernels (gfx950 only): vector types, MFMA and
// conversion traits, wait-count helpers, inline-assembly LDS reads, LDS swizzles.
#pragma once

#include "fsta_common.h"

namespace fsta {
namespace mfma {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

constexpr int kTileN = 32;     // keys per tile
constexpr int kCus = 256;      // compute units of an MI355X
constexpr int kXcds = 8;       // L2 domains of an MI355X; workgroup i runs on XCD i % 8
constexpr int kMaxStages = 4;  // ring depth limit (LDS per workgroup = stages * 4 * 32 * D bytes)
constexpr float kRescaleSlack = 8.f;  // log2 of the largest weight kept without raising the maximum

template <bool BF16> struct Mma;
template <> struct Mma<true> {
    using elem = __bf16;
    using elem2 = bf16x2;
    using frag = bf16x8;
    static __device__ __forceinline__ f32x16 mfma(frag a, frag b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ float dot2(elem2 a, elem2 b, float c) {
        return __builtin_amdgcn_fdot2_f32_bf16(a, b, c, false);
    }
    // Two floats -> two bf16 (round to nearest even) in one dword, first value in the low
    // half: one v_cvt_pk_bf16_f32.  Kept as a vector cast the compiler can see (not inline
    // assembly), so that it inserts the wait states the matrix cores need after a VALU write.
    static __device__ __forceinline__ uint32_t pack(float a, float b) {
        const f32x2 w = {a, b};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(w, bf16x2));
    }
    static __device__ __forceinline__ float low(uint32_t pk) { return __builtin_bit_cast(float, pk << 16); }
    static __device__ __forceinline__ float high(uint32_t pk) { return __builtin_bit_cast(float, pk & 0xffff0000u); }
};
template <> struct Mma<false> {
    using elem = _Float16;
    using elem2 = f16x2;
    using frag = f16x8;
    static __device__ __forceinline__ f32x16 mfma(frag a, frag b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ float dot2(elem2 a, elem2 b, float c) {
        return __builtin_amdgcn_fdot2(a, b, c, false);
    }
    static __device__ __forceinline__ uint32_t pack(float a, float b) {
        const uint32_t lo = __builtin_bit_cast(unsigned short, (_Float16)a);
        const uint32_t hi = __builtin_bit_cast(unsigned short, (_Float16)b);
        return lo | (hi << 16);
    }
    static __device__ __forceinline__ float low(uint32_t pk) {
        return (float)__builtin_bit_cast(_Float16, (unsigned short)(pk & 0xffffu));
    }
    static __device__ __forceinline__ float high(uint32_t pk) {
        return (float)__builtin_bit_cast(_Float16, (unsigned short)(pk >> 16));
    }
};

__host__ __device__ constexpr int anc_tile_capacity(int max_anc) { return (max_anc + kTileN - 1) / kTileN; }

// LDS of one workgroup: ring of K|V tiles, then 32 sanitised keys and a validity word
// per listed tile (M/32 leaf tiles, then the ancestor tiles) and M mask words per
// ancestor tile.
template <int D, int M>
__host__ __device__ constexpr size_t mfma_lds_bytes(int max_anc, int stages) {
    return (size_t)stages * 2 * kTileN * D * 2 +
           (size_t)(M / 32 + anc_tile_capacity(max_anc)) * (kTileN * 4 + 4) + 12 +
           (size_t)anc_tile_capacity(max_anc) * M * 4;
}

template <int N> __device__ __forceinline__ void wait_vmcnt() {
    // s_waitcnt immediate on gfx9: vmcnt = [3:0] and [15:14], expcnt = [6:4], lgkmcnt = [11:8];
    // the other two counters are left at "do not wait"
    static_assert(N >= 0 && N < 64, "vmcnt has 6 bits");
    __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
}

// Waits until at most `tiles` tiles' worth of this wave's global->LDS transfers
// (kPerTile instructions each, retired in order) are still outstanding.
template <int kPerTile> __device__ __forceinline__ void wait_tiles_outstanding(int tiles) {
    static_assert((kMaxStages - 1) * kPerTile < 64, "ring too deep for vmcnt");
    switch (tiles) {
        case 0: wait_vmcnt<0>(); break;
        case 1: wait_vmcnt<kPerTile>(); break;
        case 2: wait_vmcnt<2 * kPerTile>(); break;
        default: wait_vmcnt<3 * kPerTile>(); break;
    }
}

// 32-bit LDS address of a pointer into the dynamic shared segment
__device__ __forceinline__ uint32_t lds_addr(const void* ptr) {
    return (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) char*)ptr;
}

// LDS reads of tile data are issued as inline assembly on purpose: for the builtin
// forms the compiler's wait-count pass first drains every outstanding global->LDS
// transfer (s_waitcnt vmcnt(0)), which would empty the gather ring on every tile.
// A result is only valid after lds_wait() followed by lds_tie() on it.
// EVERY result must be tied behind its wait on every path, also one that nobody reads: the data
// arrives long after the statement, the compiler takes the statement itself as the write, and a
// result that is dead for the compiler has its registers handed to other values at once, which the
// late arrival then overwrites (seen on the device: wrong rows in one template instance only,
// moving with every change of register allocation).
//
// ds_read_b64_tr_b16: within each group of 16 lanes, lane i supplies the address of
// 4 consecutive 16-bit elements (think row i/4, column block i%4 of a 4 x 16 tile)
// and receives element column i of rows 0..3, i.e. component j comes from lane
// 4j + i/4, element i%4.
__device__ __forceinline__ s16x4 lds_read_tr16(uint32_t addr) {
    s16x4 out;
    asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(out) : "v"(addr) : "memory");
    return out;
}
template <int kOffset> __device__ __forceinline__ s16x4 lds_read_tr16_at(uint32_t addr) {
    s16x4 out;
    asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(out) : "v"(addr), "n"(kOffset) : "memory");
    return out;
}
__device__ __forceinline__ u32x4 lds_read_b128(uint32_t addr) {
    u32x4 out;
    asm volatile("ds_read_b128 %0, %1" : "=v"(out) : "v"(addr) : "memory");
    return out;
}
__device__ __forceinline__ uint32_t lds_read_b32(uint32_t addr) {
    uint32_t out;
    asm volatile("ds_read_b32 %0, %1" : "=v"(out) : "v"(addr) : "memory");
    return out;
}
__device__ __forceinline__ u32x2 lds_read_b64(uint32_t addr) {
    u32x2 out;
    asm volatile("ds_read_b64 %0, %1" : "=v"(out) : "v"(addr) : "memory");
    return out;
}
// 8-byte global load the compiler does not see: with global->LDS transfers in flight its own
// wait for a loaded register is always vmcnt(0), i.e. for every transfer issued since.  The
// result is valid after a wait_vmcnt<N>() that covers it, followed by lds_tie().
__device__ __forceinline__ u32x2 global_read_b64(const void* ptr) {
    u32x2 out;
    asm volatile("global_load_dwordx2 %0, %1, off" : "=v"(out) : "v"(ptr) : "memory");
    return out;
}
__device__ __forceinline__ uint32_t global_read_b32(const void* ptr) {
    uint32_t out;
    asm volatile("global_load_dword %0, %1, off" : "=v"(out) : "v"(ptr) : "memory");
    return out;
}
// LDS store the compiler does not see either (same reason); complete after lds_wait().
__device__ __forceinline__ void lds_write_b32(uint32_t addr, uint32_t value) {
    asm volatile("ds_write_b32 %0, %1" : : "v"(addr), "v"(value) : "memory");
}
__device__ __forceinline__ void lds_write_b128(uint32_t addr, u32x4 value) {
    asm volatile("ds_write_b128 %0, %1" : : "v"(addr), "v"(value) : "memory");
}
// Waits for every outstanding LDS access of this wave.
__device__ __forceinline__ void lds_wait() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }
// Orders every later use of `x` behind the preceding lds_wait().
template <typename V> __device__ __forceinline__ void lds_tie(V& x) { asm volatile("" : "+v"(x)); }

// Workgroup barrier without the memory fence of __syncthreads(): that fence waits for every
// outstanding global->LDS transfer (vmcnt(0)) and would drain the gather ring at every step.
// What must be visible across the barrier is waited for explicitly instead: the caller's own
// transfers of the tiles about to be used (wait_tiles_outstanding) and, here, its LDS accesses.
__device__ __forceinline__ void ring_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

// Sum / maximum over the four lanes l, l ^ 16, l ^ 32, l ^ 48 (one per quarter-wave), result in
// all four: v_permlane32_swap exchanges the upper half of one register with the lower half of
// another, v_permlane16_swap the odd 16-lane rows with the even ones, so two copies of x turn
// into "my half's value" and "the other half's value".  Vector ALU only, no trip through LDS
// (ds_bpermute).  All 64 lanes must be active.
__device__ __forceinline__ void swap_halves(float x, bool rows16, float& mine, float& other) {
    const uint32_t bits = __builtin_bit_cast(uint32_t, x);
    const u32x2 r = rows16 ? __builtin_amdgcn_permlane16_swap(bits, bits, false, false)
                           : __builtin_amdgcn_permlane32_swap(bits, bits, false, false);
    const uint32_t r0 = r[0], r1 = r[1];   // (copies: bit_cast straight from a vector element reads element 0)
    mine = __builtin_bit_cast(float, r0);
    other = __builtin_bit_cast(float, r1);
}
__device__ __forceinline__ float sum_quarters(float x) {
    float a, b;
    swap_halves(x, false, a, b);
    x = a + b;
    swap_halves(x, true, a, b);
    return a + b;
}
__device__ __forceinline__ float max_quarters(float x) {
    float a, b;
    swap_halves(x, false, a, b);
    x = fmaxf(a, b);
    swap_halves(x, true, a, b);
    return fmaxf(a, b);
}

struct VPair { s16x4 a, b; };   // 8 consecutive k-indices of one A-operand row

// 16-byte chunk position of (row, chunk) inside an LDS tile.  K is read as whole
// 16-byte fragments by 32 different rows at once, V as 4-row x 64-byte groups by
// the transposing read; each gets the XOR pattern that spreads its access over
// all 64 banks.
template <int D> __device__ __forceinline__ int k_chunk(int row, int c) {
    constexpr int cpr = D / 8, rpb = 16 / cpr;
    return c ^ ((row / rpb) % cpr);
}
template <int D> __device__ __forceinline__ int v_chunk(int row, int c) {
    constexpr int qpr = D / 32, rpb = 4 / qpr;
    return c ^ (4 * ((row / rpb) % qpr));
}

// V tile swizzle for the transposing read of the kernels with 16 query rows per MFMA: one read
// instruction touches 16 consecutive rows x 32 bytes, so 32-byte granules are XORed with the row.
template <int D> __device__ __forceinline__ int v16_chunk(int row, int c) {
    constexpr int gpr = D / 16, rpb = 8 / gpr;   // granules per row, rows per 256 bytes
    return c ^ (2 * ((row / rpb) % gpr));
}

typedef float f32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ f32x4 mfma16(bf16x8 a, bf16x8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ f32x4 mfma16(f16x8 a, f16x8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
}

}  // namespace mfma
}  // namespace fsta
