// Device-side helpers shared by the gfx950 kernels: vector types, wave64
// reductions through DPP, LUT staging into LDS.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

namespace ap {

typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kWave = 64;

// Compile-time loop: f(integral_constant<int,0>) ... f(integral_constant<int,N-1>).
template <int N, int I = 0, typename F>
__device__ __forceinline__ void static_for(F &&f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<N, I + 1>(f);
    }
}

// fp32 += a.x*b.x + a.y*b.y  (v_dot2c_f32_f16: fp16 products, fp32 accumulate)
__device__ __forceinline__ float dot2(uint32_t w, uint32_t x, float acc) {
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, w), __builtin_bit_cast(half2_t, x), acc, false);
}

// ((v >> 8*BYTE) & 0xff) << SHIFT in one VALU instruction: SDWA byte select on
// the shifted operand (SHIFT > 0), a bit-field extract otherwise.  This is the
// LDS byte offset of a gather whose table sits at a compile-time address.
template <int BYTE, int SHIFT>
__device__ __forceinline__ uint32_t byte_offset(uint32_t v) {
    static_assert(BYTE >= 0 && BYTE < 4 && SHIFT >= 0 && SHIFT < 8, "");
    if constexpr (SHIFT == 0) {
        return __builtin_amdgcn_ubfe(v, 8 * BYTE, 8);
    } else {
        uint32_t r;
        const uint32_t sh = SHIFT;
        if constexpr (BYTE == 0)
            asm("v_lshlrev_b32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:BYTE_0"
                : "=v"(r) : "v"(sh), "v"(v));
        else if constexpr (BYTE == 1)
            asm("v_lshlrev_b32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:BYTE_1"
                : "=v"(r) : "v"(sh), "v"(v));
        else if constexpr (BYTE == 2)
            asm("v_lshlrev_b32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:BYTE_2"
                : "=v"(r) : "v"(sh), "v"(v));
        else
            asm("v_lshlrev_b32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:BYTE_3"
                : "=v"(r) : "v"(sh), "v"(v));
        return r;
    }
}

// base + ((v >> 8*BYTE) & 0xff) in one VALU instruction (SDWA byte select on the second
// addend): the LDS byte address of a gather whose table base differs per lane, for index
// bytes that already hold the byte offset.
template <int BYTE>
__device__ __forceinline__ uint32_t byte_add(uint32_t base, uint32_t v) {
    static_assert(BYTE >= 0 && BYTE < 4, "");
    uint32_t r;
    if constexpr (BYTE == 0)
        asm("v_add_u32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:BYTE_0"
            : "=v"(r) : "v"(base), "v"(v));
    else if constexpr (BYTE == 1)
        asm("v_add_u32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:BYTE_1"
            : "=v"(r) : "v"(base), "v"(v));
    else if constexpr (BYTE == 2)
        asm("v_add_u32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:BYTE_2"
            : "=v"(r) : "v"(base), "v"(v));
    else
        asm("v_add_u32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:BYTE_3"
            : "=v"(r) : "v"(base), "v"(v));
    return r;
}

// A pointer into global memory that is the same in every lane, pinned to scalar registers: the compiler
// then adds a lane's 32-bit byte offset in the load instruction itself (scalar base + vector offset)
// instead of folding the base into 64-bit vector arithmetic per load.  The result carries the global
// address space in its type, which the round trip through integers would otherwise lose.
template <typename T>
using global_ptr = __attribute__((address_space(1))) T *;

template <typename T>
__device__ __forceinline__ global_ptr<T> scalar_ptr(T *p) {
    const uint64_t v = reinterpret_cast<uint64_t>(p);
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
    const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return (global_ptr<T>)(((uint64_t)hi << 32) | lo);
}

// Load of type V at byte offset `byte` (32 bits, per lane) from a scalar base.
template <typename V, typename T>
__device__ __forceinline__ V load_at(global_ptr<T> base, uint32_t byte) {
    return *(global_ptr<const V>)((global_ptr<const char>)base + byte);
}
template <typename V, typename T>
__device__ __forceinline__ V load_at_nt(global_ptr<T> base, uint32_t byte) {
    return __builtin_nontemporal_load((global_ptr<const V>)((global_ptr<const char>)base + byte));
}
template <typename V, typename T>
__device__ __forceinline__ void store_at_nt(global_ptr<T> base, uint32_t byte, const V &v) {
    __builtin_nontemporal_store(v, (global_ptr<V>)((global_ptr<char>)base + byte));
}

template <int CTRL>
__device__ __forceinline__ float dpp_add(float v) {
    const int moved = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true);
    return v + __builtin_bit_cast(float, moved);
}

template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_add_rows(float v) {
    const int moved = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, ROW_MASK, 0xf, false);
    return v + __builtin_bit_cast(float, moved);
}

// Sum over the 64 lanes of a wave in six DPP adds.  The total is valid in lanes
// 48..63 only (kSumLane reads it); other lanes hold partial sums.
constexpr int kSumLane = 63;
__device__ __forceinline__ float wave_sum(float v) {
    v = dpp_add<0xB1>(v);            // quad_perm [1,0,3,2]
    v = dpp_add<0x4E>(v);            // quad_perm [2,3,0,1]
    v = dpp_add<0x141>(v);           // row_half_mirror: lanes 0-3 <-> 7-4 within 8
    v = dpp_add<0x140>(v);           // row_mirror: every lane of a 16-lane row holds the row sum
    v = dpp_add_rows<0x142, 0xa>(v); // row_bcast:15 into rows 1 and 3
    v = dpp_add_rows<0x143, 0xc>(v); // row_bcast:31 into rows 2 and 3: row 3 holds the total
    return v;
}

// Copy one row's table of 2^BITS fp16 entries from global memory into this
// wave's LDS slot.  Split in two so the global load can be issued early.
template <int BITS>
struct LutRegs {
    u32x2 v;
};

template <int BITS>
__device__ __forceinline__ LutRegs<BITS> lut_fetch(global_ptr<const half_t> lut_row, int lane) {
    LutRegs<BITS> r;
    r.v = u32x2{0u, 0u};
    constexpr int dwords = (1 << BITS) / 2;          // table size in dwords
    if constexpr (dwords >= 128) {                   // 8 bits: 64 lanes x 8 B
        r.v = load_at<u32x2>(lut_row, (uint32_t)lane * 8u);
    } else if constexpr (dwords == 64) {             // 7 bits: 64 lanes x 4 B
        r.v.x = load_at<uint32_t>(lut_row, (uint32_t)lane * 4u);
    } else {                                         // <= 6 bits: first `dwords` lanes
        if (lane < dwords) r.v.x = load_at<uint32_t>(lut_row, (uint32_t)lane * 4u);
    }
    return r;
}
template <int BITS>
__device__ __forceinline__ LutRegs<BITS> lut_fetch(const half_t *lut_row, int lane) {
    return lut_fetch<BITS>(scalar_ptr(lut_row), lane);
}

// A point the fetched words cannot be used before: put between the loads a kernel issues after the table
// fetch and the staging, so that no staging work is moved up to the fetch (and the wave made to wait for its
// table before its other loads have left).
template <int BITS>
__device__ __forceinline__ void lut_arrive(LutRegs<BITS> &r) {
    if constexpr (BITS == 8) asm volatile("" : "+v"(r.v)); else asm volatile("" : "+v"(r.v.x));
}

template <int BITS>
__device__ __forceinline__ void lut_stage(const LutRegs<BITS> &r, half_t *slot, int lane) {
    constexpr int dwords = (1 << BITS) / 2;
    if constexpr (dwords >= 128) {
        reinterpret_cast<u32x2 *>(slot)[lane] = r.v;
    } else if constexpr (dwords == 64) {
        reinterpret_cast<uint32_t *>(slot)[lane] = r.v.x;
    } else {
        if (lane < dwords) reinterpret_cast<uint32_t *>(slot)[lane] = r.v.x;
    }
}

}  // namespace ap
