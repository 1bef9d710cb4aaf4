// Division of a run-time numerator by a run-time divisor that the host knows at launch: the host passes a 32-bit
// reciprocal with the kernel arguments and the kernel multiplies (a division in the kernel is a 25-instruction
// sequence through the floating-point reciprocal).  Pure integer code for the GPU (hipcc) and the host (g++: the
// launch code computes the reciprocals, and the CPU unit tests check both halves against plain division).
#pragma once
#include <stdint.h>

#if defined(__HIPCC__)
#include <hip/hip_runtime.h>
#define AP_RCP_HD __host__ __device__ __forceinline__
#else
#define AP_RCP_HD inline
#endif

namespace ap {

AP_RCP_HD uint32_t mul_hi_u32(uint32_t a, uint32_t b) {
#if defined(__HIP_DEVICE_COMPILE__)
    return __umulhi(a, b);
#else
    return (uint32_t)(((uint64_t)a * b) >> 32);
#endif
}

// floor(2^32 / d) for d >= 2, 2^32 - 1 for d = 1.
AP_RCP_HD uint32_t reciprocal_floor(uint32_t d) { return d <= 1u ? 0xffffffffu : (uint32_t)((1ull << 32) / d); }

// q = n / d, r = n % d for n < 2^31, 1 <= d < 2^31, magic = reciprocal_floor(d).  The product's high word is the
// quotient or one below it (the reciprocal is short by less than one part in 2^32 / d, and n < 2^31 keeps the
// total shortfall below one), so one correction step finishes; it is written as integer arithmetic on the sign
// bit, which stays in scalar registers where a select of 1 and 0 would travel through a vector register.
AP_RCP_HD void divmod_by_reciprocal(uint32_t n, uint32_t d, uint32_t magic, uint32_t &q, uint32_t &r) {
    q = mul_hi_u32(n, magic);
    r = n - q * d;
    const uint32_t fix = (d - 1u - r) >> 31;  // 1 when r >= d
    q += fix;
    r -= d & (0u - fix);
}

// ceil(2^32 / d) for d >= 2 (unused for d = 1: 0).
AP_RCP_HD uint32_t reciprocal_ceil(uint32_t d) { return d <= 1u ? 0u : (uint32_t)(((1ull << 32) + d - 1u) / d); }

// n / d for n * d < 2^32 (d <= 8 and n < 2^29 in the kernels that use it), magic = reciprocal_ceil(d): exact
// without a correction, because the reciprocal's excess times n stays below 1 / d.
AP_RCP_HD uint32_t div_by_reciprocal_ceil(uint32_t n, uint32_t d, uint32_t magic) {
    return d == 1u ? n : mul_hi_u32(n, magic);
}

}  // namespace ap
