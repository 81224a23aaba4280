// fp8 (e4m3fn, the OCP format: bias 7, no infinities, NaN = S.1111.111, largest finite 448)
// operands for the bf16 GEMM path, and fp32 results back to fp8.  Every e4m3 value is a bf16
// value, so the product of converted operands, accumulated in fp32, is what an fp8 matrix-core
// instruction with fp32 accumulation computes; the result is rounded once, from fp32.
// The conversions are written out in integer arithmetic (no hardware conversion instruction is
// relied on): round to nearest even; finite values beyond the largest finite one saturate to it,
// as cvt.rn.satfinite does in the code Triton generates for the reference's `.to(tl.float8e4nv)`
// (kraken/fused/all_gather_matmul.py:53,121); NaN stays NaN.
#include "common.h"

namespace kr {

__device__ __forceinline__ uint32_t e4m3_to_bf16_bits(uint32_t b) {
    const uint32_t sign = (b & 0x80u) << 8;
    const uint32_t exp = (b >> 3) & 15u, man = b & 7u;
    if (exp == 0) {
        // subnormal: man * 2^-9, exact in bf16 (man < 8)
        const float f = (float)man * 0.001953125f;
        return sign | (__builtin_bit_cast(uint32_t, f) >> 16);
    }
    if (exp == 15 && man == 7) return sign | 0x7fc0u;
    return sign | ((exp + 120u) << 7) | (man << 4);
}

__device__ __forceinline__ uint32_t f32_to_e4m3(float x) {
    const uint32_t u = __builtin_bit_cast(uint32_t, x);
    const uint32_t sign = (u >> 24) & 0x80u;
    const uint32_t a = u & 0x7fffffffu;
    if (a > 0x7f800000u) return sign | 0x7fu;                 // NaN
    if (a >= 0x43e00000u) return sign | 0x7eu;                // |x| >= 448 (infinity included): largest finite
    if (a < 0x3c800000u) {                                    // |x| < 2^-6: subnormal, steps of 2^-9
        const float m = __builtin_rintf(__builtin_bit_cast(float, a) * 512.0f);   // 0 .. 8, ties to even
        return sign | (uint32_t)m;                            // 8 is the smallest normal, 0x08
    }
    const uint32_t r = a + 0x7ffffu + ((a >> 20) & 1u);       // round the 23-bit mantissa to 3 bits, ties to even
    uint32_t e = ((r >> 23) - 120u) << 3 | ((r >> 20) & 7u);
    if (e > 0x7eu) e = 0x7eu;
    return sign | e;
}

// 16 fp8 per thread: one 128-bit load, two 128-bit stores
__global__ __launch_bounds__(256) void cast_e4m3_bf16_kernel(const u32x4* __restrict__ src, u32x4* __restrict__ dst, int64_t nvec) {
    for (int64_t v = (int64_t)blockIdx.x * 256 + threadIdx.x; v < nvec; v += (int64_t)gridDim.x * 256) {
        const u32x4 x = ld_stream(src + v);
        const uint32_t w[4] = {x.x, x.y, x.z, x.w};
        uint32_t o[8];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            o[2 * i] = e4m3_to_bf16_bits(w[i] & 0xffu) | (e4m3_to_bf16_bits((w[i] >> 8) & 0xffu) << 16);
            o[2 * i + 1] = e4m3_to_bf16_bits((w[i] >> 16) & 0xffu) | (e4m3_to_bf16_bits(w[i] >> 24) << 16);
        }
        st_stream(dst + 2 * v, u32x4{o[0], o[1], o[2], o[3]});
        st_stream(dst + 2 * v + 1, u32x4{o[4], o[5], o[6], o[7]});
    }
}

// 16 fp32 per thread: four 128-bit loads, one 128-bit store
__global__ __launch_bounds__(256) void cast_f32_e4m3_kernel(const f32x4* __restrict__ src, u32x4* __restrict__ dst, int64_t nvec) {
    for (int64_t v = (int64_t)blockIdx.x * 256 + threadIdx.x; v < nvec; v += (int64_t)gridDim.x * 256) {
        uint32_t o[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const f32x4 f = __builtin_nontemporal_load(src + 4 * v + i);
            o[i] = f32_to_e4m3(f.x) | (f32_to_e4m3(f.y) << 8) | (f32_to_e4m3(f.z) << 16) | (f32_to_e4m3(f.w) << 24);
        }
        st_stream(dst + v, u32x4{o[0], o[1], o[2], o[3]});
    }
}

}  // namespace kr

using namespace kr;

static int cast_launch_checks(const void* src, void* dst, int64_t n) {
    if (n < 0) return KR_ERR_BAD_DIM;
    if (n % 16 != 0) return KR_ERR_NUMEL_MOD8;
    if (n == 0) return KR_OK;
    if (src == nullptr || dst == nullptr) return KR_ERR_NULL_POINTER;
    if (!aligned16(src) || !aligned16(dst)) return KR_ERR_ALIGNMENT;
    return KR_OK;
}

extern "C" int kr_cast_fp8_to_bf16(const void* src, int64_t n, void* dst, void* stream) {
    const int rc = cast_launch_checks(src, dst, n);
    if (rc != KR_OK || n == 0) return rc;
    const int64_t nvec = n / 16;
    const unsigned blocks = (unsigned)std::min<int64_t>((nvec + 255) / 256, 256 * 16);
    hipLaunchKernelGGL(cast_e4m3_bf16_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream, (const u32x4*)src, (u32x4*)dst, nvec);
    return (int)hipGetLastError();
}

extern "C" int kr_cast_f32_to_fp8(const void* src, int64_t n, void* dst, void* stream) {
    const int rc = cast_launch_checks(src, dst, n);
    if (rc != KR_OK || n == 0) return rc;
    const int64_t nvec = n / 16;
    const unsigned blocks = (unsigned)std::min<int64_t>((nvec + 255) / 256, 256 * 16);
    hipLaunchKernelGGL(cast_f32_e4m3_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream, (const f32x4*)src, (u32x4*)dst, nvec);
    return (int)hipGetLastError();
}
