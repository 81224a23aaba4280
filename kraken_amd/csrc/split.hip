// fp32 GEMM operands for the bf16 matrix cores: x = hi + lo with hi = bf16(x), lo = bf16(x - hi).
// One pass over the fp32 matrix writes the three bf16 blocks the 3K-long product needs,
//   A [M, K]            -> [ a_hi | a_hi | a_lo ]   ([M, 3K], blocks side by side)
//   B [K, N] row-major  -> [ b_hi ; b_lo ; b_hi ]   ([3K, N], blocks one below the other)
//   B^T [N, K]          -> [ b_hi | b_lo | b_hi ]   ([N, 3K])
// so that  A' @ B' = a_hi b_hi + a_hi b_lo + a_lo b_hi  (everything of a @ b but a_lo b_lo).
#include "common.h"

namespace kr {

// One thread per 8 consecutive columns: two 128-bit loads, three 128-bit stores.
// SIDE: blocks side by side (block b of row r starts at out + r*ld_out + b*cols), else one below
// the other (block b of row r at out + (b*rows + r)*ld_out).  sel[b]: 0 = hi, 1 = lo.
template <bool SIDE>
__global__ __launch_bounds__(256) void split_fp32_kernel(const float* __restrict__ x, int64_t rows, int cols_v, int64_t ld_x,
                                                         uint16_t* __restrict__ out, int64_t ld_out, int sel0, int sel1, int sel2) {
    const int64_t nvec = rows * cols_v;
    for (int64_t v = (int64_t)blockIdx.x * 256 + threadIdx.x; v < nvec; v += (int64_t)gridDim.x * 256) {
        const int64_t r = v / cols_v;
        const int c = (int)(v - r * cols_v) * 8;
        const f32x4 lo4 = __builtin_nontemporal_load((const f32x4*)(x + r * ld_x + c));
        const f32x4 hi4 = __builtin_nontemporal_load((const f32x4*)(x + r * ld_x + c + 4));
        const float f[8] = {lo4.x, lo4.y, lo4.z, lo4.w, hi4.x, hi4.y, hi4.z, hi4.w};
        const u32x4 hi = pack8(f);
        float h[8], d[8];
        unpack8(hi, h);
#pragma unroll
        for (int j = 0; j < 8; ++j) d[j] = f[j] - h[j];
        const u32x4 lo = pack8(d);
        const int cols = cols_v * 8;
        const int sel[3] = {sel0, sel1, sel2};
#pragma unroll
        for (int b = 0; b < 3; ++b) {
            uint16_t* dst = SIDE ? out + r * ld_out + (int64_t)b * cols + c : out + ((int64_t)b * rows + r) * ld_out + c;
            st_stream((u32x4*)dst, sel[b] ? lo : hi);
        }
    }
}

}  // namespace kr

using namespace kr;

extern "C" int kr_split_fp32(const void* x, int64_t rows, int64_t cols, int64_t ld_x, int side_by_side, int pattern,
                             void* out, int64_t ld_out, void* stream) {
    if (rows < 0 || cols < 0 || rows > 0x7fffffffLL || cols > 0x7fffffffLL) return KR_ERR_BAD_DIM;
    if (cols % 8 != 0) return KR_ERR_NUMEL_MOD8;
    if (rows == 0 || cols == 0) return KR_OK;
    if (x == nullptr || out == nullptr) return KR_ERR_NULL_POINTER;
    if (ld_x < cols || ld_out < (side_by_side ? 3 * cols : cols)) return KR_ERR_LAYOUT;
    if (!aligned16(x) || !aligned16(out) || ld_x % 4 != 0 || ld_out % 8 != 0) return KR_ERR_ALIGNMENT;
    if (pattern != 0 && pattern != 1) return KR_ERR_BAD_DIM;
    // pattern 0: hi, hi, lo (the left operand); 1: hi, lo, hi (the right operand)
    const int s1 = pattern == 0 ? 0 : 1, s2 = pattern == 0 ? 1 : 0;
    const int64_t nvec = rows * (cols / 8);
    const unsigned blocks = (unsigned)std::min<int64_t>((nvec + 255) / 256, 256 * 16);
    hipStream_t st = (hipStream_t)stream;
    if (side_by_side)
        hipLaunchKernelGGL(split_fp32_kernel<true>, dim3(blocks), dim3(256), 0, st, (const float*)x, rows, (int)(cols / 8), ld_x,
                           (uint16_t*)out, ld_out, 0, s1, s2);
    else
        hipLaunchKernelGGL(split_fp32_kernel<false>, dim3(blocks), dim3(256), 0, st, (const float*)x, rows, (int)(cols / 8), ld_x,
                           (uint16_t*)out, ld_out, 0, s1, s2);
    return (int)hipGetLastError();
}
