// W-way elementwise reduce (+bias) over W bf16 buffers (the slices of a stacked tensor, or
// W separate allocations named by a pointer table).
//
// HBM-bound: per output vector of 8 elements the kernel reads W*16 B (+16 B of
// bias) and writes 16 B, i.e. (W+1)*2 bytes per element.  A workgroup walks the
// input in blocks of kThreads*kUnroll vectors (grid-stride, at most kMaxBlocks
// workgroups = 4 per CU: measured best on MI355X, 6.05 TB/s against 5.8 TB/s for
// one block per workgroup).  Every thread owns kUnroll 128-bit vectors that are
// kThreads vectors apart, so each wave-level load covers 1 KiB of consecutive
// addresses, and all W*kUnroll loads of a thread are issued before the first
// add (the adds keep the fixed order bias?, slice 0, 1, ... W-1, so the sum is
// reproducible bit for bit).  Loads and stores are non-temporal.
#include "common.h"

namespace kr {

constexpr int kThreads = 256;
constexpr int kMaxBlocks = 4 * 256;   // 4 workgroups per CU

enum BiasMode { kNoBias = 0, kFullBias = 1, kVectorBias = 2 };

// WT > 0: W known at compile time (loop fully unrolled); WT == 0: run-time W.
template <class SRC, int WT, int BIAS, bool BIAS_FIRST, int kUnroll>
__global__ __launch_bounds__(kThreads) void reduce_kernel(
    const SRC src, int w_rt, int64_t nvec,
    const u32x4* __restrict__ bias, uint32_t d_vec, u32x4* __restrict__ out) {
    const int W = WT > 0 ? WT : w_rt;
    for (int64_t blk = blockIdx.x; blk * (kThreads * kUnroll) < nvec; blk += gridDim.x) {
    const int64_t base = blk * (kThreads * kUnroll) + threadIdx.x;

    if (base - threadIdx.x + (int64_t)kUnroll * kThreads <= nvec) {
        // full block: no bounds checks
        float acc[kUnroll][8];
        u32x4 bv[kUnroll];
        if (BIAS != kNoBias) {
#pragma unroll
            for (int u = 0; u < kUnroll; ++u) {
                const int64_t i = base + (int64_t)u * kThreads;
                bv[u] = BIAS == kFullBias ? ld_stream(bias + i) : bias[mod_vec(i, d_vec)];
            }
        }
        if (WT > 0) {
            u32x4 v[WT > 0 ? WT : 1][kUnroll];
            if constexpr (SRC::kTable) {
                // separate buffers: each buffer's block through a descriptor (base = buffer +
                // block, in scalar registers), so all W buffers share one byte offset per (lane, u)
                constexpr uint32_t kBlockBytes = kThreads * kUnroll * 16;
#pragma unroll
                for (int r = 0; r < WT; ++r) {
                    const __amdgpu_buffer_rsrc_t rs = stream_rsrc(src.at(r) + blk * (kThreads * kUnroll), kBlockBytes);
#pragma unroll
                    for (int u = 0; u < kUnroll; ++u) v[r][u] = ld_stream(rs, (threadIdx.x + u * kThreads) * 16u);
                }
            } else {
#pragma unroll
                for (int r = 0; r < WT; ++r)
#pragma unroll
                    for (int u = 0; u < kUnroll; ++u)
                        v[r][u] = ld_stream(src.at(r) + base + (int64_t)u * kThreads);
            }
#pragma unroll
            for (int u = 0; u < kUnroll; ++u) {
                if (BIAS != kNoBias && BIAS_FIRST) {
                    unpack8(bv[u], acc[u]);
                    add8(v[0][u], acc[u]);
                } else {
                    zero8(acc[u]);  // acc = 0.0f, then += slice 0 (keeps the sign of a -0.0 sum as the reference has it)
                    add8(v[0][u], acc[u]);
                }
#pragma unroll
                for (int r = 1; r < WT; ++r) add8(v[r][u], acc[u]);
            }
        } else {
#pragma unroll
            for (int u = 0; u < kUnroll; ++u) {
                const int64_t i = base + (int64_t)u * kThreads;
                if (BIAS != kNoBias && BIAS_FIRST) {
                    unpack8(bv[u], acc[u]);
                    add8(ld_stream(src.at(0) + i), acc[u]);
                } else {
                    zero8(acc[u]);
                    add8(ld_stream(src.at(0) + i), acc[u]);
                }
                for (int r = 1; r < W; ++r) add8(ld_stream(src.at(r) + i), acc[u]);
            }
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            if (BIAS != kNoBias && !BIAS_FIRST) add8(bv[u], acc[u]);
            st_stream(out + base + (int64_t)u * kThreads, pack8(acc[u]));
        }
    } else {
        // ragged last block
        for (int u = 0; u < kUnroll; ++u) {
            const int64_t i = base + (int64_t)u * kThreads;
            if (i >= nvec) break;
            float acc[8];
            u32x4 bv = {0, 0, 0, 0};
            if (BIAS != kNoBias) bv = BIAS == kFullBias ? bias[i] : bias[mod_vec(i, d_vec)];
            if (BIAS != kNoBias && BIAS_FIRST) {
                unpack8(bv, acc);
                add8(src.at(0)[i], acc);
            } else {
                zero8(acc);
                add8(src.at(0)[i], acc);
            }
            for (int r = 1; r < W; ++r) add8(src.at(r)[i], acc);
            if (BIAS != kNoBias && !BIAS_FIRST) add8(bv, acc);
            out[i] = pack8(acc);
        }
    }
    }
}

// Striped ownership: output vector j (compact) comes from input vector
//   (j / blk_v) * blk_v * W + rank * blk_v + (j % blk_v).
template <class SRC>
__global__ __launch_bounds__(kThreads) void reduce_striped_kernel(
    const SRC src, int W, int64_t share_nvec,
    const u32x4* __restrict__ bias, uint32_t blk_v, int rank, u32x4* __restrict__ out) {
    const int64_t j = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    if (j >= share_nvec) return;
    const int64_t stripe = j / blk_v;
    const int64_t i = (stripe * W + rank) * blk_v + (j - stripe * blk_v);
    float acc[8];
    zero8(acc);
    add8(ld_stream(src.at(0) + i), acc);
    for (int r = 1; r < W; ++r) add8(ld_stream(src.at(r) + i), acc);
    if (bias != nullptr) add8(ld_stream(bias + i), acc);
    st_stream(out + j, pack8(acc));
}

// Rotated-order tile reduce of the copy-engine reduce-scatter variant:
// out[v] = sum_i in[((i + rank + 1) % W) * band_v + v], optionally rounding
// the running sum to bf16 after every add.
template <bool ACC_BF16>
__global__ __launch_bounds__(kThreads) void reduce_rotated_kernel(
    const u32x4* __restrict__ in, int W, int64_t band_v, int rank, u32x4* __restrict__ out) {
    const int64_t v = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    if (v >= band_v) return;
    float acc[8];
    int cur = (rank + 1) % W;
    unpack8(ld_stream(in + cur * band_v + v), acc);
    for (int i = 1; i < W; ++i) {
        cur = cur + 1 == W ? 0 : cur + 1;
        add8(ld_stream(in + cur * band_v + v), acc);
        if (ACC_BF16) unpack8(pack8(acc), acc);
    }
    st_stream(out + v, pack8(acc));
}

// Vectors per thread per block: 4 for large inputs (most bytes in flight per workgroup), 1
// for inputs too small to give every CU such a block (more, smaller workgroups).  Measured with
// inputs that are not in any cache: from 256 blocks of 4 x 256 vectors on (one per CU) the
// larger block wins whenever the blocks fill whole rounds of 256 CUs (32 MiB input: 9.0 -> 7.9 us,
// 64 MiB: 16.0 -> 13.5 us), and loses 5 % at one and a half rounds.
static int pick_unroll(int64_t nvec) {
    if (const int u = env_switches().reduce_unroll; u == 1 || u == 2 || u == 4) return u;
    const int64_t blocks4 = (nvec + kThreads * 4 - 1) / (kThreads * 4);
    return (blocks4 >= 768 || (blocks4 >= 256 && blocks4 % 256 == 0)) ? 4 : 1;
}

template <class SRC, int WT, int BIAS, bool BF>
static void launch_reduce3(hipStream_t s, const SRC& tab, int W, int64_t nvec, const u32x4* bias,
                           uint32_t d_vec, u32x4* out) {
    const int unroll = pick_unroll(nvec);
    const int64_t per_block = (int64_t)kThreads * unroll;
    int64_t blocks = (nvec + per_block - 1) / per_block;
    const int64_t max_blocks = env_switches().reduce_blocks > 0 ? env_switches().reduce_blocks : kMaxBlocks;
    if (blocks > max_blocks) blocks = max_blocks;
    const dim3 grid((unsigned)blocks);
    if (unroll == 2)
        hipLaunchKernelGGL((reduce_kernel<SRC, WT, BIAS, BF, 2>), grid, dim3(kThreads), 0, s, tab, W, nvec, bias,
                           d_vec, out);
    else if (unroll == 4)
        hipLaunchKernelGGL((reduce_kernel<SRC, WT, BIAS, BF, 4>), grid, dim3(kThreads), 0, s, tab, W, nvec, bias,
                           d_vec, out);
    else
        hipLaunchKernelGGL((reduce_kernel<SRC, WT, BIAS, BF, 1>), grid, dim3(kThreads), 0, s, tab, W, nvec, bias,
                           d_vec, out);
}

template <class SRC, int WT, int BIAS>
static hipError_t launch_reduce2(bool bias_first, hipStream_t s, const SRC& tab, int W,
                                 int64_t nvec, const u32x4* bias, uint32_t d_vec, u32x4* out) {
    if (bias_first)
        launch_reduce3<SRC, WT, BIAS, true>(s, tab, W, nvec, bias, d_vec, out);
    else
        launch_reduce3<SRC, WT, BIAS, false>(s, tab, W, nvec, bias, d_vec, out);
    return hipGetLastError();
}

template <class SRC, int WT>
static hipError_t launch_reduce1(int mode, bool bias_first, hipStream_t s, const SRC& tab, int W,
                                 int64_t nvec, const u32x4* bias, uint32_t d_vec, u32x4* out) {
    switch (mode) {
        case kNoBias:
            // without a bias both orders are the same kernel
            return launch_reduce2<SRC, WT, kNoBias>(true, s, tab, W, nvec, bias, d_vec, out);
        case kFullBias:
            return launch_reduce2<SRC, WT, kFullBias>(bias_first, s, tab, W, nvec, bias, d_vec, out);
        default:
            return launch_reduce2<SRC, WT, kVectorBias>(bias_first, s, tab, W, nvec, bias, d_vec, out);
    }
}

}  // namespace kr

using namespace kr;

// Argument checks shared by the stacked and the pointer-table entry points; `first` is the
// stacked tensor, or the table itself.  Returns KR_OK also for numel == 0.
static int check_reduce_common(const void* first, int W, int64_t numel, const void* out) {
    if (W < 1 || W > KR_MAX_WORLD) return KR_ERR_WORLD_SIZE;
    if (numel < 0) return KR_ERR_BAD_DIM;
    if (numel % 8 != 0) return KR_ERR_NUMEL_MOD8;
    if (numel == 0) return KR_OK;
    if (first == nullptr || out == nullptr) return KR_ERR_NULL_POINTER;
    if (!aligned16(out)) return KR_ERR_ALIGNMENT;
    return KR_OK;
}

static int check_stack(const void* stack, int64_t slice_stride) {
    if (!aligned16(stack) || slice_stride % 8 != 0) return KR_ERR_ALIGNMENT;
    if (slice_stride < 0) return KR_ERR_BAD_DIM;
    return KR_OK;
}

// bias mode from the bias arguments, or a negative argument error
static int reduce_bias_mode(const void* bias, int64_t bias_numel, int64_t numel, int64_t D) {
    if (bias == nullptr) return kNoBias;
    if (!aligned16(bias)) return KR_ERR_ALIGNMENT;
    if (bias_numel == numel) return kFullBias;
    if (D > 0 && bias_numel == D && D % 8 == 0 && numel % D == 0) return kVectorBias;
    return KR_ERR_BIAS_SHAPE;
}

template <class SRC>
static int launch_reduce(const SRC& tab, int W, int64_t numel, const void* bias, int mode, int64_t D,
                         int bias_first, void* out, void* stream) {
    const int64_t nvec = numel / 8;
    const hipStream_t s = (hipStream_t)stream;
    const u32x4* bp = (const u32x4*)bias;
    u32x4* op = (u32x4*)out;
    const uint32_t d_vec = mode == kVectorBias ? (uint32_t)(D / 8) : 1u;
    hipError_t e;
    switch (W) {
        case 2: e = launch_reduce1<SRC, 2>(mode, bias_first != 0, s, tab, W, nvec, bp, d_vec, op); break;
        case 4: e = launch_reduce1<SRC, 4>(mode, bias_first != 0, s, tab, W, nvec, bp, d_vec, op); break;
        case 8: e = launch_reduce1<SRC, 8>(mode, bias_first != 0, s, tab, W, nvec, bp, d_vec, op); break;
        default: e = launch_reduce1<SRC, 0>(mode, bias_first != 0, s, tab, W, nvec, bp, d_vec, op); break;
    }
    return (int)e;
}

extern "C" int kr_reduce_bf16(const void* stack, int W, int64_t slice_stride, int64_t numel, const void* bias,
                              int64_t bias_numel, int64_t D, int bias_first, void* out, void* stream) {
    int rc = check_reduce_common(stack, W, numel, out);
    if (rc != KR_OK) return rc;
    if (numel > 0 && (rc = check_stack(stack, slice_stride)) != KR_OK) return rc;
    const int mode = reduce_bias_mode(bias, bias_numel, numel, D);
    if (mode < 0) return mode;
    if (numel == 0) return KR_OK;
    const StackedPeers src{(const u32x4*)stack, slice_stride / 8};
    return launch_reduce(src, W, numel, bias, mode, D, bias_first, out, stream);
}

extern "C" int kr_reduce_ptrs_bf16(const void* const* bufs, int W, int64_t numel, const void* bias,
                                   int64_t bias_numel, int64_t D, int bias_first, void* out, void* stream) {
    int rc = check_reduce_common(bufs, W, numel, out);
    if (rc != KR_OK) return rc;
    const int mode = reduce_bias_mode(bias, bias_numel, numel, D);
    if (mode < 0) return mode;
    if (numel == 0) return KR_OK;
    PeerTab tab;
    if ((rc = peer_tab_from_ptrs(tab, bufs, W)) != KR_OK) return rc;
    return launch_reduce(tab, W, numel, bias, mode, D, bias_first, out, stream);
}

extern "C" int64_t kr_striped_share_numel(int64_t numel, int W, int64_t stripe_block, int rank) {
    if (W < 1 || W > KR_MAX_WORLD) return KR_ERR_WORLD_SIZE;
    if (numel < 0) return KR_ERR_BAD_DIM;
    if (numel % 8 != 0) return KR_ERR_NUMEL_MOD8;
    if (stripe_block <= 0 || stripe_block % 8 != 0 || rank < 0 || rank >= W) return KR_ERR_STRIPE;
    const int64_t stripe = stripe_block * W;
    const int64_t full = numel / stripe;
    const int64_t rem = numel - full * stripe;
    int64_t tail = rem - (int64_t)rank * stripe_block;
    if (tail < 0) tail = 0;
    if (tail > stripe_block) tail = stripe_block;
    return full * stripe_block + tail;
}

template <class SRC>
static int launch_striped(const SRC& tab, int W, int64_t share, const void* bias, int64_t stripe_block,
                          int rank, void* out, void* stream) {
    if (bias != nullptr && !aligned16(bias)) return KR_ERR_ALIGNMENT;
    const int64_t nvec = share / 8;
    const int64_t blocks = (nvec + kThreads - 1) / kThreads;
    if (blocks > 0x7fffffffLL || stripe_block / 8 > 0xffffffffLL) return KR_ERR_BAD_DIM;
    hipLaunchKernelGGL(reduce_striped_kernel<SRC>, dim3((unsigned)blocks), dim3(kThreads), 0, (hipStream_t)stream, tab,
                       W, nvec, (const u32x4*)bias, (uint32_t)(stripe_block / 8), rank, (u32x4*)out);
    return (int)hipGetLastError();
}

extern "C" int kr_reduce_striped_bf16(const void* stack, int W, int64_t slice_stride, int64_t numel,
                                      const void* bias, int64_t stripe_block, int rank, void* out,
                                      void* stream) {
    const int64_t share = kr_striped_share_numel(numel, W, stripe_block, rank);
    if (share < 0) return (int)share;
    if (share == 0) return KR_OK;
    int rc = check_reduce_common(stack, W, numel, out);
    if (rc != KR_OK) return rc;
    if ((rc = check_stack(stack, slice_stride)) != KR_OK) return rc;
    const StackedPeers src{(const u32x4*)stack, slice_stride / 8};
    return launch_striped(src, W, share, bias, stripe_block, rank, out, stream);
}

extern "C" int kr_reduce_striped_ptrs_bf16(const void* const* bufs, int W, int64_t numel, const void* bias,
                                           int64_t stripe_block, int rank, void* out, void* stream) {
    const int64_t share = kr_striped_share_numel(numel, W, stripe_block, rank);
    if (share < 0) return (int)share;
    if (share == 0) return KR_OK;
    int rc = check_reduce_common(bufs, W, numel, out);
    if (rc != KR_OK) return rc;
    PeerTab tab;
    if ((rc = peer_tab_from_ptrs(tab, bufs, W)) != KR_OK) return rc;
    return launch_striped(tab, W, share, bias, stripe_block, rank, out, stream);
}

extern "C" int kr_reduce_rotated_bf16(const void* in, int W, int64_t rows, int64_t N, int rank, int acc_bf16,
                                      void* out, void* stream) {
    if (W < 1 || W > KR_MAX_WORLD) return KR_ERR_WORLD_SIZE;
    if (rows < 0 || N < 0) return KR_ERR_BAD_DIM;
    if (rank < 0 || rank >= W) return KR_ERR_STRIPE;
    const int64_t band = rows * N;
    if (band % 8 != 0) return KR_ERR_NUMEL_MOD8;
    if (band == 0) return KR_OK;
    if (in == nullptr || out == nullptr) return KR_ERR_NULL_POINTER;
    if (!aligned16(in) || !aligned16(out)) return KR_ERR_ALIGNMENT;
    const int64_t band_v = band / 8;
    const int64_t blocks = (band_v + kThreads - 1) / kThreads;
    if (blocks > 0x7fffffffLL) return KR_ERR_BAD_DIM;
    if (acc_bf16)
        hipLaunchKernelGGL((reduce_rotated_kernel<true>), dim3((unsigned)blocks), dim3(kThreads), 0,
                           (hipStream_t)stream, (const u32x4*)in, W, band_v, rank, (u32x4*)out);
    else
        hipLaunchKernelGGL((reduce_rotated_kernel<false>), dim3((unsigned)blocks), dim3(kThreads), 0,
                           (hipStream_t)stream, (const u32x4*)in, W, band_v, rank, (u32x4*)out);
    return (int)hipGetLastError();
}
