// Row kernels: W-way reduce + bias + RMSNorm in one pass, and stand-alone RMSNorm.  The W
// inputs are the slices of a stacked tensor or the entries of a pointer table (SRC, common.h).
//
// One workgroup owns one row.  The reduced row lives in fp32 registers (VPT
// 128-bit vectors per thread), so every input byte is read exactly once:
// W*D*2 B of slices (+ D*2 bias + D*2 weight) in, D*2 B out per row.  The sum
// of squares is reduced inside each wavefront with DPP lane permutes, then
// across the wavefronts of the workgroup through a few words of LDS that every
// wavefront re-reads and sums in the same way, so all threads hold the same rstd.
#include <stdlib.h>

#include "common.h"

namespace kr {

enum RowBias { kRowNoBias = 0, kRowFullBias = 1, kRowVecBias = 2 };

constexpr int kMaxVpt = 8;       // vectors per thread  -> D <= 1024 * 8 * 8
constexpr int kMaxThreads = 1024;
constexpr int64_t kLatRows = 1024;  // at most this many rows: latency-first kernel

// LAT (few rows: the kernel's time is one workgroup's latency): every load of the thread --
// weights, bias, the W inputs -- is issued before the first is consumed and none sits under a
// branch (a lane past the end of the row re-reads the row's last vector and is masked), so the
// row costs one memory round trip instead of three.
template <class SRC, int VPT, int WT, int BIAS, bool LAT = false>
__global__ __launch_bounds__(kMaxThreads) void reduce_rmsnorm_kernel(
    const SRC src, int w_rt, int d_vec,
    const u32x4* __restrict__ bias, const u32x4* __restrict__ wgt, float eps, float inv_d,
    u32x4* __restrict__ y) {
    __shared__ float wave_part[kMaxThreads / kWave];
    const int W = WT > 0 ? WT : w_rt;
    const int tid = threadIdx.x;
    const int nthr = blockDim.x;
    const int64_t row_v = (int64_t)blockIdx.x * d_vec;

    float s[VPT][8];
    u32x4 wv[VPT];

    // issue the weight loads early (they are shared by all rows and stay in L2); rows long
    // enough to need 4+ vectors per thread fetch them after the reduction instead, to stay
    // inside the 128 registers a 1024-thread workgroup leaves per thread
    constexpr bool kEarlyWeights = VPT < 4;
    constexpr bool kLatPath = LAT && WT > 0 && WT * VPT <= 16 && VPT == 1;
    if constexpr (kLatPath) {
        u32x4 bv[VPT];
        u32x4 x[WT][VPT];
#pragma unroll
        for (int v = 0; v < VPT; ++v) {
            const int cc = min(tid + v * nthr, d_vec - 1);
            wv[v] = wgt[cc];
            if (BIAS == kRowFullBias) bv[v] = ld_stream(bias + row_v + cc);
            else if (BIAS == kRowVecBias) bv[v] = bias[cc];
        }
#pragma unroll
        for (int r = 0; r < WT; ++r)
#pragma unroll
            for (int v = 0; v < VPT; ++v) x[r][v] = ld_stream(src.at(r) + row_v + min(tid + v * nthr, d_vec - 1));
#pragma unroll
        for (int v = 0; v < VPT; ++v) {
            if (BIAS == kRowNoBias) zero8(s[v]);
            else unpack8(bv[v], s[v]);
#pragma unroll
            for (int r = 0; r < WT; ++r) add8(x[r][v], s[v]);
            const bool live = tid + v * nthr < d_vec;
#pragma unroll
            for (int j = 0; j < 8; ++j) s[v][j] = live ? s[v][j] : 0.0f;
        }
    } else {
    if (kEarlyWeights) {
#pragma unroll
        for (int v = 0; v < VPT; ++v) {
            const int c = tid + v * nthr;
            wv[v] = c < d_vec ? wgt[c] : u32x4{0, 0, 0, 0};
        }
    }

#pragma unroll
    for (int v = 0; v < VPT; ++v) {
        const int c = tid + v * nthr;
        if (BIAS == kRowNoBias || c >= d_vec) {
            zero8(s[v]);
        } else if (BIAS == kRowFullBias) {
            unpack8(ld_stream(bias + row_v + c), s[v]);
        } else {
            unpack8(bias[c], s[v]);
        }
    }

    if constexpr (WT > 0 && WT * VPT <= 16 && VPT < 4) {
        // all W*VPT loads of the thread in flight before the first add
        u32x4 x[WT][VPT];
#pragma unroll
        for (int r = 0; r < WT; ++r)
#pragma unroll
            for (int v = 0; v < VPT; ++v) {
                const int c = tid + v * nthr;
                x[r][v] = c < d_vec ? ld_stream(src.at(r) + row_v + c) : u32x4{0, 0, 0, 0};
            }
#pragma unroll
        for (int r = 0; r < WT; ++r)
#pragma unroll
            for (int v = 0; v < VPT; ++v) add8(x[r][v], s[v]);
    } else {
        // long rows (or run-time W): G slices at a time, G * VPT <= 16 loads in flight per thread
        constexpr int G = VPT >= 4 ? 8 / VPT : 16 / VPT;   // long rows keep 64 row registers: fewer loads in flight
#pragma unroll 1
        for (int r0 = 0; r0 < W; r0 += G) {
            u32x4 x[G][VPT];
#pragma unroll
            for (int gi = 0; gi < G; ++gi)
#pragma unroll
                for (int v = 0; v < VPT; ++v) {
                    const int c = tid + v * nthr;
                    x[gi][v] = (r0 + gi < W && c < d_vec)
                                   ? ld_stream(src.at(r0 + gi) + row_v + c)
                                   : u32x4{0, 0, 0, 0};
                }
#pragma unroll
            for (int gi = 0; gi < G; ++gi)
#pragma unroll
                for (int v = 0; v < VPT; ++v) add8(x[gi][v], s[v]);
        }
    }

    }   // !kLatPath

    float ss = 0.0f;
#pragma unroll
    for (int v = 0; v < VPT; ++v)
#pragma unroll
        for (int j = 0; j < 8; ++j) ss += s[v][j] * s[v][j];

    ss = wave_sum(ss);
    const int nwaves = nthr / kWave;
    float total = ss;
    if (nwaves > 1) {
        if ((tid & (kWave - 1)) == 0) wave_part[tid / kWave] = ss;
        __syncthreads();
        // lane i of every wave fetches wave i's part (one LDS read instead of nwaves in a row)
        // and the wave sums them the same way: all threads hold the same total
        const int l = tid & (kWave - 1);
        total = wave_sum(l < nwaves ? wave_part[l] : 0.0f);
    }
    const float rstd = __builtin_amdgcn_rsqf(total * inv_d + eps);

#pragma unroll
    for (int v = 0; v < VPT; ++v) {
        const int c = tid + v * nthr;
        if (c < d_vec) {
            float wf[8], o[8];
            unpack8(kEarlyWeights ? wv[v] : wgt[c], wf);
#pragma unroll
            for (int j = 0; j < 8; ++j) o[j] = (s[v][j] * rstd) * wf[j];
            st_stream(y + row_v + c, pack8(o));
        }
    }
}

template <class SRC, int VPT, int WT, bool LAT>
static hipError_t launch_row2(int mode, dim3 grid, dim3 block, hipStream_t st, const SRC& tab, int W,
                              int d_vec, const u32x4* bias, const u32x4* wgt, float eps,
                              float inv_d, u32x4* y) {
    switch (mode) {
        case kRowNoBias:
            hipLaunchKernelGGL((reduce_rmsnorm_kernel<SRC, VPT, WT, kRowNoBias, LAT>), grid, block, 0, st, tab, W,
                               d_vec, bias, wgt, eps, inv_d, y);
            break;
        case kRowFullBias:
            hipLaunchKernelGGL((reduce_rmsnorm_kernel<SRC, VPT, WT, kRowFullBias, LAT>), grid, block, 0, st, tab, W,
                               d_vec, bias, wgt, eps, inv_d, y);
            break;
        default:
            hipLaunchKernelGGL((reduce_rmsnorm_kernel<SRC, VPT, WT, kRowVecBias, LAT>), grid, block, 0, st, tab, W,
                               d_vec, bias, wgt, eps, inv_d, y);
            break;
    }
    return hipGetLastError();
}

template <class SRC, int VPT, bool LAT>
static hipError_t launch_row1(int W, int mode, dim3 grid, dim3 block, hipStream_t st, const SRC& tab,
                              int d_vec, const u32x4* bias, const u32x4* wgt, float eps,
                              float inv_d, u32x4* y) {
    switch (W) {
        case 1: return launch_row2<SRC, VPT, 1, LAT>(mode, grid, block, st, tab, W, d_vec, bias, wgt, eps, inv_d, y);
        case 2: return launch_row2<SRC, VPT, 2, LAT>(mode, grid, block, st, tab, W, d_vec, bias, wgt, eps, inv_d, y);
        case 4: return launch_row2<SRC, VPT, 4, LAT>(mode, grid, block, st, tab, W, d_vec, bias, wgt, eps, inv_d, y);
        case 8: return launch_row2<SRC, VPT, 8, LAT>(mode, grid, block, st, tab, W, d_vec, bias, wgt, eps, inv_d, y);
        default: return launch_row2<SRC, VPT, 0, LAT>(mode, grid, block, st, tab, W, d_vec, bias, wgt, eps, inv_d, y);
    }
}

// Threads per row: enough 64-lane wavefronts to give every thread at most
// `vpt` vectors, capped at 1024 threads.
static void row_geometry(int d_vec, int* threads, int* vpt) {
    int v = 1;
    while ((int64_t)v * kMaxThreads < d_vec) v *= 2;           // 1,2,4,8
    // (one vector per thread measured best: 78 % of HBM peak at D = 4096/8192 against 75-77 %
    // with two; more wavefronts per row cost less than fewer loads in flight per thread)
    // KRAKEN_AMD_ROW_VPT=1|2|4|8 overrides the vectors per thread (tuning); ignored if a row
    // would need more than 1024 threads
    if (const char* e = getenv("KRAKEN_AMD_ROW_VPT")) {
        const int o = atoi(e);
        if ((o == 1 || o == 2 || o == 4 || o == 8) && (int64_t)o * kMaxThreads >= d_vec) v = o;
    }
    int t = (d_vec + v - 1) / v;
    t = (t + kWave - 1) / kWave * kWave;
    *threads = t;
    *vpt = v;
}

template <class SRC>
static int launch_rows(const SRC& tab, int W, int64_t rows, int64_t D, const void* bias,
                       int mode, const void* w, float eps, void* y, void* stream) {
    int threads, vpt;
    const int d_vec = (int)(D / 8);
    row_geometry(d_vec, &threads, &vpt);
    // few rows of at most 8192 elements: one workgroup's latency is the kernel's time, and the
    // latency-first instantiation is 9 % faster at [256, 4096], 2.5 % at [16, 8192]; with many
    // rows it is level or up to 2 % slower (KRAKEN_AMD_ROW_LAT=0|1 overrides, for tuning)
    bool lat = rows <= kLatRows;
    if (const char* e = getenv("KRAKEN_AMD_ROW_LAT")) lat = e[0] == '1';
    const dim3 grid((unsigned)rows), block((unsigned)threads);
    const hipStream_t st = (hipStream_t)stream;
    const u32x4* bp = (const u32x4*)bias;
    const u32x4* wp = (const u32x4*)w;
    u32x4* yp = (u32x4*)y;
    const float inv_d = 1.0f / (float)D;
    hipError_t e;
    switch (vpt) {
        case 1:
            e = lat ? launch_row1<SRC, 1, true>(W, mode, grid, block, st, tab, d_vec, bp, wp, eps, inv_d, yp)
                    : launch_row1<SRC, 1, false>(W, mode, grid, block, st, tab, d_vec, bp, wp, eps, inv_d, yp);
            break;
        case 2: e = launch_row1<SRC, 2, false>(W, mode, grid, block, st, tab, d_vec, bp, wp, eps, inv_d, yp); break;
        case 4: e = launch_row1<SRC, 4, false>(W, mode, grid, block, st, tab, d_vec, bp, wp, eps, inv_d, yp); break;
        default: e = launch_row1<SRC, 8, false>(W, mode, grid, block, st, tab, d_vec, bp, wp, eps, inv_d, yp); break;
    }
    return (int)e;
}

}  // namespace kr

using namespace kr;

// Argument checks shared by the row entry points (everything but the input buffers).
// Returns KR_OK also for rows == 0.
static int check_rows(int W, int64_t rows, int64_t D, const void* bias, const void* w, const void* y) {
    if (W < 1 || W > KR_MAX_WORLD) return KR_ERR_WORLD_SIZE;
    if (rows < 0 || D <= 0) return KR_ERR_BAD_DIM;
    if (D % 8 != 0) return KR_ERR_NUMEL_MOD8;
    if (D > KR_MAX_ROW) return KR_ERR_ROW_TOO_LONG;
    if (rows > 0x7fffffffLL) return KR_ERR_BAD_DIM;
    if (rows == 0) return KR_OK;
    if (w == nullptr || y == nullptr) return KR_ERR_NULL_POINTER;
    if (!aligned16(w) || !aligned16(y)) return KR_ERR_ALIGNMENT;
    if (bias != nullptr && !aligned16(bias)) return KR_ERR_ALIGNMENT;
    return KR_OK;
}

extern "C" int kr_reduce_rmsnorm_bf16(const void* stack, int W, int64_t slice_stride, int64_t rows, int64_t D,
                                      const void* bias, int bias_is_vector, const void* w, float eps, void* y,
                                      void* stream) {
    if (W >= 1 && W <= KR_MAX_WORLD && slice_stride < 0) return KR_ERR_BAD_DIM;
    int rc = check_rows(W, rows, D, bias, w, y);
    if (rc != KR_OK || rows == 0) return rc;
    if (stack == nullptr) return KR_ERR_NULL_POINTER;
    if (!aligned16(stack) || slice_stride % 8 != 0) return KR_ERR_ALIGNMENT;
    const int mode = bias == nullptr ? kRowNoBias : (bias_is_vector ? kRowVecBias : kRowFullBias);
    const StackedPeers src{(const u32x4*)stack, slice_stride / 8};
    return launch_rows(src, W, rows, D, bias, mode, w, eps, y, stream);
}

extern "C" int kr_reduce_rmsnorm_ptrs_bf16(const void* const* bufs, int W, int64_t rows, int64_t D,
                                           const void* bias, int bias_is_vector, const void* w, float eps,
                                           void* y, void* stream) {
    int rc = check_rows(W, rows, D, bias, w, y);
    if (rc != KR_OK || rows == 0) return rc;
    PeerTab tab;
    if ((rc = peer_tab_from_ptrs(tab, bufs, W)) != KR_OK) return rc;
    const int mode = bias == nullptr ? kRowNoBias : (bias_is_vector ? kRowVecBias : kRowFullBias);
    return launch_rows(tab, W, rows, D, bias, mode, w, eps, y, stream);
}

extern "C" int kr_rmsnorm_bf16(const void* x, const void* w, float eps, int64_t rows, int64_t D, void* y,
                               void* stream) {
    int rc = check_rows(1, rows, D, nullptr, w, y);
    if (rc != KR_OK || rows == 0) return rc;
    if (x == nullptr) return KR_ERR_NULL_POINTER;
    if (!aligned16(x)) return KR_ERR_ALIGNMENT;
    const StackedPeers src{(const u32x4*)x, 0};
    return launch_rows(src, 1, rows, D, nullptr, kRowNoBias, w, eps, y, stream);
}
