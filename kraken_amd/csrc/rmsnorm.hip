// Row kernels: W-way reduce + bias + RMSNorm in one pass, and stand-alone RMSNorm.  The W
// inputs are the slices of a stacked tensor or the entries of a pointer table (SRC, common.h).
//
// One workgroup owns one row.  The reduced row lives in fp32 registers (VPT
// 128-bit vectors per thread), so every input byte is read exactly once:
// W*D*2 B of slices (+ D*2 bias + D*2 weight) in, D*2 B out per row.  The sum
// of squares is reduced inside each wavefront with DPP lane permutes, then
// across the wavefronts of the workgroup through a few words of LDS that every
// wavefront re-reads and sums in the same way, so all threads hold the same rstd.
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

// ---- few long rows: one row on many compute units --------------------------------------------
// One compute unit takes in about 55 GB/s, so a workgroup that owns a row of W * D * 2 bytes
// needs W * D * 2 / 55e9 s however few rows there are (16 rows of 8 x 8192: 2.4 us of a 4.9 us
// kernel on 16 of 256 compute units).  Here a row is cut into pieces of 64 vectors, one
// wavefront (its own workgroup, any compute unit) each.  The wavefronts of a row meet in a
// block of the caller's workspace: wavefront i stores {tag, its partial sum of squares} to slot i
// with one 8-byte store, polls the row's slots until all carry the tag, and adds the partial sums
// in slot order -- every wavefront of the row forms the same total in the same order, and the
// result does not depend on who arrives when.  The tag is the row's generation + 1, read from the
// block at the start of the kernel; wavefront 0 stores it back as the new generation once it has
// seen every slot carry it (by then every wavefront of the row has read the old one).  No
// read-modify-write, no reset, nothing to clear between calls: a slot left by an earlier call
// carries a tag at or below the generation and never matches.  The accesses are relaxed atomics at
// agent scope (they are served by the memory side, about 1 us a round trip, which is the price
// of the exchange).  All wavefronts of a row are resident together (the grid is at most
// kSplitMaxWaves one-wave workgroups, dispatched in order), so the poll ends; it is bounded all
// the same: after kSplitSpinLimit polls (seconds) the wavefront gives up and its piece of the row
// is written as NaN (and 1 + row goes to the caller's status word).  After such a time-out the
// workspace is no longer consistent -- a wavefront of the failed call that starts after wavefront 0
// gave up reads the new generation and leaves a slot that the next call takes for a fresh one -- so
// it must be zeroed before it is used again.  Tags are 32 bits: a slot left by an earlier call could only be mistaken for
// a fresh one if exactly 2^32 calls on the workspace lay between two uses of that slot.
constexpr int kSplitSlots = 64;                       // wavefronts per row at most -> D <= 32768
constexpr int kSplitMaxRows = 64;
constexpr int kSplitMaxWaves = 1024;
constexpr int kSplitBlockWords = 16 + kSplitSlots;    // 8-byte words per row: generation (+ padding to 128 B), slots
constexpr int64_t kSplitWorkspaceBytes = (int64_t)kSplitMaxRows * kSplitBlockWords * 8;
constexpr int kSplitSpinLimit = 1 << 22;

template <class SRC, int WT, int BIAS>
__global__ __launch_bounds__(kWave) void reduce_rmsnorm_split_kernel(
    const SRC src, int d_vec, int nw,
    const u32x4* __restrict__ bias, const u32x4* __restrict__ wgt, float eps, float inv_d,
    u32x4* __restrict__ y, uint64_t* __restrict__ ws, int* __restrict__ status) {
    const int row = blockIdx.x / nw;
    const int piece = blockIdx.x - row * nw;
    const int lane = threadIdx.x;
    const int c = piece * kWave + lane;
    const int cc = min(c, d_vec - 1);
    const int64_t row_v = (int64_t)row * d_vec;
    uint64_t* block = ws + (int64_t)row * kSplitBlockWords;
    uint64_t* slots = block + 16;

    // every load of the wavefront is issued before the first is used
    u32x4 x[WT];
#pragma unroll
    for (int r = 0; r < WT; ++r) x[r] = ld_stream(src.at(r) + row_v + cc);
    u32x4 bv = {0, 0, 0, 0};
    if (BIAS == kRowFullBias) bv = ld_stream(bias + row_v + cc);
    else if (BIAS == kRowVecBias) bv = bias[cc];
    const u32x4 wv = wgt[cc];
    const uint32_t tag = (uint32_t)__hip_atomic_load(block, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1u;

    float s[8];
    if (BIAS == kRowNoBias) zero8(s);
    else unpack8(bv, s);
#pragma unroll
    for (int r = 0; r < WT; ++r) add8(x[r], s);
    float ss = 0.0f;
    if (c < d_vec) {
#pragma unroll
        for (int j = 0; j < 8; ++j) ss += s[j] * s[j];
    }
    ss = wave_sum(ss);

    if (lane == 0)
        __hip_atomic_store(slots + piece, ((uint64_t)tag << 32) | __builtin_bit_cast(uint32_t, ss), __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
    uint64_t v = (uint64_t)tag << 32;
    bool met = false;
    for (int spin = 0; spin < kSplitSpinLimit && !met; ++spin) {
        if (lane < nw) v = __hip_atomic_load(slots + lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        met = __all((uint32_t)(v >> 32) == tag);
        if (!met) __builtin_amdgcn_s_sleep(1);
    }
    if (piece == 0 && lane == 0)
        __hip_atomic_store(block, (uint64_t)tag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    float total = 0.0f;
    const int part = (int)(uint32_t)v;
    for (int k = 0; k < nw; ++k) total += __builtin_bit_cast(float, __builtin_amdgcn_readlane(part, k));
    // a row whose wavefronts did not meet within the bound comes out as NaN, not as a plausible wrong
    // value, and the caller's status word (if any) names it
    const float rstd = met ? __builtin_amdgcn_rsqf(total * inv_d + eps) : __builtin_nanf("");
    if (!met && status != nullptr && lane == 0) __hip_atomic_store(status, 1 + row, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);

    if (c < d_vec) {
        float wf[8], o[8];
        unpack8(wv, wf);
#pragma unroll
        for (int j = 0; j < 8; ++j) o[j] = (s[j] * rstd) * wf[j];
        st_stream(y + row_v + c, pack8(o));
    }
}

// Whether a call takes the split kernel (given a workspace).  Measured against one workgroup per
// row with W = 8, inputs from HBM, rows = 1..64: D = 8192 wins up to 32 rows (1 row 4.0 -> 3.4 us,
// 16 rows 5.0 -> 4.0 us, 32 rows 5.1 -> 5.0 us; 64 rows lose, 5.4 -> 6.4 us), D = 16384 up to 32 rows
// (7.7 -> 6.0 us at 16), D = 32768 up to 16 rows (13.3 -> 9.4 us); D = 5120 is level and D <= 4096
// loses 0.1 - 0.8 us: the exchange costs about 1.2 us, which a row of less than ~96 KiB does not
// win back.
static bool row_split_pays(int W, int64_t rows, int64_t D) {
    if (!(W == 1 || W == 2 || W == 4 || W == 8)) return false;
    const int64_t d_vec = D / 8;
    const int64_t nw = (d_vec + kWave - 1) / kWave;
    if (rows < 1 || rows > kSplitMaxRows || nw < 2 || nw > kSplitSlots || rows * nw > kSplitMaxWaves) return false;
    if (env_switches().row_split >= 0) return env_switches().row_split != 0;
    const int64_t row_bytes = (int64_t)W * D * 2;
    return row_bytes >= 96 * 1024 && rows * nw <= (row_bytes >= 256 * 1024 ? 1024 : 512);
}

template <class SRC, int WT>
static hipError_t launch_split2(int mode, dim3 grid, hipStream_t st, const SRC& tab, int d_vec, int nw,
                                const u32x4* bias, const u32x4* wgt, float eps, float inv_d, u32x4* y, uint64_t* ws, int* status) {
    switch (mode) {
        case kRowNoBias:
            hipLaunchKernelGGL((reduce_rmsnorm_split_kernel<SRC, WT, kRowNoBias>), grid, dim3(kWave), 0, st, tab, d_vec,
                               nw, bias, wgt, eps, inv_d, y, ws, status);
            break;
        case kRowFullBias:
            hipLaunchKernelGGL((reduce_rmsnorm_split_kernel<SRC, WT, kRowFullBias>), grid, dim3(kWave), 0, st, tab, d_vec,
                               nw, bias, wgt, eps, inv_d, y, ws, status);
            break;
        default:
            hipLaunchKernelGGL((reduce_rmsnorm_split_kernel<SRC, WT, kRowVecBias>), grid, dim3(kWave), 0, st, tab, d_vec,
                               nw, bias, wgt, eps, inv_d, y, ws, status);
            break;
    }
    return hipGetLastError();
}

template <class SRC>
static int launch_split(const SRC& tab, int W, int64_t rows, int64_t D, const void* bias, int mode, const void* w,
                        float eps, void* y, void* workspace, int* status, void* stream) {
    const int d_vec = (int)(D / 8);
    const int nw = (d_vec + kWave - 1) / kWave;
    const dim3 grid((unsigned)(rows * nw));
    const hipStream_t st = (hipStream_t)stream;
    const u32x4* bp = (const u32x4*)bias;
    const u32x4* wp = (const u32x4*)w;
    const float inv_d = 1.0f / (float)D;
    switch (W) {
        case 1: return (int)launch_split2<SRC, 1>(mode, grid, st, tab, d_vec, nw, bp, wp, eps, inv_d, (u32x4*)y, (uint64_t*)workspace, status);
        case 2: return (int)launch_split2<SRC, 2>(mode, grid, st, tab, d_vec, nw, bp, wp, eps, inv_d, (u32x4*)y, (uint64_t*)workspace, status);
        case 4: return (int)launch_split2<SRC, 4>(mode, grid, st, tab, d_vec, nw, bp, wp, eps, inv_d, (u32x4*)y, (uint64_t*)workspace, status);
        default: return (int)launch_split2<SRC, 8>(mode, grid, st, tab, d_vec, nw, bp, wp, eps, inv_d, (u32x4*)y, (uint64_t*)workspace, status);
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
    if (const int o = env_switches().row_vpt; (o == 1 || o == 2 || o == 4 || o == 8) && (int64_t)o * kMaxThreads >= d_vec)
        v = o;
    int t = (d_vec + v - 1) / v;
    t = (t + kWave - 1) / kWave * kWave;
    *threads = t;
    *vpt = v;
}

template <class SRC>
static int launch_rows(const SRC& tab, int W, int64_t rows, int64_t D, const void* bias,
                       int mode, const void* w, float eps, void* y, void* stream,
                       void* workspace = nullptr, int64_t workspace_bytes = 0, int* status = nullptr) {
    if (workspace != nullptr && workspace_bytes >= kSplitWorkspaceBytes && row_split_pays(W, rows, D))
        return launch_split(tab, W, rows, D, bias, mode, w, eps, y, workspace, status, stream);
    int threads, vpt;
    const int d_vec = (int)(D / 8);
    row_geometry(d_vec, &threads, &vpt);
    // few rows of at most 8192 elements: one workgroup's latency is the kernel's time, and the
    // latency-first instantiation is 9 % faster at [256, 4096], 2.5 % at [16, 8192]; with many
    // rows it is level or up to 2 % slower (KRAKEN_AMD_ROW_LAT=0|1 overrides, for tuning)
    bool lat = rows <= kLatRows;
    if (env_switches().row_lat >= 0) lat = env_switches().row_lat == 1;
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

extern "C" int64_t kr_rmsnorm_workspace_bytes(int W, int64_t rows, int64_t D) {
    if (D <= 0 || D % 8 != 0) return 0;
    return row_split_pays(W, rows, D) ? kSplitWorkspaceBytes : 0;
}

extern "C" int kr_reduce_rmsnorm_ws_bf16(const void* stack, int W, int64_t slice_stride, int64_t rows, int64_t D,
                                         const void* bias, int bias_is_vector, const void* w, float eps, void* y,
                                         void* workspace, int64_t workspace_bytes, int32_t* status, void* stream) {
    if (W >= 1 && W <= KR_MAX_WORLD && slice_stride < 0) return KR_ERR_BAD_DIM;
    int rc = check_rows(W, rows, D, bias, w, y);
    if (rc != KR_OK || rows == 0) return rc;
    if (stack == nullptr) return KR_ERR_NULL_POINTER;
    if (!aligned16(stack) || slice_stride % 8 != 0 || !aligned16(workspace)) return KR_ERR_ALIGNMENT;
    if ((reinterpret_cast<uintptr_t>(status) & 3u) != 0) return KR_ERR_ALIGNMENT;
    const int mode = bias == nullptr ? kRowNoBias : (bias_is_vector ? kRowVecBias : kRowFullBias);
    const StackedPeers src{(const u32x4*)stack, slice_stride / 8};
    return launch_rows(src, W, rows, D, bias, mode, w, eps, y, stream, workspace, workspace_bytes, status);
}

extern "C" int kr_reduce_rmsnorm_bf16(const void* stack, int W, int64_t slice_stride, int64_t rows, int64_t D,
                                      const void* bias, int bias_is_vector, const void* w, float eps, void* y,
                                      void* stream) {
    return kr_reduce_rmsnorm_ws_bf16(stack, W, slice_stride, rows, D, bias, bias_is_vector, w, eps, y, nullptr, 0,
                                     nullptr, stream);
}

extern "C" int kr_reduce_rmsnorm_ptrs_ws_bf16(const void* const* bufs, int W, int64_t rows, int64_t D,
                                              const void* bias, int bias_is_vector, const void* w, float eps,
                                              void* y, void* workspace, int64_t workspace_bytes, int32_t* status,
                                              void* stream) {
    int rc = check_rows(W, rows, D, bias, w, y);
    if (rc != KR_OK || rows == 0) return rc;
    PeerTab tab;
    if ((rc = peer_tab_from_ptrs(tab, bufs, W)) != KR_OK) return rc;
    if (!aligned16(workspace) || (reinterpret_cast<uintptr_t>(status) & 3u) != 0) return KR_ERR_ALIGNMENT;
    const int mode = bias == nullptr ? kRowNoBias : (bias_is_vector ? kRowVecBias : kRowFullBias);
    return launch_rows(tab, W, rows, D, bias, mode, w, eps, y, stream, workspace, workspace_bytes, status);
}

extern "C" int kr_reduce_rmsnorm_ptrs_bf16(const void* const* bufs, int W, int64_t rows, int64_t D,
                                           const void* bias, int bias_is_vector, const void* w, float eps,
                                           void* y, void* stream) {
    return kr_reduce_rmsnorm_ptrs_ws_bf16(bufs, W, rows, D, bias, bias_is_vector, w, eps, y, nullptr, 0, nullptr, stream);
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
