// Pieces shared by the GEMM kernels: argument block, tile schedule, fused epilogue.
#pragma once

#include <atomic>
#include <type_traits>

#include "common.h"

namespace kr {

struct GemmArgs {
    const uint16_t* A;
    const uint16_t* B;
    int64_t lda;   // elements between rows of A (k is contiguous)
    int64_t ldb;   // NT: elements between n-rows of B^T; NN: elements between k-rows of B
    int M, N, K;
    PeerTab peer;        // peer.p[j]: partial sums of peer j, [band_rows, N] bf16 (j < n_peers)
    int n_peers;
    const uint16_t* bias;
    int band_row0, band_rows;
    uint16_t* c_full;
    void* out;
    int out_is_fp32;
    int out_fp8;       // fp8 kernel only: the result is fp8 (e4m3fn), [M, N] bytes
    int pivot_tiles;   // rotation of the M-tile order
    int tiles_m, tiles_n;
    // all-gather matmul with arrival flags (progress == nullptr: A is complete, nothing waits)
    const uint32_t* progress;   // progress[b] == 1 once rows [b*comm_rows, (b+1)*comm_rows) of A have arrived
    int comm_rows;
    const uint16_t* a_local;    // this rank's own shard, rows [local_row0, local_row0+local_rows) of A: never waits
    int64_t lda_local;
    int local_row0, local_rows;
    uint64_t wait_ticks;        // bound of one tile's wait, in ticks of the 100 MHz constant clock
    int* status;                // set to 1 + block index by a tile whose wait ran out (may be nullptr)
    // split K loop of the 128x128 kernel (k_splits == 1: off)
    int k_splits;               // workgroups per tile, each with its share of the k-steps (grid y)
    int64_t split_out_stride;   // elements between the fp32 outputs of consecutive splits (0: one output)
    // 256x256 kernel, split of the last partial round of tiles (tail_tiles == 0: off): the main
    // launch runs the first tiles_m*tiles_n - tail_tiles tiles of the schedule, a second launch
    // the remaining ones with k_splits workgroups per tile, a third sums the parts
    int tail_tiles;
    int group_n;         // column panels per scheduling group (tile_schedule)
    int peers_on_mfma;   // 256x256 kernel: add whole-band tiles' peers through the matrix cores
    int mi16;            // 256x256 kernel: k loop and peer phase on 16x16x32 MFMA blocks
    int n224;            // 256x224 tiles (tiles_n counts them): plain product, transposed-contiguous B, whole rounds
    // producer of the copy-engine reduce-scatter (band_counter == nullptr: off): finished tiles are
    // counted per destination rank, whose band is count_rows rows of C
    uint32_t* band_counter;   // [M / count_rows] tiles finished that touch the band
    uint32_t* band_signal;    // [M / count_rows] set to 1 by the workgroup that finishes the band's last tile
    int count_rows;
};

// Opt a kernel into more than 64 KiB of dynamic LDS, once per device: the attribute belongs to the
// current device's copy of the code.  `done`: the call site's own bit mask of devices.
inline hipError_t lds_opt_in(const void* fn, int bytes, std::atomic<uint64_t>& done) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    const uint64_t bit = 1ull << (dev & 63);
    if (done.load(std::memory_order_acquire) & bit) return hipSuccess;
    e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e != hipSuccess) return e;
    done.fetch_or(bit, std::memory_order_release);
    return hipSuccess;
}

// LDS-DMA kernel for shapes the 256x256 tile divides (gemm_dtl.hip)
bool gemm_dtl_supported(const GemmArgs& g);
hipError_t launch_gemm_dtl(const GemmArgs& g, bool b_nt, hipStream_t st, void* workspace);
hipError_t launch_gemm_dtl8(const GemmArgs& g, hipStream_t st);   // fp8 operands (gemm_dtl.hip)

constexpr int kXcds = 8;

// A operand of the tile that starts at row m0 (bm rows), for the all-gather matmul: rows arrive
// in blocks of g.comm_rows while the kernel runs, each block's flag in g.progress set to 1 by a
// stream-ordered write behind its copy (kraken/fused/all_gather_matmul.py:95-110: a tile of
// the local shard reads the shard itself, any other tile waits for its block's flag).  Called by
// every wave of the workgroup: each polls the flags of the blocks the tile covers with
// device-scope loads and a short sleep, then an acquire fence orders its own loads behind the
// flag (so no workgroup barrier is needed); the wait is bounded (g.wait_ticks): a tile whose flag does not come records
// 1 + block in g.status and goes on (its result is then meaningless), and later tiles see
// the status and do not wait at all, so the grid always drains.
__device__ __forceinline__ void gathered_a_tile(const GemmArgs& g, int m0, int bm, const uint16_t*& a_tile,
                                                int64_t& lda) {
    a_tile = g.A + (int64_t)m0 * g.lda;
    lda = g.lda;
    if (g.progress == nullptr) return;
    const int m1 = min(m0 + bm, g.M);
    if (g.a_local != nullptr && m0 >= g.local_row0 && m1 <= g.local_row0 + g.local_rows) {
        a_tile = g.a_local + (int64_t)(m0 - g.local_row0) * g.lda_local;
        lda = g.lda_local;
        return;
    }
    const int b_hi = (m1 - 1) / g.comm_rows;
    const uint64_t t0 = __builtin_amdgcn_s_memrealtime();
    bool give_up = g.status != nullptr && __hip_atomic_load(g.status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0;
    for (int b = m0 / g.comm_rows; b <= b_hi && !give_up; ++b) {
        while (__hip_atomic_load(g.progress + b, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 1u) {
            if (__builtin_amdgcn_s_memrealtime() - t0 > g.wait_ticks) {
                give_up = true;
                if (g.status != nullptr) __hip_atomic_store(g.status, b + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                break;
            }
            __builtin_amdgcn_s_sleep(16);
        }
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
}

// a value every lane of the wave holds, moved to scalar registers
__device__ __forceinline__ int64_t wave_uniform(int64_t v) {
    const uint32_t lo = __builtin_amdgcn_readfirstlane((int)(uint32_t)v);
    const uint32_t hi = __builtin_amdgcn_readfirstlane((int)(uint32_t)((uint64_t)v >> 32));
    return (int64_t)(((uint64_t)hi << 32) | lo);
}

// Position in the tile order of workgroup `wg` of a launch over the first `count` tiles.
// Workgroups are dealt round-robin to the 8 XCDs (each with its own L2), so workgroup ids are
// re-numbered to give every XCD a contiguous range of the order: XCD x owns positions
// [x * ntiles/8, (x+1) * ntiles/8) and a launch over fewer tiles takes the first count/8 of each
// range (`first` skips positions an earlier launch has taken).
__device__ __forceinline__ int schedule_position(const GemmArgs& g, int wg, int first = 0) {
    const int ntiles = g.tiles_m * g.tiles_n;
    if (ntiles % kXcds != 0 || first % kXcds != 0) return first + wg;
    return (wg % kXcds) * (ntiles / kXcds) + first / kXcds + wg / kXcds;
}

// Map a position in the tile order to its tile (tile_m, tile_n).
__device__ __forceinline__ void tile_schedule(const GemmArgs& g, int pid, int& tile_m_out, int& tile_n_out) {
    // ---- tile schedule -------------------------------------------------------------------
    // Tiles are ordered in groups of g.group_n column panels, M fastest in steps of g.group_n
    // columns: the ~32 tiles an XCD runs at a time form a (32 / group_n) x group_n block that
    // shares its A and B panels through the XCD's L2 (a dozen panels for 32 tiles), and every
    // XCD works on all row bands -- the rows of the reduce band (whose tiles also stream the
    // peers' partial sums) are spread over all XCDs instead of landing on one.  The M order is
    // rotated by the pivot, so the band's (or the local shard's) tiles are the first ones of
    // every XCD.
    const int per_group = g.group_n * g.tiles_m;
    const int group = pid / per_group;
    const int first_n = group * g.group_n;
    const int gsz = min(g.tiles_n - first_n, g.group_n);
    const int tile_n = first_n + (pid % per_group) % gsz;
    int tile_m = (pid % per_group) / gsz;
    tile_m += g.pivot_tiles;
    if (tile_m >= g.tiles_m) tile_m -= g.tiles_m;
    tile_m_out = tile_m;
    tile_n_out = tile_n;
}

// Fused epilogue of one workgroup tile.  `acc` are this wave's 32x32 MFMA accumulators (TM x TN
// blocks) in the TRANSPOSED layout the kernels produce by passing the B fragment as the first
// MFMA operand: lane holds row (lane & 31) of the block, register v is column
// 8*(v/4) + 4*(lane>>5) + v%4 -- four consecutive columns per register quad, so a quad is one
// contiguous store into a row-major LDS patch.  `smem` is the workgroup's LDS (free for reuse:
// every wave has passed a barrier after its last read of the operand stages).
//
// F32 = false (bf16 result): the product is rounded to bf16 on its way into the patch, as the
// reference's reduce-scatter rounds a rank's partial product before the partials are summed
// (kraken/fused/gemm_reduce_scatter_fused.py:72, summed in fp32 at :118-145); partial sums of
// the peers and the bias are then added in fp32 in the order own, peer 0, 1, ..., bias.
// F32 = true (fp32 result: the reference's fused all-reduce keeps fp32 from the accumulator to
// the output, kraken/fused/gemm_one_shot_all_reduce_fused.py:65-99): the patch holds fp32.
//
// ACC is either f32x16[TM][TN] (32x32 MFMA blocks: lane l holds row l%32 of a block and the
// columns 8(v/4) + 4(l/32) + v%4 of register v) or f32x4[2*TM][2*TN] (16x16 blocks: lane l
// holds row l%16 and the columns 4(l/16) + v); only the copy into the patch knows which.
template <bool F32, int BM, int WTM, int WTN, int TM, int TN, bool EVEN, int EP_WAVE, class ACC>
__device__ __forceinline__ void gemm_epilogue_impl(const GemmArgs& g, const int n_peers, const uint16_t* bias,
                                                   const ACC& acc, unsigned char* smem,
                                                   int m0, int n0, int wm, int wn, int lane, int wave) {
    constexpr bool MI16 = std::is_same<ACC, f32x4[2 * TM][2 * TN]>::value;
    static_assert(MI16 || std::is_same<ACC, f32x16[TM][TN]>::value, "unknown accumulator layout");
    // After the barrier above no wave reads the pipeline stages any more, and from here on
    // every wave touches only its own LDS patch, so no further workgroup barrier is needed
    // (LDS requests of one wave are served in order).  Per 32-row slab the accumulators are
    // written to the patch and read back as row-contiguous 8-element chunks.
    //
    // Loads and stores share one in-order counter on this hardware: waiting for a load that
    // was issued after a store also waits until that store has been acknowledged by memory,
    // a round trip of thousands of cycles.  So nothing in the store path may depend on a
    // load issued behind a store: the bias is fetched once, before the first store, and the
    // partial sums of the other ranks are fetched one batch ahead (the loads of batch b+1 are
    // issued before the stores of batch b), so every wait leaves the younger stores pending.
    typedef typename std::conditional<F32, float, uint16_t>::type patch_t;
    // row pitch in elements: 16 bytes of padding keep the quad stores of 16 (bf16: 8-byte) or
    // 8 (fp32: 16-byte) lanes on distinct banks and the rows 16-byte aligned
    constexpr int LD = WTN + (F32 ? 4 : 8);
    static_assert(32 * LD * (int)sizeof(patch_t) <= EP_WAVE, "patch exceeds the wave's share of LDS");
    patch_t* patch = (patch_t*)(smem + wave * EP_WAVE);
    constexpr int CPR = WTN / 8;            // 8-element chunks per patch row
    constexpr int EP_ITERS = 32 * CPR / 64; // chunks per lane per 32-row slab
    constexpr int kChunkBatch = BM >= 256 ? 4 : 2;   // the small tile keeps its register count low (occupancy)
    constexpr int kPeerGroup = 4;           // peers fetched together by the generic path
    const int band_lo = g.band_row0, band_hi = g.band_row0 + g.band_rows;
    const int lane_r = lane / CPR, lane_cc = lane % CPR;   // chunk (it*64 + lane): row it*(64/CPR) + lane_r
    const int n = n0 + wn * WTN + lane_cc * 8;             // first of the lane's 8 columns, same for every chunk

    float bias_f[8];
    zero8(bias_f);
    const bool has_bias = bias != nullptr;
    if (has_bias) add8(*(const u32x4*)(bias + (EVEN ? n : min(n, g.N - 8))), bias_f);

    // Round-to-nearest-even pack of two fp32 to bf16, pinned where it is written: the
    // accumulators do not change inside the slab loop, so an ordinary conversion -- or, for
    // accumulators held in AGPRs, even just the copy to a VALU-readable register -- would be
    // hoisted out of it for all slabs at once, at the price of 128 or more live registers.
    auto pack_here = [](float lo, float hi) __attribute__((always_inline)) {
        uint32_t r;
        if constexpr (BM >= 256) {   // 256 accumulators: they live in AGPRs
            uint32_t t;
            asm volatile("v_accvgpr_read_b32 %0, %2\n\tv_accvgpr_read_b32 %1, %3\n\tv_cvt_pk_bf16_f32 %0, %0, %1"
                         : "=&v"(r), "=&v"(t)
                         : "a"(lo), "a"(hi));
        } else {
            asm volatile("v_cvt_pk_bf16_f32 %0, %1, %2" : "=v"(r) : "v"(lo), "v"(hi));
        }
        return r;
    };
    // copy of slab i's accumulators to the patch.  Accumulator registers can only be indexed
    // statically, hence the uniform if-chain inside a rolled slab loop.
    auto copy_slab = [&](int i) __attribute__((always_inline)) {
        patch_t* row = MI16 ? patch + (lane & 15) * LD + 4 * (lane >> 4) : patch + (lane & 31) * LD + 4 * (lane >> 5);
#pragma unroll
        for (int ii = 0; ii < TM; ++ii) {
            if (i == ii) {
                if constexpr (MI16) {
                    // slab = block rows 2i and 2i+1 (patch rows 0..15 and 16..31), 2*TN column blocks
#pragma unroll
                    for (int h = 0; h < 2; ++h)
#pragma unroll
                        for (int j = 0; j < 2 * TN; ++j) {
                            const f32x4& a = acc[2 * ii + h][j];
                            if constexpr (F32) {
                                *(f32x4*)(row + h * 16 * LD + j * 16) = a;
                            } else {
                                typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
                                *(u32x2*)(row + h * 16 * LD + j * 16) = u32x2{pack_here(a[0], a[1]), pack_here(a[2], a[3])};
                            }
                        }
                } else {
#pragma unroll
                for (int j = 0; j < TN; ++j)
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const f32x16& a = acc[ii][j];
                        if constexpr (F32) {
                            *(f32x4*)(row + j * 32 + 8 * q) = f32x4{a[4 * q], a[4 * q + 1], a[4 * q + 2], a[4 * q + 3]};
                        } else {
                            typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
                            *(u32x2*)(row + j * 32 + 8 * q) =
                                u32x2{pack_here(a[4 * q], a[4 * q + 1]), pack_here(a[4 * q + 2], a[4 * q + 3])};
                        }
                    }
                }
                // a distinct statement per case: identical case bodies would be merged into one
                // with a run-time accumulator index, which forces the accumulators into memory
                asm volatile("; accumulators of slab %0 copied" ::"n"(ii));
            }
        }
        // keep the scheduler from pulling the accumulator reads of later slabs (256 registers
        // in all) ahead of this point
        __builtin_amdgcn_sched_barrier(0);
    };
    // one chunk of the current slab: as stored (bf16 patch) or as fp32 values
    auto read_raw = [&](int chunk) __attribute__((always_inline)) {
        const int r = chunk * (64 / CPR) + lane_r;
        return *(const u32x4*)(patch + r * LD + lane_cc * 8);
    };
    auto read_chunk = [&](int chunk, float (&f)[8]) __attribute__((always_inline)) {
        if constexpr (F32) {
            const int r = chunk * (64 / CPR) + lane_r;
            const f32x4 lo = *(const f32x4*)(patch + r * LD + lane_cc * 8);
            const f32x4 hi = *(const f32x4*)(patch + r * LD + lane_cc * 8 + 4);
            f[0] = lo.x; f[1] = lo.y; f[2] = lo.z; f[3] = lo.w;
            f[4] = hi.x; f[5] = hi.y; f[6] = hi.z; f[7] = hi.w;
        } else {
            unpack8(read_raw(chunk), f);
        }
    };
    auto store_out = [&](int64_t off, const float (&f)[8]) __attribute__((always_inline)) {
        if constexpr (F32) {
            float* o = (float*)g.out + (int64_t)blockIdx.y * g.split_out_stride + off;
            *(f32x4*)o = f32x4{f[0], f[1], f[2], f[3]};
            *(f32x4*)(o + 4) = f32x4{f[4], f[5], f[6], f[7]};
        } else {
            st_stream((u32x4*)((uint16_t*)g.out + off), pack8(f));
        }
    };

    // the wave's first row, as a scalar: the classification below must branch uniformly
    const int wave_m0 = __builtin_amdgcn_readfirstlane(m0 + wm * WTM);

    // ---- every row of the wave lies in the band and there are exactly 7 peers ---------------
    // (the eight-rank case of the reference benchmarks): straight-line batches of kFastBatch
    // chunks, peer loads double-buffered one batch ahead across slab boundaries.
    if constexpr (!F32) {
        constexpr int kFastPeers = 7;
        constexpr int kFastBatch = BM >= 256 ? 2 : 1;   // chunks per batch (the small tile keeps two workgroups per CU)
        constexpr int kFastBatches = EP_ITERS / kFastBatch;
        static_assert(kFastBatches % 2 == 0, "the two peer buffers alternate with a static parity");
        if (EVEN && n_peers == kFastPeers && wave_m0 >= band_lo && wave_m0 + WTM <= band_hi) {
            u32x4 pv[2][kFastBatch][kFastPeers];
            const int64_t peer_off = (int64_t)(wave_m0 - band_lo + lane_r) * g.N + n;
            const int64_t chunk_step = (int64_t)(64 / CPR) * g.N;   // elements between consecutive chunks of a lane
            auto issue = [&](auto buf_c, int chunk_abs) __attribute__((always_inline)) {
                constexpr int buf = decltype(buf_c)::value;
#pragma unroll
                for (int c = 0; c < kFastBatch; ++c)
#pragma unroll
                    for (int q = 0; q < kFastPeers; ++q)
                        pv[buf][c][q] =
                            ld_stream((const u32x4*)((const uint16_t*)g.peer.p[q] + peer_off + (chunk_abs + c) * chunk_step));
            };
            issue(std::integral_constant<int, 0>{}, 0);
#pragma nounroll
            for (int i = 0; i < TM; ++i) {
                copy_slab(i);
                const int chunk0 = i * EP_ITERS;   // chunks are numbered through all slabs of the wave
#pragma unroll
                for (int b = 0; b < kFastBatches; ++b) {
                    // unconditional (the very last batch re-fetches itself, unused): a prefetch under
                    // a branch would make the wait below assume the shorter queue and stall on stores
                    const int next_chunk = min(chunk0 + (b + 1) * kFastBatch, TM * EP_ITERS - kFastBatch);
                    if (b & 1) issue(std::integral_constant<int, 0>{}, next_chunk);
                    else issue(std::integral_constant<int, 1>{}, next_chunk);
                    float f[kFastBatch][8];
#pragma unroll
                    for (int c = 0; c < kFastBatch; ++c) read_chunk(b * kFastBatch + c, f[c]);
#pragma unroll
                    for (int c = 0; c < kFastBatch; ++c) {
#pragma unroll
                        for (int q = 0; q < kFastPeers; ++q) add8(pv[b & 1][c][q], f[c]);
#pragma unroll
                        for (int e = 0; e < 8; ++e) f[c][e] += bias_f[e];
                    }
#pragma unroll
                    for (int c = 0; c < kFastBatch; ++c) {
                        const int m = wave_m0 + (chunk0 + b * kFastBatch + c) * (64 / CPR) + lane_r;
                        store_out((int64_t)(m - band_lo) * g.N + n, f[c]);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            return;
        }
    }

    // ---- every other case, one slab at a time ------------------------------------------------
    // One batch of kChunkBatch chunks of the current slab.  NP == 0: every row of the slab lies
    // in the band and there are no peers; NP == -2: no row of the slab lies in the band (both
    // straight-line code without loads); NP == -1: generic per-lane handling (band edge inside
    // the slab, ragged tile, any peer count).
    auto slab_batch = [&](auto np_c, int slab_m0, int b0) __attribute__((always_inline)) {
        constexpr int NP = decltype(np_c)::value;
        int64_t off[kChunkBatch];
        bool in_band[kChunkBatch], valid[kChunkBatch];
#pragma unroll
        for (int c = 0; c < kChunkBatch; ++c) {
            const int m = slab_m0 + (b0 + c) * (64 / CPR) + lane_r;
            valid[c] = EVEN || (m < g.M && n < g.N);
            in_band[c] = NP == 0 ? true : NP == -2 ? false : (valid[c] && m >= band_lo && m < band_hi);
            off[c] = in_band[c] ? (int64_t)(m - band_lo) * g.N + n : (int64_t)m * g.N + n;
        }
        if constexpr (!F32 && NP != -1) {
            // nothing to add but perhaps the bias: the bf16 chunks go out as they are
            if (NP == -2 || !has_bias) {
                if (NP == 0 || g.c_full != nullptr) {
                    uint16_t* dst = NP == 0 ? (uint16_t*)g.out : g.c_full;
#pragma unroll
                    for (int c = 0; c < kChunkBatch; ++c) st_stream((u32x4*)(dst + off[c]), read_raw(b0 + c));
                }
                return;
            }
        }
        float f[kChunkBatch][8];
#pragma unroll
        for (int c = 0; c < kChunkBatch; ++c) read_chunk(b0 + c, f[c]);
        if constexpr (NP == -1) {
            // Peers in groups of kPeerGroup, all loads of a group issued before its first add;
            // the groups are unrolled, each under one uniform test.  No load is predicated:
            // a chunk outside the band reads a valid in-band address instead, a peer index
            // past the last repeats the last peer, and such values are masked to +0.0 (loads
            // under branches would make every later load wait for the whole queue).
            const int64_t safe_off = min(n, g.N - 8);
#pragma unroll
            for (int q0 = 0; q0 < KR_MAX_WORLD - 1; q0 += kPeerGroup) {
                if (q0 < n_peers) {
                    u32x4 pv[kChunkBatch][kPeerGroup];
#pragma unroll
                    for (int c = 0; c < kChunkBatch; ++c)
#pragma unroll
                        for (int q = 0; q < kPeerGroup; ++q) {
                            const int qq = min(q0 + q, n_peers - 1);
                            pv[c][q] = ld_stream(
                                (const u32x4*)((const uint16_t*)g.peer.p[qq] + (in_band[c] ? off[c] : safe_off)));
                        }
#pragma unroll
                    for (int c = 0; c < kChunkBatch; ++c)
#pragma unroll
                        for (int q = 0; q < kPeerGroup; ++q) {
                            const uint32_t keep = (in_band[c] && q0 + q < n_peers) ? 0xffffffffu : 0u;
                            add8(u32x4{pv[c][q].x & keep, pv[c][q].y & keep, pv[c][q].z & keep, pv[c][q].w & keep}, f[c]);
                        }
                }
            }
        }
#pragma unroll
        for (int c = 0; c < kChunkBatch; ++c) {
            if (in_band[c]) {
#pragma unroll
                for (int e = 0; e < 8; ++e) f[c][e] += bias_f[e];
                store_out(off[c], f[c]);
            } else if (valid[c] && g.c_full != nullptr) {
                st_stream((u32x4*)(g.c_full + off[c]), pack8(f[c]));
            }
        }
    };

#pragma nounroll
    for (int i = 0; i < TM; ++i) {
        copy_slab(i);
        const int slab_m0 = wave_m0 + i * 32;
        const bool all_in = EVEN && slab_m0 >= band_lo && slab_m0 + 32 <= band_hi;
        const bool all_out = EVEN && (slab_m0 + 32 <= band_lo || slab_m0 >= band_hi);
#pragma unroll
        for (int b0 = 0; b0 < EP_ITERS; b0 += kChunkBatch) {
            if (all_out) {
                slab_batch(std::integral_constant<int, -2>{}, slab_m0, b0);
            } else if (all_in && n_peers == 0) {
                slab_batch(std::integral_constant<int, 0>{}, slab_m0, b0);
            } else {
                slab_batch(std::integral_constant<int, -1>{}, slab_m0, b0);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    }
}

// Producer side of the copy-engine reduce-scatter, called by the whole workgroup once its tile
// (rows m0 .. m0+bm-1) is stored (kraken/fused/gemm_reduce_scatter_ce_persistent.py:117-132):
// the tile is counted into the counter of every destination rank whose band of g.count_rows rows
// it touches, and the workgroup whose count completes a band (all column tiles of all row tiles
// that overlap it) sets the band's flag, on which a stream-ordered wait in front of the band's
// copy is parked.  Order: every wave's stores are complete at the barrier; thread 0's release
// fence then writes them back to memory before its count becomes visible, and the workgroup that
// sees the last count acquires the others' before it publishes the flag.
__device__ __forceinline__ void count_finished_tile(const GemmArgs& g, int m0, int bm) {
    __syncthreads();
    if (threadIdx.x != 0) return;
    __atomic_thread_fence(__ATOMIC_RELEASE);   // system scope
    const int m_last = min(m0 + bm, g.M) - 1;
    for (int r = m0 / g.count_rows; r <= m_last / g.count_rows; ++r) {
        const int t_lo = (int)(((int64_t)r * g.count_rows) / bm);
        const int t_hi = (int)(((int64_t)(r + 1) * g.count_rows - 1) / bm);
        const uint32_t band_tiles = (uint32_t)(t_hi - t_lo + 1) * (uint32_t)g.tiles_n;
        const uint32_t before = __hip_atomic_fetch_add(g.band_counter + r, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (before + 1 == band_tiles) {
            __atomic_thread_fence(__ATOMIC_ACQ_REL);
            __hip_atomic_store(g.band_signal + r, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        }
    }
}

// n_peers and bias are what is still to be added here (a kernel that has already put the
// peers or the bias into the accumulators passes 0 / nullptr); g is only read, never copied,
// so the peer table stays in kernel-argument memory.
template <int BM, int WTM, int WTN, int TM, int TN, bool EVEN, int EP_WAVE, class ACC>
__device__ __forceinline__ void gemm_epilogue(const GemmArgs& g, int n_peers, const uint16_t* bias,
                                              const ACC& acc, unsigned char* smem,
                                              int m0, int n0, int wm, int wn, int lane, int wave) {
    if (g.out_is_fp32) gemm_epilogue_impl<true, BM, WTM, WTN, TM, TN, EVEN, EP_WAVE, ACC>(g, n_peers, bias, acc, smem, m0, n0, wm, wn, lane, wave);
    else gemm_epilogue_impl<false, BM, WTM, WTN, TM, TN, EVEN, EP_WAVE, ACC>(g, n_peers, bias, acc, smem, m0, n0, wm, wn, lane, wave);
    if (g.band_counter != nullptr) count_finished_tile(g, m0, BM);
}

}  // namespace kr
