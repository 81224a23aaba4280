// Pieces shared by the GEMM kernels: argument block, tile schedule, fused epilogue.
#pragma once

#include <type_traits>

#include "common.h"

namespace kr {

struct GemmArgs {
    const uint16_t* A;
    const uint16_t* B;
    int64_t lda;   // elements between rows of A (k is contiguous)
    int64_t ldb;   // NT: elements between n-rows of B^T; NN: elements between k-rows of B
    int M, N, K;
    const uint16_t* peers;
    int n_peers;
    int64_t peers_stride;
    const uint16_t* bias;
    int band_row0, band_rows;
    uint16_t* c_full;
    void* out;
    int out_is_fp32;
    int pivot_tiles;   // rotation of the M-tile order
    int tiles_m, tiles_n;
};

// LDS-DMA kernel for shapes the 256x256 tile divides (gemm_dtl.hip)
bool gemm_dtl_supported(const GemmArgs& g);
hipError_t launch_gemm_dtl(const GemmArgs& g, bool b_nt, hipStream_t st);

constexpr int kGroupN = 4;        // column panels per scheduling group
constexpr int kXcds = 8;

// Map the workgroup id to its tile (tile_m, tile_n).
__device__ __forceinline__ void tile_schedule(const GemmArgs& g, int& tile_m_out, int& tile_n_out) {
    // ---- tile schedule -------------------------------------------------------------------
    // Workgroups are dealt round-robin to the 8 XCDs (each with its own L2), so workgroup ids
    // are first re-numbered to give every XCD a contiguous range of tiles.  Tiles are then
    // ordered in groups of kGroupN column panels, M fastest in steps of kGroupN columns: the
    // ~32 tiles an XCD runs at a time form an 8 x 4 block that shares 8 A panels and 4 B
    // panels through its L2, and every XCD works on all row bands -- the rows of the reduce
    // band (whose tiles also stream the peers' partial sums) are spread over all XCDs
    // instead of landing on one.  The M order is rotated by the pivot, so the band's (or the
    // local shard's) tiles are the first ones of every XCD.
    int pid = blockIdx.x;
    const int ntiles = g.tiles_m * g.tiles_n;
    if (ntiles % kXcds == 0) pid = (pid % kXcds) * (ntiles / kXcds) + pid / kXcds;
    const int per_group = kGroupN * g.tiles_m;
    const int group = pid / per_group;
    const int first_n = group * kGroupN;
    const int gsz = min(g.tiles_n - first_n, kGroupN);
    const int tile_n = first_n + (pid % per_group) % gsz;
    int tile_m = (pid % per_group) / gsz;
    tile_m += g.pivot_tiles;
    if (tile_m >= g.tiles_m) tile_m -= g.tiles_m;
    tile_m_out = tile_m;
    tile_n_out = tile_n;
}

// Fused epilogue of one workgroup tile.  `acc` are the 32x32 MFMA accumulators of this wave
// (TM x TN blocks), `smem` the workgroup's LDS (free for reuse: every wave has passed a
// barrier after its last read of the operand stages).
template <int BM, int WTM, int WTN, int TM, int TN, bool EVEN, int EP_LD, int EP_WAVE>
__device__ __forceinline__ void gemm_epilogue(const GemmArgs& g, const f32x16 (&acc)[TM][TN], unsigned char* smem,
                                              int m0, int n0, int wm, int wn, int lane, int wave) {
    // After the barrier above no wave reads the pipeline stages any more, and from here on
    // every wave touches only its own LDS patch, so no further workgroup barrier is needed
    // (LDS requests of one wave are served in order).  Per 32-row slab the accumulators are
    // written to the patch in MFMA layout and read back as row-contiguous 8-element chunks.
    // The partial sums of the other ranks are fetched kPeerGroup peers x kChunkBatch chunks at
    // a time, all loads issued before the first add, so a band tile keeps dozens of 1 KiB
    // wave-loads in flight instead of waiting for one HBM round trip per peer.
    float* patch = (float*)(smem + wave * EP_WAVE);
    constexpr int CPR = WTN / 8;            // 8-element chunks per patch row
    constexpr int EP_ITERS = 32 * CPR / 64; // chunks per lane per 32-row slab
    constexpr int kChunkBatch = BM >= 256 ? 4 : 2;   // the small tile keeps its register count low (occupancy)
    constexpr int kPeerGroup = 8;
    static_assert(2 * kPeerGroup >= KR_MAX_WORLD - 1, "two peer groups must cover every world size");
    const int band_lo = g.band_row0, band_hi = g.band_row0 + g.band_rows;
    const int lane_r = lane / CPR, lane_cc = lane % CPR;   // chunk (it*64 + lane): row it*(64/CPR) + lane_r

    // One batch of kChunkBatch chunks of the current slab.  NP >= 0: every row of the slab lies
    // in the band and there are exactly NP peers (straight-line code, no per-lane branches);
    // NP == -1: generic per-lane handling (band edge inside the slab, ragged tile, any peer
    // count); NP == -2: no row of the slab lies in the band.
    auto slab_batch = [&](auto np_c, int slab_m0, int b0) {
        constexpr int NP = decltype(np_c)::value;
        float f[kChunkBatch][8];
        int64_t off[kChunkBatch];
        bool in_band[kChunkBatch], valid[kChunkBatch];
        const int n = n0 + wn * WTN + lane_cc * 8;
#pragma unroll
        for (int c = 0; c < kChunkBatch; ++c) {
            const int m = slab_m0 + (b0 + c) * (64 / CPR) + lane_r;
            valid[c] = EVEN || (m < g.M && n < g.N);
            in_band[c] = NP >= 0 ? true : NP == -2 ? false : (valid[c] && m >= band_lo && m < band_hi);
            off[c] = in_band[c] ? (int64_t)(m - band_lo) * g.N + n : (int64_t)m * g.N + n;
        }
        constexpr int NG = NP >= 0 ? NP : kPeerGroup;   // peers fetched in the first group
        u32x4 pv[kChunkBatch][NG > 0 ? NG : 1];
        if constexpr (NP > 0) {
#pragma unroll
            for (int c = 0; c < kChunkBatch; ++c)
#pragma unroll
                for (int q = 0; q < NP; ++q)
                    pv[c][q] = ld_stream((const u32x4*)(g.peers + q * g.peers_stride + off[c]));
        } else if constexpr (NP == -1) {
#pragma unroll
            for (int c = 0; c < kChunkBatch; ++c)
#pragma unroll
                for (int q = 0; q < kPeerGroup; ++q)
                    if (in_band[c] && q < g.n_peers)
                        pv[c][q] = ld_stream((const u32x4*)(g.peers + q * g.peers_stride + off[c]));
        }
#pragma unroll
        for (int c = 0; c < kChunkBatch; ++c) {
            const int r = (b0 + c) * (64 / CPR) + lane_r;
            const f32x4 lo = *(const f32x4*)(patch + r * EP_LD + lane_cc * 8);
            const f32x4 hi = *(const f32x4*)(patch + r * EP_LD + lane_cc * 8 + 4);
            f[c][0] = lo.x; f[c][1] = lo.y; f[c][2] = lo.z; f[c][3] = lo.w;
            f[c][4] = hi.x; f[c][5] = hi.y; f[c][6] = hi.z; f[c][7] = hi.w;
        }
        if constexpr (NP > 0) {
#pragma unroll
            for (int c = 0; c < kChunkBatch; ++c)
#pragma unroll
                for (int q = 0; q < NP; ++q) add8(pv[c][q], f[c]);
        } else if constexpr (NP == -1) {
#pragma unroll
            for (int c = 0; c < kChunkBatch; ++c)
#pragma unroll
                for (int q = 0; q < kPeerGroup; ++q)
                    if (in_band[c] && q < g.n_peers) add8(pv[c][q], f[c]);
            // second group (9..15 peers), same pattern
            if (g.n_peers > kPeerGroup) {
#pragma unroll
                for (int c = 0; c < kChunkBatch; ++c)
#pragma unroll
                    for (int q = 0; q < kPeerGroup; ++q)
                        if (in_band[c] && kPeerGroup + q < g.n_peers)
                            pv[c][q] = ld_stream(
                                (const u32x4*)(g.peers + (kPeerGroup + q) * g.peers_stride + off[c]));
#pragma unroll
                for (int c = 0; c < kChunkBatch; ++c)
#pragma unroll
                    for (int q = 0; q < kPeerGroup; ++q)
                        if (in_band[c] && kPeerGroup + q < g.n_peers) add8(pv[c][q], f[c]);
            }
        }
        if constexpr (NP != -2) {
            if (g.bias != nullptr) {
                const u32x4 bv = *(const u32x4*)(g.bias + (EVEN ? n : min(n, g.N - 8)));
#pragma unroll
                for (int c = 0; c < kChunkBatch; ++c)
                    if (in_band[c]) add8(bv, f[c]);
            }
        }
#pragma unroll
        for (int c = 0; c < kChunkBatch; ++c) {
            if (in_band[c]) {
                if (g.out_is_fp32) {
                    float* o = (float*)g.out + off[c];
                    *(f32x4*)o = f32x4{f[c][0], f[c][1], f[c][2], f[c][3]};
                    *(f32x4*)(o + 4) = f32x4{f[c][4], f[c][5], f[c][6], f[c][7]};
                } else {
                    st_stream((u32x4*)((uint16_t*)g.out + off[c]), pack8(f[c]));
                }
            } else if (valid[c] && g.c_full != nullptr) {
                st_stream((u32x4*)(g.c_full + off[c]), pack8(f[c]));
            }
        }
    };

    // the wave's first row, as a scalar: the slab classification below must branch uniformly
    const int wave_m0 = __builtin_amdgcn_readfirstlane(m0 + wm * WTM);
    // The slab loop is a real loop (its body, with the specialised batch variants, exists
    // once); only the copy of slab i's accumulators to the patch is selected by a uniform
    // if-chain, because accumulator registers can only be indexed statically.
#pragma nounroll
    for (int i = 0; i < TM; ++i) {
        // MFMA layout: lane holds column (lane & 31); register v is row 8*(v/4) + 4*(lane>>5) + v%4
#pragma unroll
        for (int ii = 0; ii < TM; ++ii) {
            if (i == ii) {
#pragma unroll
                for (int j = 0; j < TN; ++j)
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        const int r = 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
                        patch[r * EP_LD + j * 32 + (lane & 31)] = acc[ii][j][v];
                    }
            }
        }
        // keep the scheduler from pulling the accumulator reads of later slabs (256 registers
        // in all) ahead of this point
        __builtin_amdgcn_sched_barrier(0);
        const int slab_m0 = wave_m0 + i * 32;
        const bool all_in = EVEN && slab_m0 >= band_lo && slab_m0 + 32 <= band_hi;
        const bool all_out = EVEN && (slab_m0 + 32 <= band_lo || slab_m0 >= band_hi);
#pragma unroll
        for (int b0 = 0; b0 < EP_ITERS; b0 += kChunkBatch) {
            if (all_out) {
                slab_batch(std::integral_constant<int, -2>{}, slab_m0, b0);
            } else if (all_in && g.n_peers == 7) {
                slab_batch(std::integral_constant<int, 7>{}, slab_m0, b0);
            } else if (all_in && g.n_peers == 0) {
                slab_batch(std::integral_constant<int, 0>{}, slab_m0, b0);
            } else {
                slab_batch(std::integral_constant<int, -1>{}, slab_m0, b0);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    }
}

}  // namespace kr
