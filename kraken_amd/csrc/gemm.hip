// bf16 GEMM on the gfx950 matrix cores with a fused reduce(+bias) epilogue.
//
//   C = A[M,K] @ B[K,N]                      (fp32 accumulate, v_mfma_f32_32x32x16_bf16)
//   out  = C[band] + sum_j peers[j] + bias   (rows of the band; one store, no C round trip)
//   c_full[rows outside the band] = bf16(C)
//
// Workgroup tile BM x BN x 64, WM x WN wavefronts, each owning a
// (BM/WM) x (BN/WN) block of C as 32x32 MFMA accumulators.  A and B tiles are
// staged in LDS as [row][64 k] bf16 (128-byte rows) with the 16-byte chunks of
// a row XOR-swizzled by the row index, so that the 128-bit fragment reads of 8
// consecutive rows land in 8 different bank groups.  Two LDS stages: the
// global loads of k-step t+1 are issued before the MFMAs of step t and written
// to the other stage afterwards (one workgroup barrier per k-step).
// Row-major B ([K,N], N contiguous) is transposed on its way into LDS: a
// thread loads an 8(k) x 8(n) block with eight 128-bit loads, transposes it in
// registers with byte permutes and writes eight 128-bit [n][8 k] chunks.
// Epilogue (shared with the LDS-DMA kernel for 256x256 tiles): accumulators go
// through a per-wave LDS patch to turn the MFMA layout into row-contiguous
// 8-element vectors, so peers, bias and output are all moved with 128-bit
// accesses covering whole row segments.  This file also holds the C entry point
// and the choice between the two kernels.
#include <stdlib.h>

#include <type_traits>

#include <algorithm>
#include <mutex>

#include "gemm_common.h"

namespace kr {


constexpr int BK = 64;            // k extent of one LDS stage
constexpr int kRowBytes = BK * 2; // 128-byte LDS rows

// 16-byte chunk swizzle inside a 128-byte LDS row
__device__ __forceinline__ int swz(int row, int chunk) { return chunk ^ ((row ^ (row >> 3)) & 7); }

__device__ __forceinline__ uint32_t perm_lo(uint32_t hi_src, uint32_t lo_src) {
    // {lo16(hi_src), lo16(lo_src)}
    return __builtin_amdgcn_perm(hi_src, lo_src, 0x05040100u);
}
__device__ __forceinline__ uint32_t perm_hi(uint32_t hi_src, uint32_t lo_src) {
    // {hi16(hi_src), hi16(lo_src)}
    return __builtin_amdgcn_perm(hi_src, lo_src, 0x07060302u);
}

template <int BM, int BN, int WM, int WN, bool B_NT, bool EVEN>
__global__ __launch_bounds__(WM* WN * 64) void gemm_reduce_kernel(const GemmArgs g) {
    constexpr int T = WM * WN * 64;
    constexpr int WTM = BM / WM, WTN = BN / WN;   // wave tile
    constexpr int TM = WTM / 32, TN = WTN / 32;   // 32x32 MFMA blocks per wave
    constexpr int A_STAGE = BM * kRowBytes, B_STAGE = BN * kRowBytes;
    constexpr int STAGE = A_STAGE + B_STAGE;
    constexpr int A_ITERS = BM * 8 / T;           // 16-byte chunks per thread per stage
    constexpr int B_ITERS_NT = BN * 8 / T;
    constexpr int B_BLOCKS = BN / T > 0 ? BN / T : 1;  // NN: 8x8 blocks per thread per stage
    static_assert(BM % (WM * 32) == 0 && BN % (WN * 32) == 0, "wave tile must be a multiple of 32");
    static_assert((BM * 8) % T == 0 && (BN * 8) % T == 0 && (BN % T == 0 || BN < T), "load split");
    // epilogue patch: 32 rows x WTN fp32 per wave, rows padded by 4 floats
    constexpr int EP_WAVE = 32 * (WTN + 4) * 4;
    static_assert(EP_WAVE * WM * WN <= 2 * STAGE, "epilogue patch must fit in the pipeline LDS");

    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave / WN, wn = wave % WN;

    int tile_m, tile_n;
    tile_schedule(g, schedule_position(g, blockIdx.x), tile_m, tile_n);
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const uint16_t* a_tile;   // first row of the tile's A panel (gathered matrix or local shard)
    int64_t lda;
    gathered_a_tile(g, m0, BM, a_tile, lda);
    // k range of this workgroup: all of K, or with a split K loop (g.k_splits > 1, split index
    // in blockIdx.y) the split's share of the k-steps; k_begin enters every operand offset
    const int kt_all = (g.K + BK - 1) / BK;
    const int kt_begin = g.k_splits > 1 ? (int)((int64_t)kt_all * blockIdx.y / g.k_splits) : 0;
    const int kt_total = g.k_splits > 1 ? (int)((int64_t)kt_all * (blockIdx.y + 1) / g.k_splits) - kt_begin : kt_all;
    const int k_begin = kt_begin * BK;

    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

    // ---- operand staging: global -> registers -> LDS, one 16-byte chunk per "unit" ------
    // Global loads are buffer loads: a wave-uniform resource descriptor (tile base), a
    // per-thread 32-bit byte offset that never changes, and a wave-uniform scalar offset that
    // advances with k.  No per-load address arithmetic is left in the main loop.
    constexpr int NB_LD = B_NT ? B_ITERS_NT : B_BLOCKS * 8;   // 128-bit global loads of B per thread per stage
    constexpr int NB_ST = B_NT ? B_ITERS_NT : B_BLOCKS * 4;   // B store units per thread per stage
    constexpr uint32_t kOob = 0x80000000u;                     // offset beyond num_records: the load returns 0
    // two register sets: set (t & 1) holds tile t+1 during iteration t and is re-filled with
    // tile t+3, so a global load has two iterations to land
    u32x4 a_reg[2][A_ITERS];
    u32x4 b_reg[2][NB_LD];
    uint32_t a_goff[A_ITERS], a_loff[A_ITERS];
    uint32_t b_goff[B_NT ? B_ITERS_NT : B_BLOCKS], b_loff[B_NT ? B_ITERS_NT : B_BLOCKS];
    const int ld_kc = tid & 7;        // 16-byte chunk inside a 128-byte k-row (T % 8 == 0)
    bool nn_active = true;            // NN: this thread owns an 8x8 block of the B stage
#pragma unroll
    for (int i = 0; i < A_ITERS; ++i) {
        const int row = (i * T + tid) >> 3;
        int m = m0 + row;
        if (!EVEN) m = min(m, g.M - 1);
        a_goff[i] = (uint32_t)(((int64_t)(m - m0) * lda + ld_kc * 8) * 2);
        a_loff[i] = row * kRowBytes + swz(row, ld_kc) * 16;
    }
    if (B_NT) {
#pragma unroll
        for (int i = 0; i < B_ITERS_NT; ++i) {
            const int row = (i * T + tid) >> 3;
            int n = n0 + row;
            if (!EVEN) n = min(n, g.N - 1);
            b_goff[i] = (uint32_t)(((int64_t)(n - n0) * g.ldb + ld_kc * 8) * 2);
            b_loff[i] = A_STAGE + row * kRowBytes + swz(row, ld_kc) * 16;
        }
    } else {
#pragma unroll
        for (int i = 0; i < B_BLOCKS; ++i) {
            const int blk = i * T + tid;
            const int nc = blk % (BN / 8), kg = blk / (BN / 8);
            if (BN < T && kg >= 8) nn_active = false;     // more threads than 8x8 blocks
            int n = n0 + nc * 8;
            if (!EVEN) n = min(n, g.N - 8);
            b_goff[i] = (uint32_t)(((int64_t)(kg & 7) * 8 * g.ldb + (n - n0)) * 2);
            b_loff[i] = (uint32_t)(nc | ((kg & 7) << 16));   // packed (nc, kg); expanded at the store
        }
    }
    // descriptors: 48-bit base, stride 0 (raw), num_records 2^31-1 bytes, 32-bit data format.
    // Rows are clamped into the matrix above, so only the K tail needs the out-of-range path.
    const __amdgpu_buffer_rsrc_t a_rsrc =
        __builtin_amdgcn_make_buffer_rsrc((void*)a_tile, 0, 0x7fffffff, 0x00020000);
    const __amdgpu_buffer_rsrc_t bt_rsrc =
        __builtin_amdgcn_make_buffer_rsrc((void*)(g.B + (int64_t)n0 * g.ldb), 0, 0x7fffffff, 0x00020000);

    auto load_a_unit = [&](int rs, int i, int k_rel) {
        const int k0 = k_begin + k_rel;
        uint32_t off = a_goff[i];
        if (!EVEN && k0 + ld_kc * 8 >= g.K) off = kOob;
        a_reg[rs][i] = __builtin_amdgcn_raw_buffer_load_b128(a_rsrc, off, k0 * 2, 0);
    };
    auto load_b_unit = [&](int rs, int u, int k_rel) {
        const int k0 = k_begin + k_rel;
        if (B_NT) {
            uint32_t off = b_goff[u];
            if (!EVEN && k0 + ld_kc * 8 >= g.K) off = kOob;
            b_reg[rs][u] = __builtin_amdgcn_raw_buffer_load_b128(bt_rsrc, off, k0 * 2, 0);
        } else {
            const int i = u >> 3, j = u & 7;             // block i, k-row j of the 8x8 block
            if (!nn_active) return;
            // re-based on the k-row so that the scalar offset stays small for any matrix size
            const __amdgpu_buffer_rsrc_t brs = __builtin_amdgcn_make_buffer_rsrc(
                (void*)(g.B + (int64_t)(k0 + j) * g.ldb + n0), 0, 0x7fffffff, 0x00020000);
            uint32_t off = b_goff[i];
            if (!EVEN && k0 + (int)(b_loff[i] >> 16) * 8 + j >= g.K) off = kOob;
            b_reg[rs][u] = __builtin_amdgcn_raw_buffer_load_b128(brs, off, 0, 0);
        }
    };
    // LDS is addressed by raw byte offsets: this kernel declares no static LDS, so its dynamic
    // array starts at LDS address 0.  Offsets are relative to stage 0; `st` (0 or STAGE, a power
    // of two above every in-stage offset) selects the stage by XOR.
    typedef __attribute__((address_space(3))) u32x4* lds_u32x4;
    typedef const __attribute__((address_space(3))) bf16x8* lds_frag;
    auto store_a_unit = [&](int rs, int i, uint32_t st) { *(lds_u32x4)(size_t)(a_loff[i] ^ st) = a_reg[rs][i]; };
    auto store_b_unit = [&](int rs, int u, uint32_t st) {
        if (B_NT) {
            *(lds_u32x4)(size_t)(b_loff[u] ^ st) = b_reg[rs][u];
        } else {
            // unit u = (block i, word q): columns 2q and 2q+1 of the 8x8 block, all 8 k
            const int i = u >> 2, q = u & 3;
            if (!nn_active) return;
            const int nc = (int)(b_loff[i] & 0xffff), kg = (int)(b_loff[i] >> 16);
            u32x4 even, odd;               // [n = 2q][k 0..7], [n = 2q+1][k 0..7]
            even.x = perm_lo(b_reg[rs][i * 8 + 1][q], b_reg[rs][i * 8 + 0][q]);
            even.y = perm_lo(b_reg[rs][i * 8 + 3][q], b_reg[rs][i * 8 + 2][q]);
            even.z = perm_lo(b_reg[rs][i * 8 + 5][q], b_reg[rs][i * 8 + 4][q]);
            even.w = perm_lo(b_reg[rs][i * 8 + 7][q], b_reg[rs][i * 8 + 6][q]);
            odd.x = perm_hi(b_reg[rs][i * 8 + 1][q], b_reg[rs][i * 8 + 0][q]);
            odd.y = perm_hi(b_reg[rs][i * 8 + 3][q], b_reg[rs][i * 8 + 2][q]);
            odd.z = perm_hi(b_reg[rs][i * 8 + 5][q], b_reg[rs][i * 8 + 4][q]);
            odd.w = perm_hi(b_reg[rs][i * 8 + 7][q], b_reg[rs][i * 8 + 6][q]);
            const int r0 = nc * 8 + 2 * q, r1 = r0 + 1;
            *(lds_u32x4)(size_t)((uint32_t)(A_STAGE + r0 * kRowBytes + swz(r0, kg) * 16) ^ st) = even;
            *(lds_u32x4)(size_t)((uint32_t)(A_STAGE + r1 * kRowBytes + swz(r1, kg) * 16) ^ st) = odd;
        }
    };

    // ---- MFMA fragments ---------------------------------------------------------------
    // lane -> row (A) / column (B) of a 32x32 block and which 8-wide half of the 16-wide k step
    const int frag_row = lane & 31, frag_kc = lane >> 5;
    uint32_t fa_off[TM], fb_off[TN];   // LDS byte offset of the lane's chunk at ks = 0
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        const int row = wm * WTM + i * 32 + frag_row;
        fa_off[i] = row * kRowBytes + swz(row, frag_kc) * 16;
    }
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        const int row = wn * WTN + j * 32 + frag_row;
        fb_off[j] = A_STAGE + row * kRowBytes + swz(row, frag_kc) * 16;   // A_STAGE < STAGE: survives the XOR
    }
    bf16x8 af[2][TM], bfr[2][TN];
    // chunk (2*ks + kc) ^ f(row) == (kc ^ f(row)) ^ 2*ks: the k sub-step only flips address bits 5..6
    // fa_off / fb_off carry the stage bit of the tile being computed (toggled every iteration);
    // `other` = STAGE reads from the other stage.
    auto read_frag = [&](int q, int ks, uint32_t other, int buf) {
        if (q < TM) af[buf][q] = *(lds_frag)(size_t)(fa_off[q] ^ (uint32_t)(ks << 5) ^ other);
        else bfr[buf][q - TM] = *(lds_frag)(size_t)(fb_off[q - TM] ^ (uint32_t)(ks << 5) ^ other);
    };

    // ---- software pipeline ---------------------------------------------------------------
    // Iteration t computes tile t from LDS stage t&1 while (a) the registers holding tile
    // t+1 (loaded from global memory during iteration t-1) are written to stage (t+1)&1 and
    // (b) tile t+2 is loaded into those registers.  MFMA fragments are double-buffered in
    // registers one 16-wide k sub-step ahead.  One workgroup barrier per iteration, placed
    // before the last sub-step: by then every wave has written its part of tile t+1 and has
    // issued (and waited for) its last reads of tile t.  All side work is spread between the
    // MFMAs in a fixed order.
    constexpr int NM = TM * TN, NF = TM + TN;
    const int k_last = (kt_total - 1) * BK;

#define KR_SCHED_FENCE() __builtin_amdgcn_sched_barrier(0)
    // Side work of one iteration, in the order it is issued: A units, then B units; a unit is
    // "write the registers of tile t+1 to LDS, then re-fill them with tile t+2" (so those
    // loads have a whole iteration to land).  Row-major B consumes the 8 registers of a block
    // in 4 store units before the block is re-loaded.  The jobs are spread evenly over the MFMA
    // slots of sub-steps 0..2; sub-step 3 follows the barrier.
    constexpr int NJ = A_ITERS + (B_NT ? NB_ST : NB_ST + NB_LD);
    constexpr int NSL = 3 * NM;
    uint32_t nxt = STAGE;   // stage (relative to stage 0) that receives tile t+1
    static_assert((STAGE & (STAGE - 1)) == 0, "stage selection by XOR needs a power-of-two stage size");
    auto staging_job = [&](int rs, int j, int k2) {
        if (j < A_ITERS) {
            store_a_unit(rs, j, nxt);
            load_a_unit(rs, j, k2);
        } else if (B_NT) {
            store_b_unit(rs, j - A_ITERS, nxt);
            load_b_unit(rs, j - A_ITERS, k2);
        } else if (j - A_ITERS < NB_ST) {
            store_b_unit(rs, j - A_ITERS, nxt);
        } else {
            load_b_unit(rs, j - A_ITERS - NB_ST, k2);
        }
    };
    // one 16-wide k sub-step: NM MFMAs on fragment buffer `buf`; after each MFMA the fragment
    // reads of the next sub-step (into the other buffer) and the staging jobs of that slot
    auto mfma_step = [&](auto ks_c, auto rs_c, int k2) {
        constexpr int ks = decltype(ks_c)::value;
        constexpr int rs = decltype(rs_c)::value;
        constexpr int buf = ks & 1;
        constexpr bool staging = ks < 3;
#pragma unroll
        for (int s = 0; s < NM; ++s) {
            const int i = s / TN, j = s % TN;
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bfr[buf][j], af[buf][i], acc[i][j], 0, 0, 0);
#pragma unroll
            for (int q = s * NF / NM; q < (s + 1) * NF / NM; ++q)
                read_frag(q, (ks + 1) & 3, ks == 3 ? STAGE : 0, buf ^ 1);
            if constexpr (staging) {
                const int slot = ks * NM + s;
#pragma unroll
                for (int jj = slot * NJ / NSL; jj < (slot + 1) * NJ / NSL; ++jj) staging_job(rs, jj, k2);
            }
            KR_SCHED_FENCE();
        }
    };
    auto iteration = [&](int t, auto rs_c) {
        const int k2 = min((t + 3) * BK, k_last);   // tile t+3, clamped: the tail re-loads the last tile
        // The LDS offsets flip between the two stages every iteration.  Hide their values from
        // the optimiser here, or it pre-computes every (stage, sub-step) address variant outside
        // the loop and runs out of registers; the XORs it keeps inside are free next to the MFMAs.
#pragma unroll
        for (int i = 0; i < TM; ++i) asm volatile("" : "+v"(fa_off[i]));
#pragma unroll
        for (int j = 0; j < TN; ++j) asm volatile("" : "+v"(fb_off[j]));
#pragma unroll
        for (int i = 0; i < A_ITERS; ++i) asm volatile("" : "+v"(a_loff[i]));
        if (B_NT) {
#pragma unroll
            for (int i = 0; i < B_ITERS_NT; ++i) asm volatile("" : "+v"(b_loff[i]));
        }
        asm volatile("" : "+s"(nxt));
        mfma_step(std::integral_constant<int, 0>{}, rs_c, k2);
        mfma_step(std::integral_constant<int, 1>{}, rs_c, k2);
        mfma_step(std::integral_constant<int, 2>{}, rs_c, k2);
        // every LDS access of this wave so far has completed; then all waves meet
        __builtin_amdgcn_s_waitcnt(0xc07f);   // lgkmcnt(0) only: the global loads stay in flight
        __builtin_amdgcn_s_barrier();
        KR_SCHED_FENCE();
        // sub-step 3 reads the fragments of sub-step 0 of tile t+1
        mfma_step(std::integral_constant<int, 3>{}, rs_c, k2);
        // switch stages: the fragment offsets follow the tile being computed
#pragma unroll
        for (int i = 0; i < TM; ++i) fa_off[i] ^= STAGE;
#pragma unroll
        for (int j = 0; j < TN; ++j) fb_off[j] ^= STAGE;
        nxt ^= STAGE;
    };

    // prologue: tile 0 -> stage 0, tiles 1 and 2 -> the two register sets, first fragments
#pragma unroll
    for (int i = 0; i < A_ITERS; ++i) load_a_unit(0, i, 0);
#pragma unroll
    for (int u = 0; u < NB_LD; ++u) load_b_unit(0, u, 0);
#pragma unroll
    for (int i = 0; i < A_ITERS; ++i) store_a_unit(0, i, 0);
#pragma unroll
    for (int u = 0; u < NB_ST; ++u) store_b_unit(0, u, 0);
    {
        const int k1 = min(BK, k_last), k2 = min(2 * BK, k_last);
#pragma unroll
        for (int i = 0; i < A_ITERS; ++i) load_a_unit(0, i, k1);
#pragma unroll
        for (int u = 0; u < NB_LD; ++u) load_b_unit(0, u, k1);
#pragma unroll
        for (int i = 0; i < A_ITERS; ++i) load_a_unit(1, i, k2);
#pragma unroll
        for (int u = 0; u < NB_LD; ++u) load_b_unit(1, u, k2);
    }
    __builtin_amdgcn_s_waitcnt(0xc07f);
    __builtin_amdgcn_s_barrier();
    KR_SCHED_FENCE();
#pragma unroll
    for (int q = 0; q < NF; ++q) read_frag(q, 0, 0, 0);

    // branch-free body (a conditional second half would put 256 live accumulators through
    // control-flow merges); an odd last tile is peeled
    int t = 0;
    for (; t + 1 < kt_total; t += 2) {
        iteration(t, std::integral_constant<int, 0>{});
        iteration(t + 1, std::integral_constant<int, 1>{});
    }
    if (t < kt_total) iteration(t, std::integral_constant<int, 0>{});
#undef KR_SCHED_FENCE
    // the tail iterations re-load and re-store the last tile: drain everything before the
    // LDS is reused by the epilogue
    __syncthreads();

    gemm_epilogue<BM, WTM, WTN, TM, TN, EVEN, EP_WAVE>(g, g.n_peers, g.bias, acc, smem, m0, n0, wm, wn, lane, wave);
}

// Second pass of the split K loop: sums the S fp32 partial products [S][M][N] in the order
// 0..S-1 and applies the epilogue of the one-pass kernel (same order of the adds, same
// rounding: with a bf16 result and peers the product is rounded to bf16 before the peers'
// partial sums are added).  One thread per 8 consecutive columns.
__global__ __launch_bounds__(256) void splitk_finish_kernel(const GemmArgs g, const float* __restrict__ parts, int S) {
    const int64_t v = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int nv = g.N / 8;
    if (v >= (int64_t)g.M * nv) return;
    const int m = (int)(v / nv), n = (int)(v - (int64_t)m * nv) * 8;
    const int64_t mn = (int64_t)g.M * g.N;
    const float* p = parts + (int64_t)m * g.N + n;
    float f[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) f[j] = 0.0f;
    for (int sp = 0; sp < S; ++sp) {
        const f32x4 lo = __builtin_nontemporal_load((const f32x4*)(p + sp * mn));
        const f32x4 hi = __builtin_nontemporal_load((const f32x4*)(p + sp * mn + 4));
        f[0] += lo.x; f[1] += lo.y; f[2] += lo.z; f[3] += lo.w;
        f[4] += hi.x; f[5] += hi.y; f[6] += hi.z; f[7] += hi.w;
    }
    const int mb = m - g.band_row0;
    if (mb < 0 || mb >= g.band_rows) {
        if (g.c_full != nullptr) st_stream((u32x4*)(g.c_full + (int64_t)m * g.N + n), pack8(f));
        return;
    }
    const int64_t off = (int64_t)mb * g.N + n;
    if (!g.out_is_fp32) unpack8(pack8(f), f);   // the one-pass kernel rounds the product on its way to the epilogue
    for (int q = 0; q < g.n_peers; ++q) add8(ld_stream((const u32x4*)((const uint16_t*)g.peer.p[q] + off)), f);
    if (g.bias != nullptr) add8(*(const u32x4*)(g.bias + n), f);
    if (g.out_is_fp32) {
        float* o = (float*)g.out + off;
        *(f32x4*)o = f32x4{f[0], f[1], f[2], f[3]};
        *(f32x4*)(o + 4) = f32x4{f[4], f[5], f[6], f[7]};
    } else {
        st_stream((u32x4*)((uint16_t*)g.out + off), pack8(f));
    }
}

template <int BM, int BN, int WM, int WN>
static hipError_t launch_gemm(const GemmArgs& g, bool b_nt, bool even, hipStream_t st) {
    constexpr int T = WM * WN * 64;
    constexpr int LDS = 2 * (BM + BN) * kRowBytes;
    const dim3 grid((unsigned)(g.tiles_m * g.tiles_n), (unsigned)g.k_splits), block(T);
#define KR_LAUNCH(NT, EV)                                                                             \
    do {                                                                                              \
        auto kfn = gemm_reduce_kernel<BM, BN, WM, WN, NT, EV>;                                        \
        static std::atomic<uint64_t> opted{0};                                                        \
        if (hipError_t e = lds_opt_in((const void*)kfn, LDS, opted); e != hipSuccess) return e;       \
        hipLaunchKernelGGL(kfn, grid, block, LDS, st, g);                                             \
    } while (0)
    if (b_nt) {
        if (even) KR_LAUNCH(true, true); else KR_LAUNCH(true, false);
    } else {
        if (even) KR_LAUNCH(false, true); else KR_LAUNCH(false, false);
    }
#undef KR_LAUNCH
    return hipGetLastError();
}

}  // namespace kr

using namespace kr;

// ---- split K loop: how many workgroups share a tile ------------------------------------------
// A tile's K loop is split when the tiles alone leave CUs empty: into as many parts as fill the
// 256 CUs once (measured on M = 128..1024, N = 6656, K = 4096 and 16384: 52 tiles -> 4 parts,
// 104 -> 2, 208 and more -> 1 were the fastest or within a few percent of it; more parts only
// add partial products to write and read), each with at least kMinSplitSteps k-steps of 64.
constexpr int kMaxSplits = 16;
constexpr int kMinSplitSteps = 8;
static int split_k_factor(int64_t tiles, int64_t K) {
    if (const int v = env_switches().gemm_splitk; v >= 1 && v <= kMaxSplits)   // testing and tuning
        return (int)std::min<int64_t>(v, std::max<int64_t>(1, (K + BK - 1) / BK));
    // (up to 256 tiles a second workgroup per tile still finds a place next to the first; it pays
    // once the K loop is long: 208 tiles at K = 16384 measured 197 -> 178 us, at K = 4096 54 -> 62 us)
    if (tiles > 128 && tiles <= 256 && K >= 12288) return 2;
    if (tiles <= 0 || tiles * 2 > 256) return 1;
    int64_t s = 256 / tiles;
    s = std::min<int64_t>(s, ((K + BK - 1) / BK) / kMinSplitSteps);
    s = std::min<int64_t>(s, kMaxSplits);
    return (int)std::max<int64_t>(s, 1);
}
// ---- 256x256 kernel: split of the last partial round ------------------------------------------
// 256 tiles run at a time (one per CU).  When the tile count leaves a last round that is at most
// 3/8 full and K is long enough, its tiles get S = 256 / tail workgroups each (at least kMinSplitSteps k-steps per
// part, at most kMaxTailSplits parts), which turns that round from a whole one into tail/256
// of one; the price is tail * S partial tiles of 256 KiB written and read once.
constexpr int kMaxTailSplits = 8;
static void tail_split_plan(int64_t tiles, int64_t K, int* tail_out, int* splits_out) {
    *tail_out = 0;
    *splits_out = 1;
    const int64_t force = env_switches().gemm_tailsplit;   // 0: off, n: n parts (testing)
    if (force == 0 || (tiles > 128 && tiles <= 256)) return;
    // up to 128 tiles the whole launch is one partial round
    const int64_t tail = tiles % 256;
    // (measured: 16..64 tail tiles gain 5-25 % from K = 4096 on; 128 tail tiles at K = 2048 lose
    // 12 %: half a round saved does not pay for two more launches and 64 MiB of parts)
    if (tail == 0 || (tail > 96 && tiles > 128) || (K < 4096 && force <= 0)) return;
    int64_t s = std::min<int64_t>(256 / tail, kMaxTailSplits);
    s = std::min<int64_t>(s, (K / 64) / kMinSplitSteps);
    if (force > 0) s = std::min<int64_t>(force, K / 64);
    if (s < 2) return;
    *tail_out = (int)tail;
    *splits_out = (int)s;
}
static int64_t gemm_dtl_tail_workspace_bytes(int tail_tiles, int splits) {
    return (int64_t)tail_tiles * splits * (256 * 256 * 4);
}

// Few rows, long K: whether the 256x256 kernel with every tile's K loop split (the whole launch
// treated as a partial round) beats the 128x128 kernel with its split.  Measured on N = 6656,
// M = 256 / 512 / 1024 (26 / 52 / 104 tiles), caches flushed: row-major B wins from K = 4096 on
// (M = 512, K = 16384: 200 -> 146 us; M = 1024, K = 32768: 622 -> 434 us) except 104 tiles at
// K = 4096; transposed-contiguous B only with much work per tile (52 tiles at K = 32768
// 308 -> 279 us, 104 tiles at K = 16384 287 -> 281 us; below that up to 15 % slower).
// (plain: a product without peers, band or second output.  There the finishing pass only sums and
// stores, and with the 16x16x32 kernels transposed B pays from 48 tiles and K = 8192 on: 52 tiles
// 99 -> 94 us, 104 tiles 144 -> 139 us; with a reduce-scatter epilogue the same shapes lose 5-10 %.)
static bool whole_launch_split_pays(int64_t M, int64_t N, int64_t K, bool b_nt, bool plain) {
    if (M <= 0 || N <= 0 || M % 256 != 0 || N % 256 != 0 || K % 64 != 0) return false;
    const int64_t tiles = (M / 256) * (N / 256);
    if (tiles < 24 || tiles > 128) return false;
    if (b_nt) return tiles * K >= (int64_t)52 * 32768 || (plain && tiles >= 48 && K >= 8192);
    return K >= 8192 || (K >= 4096 && tiles <= 64);
}

// workspace of the two-pass form: S fp32 partial products of the whole [M, N] result
static int64_t split_k_workspace_bytes(int64_t M, int64_t N, int S) { return (int64_t)S * M * N * 4; }

// ---- the workspace form for callers that cannot allocate ------------------------------------------
// The split-K workspace lives in a device array of the library instead of caller memory.  Host code
// never uses the array's name as an address: each device's copy is looked up once, with that device
// current, and the pointer kept is what the kernels get, exactly as they get the caller's workspace.
static __device__ __align__(256) unsigned char scratch[KR_STATIC_SCRATCH_BYTES];

constexpr int kMaxDevices = 64;
static int static_scratch(void** out) {
    static std::mutex mu;
    static void* ptr_of_device[kMaxDevices] = {};
    int dev = -1;
    if (hipError_t e = hipGetDevice(&dev); e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= kMaxDevices) return (int)hipErrorInvalidDevice;
    std::lock_guard<std::mutex> lock(mu);
    if (ptr_of_device[dev] == nullptr) {
        void* ptr = nullptr;
        if (hipError_t e = hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch)); e != hipSuccess) return (int)e;
        if (ptr == nullptr) return (int)hipErrorInvalidSymbol;
        ptr_of_device[dev] = ptr;
    }
    *out = ptr_of_device[dev];
    return KR_OK;
}

// ---- which kernel a call gets ----------------------------------------------------------------
// One place decides it, for the launch and for kr_gemm_plan (which reports the decision).
struct GemmPlan {
    int tile;            // 256: LDS-DMA kernel (gemm_dtl.hip); 128: register-staged kernel (this file)
    int mi16;            // 256x256 kernel: k loop on 16x16x32 blocks (else 32x32x16)
    int peers_on_mfma;   // 256x256 kernel, 32x32x16 form: whole-band tiles add their peers on the matrix cores
    int group_n;         // column panels per scheduling group
    int tail_tiles;      // 256x256 kernel: tiles of the last partial round that are split ...
    int tail_splits;     // ... into this many parts each
    int splits;          // 128x128 kernel: workgroups per tile (split K loop), 1 = one pass
    int n224;            // 256x224 tiles instead of 256x256 (whole rounds of compute units where those leave a partial one)
};
static GemmPlan plan_gemm(int64_t M, int64_t N, int64_t K, bool b_nt, int n_peers, int64_t band_rows, bool plain,
                          bool plain_bf16_all_rows, bool has_workspace, int64_t workspace_bytes, bool has_gather, bool has_progress, bool flagged,
                          bool dtl_ok) {
    GemmPlan p{};
    // Tile choice: the 256x256 tile of the LDS-DMA kernel (4 waves x 128x128) has the highest
    // MFMA work per LDS/HBM byte; it needs K % 64 == 0 and a K loop long enough to amortise
    // its epilogue.  Otherwise 128x128 tiles, two of which share a CU so that one
    // tile's epilogue overlaps the other's MFMAs; they also win while all of them fit on the
    // 256 CUs at once (512 tiles = 128 of the large ones): measured, the large tile is 15-30 %
    // faster from 144 tiles on and 5-10 % slower at 128, for K from 1024 to 8192.
    bool big = ((M + 255) / 256) * ((N + 255) / 256) > 128 && K >= 256;
    // (few rows and a long K loop: the large tile again, with every tile's K loop split)
    if (!big && has_workspace && !has_gather && whole_launch_split_pays(M, N, K, b_nt, plain)) {
        int tail, ts;
        tail_split_plan((M / 256) * (N / 256), K, &tail, &ts);
        big = tail > 0 && gemm_dtl_tail_workspace_bytes(tail, ts) <= workspace_bytes;
    }
    // KRAKEN_AMD_GEMM_TILE=128|256 overrides the choice (testing and tuning)
    if (env_switches().gemm_tile == 128) big = false;
    if (env_switches().gemm_tile == 256) big = true;
    const bool dtl = big && dtl_ok;
    p.tile = dtl ? 256 : 128;
    // KRAKEN_AMD_GEMM_PEERS=epilogue keeps the peers' partial sums out of the matrix cores
    // (they are then added in the epilogue, where a non-finite value stays in its element)
    p.peers_on_mfma = 1;
    if (env_switches().gemm_peers >= 0) p.peers_on_mfma = env_switches().gemm_peers;
    // MFMA block shape of the 256x256 kernel: 16x16x32 draws less power per flop than 32x32x16 and
    // the chip is power-limited (k loop 5-10 % faster with warm operands; results agree to fp32
    // rounding), and its peer phase takes two peers per MFMA.  KRAKEN_AMD_GEMM_MFMA=16|32 overrides.
    p.mi16 = 1;
    if (env_switches().gemm_mfma > 0) p.mi16 = env_switches().gemm_mfma == 16;
    const int bm = p.tile;
    const int64_t tiles_m = (M + bm - 1) / bm, tiles_n = (N + bm - 1) / bm;
    // Column panels per scheduling group: the tiles an XCD runs at a time form a block that is
    // group_n panels wide.  8 measured best for the compute-bound shapes; where most tiles also
    // stream the peers' partial sums (HBM-bound), 16 lets neighbouring CUs read longer runs of
    // the same rows at about the same time.
    // (transposed-contiguous B: 4 measured 1-3 % ahead of 8 on 8192x3584x8192 and on the K = 16384
    // shapes with N = 6656, level elsewhere; row-major B: 8 and 4 level)
    p.group_n = (n_peers > 0 && band_rows * 2 >= M) ? 16 : (b_nt ? 4 : 8);
    // Rows that arrive while the kernel runs: narrow groups, so that the range of tiles each XCD
    // walks spans all row blocks in the order of their arrival (every XCD then starts on the
    // local shard and waits little); with wide groups the XCDs that own the last blocks idle
    // until those have arrived.
    // The same for row bands that are flagged as they complete: every XCD then moves from band to
    // band in the order of the destinations, and a band is complete once all eight have passed it
    // (with wide groups every band would only be complete when the last group is).
    if (flagged) p.group_n = (int)((tiles_n + kXcds - 1) / kXcds);
    if (const int v = env_switches().gemm_group; v >= 1 && v <= 64) p.group_n = v;
    // 256x256 kernel: the last partial round of tiles, split over the idle CUs (workspace given)
    p.tail_tiles = 0;
    p.tail_splits = 1;
    if (dtl && has_workspace && !has_progress && M % 256 == 0 && N % 256 == 0) {
        int tail, ts;
        tail_split_plan(tiles_m * tiles_n, K, &tail, &ts);
        if (tail > 0 && gemm_dtl_tail_workspace_bytes(tail, ts) <= workspace_bytes) {
            p.tail_tiles = tail;
            p.tail_splits = ts;
        }
    }
    // 256x224 tiles: a plain product (no peers, bias, band or second output; bf16 result, which the
    // caller vouches for) with transposed-contiguous B whose columns 224 divides, when that tiling
    // needs fewer column-units of work than 256-column tiles rounded up to whole rounds of the
    // 256 compute units (8192 x 3584: 448 tiles = 2 rounds of 256 columns against 512 tiles = 2
    // rounds of 224: measured 340 -> 320 us at K = 8192); a 224-column tile costs about 3 % more
    // per flop (A is read from LDS and L2 for fewer columns).  KRAKEN_AMD_GEMM_N224=0|1 overrides.
    // (An A that arrives while the kernel runs is fine: the tile waits for its rows' flags before its
    // first load, whatever its width.)
    p.n224 = 0;
    if (dtl && p.mi16 && b_nt && plain && plain_bf16_all_rows && M % 256 == 0 && N % 224 == 0) {
        const int64_t t8 = tiles_m * tiles_n, t7 = (M / 256) * (N / 224);
        const double cost8 = (double)((t8 + 255) / 256) * 256.0, cost7 = (double)((t7 + 255) / 256) * 224.0 * 1.03;
        bool use = cost7 < cost8;
        if (env_switches().gemm_n224 >= 0) use = env_switches().gemm_n224 != 0;
        if (use) {
            p.n224 = 1;
            p.tail_tiles = 0;
            p.tail_splits = 1;
        }
    }
    // Split K loop (128x128 kernel, workspace given): with few tiles most CUs would idle, so S
    // workgroups share a tile's K loop and meet in the workspace.
    p.splits = 1;
    if (!dtl && has_workspace) {
        p.splits = split_k_factor(tiles_m * tiles_n, K);
        if (p.splits > 1 && split_k_workspace_bytes(M, N, p.splits) > workspace_bytes) p.splits = 1;
    }
    return p;
}

// Everything kr_gemm_reduce_noalloc_bf16 would otherwise do on its first call on a device: loads
// the library's code for the current device (a lazily loaded code object is what allocates the
// device memory of the scratch array) and looks the array up.
extern "C" int kr_init(void) {
    void* p = nullptr;
    return static_scratch(&p);
}

// What the kernel exchanges with other streams while it runs (null pointer to gemm_reduce:
// nothing): the arrival flags of the all-gather matmul (progress == nullptr: A is complete) and
// the per-band counters of the producer GEMM (band_counter == nullptr: none).
struct GatherSpec {
    const void* a_local;
    int64_t lda_local;
    int64_t local_row0, local_rows;
    const uint32_t* progress;
    int64_t comm_rows;
    int64_t wait_limit_us;
    int* status;
    uint32_t* band_counter;
    uint32_t* band_signal;
    int64_t count_rows;
};

// Everything of the entry points except the peers: argument checks in the documented
// order, then tile choice and launch.  `peers_given` is the stacked base or the table.
static int gemm_reduce(const void* A, int64_t lda_m, int64_t lda_k, const void* B, int64_t ldb_k, int64_t ldb_n,
                       int64_t M, int64_t N, int64_t K, const void* peers_given, int n_peers,
                       const void* const* peer_ptrs, int64_t peers_stride, const void* bias,
                       int64_t band_row0, int64_t band_rows, void* c_full, void* out, int out_is_fp32,
                       int64_t tile_pivot, void* stream, const GatherSpec* gather = nullptr,
                       void* workspace = nullptr, int64_t workspace_bytes = 0, bool static_ws = false) {
    if (M < 0 || N < 0 || K < 0 || M > 0x7fffffffLL || N > 0x7fffffffLL || K > 0x7fffffffLL)
        return KR_ERR_BAD_DIM;
    if (n_peers < 0 || n_peers >= KR_MAX_WORLD) return KR_ERR_WORLD_SIZE;
    if (band_row0 < 0 || band_rows < 0 || band_row0 + band_rows > M) return KR_ERR_BAND;
    if (K % 8 != 0 || N % 8 != 0) return KR_ERR_NUMEL_MOD8;
    if (M == 0 || N == 0) return KR_OK;
    if (K == 0) return KR_ERR_BAD_DIM;
    if (A == nullptr || B == nullptr) return KR_ERR_NULL_POINTER;
    if (band_rows > 0 && out == nullptr) return KR_ERR_NULL_POINTER;
    if (n_peers > 0 && peers_given == nullptr) return KR_ERR_NULL_POINTER;
    if (lda_k != 1) return KR_ERR_LAYOUT;
    const bool b_nt = (ldb_k == 1 && (ldb_n != 1 || N == 1));
    if (!b_nt && ldb_n != 1) return KR_ERR_LAYOUT;
    const int64_t ldb = b_nt ? ldb_n : ldb_k;
    if (lda_m < K || (b_nt ? ldb < K : ldb < N)) return KR_ERR_LAYOUT;
    if (lda_m % 8 != 0 || ldb % 8 != 0) return KR_ERR_ALIGNMENT;
    if (!aligned16(A) || !aligned16(B) || !aligned16(bias) || !aligned16(c_full) || !aligned16(out))
        return KR_ERR_ALIGNMENT;
    // (arguments are checked; a shape that is split now gets the library's own workspace)
    if (static_ws && kr_gemm_workspace_bytes(M, N, K) > KR_STATIC_SCRATCH_BYTES) return KR_ERR_SCRATCH;
    if (static_ws && kr_gemm_workspace_bytes(M, N, K) > 0) {
        const int rc = static_scratch(&workspace);
        if (rc != KR_OK) return rc;
        workspace_bytes = KR_STATIC_SCRATCH_BYTES;
    }

    GemmArgs g;
    if (peer_ptrs != nullptr) {
        // separate allocations: a table of n_peers device pointers
        const int rc = n_peers > 0 ? peer_tab_from_ptrs(g.peer, peer_ptrs, n_peers) : KR_OK;
        if (rc != KR_OK) return rc;
        if (n_peers == 0) peer_tab_stacked(g.peer, A, 0, 0);
    } else {
        if (peers_stride % 8 != 0 || !aligned16(peers_given)) return KR_ERR_ALIGNMENT;
        if (n_peers > 0 && peers_stride < band_rows * N) return KR_ERR_BAD_DIM;
        peer_tab_stacked(g.peer, n_peers > 0 ? peers_given : A, n_peers, peers_stride);
    }
    g.A = (const uint16_t*)A;
    g.B = (const uint16_t*)B;
    g.lda = lda_m;
    g.ldb = ldb;
    g.M = (int)M; g.N = (int)N; g.K = (int)K;
    g.n_peers = n_peers;
    g.progress = nullptr;
    g.comm_rows = 1;
    g.a_local = nullptr;
    g.lda_local = 0;
    g.local_row0 = g.local_rows = 0;
    g.wait_ticks = 0;
    g.status = nullptr;
    if (gather != nullptr && gather->progress != nullptr) {
        g.progress = gather->progress;
        g.comm_rows = (int)gather->comm_rows;
        g.a_local = (const uint16_t*)gather->a_local;
        g.lda_local = gather->lda_local;
        g.local_row0 = (int)gather->local_row0;
        g.local_rows = (int)gather->local_rows;
        g.wait_ticks = (uint64_t)gather->wait_limit_us * 100u;   // 100 MHz constant clock
        g.status = gather->status;
    }
    g.band_counter = nullptr;
    g.band_signal = nullptr;
    g.count_rows = 1;
    if (gather != nullptr && gather->band_counter != nullptr) {
        g.band_counter = gather->band_counter;
        g.band_signal = gather->band_signal;
        g.count_rows = (int)gather->count_rows;
    }
    g.bias = (const uint16_t*)bias;
    g.band_row0 = (int)band_row0;
    g.band_rows = (int)band_rows;
    g.c_full = (uint16_t*)c_full;
    g.out = out;
    g.out_is_fp32 = out_is_fp32;
    g.out_fp8 = 0;

    const GemmPlan plan = plan_gemm(M, N, K, b_nt, n_peers, band_rows, n_peers == 0 && c_full == nullptr && bias == nullptr,
                                    !out_is_fp32 && band_row0 == 0 && band_rows == M, workspace != nullptr, workspace_bytes, gather != nullptr, g.progress != nullptr,
                                    g.progress != nullptr || g.band_counter != nullptr,
                                    gemm_dtl_supported(g) && (g.a_local == nullptr || (int64_t)256 * g.lda_local * 2 < 0x7fffffffLL));
    const bool dtl = plan.tile == 256;
    // The 128x128 kernel addresses a tile's operand panels with 32-bit byte offsets from the
    // panel's first row (through a 2 GiB buffer descriptor): row strides beyond that reach are
    // refused rather than read as zeros.
    if (!dtl) {
        const int64_t reach = std::max<int64_t>(std::max(lda_m, ldb), g.a_local != nullptr ? g.lda_local : 0);
        if ((128 * reach + std::max(K, N)) * 2 >= 0x7fffffffLL) return KR_ERR_LAYOUT;
    }
    g.peers_on_mfma = plan.peers_on_mfma;
    g.mi16 = plan.mi16;
    g.n224 = plan.n224;
    const int bm = plan.tile, bn = plan.n224 ? 224 : bm;
    g.tiles_m = (int)((M + bm - 1) / bm);
    g.tiles_n = (int)((N + bn - 1) / bn);
    if ((int64_t)g.tiles_m * g.tiles_n > 0x7fffffffLL) return KR_ERR_BAD_DIM;
    g.group_n = plan.group_n;
    g.k_splits = 1;
    g.split_out_stride = 0;
    g.tail_tiles = 0;
    if (plan.tail_tiles > 0) {
        if (!aligned16(workspace)) return KR_ERR_ALIGNMENT;
        g.tail_tiles = plan.tail_tiles;
        g.k_splits = plan.tail_splits;
    }
    const int splits = plan.splits;
    if (splits > 1 && !aligned16(workspace)) return KR_ERR_ALIGNMENT;
    int64_t pt = tile_pivot / bm;
    g.pivot_tiles = (int)(((pt % g.tiles_m) + g.tiles_m) % g.tiles_m);
    const bool even = (M % bm == 0 && N % bn == 0 && K % BK == 0);
    if (splits > 1) {
        // pass 1: S partial products, fp32, no epilogue work; pass 2: sum + epilogue
        GemmArgs g1 = g;
        g1.k_splits = splits;
        g1.split_out_stride = M * N;
        g1.out = workspace;
        g1.out_is_fp32 = 1;
        g1.n_peers = 0;
        g1.bias = nullptr;
        g1.band_row0 = 0;
        g1.band_rows = (int)M;
        g1.c_full = nullptr;
        hipError_t e = launch_gemm<128, 128, 2, 2>(g1, b_nt, even, (hipStream_t)stream);
        if (e != hipSuccess) return (int)e;
        const int64_t vecs = M * (N / 8);
        hipLaunchKernelGGL(splitk_finish_kernel, dim3((unsigned)((vecs + 255) / 256)), dim3(256), 0,
                           (hipStream_t)stream, g, (const float*)workspace, splits);
        return (int)hipGetLastError();
    }
    hipError_t e = dtl ? launch_gemm_dtl(g, b_nt, (hipStream_t)stream, workspace)
                       : launch_gemm<128, 128, 2, 2>(g, b_nt, even, (hipStream_t)stream);
    return (int)e;
}

extern "C" int kr_gemm_reduce_bf16(const void* A, int64_t lda_m, int64_t lda_k, const void* B, int64_t ldb_k,
                                   int64_t ldb_n, int64_t M, int64_t N, int64_t K, const void* peers,
                                   int n_peers, int64_t peers_stride, const void* bias, int64_t band_row0,
                                   int64_t band_rows, void* c_full, void* out, int out_is_fp32,
                                   int64_t tile_pivot, void* stream) {
    return gemm_reduce(A, lda_m, lda_k, B, ldb_k, ldb_n, M, N, K, peers, n_peers, nullptr, peers_stride, bias,
                       band_row0, band_rows, c_full, out, out_is_fp32, tile_pivot, stream);
}

extern "C" int kr_gemm_reduce_ptrs_bf16(const void* A, int64_t lda_m, int64_t lda_k, const void* B,
                                        int64_t ldb_k, int64_t ldb_n, int64_t M, int64_t N, int64_t K,
                                        const void* const* peers, int n_peers, const void* bias,
                                        int64_t band_row0, int64_t band_rows, void* c_full, void* out,
                                        int out_is_fp32, int64_t tile_pivot, void* stream) {
    // an empty table with n_peers == 0 is a plain GEMM; the flag below still selects the table path
    static const void* const kNoPeers[1] = {nullptr};
    return gemm_reduce(A, lda_m, lda_k, B, ldb_k, ldb_n, M, N, K, peers, n_peers,
                       peers != nullptr ? peers : kNoPeers, 0, bias, band_row0, band_rows, c_full, out,
                       out_is_fp32, tile_pivot, stream);
}

extern "C" int kr_all_gather_matmul_bf16(const void* A, int64_t lda_m, const void* A_local, int64_t lda_local,
                                         const void* B, int64_t ldb_k, int64_t ldb_n, int64_t M, int64_t N,
                                         int64_t K, int W, int rank, int splits_per_rank,
                                         const uint32_t* progress, int64_t wait_limit_us, int32_t* status,
                                         void* C, void* stream) {
    if (W < 1 || W > KR_MAX_WORLD) return KR_ERR_WORLD_SIZE;
    if (rank < 0 || rank >= W || splits_per_rank < 1) return KR_ERR_STRIPE;
    if (M < 0 || M % ((int64_t)W * splits_per_rank) != 0) return KR_ERR_BAND;
    if (A_local != nullptr && (!aligned16(A_local) || lda_local % 8 != 0)) return KR_ERR_ALIGNMENT;
    if (A_local != nullptr && lda_local < K) return KR_ERR_LAYOUT;
    if ((reinterpret_cast<uintptr_t>(progress) & 3u) != 0 || (reinterpret_cast<uintptr_t>(status) & 3u) != 0)
        return KR_ERR_ALIGNMENT;
    GatherSpec gs{};
    gs.a_local = A_local;
    gs.lda_local = lda_local;
    gs.local_rows = M / W;
    gs.local_row0 = gs.local_rows * rank;
    gs.progress = progress;
    gs.comm_rows = M > 0 ? M / ((int64_t)W * splits_per_rank) : 1;
    gs.wait_limit_us = wait_limit_us > 0 ? wait_limit_us : 5000000;   // 5 s
    gs.status = status;
    // no reduce: the band is every row, no peers, no bias; tile order rotated to the local shard
    return gemm_reduce(A, lda_m, 1, B, ldb_k, ldb_n, M, N, K, nullptr, 0, nullptr, 0, nullptr, 0, M, nullptr, C, 0,
                       gs.local_row0, stream, &gs);
}

extern "C" int kr_gemm_producer_bf16(const void* A, int64_t lda_m, int64_t lda_k, const void* B, int64_t ldb_k,
                                     int64_t ldb_n, int64_t M, int64_t N, int64_t K, void* C, int W, int rank,
                                     uint32_t* progress, uint32_t* signal_pad, void* stream) {
    if (W < 1 || W > KR_MAX_WORLD) return KR_ERR_WORLD_SIZE;
    if (rank < 0 || rank >= W) return KR_ERR_BAND;
    if (M < 0 || M % W != 0) return KR_ERR_BAD_DIM;
    if (progress == nullptr || signal_pad == nullptr || (M > 0 && N > 0 && C == nullptr)) return KR_ERR_NULL_POINTER;
    if ((reinterpret_cast<uintptr_t>(progress) & 3u) != 0 || (reinterpret_cast<uintptr_t>(signal_pad) & 3u) != 0)
        return KR_ERR_ALIGNMENT;
    GatherSpec ps{};
    ps.band_counter = progress;
    ps.band_signal = signal_pad;
    ps.count_rows = M > 0 ? M / W : 1;
    // no reduce band: every row of C goes to `C`; tile order rotated to the band of rank + 1
    return gemm_reduce(A, lda_m, lda_k, B, ldb_k, ldb_n, M, N, K, nullptr, 0, nullptr, 0, nullptr, 0, 0, C, nullptr,
                       0, ((int64_t)(rank + 1) % W) * (M / W), stream, &ps);
}

// Product of fp8 (e4m3fn) operands on the fp8 matrix-core instruction (all_gather_matmul.py:53,121,213: fp8 shards and
// weight, fp8 result).  The kernel is the 256x256 LDS-DMA kernel with its k-step on 16x16x128 blocks; it reads the operands
// as matrices of two-byte units, hence the halved K and row strides below.  `gather`: rows of A that arrive while the
// kernel runs (flags, local shard), as for the bf16 all-gather matmul.
static int gemm_fp8(const void* A, int64_t lda, const void* Bt, int64_t ldb, int64_t M, int64_t N, int64_t K,
                    void* out, int out_kind, void* stream, const GatherSpec* gather) {
    if (M < 0 || N < 0 || K < 0 || M > 0x7fffffffLL || N > 0x7fffffffLL || K > 0x7fffffffLL) return KR_ERR_BAD_DIM;
    if (out_kind < 0 || out_kind > 2) return KR_ERR_BAD_DIM;
    if (M % 256 != 0 || N % 256 != 0 || K % 128 != 0) return KR_ERR_BAD_DIM;
    if (M == 0 || N == 0) return KR_OK;
    if (K == 0) return KR_ERR_BAD_DIM;
    if (A == nullptr || Bt == nullptr || out == nullptr) return KR_ERR_NULL_POINTER;
    if (lda < K || ldb < K) return KR_ERR_LAYOUT;
    if (lda % 16 != 0 || ldb % 16 != 0 || !aligned16(A) || !aligned16(Bt) || !aligned16(out)) return KR_ERR_ALIGNMENT;
    GemmArgs g{};
    peer_tab_stacked(g.peer, A, 0, 0);
    g.A = (const uint16_t*)A;
    g.B = (const uint16_t*)Bt;
    g.lda = lda / 2;
    g.ldb = ldb / 2;
    g.M = (int)M; g.N = (int)N; g.K = (int)(K / 2);
    g.comm_rows = 1;
    g.count_rows = 1;
    int64_t pivot_row = 0;
    if (gather != nullptr && gather->progress != nullptr) {
        g.progress = gather->progress;
        g.comm_rows = (int)gather->comm_rows;
        g.a_local = (const uint16_t*)gather->a_local;
        g.lda_local = gather->lda_local / 2;
        g.local_row0 = (int)gather->local_row0;
        g.local_rows = (int)gather->local_rows;
        g.wait_ticks = (uint64_t)gather->wait_limit_us * 100u;   // 100 MHz constant clock
        g.status = gather->status;
    }
    if (gather != nullptr) pivot_row = gather->local_row0;
    if (!gemm_dtl_supported(g) || (g.a_local != nullptr && (int64_t)256 * g.lda_local * 2 >= 0x7fffffffLL)) return KR_ERR_LAYOUT;
    g.band_row0 = 0;
    g.band_rows = (int)M;
    g.out = out;
    g.out_is_fp32 = out_kind == 1;
    g.out_fp8 = out_kind == 2;
    g.tiles_m = (int)(M / 256);
    g.tiles_n = (int)(N / 256);
    g.pivot_tiles = (int)((pivot_row / 256) % g.tiles_m);
    g.group_n = env_switches().gemm_group > 0 ? env_switches().gemm_group : 4;
    g.k_splits = 1;
    g.mi16 = 1;
    return (int)launch_gemm_dtl8(g, (hipStream_t)stream);
}

extern "C" int kr_gemm_fp8(const void* A, int64_t lda, const void* Bt, int64_t ldb, int64_t M, int64_t N, int64_t K,
                           void* out, int out_kind, void* stream) {
    return gemm_fp8(A, lda, Bt, ldb, M, N, K, out, out_kind, stream, nullptr);
}

extern "C" int kr_all_gather_matmul_fp8(const void* A, int64_t lda, const void* A_local, int64_t lda_local, const void* Bt,
                                        int64_t ldb, int64_t M, int64_t N, int64_t K, int W, int rank, int splits_per_rank,
                                        const uint32_t* progress, int64_t wait_limit_us, int32_t* status, void* out,
                                        int out_kind, void* stream) {
    if (W < 1 || W > KR_MAX_WORLD) return KR_ERR_WORLD_SIZE;
    if (rank < 0 || rank >= W || splits_per_rank < 1) return KR_ERR_STRIPE;
    if (M < 0 || M % ((int64_t)W * splits_per_rank) != 0) return KR_ERR_BAND;
    if (A_local != nullptr && (!aligned16(A_local) || lda_local % 16 != 0)) return KR_ERR_ALIGNMENT;
    if (A_local != nullptr && lda_local < K) return KR_ERR_LAYOUT;
    if ((reinterpret_cast<uintptr_t>(progress) & 3u) != 0 || (reinterpret_cast<uintptr_t>(status) & 3u) != 0)
        return KR_ERR_ALIGNMENT;
    GatherSpec gs{};
    gs.a_local = A_local;
    gs.lda_local = lda_local;
    gs.local_rows = M / W;
    gs.local_row0 = gs.local_rows * rank;
    gs.progress = progress;
    gs.comm_rows = M > 0 ? M / ((int64_t)W * splits_per_rank) : 1;
    gs.wait_limit_us = wait_limit_us > 0 ? wait_limit_us : 5000000;   // 5 s
    gs.status = status;
    return gemm_fp8(A, lda, Bt, ldb, M, N, K, out, out_kind, stream, &gs);
}

extern "C" int kr_gemm_plan(int64_t M, int64_t N, int64_t K, int b_transposed, int n_peers, int64_t band_rows,
                            int has_bias, int has_c_full, int64_t workspace_bytes, int32_t plan[8]) {
    if (plan == nullptr) return KR_ERR_NULL_POINTER;
    if (M <= 0 || N <= 0 || K <= 0 || M > 0x7fffffffLL || N > 0x7fffffffLL || K > 0x7fffffffLL) return KR_ERR_BAD_DIM;
    if (n_peers < 0 || n_peers >= KR_MAX_WORLD) return KR_ERR_WORLD_SIZE;
    if (band_rows < 0 || band_rows > M) return KR_ERR_BAND;
    // contiguous operands: the only other input of the choice is whether the 256-row panels stay
    // within the 2 GiB reach of a buffer descriptor
    GemmArgs g{};
    g.K = (int)K;
    g.lda = K;
    g.ldb = b_transposed ? K : N;
    const GemmPlan p = plan_gemm(M, N, K, b_transposed != 0, n_peers, band_rows, n_peers == 0 && !has_c_full && !has_bias,
                                 band_rows == M, workspace_bytes > 0, workspace_bytes, false, false, false, gemm_dtl_supported(g));
    const bool whole_band_peers = p.tile == 256 && n_peers > 0 && p.peers_on_mfma != 0;
    plan[0] = p.tile;
    plan[1] = p.tile == 256 ? (p.mi16 ? 16 : 32) : 32;   // MFMA block rows: 16x16x32 or 32x32x16
    plan[2] = p.splits;
    plan[3] = p.tail_tiles;
    plan[4] = p.tail_splits;
    plan[5] = p.group_n;
    plan[6] = whole_band_peers ? 1 : 0;
    plan[7] = (M % p.tile != 0 || N % p.tile != 0) ? 1 : 0;
    if (p.n224) plan[7] |= 2;   // bit 1: 256 x 224 tiles
    return KR_OK;
}

extern "C" int64_t kr_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K) {
    if (M <= 0 || N <= 0 || K <= 0) return 0;
    // the large-tile kernel (same rule as the launch; strides are not known here)
    const int force_tile = env_switches().gemm_tile;
    bool big = ((M + 255) / 256) * ((N + 255) / 256) > 128 && K >= 256;
    if (force_tile == 128) big = false;
    if (force_tile == 256) big = true;
    if (big && K % 64 == 0 && K >= 64) {
        if (M % 256 != 0 || N % 256 != 0) return 0;
        int tail, ts;
        tail_split_plan((M / 256) * (N / 256), K, &tail, &ts);
        return tail > 0 ? gemm_dtl_tail_workspace_bytes(tail, ts) : 0;
    }
    const int64_t tiles = ((M + 127) / 128) * ((N + 127) / 128);
    const int S = split_k_factor(tiles, K);
    int64_t bytes = S > 1 ? split_k_workspace_bytes(M, N, S) : 0;
    // the layout of B is not known here: enough for either kernel
    if (force_tile < 0 && (whole_launch_split_pays(M, N, K, true, true) || whole_launch_split_pays(M, N, K, false, true))) {
        int tail, ts;
        tail_split_plan((M / 256) * (N / 256), K, &tail, &ts);
        if (tail > 0) bytes = std::max(bytes, gemm_dtl_tail_workspace_bytes(tail, ts));
    }
    return bytes;
}

extern "C" int kr_gemm_reduce_ws_bf16(const void* A, int64_t lda_m, int64_t lda_k, const void* B, int64_t ldb_k,
                                      int64_t ldb_n, int64_t M, int64_t N, int64_t K, const void* peers,
                                      int n_peers, int64_t peers_stride, const void* bias, int64_t band_row0,
                                      int64_t band_rows, void* c_full, void* out, int out_is_fp32,
                                      int64_t tile_pivot, void* workspace, int64_t workspace_bytes,
                                      void* stream) {
    return gemm_reduce(A, lda_m, lda_k, B, ldb_k, ldb_n, M, N, K, peers, n_peers, nullptr, peers_stride, bias,
                       band_row0, band_rows, c_full, out, out_is_fp32, tile_pivot, stream, nullptr, workspace,
                       workspace_bytes);
}

extern "C" int kr_gemm_reduce_ptrs_ws_bf16(const void* A, int64_t lda_m, int64_t lda_k, const void* B,
                                           int64_t ldb_k, int64_t ldb_n, int64_t M, int64_t N, int64_t K,
                                           const void* const* peers, int n_peers, const void* bias,
                                           int64_t band_row0, int64_t band_rows, void* c_full, void* out,
                                           int out_is_fp32, int64_t tile_pivot, void* workspace,
                                           int64_t workspace_bytes, void* stream) {
    static const void* const kNoPeers[1] = {nullptr};
    return gemm_reduce(A, lda_m, lda_k, B, ldb_k, ldb_n, M, N, K, peers, n_peers,
                       peers != nullptr ? peers : kNoPeers, 0, bias, band_row0, band_rows, c_full, out,
                       out_is_fp32, tile_pivot, stream, nullptr, workspace, workspace_bytes);
}

extern "C" int kr_gemm_reduce_noalloc_bf16(const void* A, int64_t lda_m, int64_t lda_k, const void* B,
                                           int64_t ldb_k, int64_t ldb_n, int64_t M, int64_t N, int64_t K,
                                           const void* peers, int n_peers, int64_t peers_stride,
                                           const void* bias, int64_t band_row0, int64_t band_rows,
                                           void* c_full, void* out, int out_is_fp32, int64_t tile_pivot,
                                           void* stream) {
    return gemm_reduce(A, lda_m, lda_k, B, ldb_k, ldb_n, M, N, K, peers, n_peers, nullptr, peers_stride, bias,
                       band_row0, band_rows, c_full, out, out_is_fp32, tile_pivot, stream, nullptr, nullptr, 0,
                       /*static_ws=*/true);
}
