// bf16 GEMM main loop with direct global->LDS loads ("LDS DMA") for shapes the 256x256 tile
// divides:  M % 256 == 0, N % 256 == 0, K % 32 == 0.
//
// Workgroup tile 256 x 256, four wavefronts (2 x 2), each owning 128 x 128 of C as 4 x 4
// v_mfma_f32_32x32x16_bf16 accumulators (256 AGPRs).  The k loop advances 32 at a time; the
// operand tiles of four k-steps live in a ring of LDS stages (A: 4 x 16 KiB at 0, B: 4 x 16 KiB
// at 64 KiB) that is filled by buffer_load ... lds: the data never passes through VGPRs, no
// ds_write is issued, and a tile is requested three k-steps before it is used.
//
// LDS layouts (per stage)
//   A and transposed-contiguous B: [256 rows][64 B] (32 k), the four 16-byte chunks of a row
//     XOR-swizzled with (row >> 2) & 3.  One wave-wide LDS-DMA load fills 16 rows (1 KiB,
//     lane l -> row l/4, chunk slot l%4); the 128-bit fragment reads of 16 consecutive rows
//     then touch all 64 banks once.
//   row-major B: [32 k][512 B] (256 n), the 16-byte pieces of a k-row XOR-swizzled with
//     4*(k & 3): the 32 lanes of two neighbouring 16-lane blocks (4 k-rows x 32 columns) then
//     cover 16 different pieces = all 64 banks.  Fragments are read with ds_read_b64_tr_b16:
//     16 lanes read a 4(k) x 16(n) block, four n each, and the hardware hands lane i the four
//     k of column i -- two such reads give the eight k per lane the MFMA wants, with no
//     transpose in registers.
// A lane's fragment addresses differ between the 32x32 blocks, the two 16-wide k sub-steps
// and the stages only by compile-time constants, so they are immediate offsets on two (A),
// two (B transposed) or four (B row-major) address registers.
//
// The B fragment is the first MFMA operand and the A fragment the second, so the accumulators
// hold C transposed: a lane owns one row m and four consecutive columns n per register quad,
// which is what the fused epilogue (gemm_common.h) stores and what lets the partial sums of the
// other ranks be added by the matrix cores themselves (peer_phase below).
#include "gemm_common.h"

namespace kr {

namespace {

constexpr int BM = 256, BN = 256, WM = 2, WN = 2;
constexpr int WTM = BM / WM, WTN = BN / WN, TM = WTM / 32, TN = WTN / 32;
constexpr int BKD = 32;                       // k extent of one stage
constexpr int NSTAGE = 4;                     // LDS ring depth: tiles are requested NSTAGE-1 k-steps ahead
                                              // (a fifth stage, all 160 KiB, measured no faster)
constexpr int A_ST = BM * BKD * 2;            // 16 KiB
constexpr int B_ST = BN * BKD * 2;            // 16 KiB
constexpr uint32_t B_BASE = NSTAGE * A_ST;
constexpr int LDS_BYTES = NSTAGE * (A_ST + B_ST);
constexpr int LOADS_PER_TILE = 8;             // LDS-DMA loads per wave per k-step (4 A + 4 B)
constexpr int EP_WAVE = 32 * (WTN + 4) * 4;     // epilogue patch of a wave: 32 rows x WTN fp32, padded
static_assert(EP_WAVE * WM * WN <= LDS_BYTES, "epilogue patch must fit in the operand ring");

typedef __attribute__((address_space(3))) void* lds_void;
typedef const __attribute__((address_space(3))) bf16x8* lds_frag;
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) s16x4* lds_tr;

// s_waitcnt vmcnt(n) only (expcnt and lgkmcnt left at "no wait")
constexpr int vmcnt_imm(int n) { return (n & 15) | (7 << 4) | (15 << 8) | ((n >> 4) << 14); }
constexpr int kLgkm0 = 0xc07f;   // s_waitcnt lgkmcnt(0) only

// One workgroup tile.  PEERS_FIRST picks the order of the two accumulation phases (peers'
// partial sums, k loop) for tiles whose peers are added on the matrix cores.
template <bool B_NT, bool PEERS_FIRST>
__device__ __forceinline__ void gemm_dtl_tile(const GemmArgs& g, unsigned char* smem) {
    // Nothing is outstanding at kernel entry; saying so keeps the compiler's own wait-count
    // bookkeeping from carrying the pending loads and stores of the other copy of this code
    // (which never runs in the same workgroup) into this one, where it cannot see the LDS-DMA
    // loads retire them and would re-wait for them in every k-step.
    __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WN, wn = wave % WN;

    int tile_m, tile_n;
    tile_schedule(g, tile_m, tile_n);
    const int m0 = tile_m * BM, n0 = tile_n * BN;

    // ---- LDS-DMA addressing ----------------------------------------------------------------
    // A wave loads the 1 KiB chunks  wave, wave+4, wave+8, wave+12  of a stage.
    // A / transposed B: chunk = 16 rows; lane l -> row l/4, slot l%4 holds chunk slot ^ ((row>>2)&3).
    // Only the wave-uniform part (chunk row, k) changes between loads: it goes to the scalar
    // offset; the per-lane byte offset is computed once.
    const uint32_t a_voff_lane =
        (uint32_t)(((int64_t)(lane >> 2) * g.lda + (((lane & 3) ^ ((lane >> 4) & 3)) << 3)) * 2);
    uint32_t b_voff_lane;
    if (B_NT) {
        b_voff_lane = (uint32_t)(((int64_t)(lane >> 2) * g.ldb + (((lane & 3) ^ ((lane >> 4) & 3)) << 3)) * 2);
    } else {
        // row-major B: chunk = 2 k-rows of 512 B; lane l -> k-row l/32, piece slot l%32 holds piece
        // slot ^ 4*(k & 3); k & 3 = 2*(chunk & 1) + l/32 and chunk & 1 == wave & 1
        const int kq = ((wave & 1) << 1) | (lane >> 5);
        b_voff_lane = (uint32_t)(((int64_t)(lane >> 5) * g.ldb + (((lane & 31) ^ (kq << 2)) << 3)) * 2);
    }
    // Buffer resource descriptor: 48-bit base, stride 0 (raw), 2^31-1 bytes, 32-bit data format.
    typedef int i32x4 __attribute__((ext_vector_type(4)));
    auto make_rsrc = [](const void* base) {
        const uint64_t b = (uint64_t)base;
        return i32x4{(int)(uint32_t)b, (int)(uint32_t)((b >> 32) & 0xffff), 0x7fffffff, 0x00020000};
    };
    // The LDS-DMA load is issued through inline assembly on purpose: the compiler then does not
    // know that LDS is written behind its back and leaves the ordering to the explicit
    // s_waitcnt vmcnt / s_barrier pairs below (told about it, it waits for vmcnt(0) in front of
    // every transposing LDS read, which serialises the whole pipeline).
    auto lds_dma_b128 = [](i32x4 rsrc, uint32_t lds_addr, uint32_t voff, int soff) {
        // (one wait state between the scalar write of M0 and the LDS-DMA instruction that reads it)
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                     :
                     : "s"(lds_addr), "v"(voff), "s"(rsrc), "s"(soff)
                     : "memory", "m0");
    };
    // same with the non-temporal hint, for data that is read exactly once (the peers' sums)
    auto lds_dma_b128_stream = [](i32x4 rsrc, uint32_t lds_addr, uint32_t voff, int soff) {
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen nt lds"
                     :
                     : "s"(lds_addr), "v"(voff), "s"(rsrc), "s"(soff)
                     : "memory", "m0");
    };
    const i32x4 a_rsrc = make_rsrc(g.A + (int64_t)m0 * g.lda);
    const i32x4 bt_rsrc = make_rsrc(g.B + (int64_t)n0 * g.ldb);

    const int kt_total = g.K / BKD;
    // one LDS-DMA load of k-step t (clamped: the tail re-requests the last tile into a free stage)
    auto issue_load = [&](int t, uint32_t stage, int q) {
        // past the end nothing new is needed, but the per-step load count must not change (the
        // vmcnt arithmetic relies on it): every lane then re-reads the first 16 bytes of the
        // last tile's chunk into the free stage -- one cache line instead of a kilobyte
        const bool live = t < kt_total;
        const int tt = min(t, kt_total - 1);
        const int k0 = tt * BKD;
        const uint32_t a_voff = live ? a_voff_lane : 0u, b_voff = live ? b_voff_lane : 0u;
        const int ch = wave + 4 * (q & 3);
        if (q < 4) {
            lds_dma_b128(a_rsrc, stage * A_ST + ch * 1024, a_voff, (int)(((int64_t)16 * ch * g.lda + k0) * 2));
        } else if (B_NT) {
            lds_dma_b128(bt_rsrc, B_BASE + stage * B_ST + ch * 1024, b_voff,
                         (int)(((int64_t)16 * ch * g.ldb + k0) * 2));
        } else {
            // re-based on the first k-row of the step: the scalar offset stays small for any K
            lds_dma_b128(make_rsrc(g.B + (int64_t)k0 * g.ldb + n0), B_BASE + stage * B_ST + ch * 1024, b_voff,
                         (int)(((int64_t)2 * ch * g.ldb) * 2));
        }
    };

    // ---- fragment addressing -----------------------------------------------------------------
    // A (and transposed B): lane -> row (lane & 31) of the 32-row block, 8 k at chunk 2*ks + (lane>>5)
    const int frow = lane & 31, fkc = lane >> 5;
    const int fsw = (frow >> 2) & 3;            // same for all blocks: block rows differ by 32
    // byte address at ks = 0; ks = 1 flips bit 5 (chunk ^ 2)
    const uint32_t fa0 = (uint32_t)((wm * WTM + frow) * 64 + (((fsw & 2) | (fkc ^ (fsw & 1))) << 4));
    const uint32_t fa1 = fa0 ^ 32u;
    uint32_t fb[4];
    if (B_NT) {
        fb[0] = B_BASE + (uint32_t)((wn * WTN + frow) * 64 + (((fsw & 2) | (fkc ^ (fsw & 1))) << 4));
        fb[1] = fb[0] ^ 32u;
        fb[2] = fb[3] = 0;
    } else {
        // transposing read: 16-lane block b = lane/16, i = lane%16 reads k-row 8*(b>>1) + i/4,
        // columns 16*(b&1) + 4*(i%4) .. +3 of the 32-column block j
        const int b = lane >> 4, i = lane & 15;
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int nl = wn * WTN + j * 32 + 16 * (b & 1) + 4 * (i & 3);
            const int kr = 8 * (b >> 1) + (i >> 2);
            const int piece = (nl >> 3) ^ (((i >> 2) & 3) << 2);
            fb[j] = B_BASE + (uint32_t)(kr * 512 + piece * 16 + (nl & 7) * 2);
        }
    }

    bf16x8 af[2][TM], bfr[2][TN];
    auto read_a = [&](int buf, int i, int ks, uint32_t stage_off) {
        af[buf][i] = *(lds_frag)(size_t)((ks ? fa1 : fa0) + stage_off + i * 2048);
    };
    auto read_b = [&](int buf, int j, int ks, uint32_t stage_off) {
        if (B_NT) {
            bfr[buf][j] = *(lds_frag)(size_t)((ks ? fb[1] : fb[0]) + stage_off + j * 2048);
        } else {
            const uint32_t a = fb[j] + stage_off + ks * 8192;
            const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_tr)(size_t)a);
            const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_tr)(size_t)(a + 2048));
            typedef short s16x8 __attribute__((ext_vector_type(8)));
            const s16x8 v = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
            bfr[buf][j] = __builtin_bit_cast(bf16x8, v);
        }
    };

    // The accumulators start at the bias instead of zero when the whole tile lies in the reduce
    // band and nothing is left for the epilogue to add in bf16 (no peers, or peers added on the
    // matrix cores): product, partial sums and bias are then summed in fp32 and rounded once,
    // and the epilogue just converts and stores.  Lane holds row m; register v of block j is
    // column 32j + 8(v/4) + 4(lane/32) + v%4, so a lane needs 16 groups of 4 consecutive bias
    // values, the same for all four row blocks.
    const int band_lo = g.band_row0;
    const bool tile_in_band = m0 >= band_lo && m0 + BM <= band_lo + g.band_rows;
    const bool mfma_peers = g.peers_on_mfma && g.n_peers > 0 && tile_in_band;
    const bool bias_in_acc = g.bias != nullptr && tile_in_band && (g.n_peers == 0 || mfma_peers);
    f32x16 acc[TM][TN];
    {
        f32x16 init[TN];
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) init[j][v] = 0.0f;
        if (bias_in_acc) {
            typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
            const uint16_t* bp = g.bias + n0 + wn * WTN + 4 * (lane >> 5);
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const u32x2 b4 = *(const u32x2*)(bp + j * 32 + 8 * q);
                    init[j][4 * q + 0] = bf16_lo(b4.x);
                    init[j][4 * q + 1] = bf16_hi(b4.x);
                    init[j][4 * q + 2] = bf16_lo(b4.y);
                    init[j][4 * q + 3] = bf16_hi(b4.y);
                }
        }
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) acc[i][j] = init[j];
    }

#define KR_SCHED_FENCE() __builtin_amdgcn_sched_barrier(0)
    // ---- partial sums of the other ranks, added on the matrix cores ---------------------------
    // For a tile that lies in the reduce band as a whole, the peers' partial sums P_q[m][n] are
    // accumulated into the same registers as the product, as  acc[n][m] += sum_k X_h[n][k] *
    // P_q[m][16h + k]  with X_h[n][k] = (n == 16h + k): the second MFMA operand wants, per lane,
    // 8 consecutive n of one row m -- 16 contiguous bytes of the peer's row-major buffer.  Each
    // wave streams its 128 x 128 part of every peer through a private quarter of the operand
    // ring (four stages of 32 rows x 256 B, filled by LDS-DMA four items ahead, 16-byte pieces
    // XOR-swizzled with the row so the fragment reads are conflict-free).  1.0 * bf16 products
    // and the fp32 accumulation are exact, so this is the fp32 sum  product + P_0 + ... + P_{W-2}
    // rounded once -- but 0 * Inf = NaN: a non-finite partial sum spoils the 32-column block of its
    // row that share its MFMA, not just its own element.
    // The phase is bound by HBM, the k loop by the matrix cores: workgroups alternate the order
    // of the two, so at any time about half the CUs stream peers while the other half multiply.
    auto peer_phase = [&]() __attribute__((always_inline)) {
        constexpr int kItemLoads = 8;          // 1 KiB LDS-DMA loads per item (32 rows x 256 B)
        constexpr int kItemBytes = kItemLoads * 1024;
        constexpr int kAhead = 4;              // items in flight = stages per wave
        static_assert(TM == 4 && kAhead * kItemBytes * WM * WN <= LDS_BYTES, "peer stages must fit in the ring");
        typedef short s16x8 __attribute__((ext_vector_type(8)));
        bf16x8 xid[2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            s16x8 x;
#pragma unroll
            for (int e = 0; e < 8; ++e) x[e] = ((lane & 31) == 16 * h + 8 * (lane >> 5) + e) ? (short)0x3f80 : (short)0;
            xid[h] = __builtin_bit_cast(bf16x8, x);
        }
        const uint32_t region = (uint32_t)wave * (kAhead * kItemBytes);
        // load r of an item fills rows 4r .. 4r+3: lane l -> row 4r + l/16, piece slot l%16 holds
        // piece slot ^ (row & 15); r = 4a + b puts 16a rows into the scalar offset
        uint32_t pvoff[4];
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            const int row = 4 * b + (lane >> 4);
            pvoff[b] = (uint32_t)(((int64_t)row * g.N + (((lane & 15) ^ row) << 3)) * 2);
        }
        // fragment (j, h): lane l -> row l%32, piece 4j + 2h + l/32
        uint32_t pa[2 * TN];
#pragma unroll
        for (int jh = 0; jh < 2 * TN; ++jh) {
            const int row = lane & 31;
            pa[jh] = region + (uint32_t)(row * 256 + (((2 * jh + (lane >> 5)) ^ (row & 15)) << 4));
        }
        const int n_items = g.n_peers * TM;    // item = (peer q, slab i), q-major
        const uint16_t* wave_base = g.peers + ((int64_t)(m0 + wm * WTM - band_lo) * g.N + n0 + wn * WTN);
        auto issue_item = [&](int it, int stage) __attribute__((always_inline)) {
            // past the end: all lanes re-read 16 bytes of the last item (the load count per item
            // is fixed for the vmcnt arithmetic; the data is never used)
            const bool live = it < n_items;
            const int itc = min(it, n_items - 1);
            const i32x4 rs = make_rsrc(wave_base + (int64_t)(itc >> 2) * g.peers_stride + (int64_t)(itc & 3) * 32 * g.N);
#pragma unroll
            for (int r = 0; r < kItemLoads; ++r)
                lds_dma_b128_stream(rs, region + stage * kItemBytes + r * 1024, live ? pvoff[r & 3] : 0u,
                             live ? (int)((int64_t)(r >> 2) * 16 * g.N * 2) : 0);
        };
#pragma unroll
        for (int it = 0; it < kAhead; ++it) issue_item(it, it);
#pragma nounroll
        for (int q = 0; q < g.n_peers; ++q) {
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                // item (q, i) has landed when at most the three younger items are outstanding; the
                // stages are private to the wave, so no barrier
                __builtin_amdgcn_s_waitcnt(vmcnt_imm((kAhead - 1) * kItemLoads));
                KR_SCHED_FENCE();
                bf16x8 y[2 * TN];
#pragma unroll
                for (int jh = 0; jh < 2 * TN; ++jh) y[jh] = *(lds_frag)(size_t)(pa[jh] + i * kItemBytes);
                KR_SCHED_FENCE();   // all eight reads in flight before the first MFMA waits for one
#pragma unroll
                for (int jh = 0; jh < 2 * TN; ++jh)
                    acc[i][jh >> 1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xid[jh & 1], y[jh], acc[i][jh >> 1], 0, 0, 0);
                // every fragment read has returned before the stage is handed back to the DMA
                __builtin_amdgcn_s_waitcnt(kLgkm0);
                KR_SCHED_FENCE();
                issue_item(q * TM + i + kAhead, i);
                KR_SCHED_FENCE();
            }
        }
        __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
        __syncthreads();   // the ring is handed on (k loop or epilogue patches of other waves)
    };
    // An empty statement that names every accumulator as an AGPR operand, placed between the
    // phases: with the live ranges cut here the register allocator keeps the accumulators
    // where the MFMAs left them instead of moving them to VGPRs and memory for the next phase.
    auto pin_accumulators = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) asm volatile("" : "+a"(acc[i][j]));
    };
    if (PEERS_FIRST && mfma_peers) peer_phase();
    pin_accumulators();

    // ---- prologue: request k-steps 0 .. NSTAGE-2; wait for step 0 -----------------------------
#pragma unroll
    for (int t = 0; t < NSTAGE - 1; ++t)
#pragma unroll
        for (int q = 0; q < LOADS_PER_TILE; ++q) issue_load(t, (uint32_t)t, q);
    __builtin_amdgcn_s_waitcnt(vmcnt_imm((NSTAGE - 2) * LOADS_PER_TILE));
    __builtin_amdgcn_s_barrier();
    KR_SCHED_FENCE();
#pragma unroll
    for (int i = 0; i < TM; ++i) read_a(0, i, 0, 0);
#pragma unroll
    for (int j = 0; j < TN; ++j) read_b(0, j, 0, 0);

    // ---- main loop ---------------------------------------------------------------------------
    // k-step t: 2 sub-steps of 16 MFMAs.  Sub-step 0 computes on fragment buffer 0 while the
    // fragments of sub-step 1 are read into buffer 1; sub-step 1 computes on buffer 1 while the
    // first fragments of k-step t+1 are read into buffer 0.  After the first MFMAs of the step
    // the wave waits until its own loads of step t+1 have landed (those of the later steps may
    // still be in flight) and meets the other waves: from then on step t+1 is complete in LDS
    // and the stage of step t-1 is free, so the loads of step t+NSTAGE-1 go out into it, one
    // every third MFMA.
    constexpr int NM = TM * TN;
    // one k-step; `stage_c` is t % NSTAGE, as a compile-time constant in the unrolled loop
    auto k_step = [&](int t, auto stage_c) __attribute__((always_inline)) {
        const uint32_t stage_cur = stage_c;
        const uint32_t stage_nxt = stage_cur + 1 == NSTAGE ? 0 : stage_cur + 1;
        const uint32_t stage_ld = stage_cur == 0 ? NSTAGE - 1 : stage_cur - 1;   // (t + NSTAGE - 1) % NSTAGE
        const uint32_t st_cur = stage_cur * A_ST, st_nxt = stage_nxt * A_ST;
#pragma unroll
        for (int s = 0; s < NM; ++s) {
            const int i = s / TN, j = s % TN;
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bfr[0][j], af[0][i], acc[i][j], 0, 0, 0);
            // fragments of sub-step 1, this stage: A blocks next to MFMAs 0..3, B blocks 4..7 / 4..11
            if (s < TM) read_a(1, s, 1, st_cur);
            else if (s < TM + TN) read_b(1, s - TM, 1, st_cur);
            if (s == 3) {
                KR_SCHED_FENCE();
                __builtin_amdgcn_s_waitcnt(vmcnt_imm((NSTAGE - 3) * LOADS_PER_TILE));
                __builtin_amdgcn_s_barrier();
            }
            // one load every third MFMA (continued in sub-step 1): four waves issuing a load per
            // MFMA ask twice what the CU's address unit takes, and the waves stall at issue
            if (s >= 4 && (s - 4) % 3 == 0 && (s - 4) / 3 < LOADS_PER_TILE / 2) issue_load(t + NSTAGE - 1, stage_ld, (s - 4) / 3);
            KR_SCHED_FENCE();
        }
#pragma unroll
        for (int s = 0; s < NM; ++s) {
            const int i = s / TN, j = s % TN;
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bfr[1][j], af[1][i], acc[i][j], 0, 0, 0);
            // first fragments of k-step t+1 (its stage is complete since the barrier above)
            if (s < TM) read_a(0, s, 0, st_nxt);
            else if (s < TM + TN) read_b(0, s - TM, 0, st_nxt);
            if (s % 3 == 0 && s / 3 < LOADS_PER_TILE / 2) issue_load(t + NSTAGE - 1, stage_ld, LOADS_PER_TILE / 2 + s / 3);
            KR_SCHED_FENCE();
        }
    };
    // Main part: one trip = NSTAGE k-steps, so every LDS stage offset is a compile-time constant
    // (immediate offsets on the fragment reads, no per-step address arithmetic) and the loop
    // branch is taken once per NSTAGE steps.  The at most NSTAGE-1 remaining steps follow.
    static_assert(NSTAGE == 4, "the unrolled trip below spells out four stages");
    int t = 0;
#pragma nounroll
    for (; t + NSTAGE <= kt_total; t += NSTAGE) {
        k_step(t, std::integral_constant<uint32_t, 0>{});
        k_step(t + 1, std::integral_constant<uint32_t, 1>{});
        k_step(t + 2, std::integral_constant<uint32_t, 2>{});
        k_step(t + 3, std::integral_constant<uint32_t, 3>{});
    }
    pin_accumulators();
    {
        uint32_t stage_cur = 0;   // t is a multiple of NSTAGE here
#pragma nounroll
        for (; t < kt_total; ++t) {
            k_step(t, stage_cur);
            stage_cur = stage_cur + 1 == NSTAGE ? 0 : stage_cur + 1;
        }
    }
    // drain the tail's surplus loads before the LDS is reused
    __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
    __syncthreads();

    pin_accumulators();
    if (!PEERS_FIRST && mfma_peers) peer_phase();
    pin_accumulators();
    GemmArgs ge = g;
    if (mfma_peers) ge.n_peers = 0;   // already in the accumulators
    if (bias_in_acc) ge.bias = nullptr;
    gemm_epilogue<BM, WTM, WTN, TM, TN, true, EP_WAVE>(ge, acc, smem, m0, n0, wm, wn, lane, wave);
}
#undef KR_SCHED_FENCE

// The two phase orders are two complete copies of the tile code under one uniform branch: each
// copy is straight-line (phase, phase, epilogue), which keeps the 256 accumulators in their
// registers; one copy with a run-time order has the register allocator move them through memory.
template <bool B_NT>
__global__ __launch_bounds__(WM* WN * 64) void gemm_dtl_kernel(const GemmArgs g) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];   // starts at LDS address 0
    if (g.peers_on_mfma && g.n_peers > 0 && (g.peers_on_mfma == 1 ? ((blockIdx.x >> 3) & 1) : g.peers_on_mfma == 2)) gemm_dtl_tile<B_NT, true>(g, smem);
    else gemm_dtl_tile<B_NT, false>(g, smem);
}

}  // namespace

bool gemm_dtl_supported(const GemmArgs& g) {
    return g.M % BM == 0 && g.N % BN == 0 && g.K % BKD == 0 && g.K >= (NSTAGE - 1) * BKD &&
           (int64_t)BM * g.lda * 2 < 0x7fffffffLL && (int64_t)(BN > 64 ? BN : 64) * g.ldb * 2 < 0x7fffffffLL;
}

hipError_t launch_gemm_dtl(const GemmArgs& g, bool b_nt, hipStream_t st) {
    const dim3 grid((unsigned)(g.tiles_m * g.tiles_n)), block(WM * WN * 64);
    static bool opt_in[2] = {false, false};   // benign race: the attribute call is idempotent
    if (!opt_in[b_nt]) {
        hipError_t e = b_nt ? hipFuncSetAttribute((const void*)gemm_dtl_kernel<true>,
                                                  hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES)
                            : hipFuncSetAttribute((const void*)gemm_dtl_kernel<false>,
                                                  hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES);
        if (e != hipSuccess) return e;
        opt_in[b_nt] = true;
    }
    if (b_nt)
        hipLaunchKernelGGL(gemm_dtl_kernel<true>, grid, block, LDS_BYTES, st, g);
    else
        hipLaunchKernelGGL(gemm_dtl_kernel<false>, grid, block, LDS_BYTES, st, g);
    return hipGetLastError();
}

}  // namespace kr
