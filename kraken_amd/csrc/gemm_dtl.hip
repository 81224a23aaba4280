// bf16 GEMM main loop with direct global->LDS loads ("LDS DMA"), 256x256 tiles, for K % 64 == 0
// (M and N may be ragged: the tiles at the lower and right edge are handled below).
//
// Workgroup tile 256 x 256, four wavefronts (2 x 2), each owning 128 x 128 of C as 4 x 4
// v_mfma_f32_32x32x16_bf16 accumulators (256 AGPRs).  The k loop advances 64 at a time through a
// double buffer of LDS stages (A: 2 x 32 KiB at 0, B: 2 x 32 KiB at 64 KiB) that is filled by
// buffer_load ... lds: the data never passes through VGPRs and no ds_write is issued.  With 64 k
// per stage a row of A (or of transposed B) is 128 contiguous bytes, one L2 cache line per row
// and load: a four-stage ring of 32-k stages, tried first, was more tolerant of load latency but
// asked the L2 for every line twice (twice the L1-to-L2 requests of hipBLASLt's kernel in the
// counters) and measured 3-7 % slower.
//
// LDS layouts (per stage)
//   A and transposed-contiguous B: [256 rows][128 B] (64 k), the eight 16-byte pieces of a row
//     XOR-swizzled with (row >> 1) & 7.  One wave-wide LDS-DMA load fills 8 rows (1 KiB,
//     lane l -> row l/8, piece slot l%8); the 128-bit fragment reads of 16 consecutive rows
//     then touch all 64 banks once.
//   row-major B: [64 k][512 B] (256 n), the 16-byte pieces of a k-row XOR-swizzled with
//     4*(k & 3): the 32 lanes of two neighbouring 16-lane blocks (4 k-rows x 32 columns) then
//     cover 16 different pieces = all 64 banks.  Fragments are read with ds_read_b64_tr_b16:
//     16 lanes read a 4(k) x 16(n) block, four n each, and the hardware hands lane i the four
//     k of column i -- two such reads give the eight k per lane the MFMA wants, with no
//     transpose in registers.
// A lane's fragment addresses differ between the 32x32 blocks and the stages only by compile-time
// constants (immediate offsets); the four 16-wide k sub-steps of a stage take one address
// register each (A, B transposed) or an immediate (B row-major, one register per column block).
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
constexpr int BKD = 64;                       // k extent of one stage: 128-byte rows, one L2 line per row and load
constexpr int NSTAGE = 2;                     // double buffer
constexpr int A_ST = BM * BKD * 2;            // 32 KiB
constexpr int B_ST = BN * BKD * 2;            // 32 KiB
constexpr uint32_t B_BASE = NSTAGE * A_ST;    // 64 KiB
constexpr int LDS_BYTES = NSTAGE * (A_ST + B_ST);
constexpr int LOADS_A = A_ST / 1024 / (WM * WN);   // LDS-DMA loads (1 KiB each) per wave per k-step: 8 A ...
constexpr int LOADS_PER_TILE = 2 * LOADS_A;        // ... + 8 B
constexpr int EP_WAVE = 32 * (WTN + 4) * 4;     // epilogue patch of a wave: 32 rows x WTN fp32, padded
static_assert(EP_WAVE * WM * WN <= LDS_BYTES, "epilogue patch must fit in the operand ring");

typedef __attribute__((address_space(3))) void* lds_void;
typedef const __attribute__((address_space(3))) bf16x8* lds_frag;
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) s16x4* lds_tr;

// s_waitcnt vmcnt(n) only (expcnt and lgkmcnt left at "no wait")
constexpr int vmcnt_imm(int n) { return (n & 15) | (7 << 4) | (15 << 8) | ((n >> 4) << 14); }
constexpr int kLgkm0 = 0xc07f;   // s_waitcnt lgkmcnt(0) only

// bf16 store of a wave's 128 x (NB*16) part of a tile held as 8 x NB accumulator blocks of 16 x 16
// (lane l: row l%16, columns 4(l/16) .. +3 of a block): per 16-row slab the blocks are rounded to
// bf16 into a per-wave LDS patch [16][NB*16 + 8] and leave as 16-byte chunks of whole rows.
// `smem`: the workgroup's LDS, free for reuse; `dst`: the wave's first row and column; ld in elements.
template <int NB>
__device__ __forceinline__ void store_tile_bf16_blocks(const f32x4 (&acc16)[2 * TM][NB], unsigned char* smem, uint16_t* dst, int64_t ld,
                                                       int lane, int wave) {
    constexpr int COLS = NB * 16, LD = COLS + 8, CPR = COLS / 8, CHUNKS = 16 * CPR;
    static_assert(16 * LD * 2 <= 4096, "patch of a wave");
    uint16_t* patch = (uint16_t*)(smem + wave * 4096);
    typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
#pragma unroll
    for (int i = 0; i < 2 * TM; ++i) {
#pragma unroll
        for (int j = 0; j < NB; ++j) {
            // (pinned here: a conversion the compiler may hoist would keep all blocks' halves alive at once)
            uint32_t lo, hi, t;
            asm volatile("v_accvgpr_read_b32 %0, %2\n\tv_accvgpr_read_b32 %1, %3\n\tv_cvt_pk_bf16_f32 %0, %0, %1"
                         : "=&v"(lo), "=&v"(t) : "a"(acc16[i][j][0]), "a"(acc16[i][j][1]));
            asm volatile("v_accvgpr_read_b32 %0, %2\n\tv_accvgpr_read_b32 %1, %3\n\tv_cvt_pk_bf16_f32 %0, %0, %1"
                         : "=&v"(hi), "=&v"(t) : "a"(acc16[i][j][2]), "a"(acc16[i][j][3]));
            *(u32x2*)(patch + (lane & 15) * LD + 16 * j + 4 * (lane >> 4)) = u32x2{lo, hi};
        }
        asm volatile("" ::: "memory");   // the reads below see the stores above (different vector types, same bytes)
#pragma unroll
        for (int it = 0; it < (CHUNKS + 63) / 64; ++it) {
            const int idx = it * 64 + lane;
            if (idx < CHUNKS) {
                const int r = idx / CPR, c = idx - r * CPR;
                const u32x4 v = *(const u32x4*)(patch + r * LD + c * 8);
                st_stream((u32x4*)(dst + (int64_t)(16 * i + r) * ld + c * 8), v);
            }
        }
        asm volatile("" ::: "memory");   // the next slab's stores stay behind these reads
    }
}

// fp32 -> fp8 (e4m3fn) of two values into one half of a word: nearest even; magnitudes from 448 on
// (infinities included) give +-448, NaN stays NaN -- the conversion kr_cast_f32_to_fp8 defines.  The
// clamp is explicit, so the instruction's own overflow handling never comes into play.
template <bool HIGH_HALF>
__device__ __forceinline__ uint32_t pack2_e4m3(float a, float b, uint32_t old) {
    const float ca = __builtin_fminf(__builtin_fmaxf(a, -448.0f), 448.0f), cb = __builtin_fminf(__builtin_fmaxf(b, -448.0f), 448.0f);
    return (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(a != a ? a : ca, b != b ? b : cb, (int)old, HIGH_HALF);
}

// fp8 store of a wave's 128 x 128 part of a tile held as 8 x 8 accumulator blocks of 16 x 16 (lane l:
// row l%16, columns 4(l/16) .. +3 of a block): per 16-row slab a lane's four values of a block become
// one word of a per-wave LDS patch [16][128 + 16] bytes (the pad keeps the 64 word stores of a block on
// 64 banks), and the slab leaves as 16-byte chunks of whole 128-byte rows.  `dst`: the wave's first
// row and column; ld in bytes.
__device__ __forceinline__ void store_tile_fp8_blocks(const f32x4 (&acc16)[2 * TM][2 * TN], unsigned char* smem, uint8_t* dst, int64_t ld,
                                                      int lane, int wave) {
    constexpr int COLS = 2 * TN * 16, LD = COLS + 16, CPR = COLS / 16;
    static_assert(16 * CPR == 128, "two chunks per lane and slab");
    unsigned char* patch = smem + wave * 4096;
#pragma unroll
    for (int i = 0; i < 2 * TM; ++i) {
#pragma unroll
        for (int j = 0; j < 2 * TN; ++j) {
            // (pinned here: copies the compiler may hoist would keep all blocks' values alive at once)
            float x0, x1, x2, x3;
            asm volatile("v_accvgpr_read_b32 %0, %2\n\tv_accvgpr_read_b32 %1, %3" : "=&v"(x0), "=&v"(x1) : "a"(acc16[i][j][0]), "a"(acc16[i][j][1]));
            asm volatile("v_accvgpr_read_b32 %0, %2\n\tv_accvgpr_read_b32 %1, %3" : "=&v"(x2), "=&v"(x3) : "a"(acc16[i][j][2]), "a"(acc16[i][j][3]));
            const uint32_t w = pack2_e4m3<true>(x2, x3, pack2_e4m3<false>(x0, x1, 0u));
            *(uint32_t*)(patch + (lane & 15) * LD + 16 * j + 4 * (lane >> 4)) = w;
        }
        asm volatile("" ::: "memory");   // the reads below see the stores above (different types, same bytes)
#pragma unroll
        for (int it = 0; it < 2; ++it) {
            const int idx = it * 64 + lane, r = idx / CPR, c = idx % CPR;
            const u32x4 v = *(const u32x4*)(patch + r * LD + c * 16);
            st_stream((u32x4*)(dst + (int64_t)(16 * i + r) * ld + c * 16), v);
        }
        asm volatile("" ::: "memory");   // the next slab's stores stay behind these reads
    }
}

// One workgroup tile.  PEERS_FIRST picks the order of the two accumulation phases (peers'
// partial sums, k loop) for tiles whose peers are added on the matrix cores.
// SPLIT: the workgroup is one of g.k_splits that share a tile of the last partial round: it
// runs its share of the k-steps and leaves its accumulators in the workspace (no epilogue).
// RAGGED: M or N is not a multiple of 256 (edge tiles get the bounds-checked epilogue).
// MI16: the k loop uses v_mfma_f32_16x16x32_bf16 (8 x 8 blocks of 16 x 16 per wave) instead of
// 32x32x16 (4 x 4 blocks of 32 x 32): same operand traffic, but the matrix cores draw less power
// per flop with it (under the power limit, matrix-core-only loops on random operands sustain
// 2.04 PFLOP/s with 16x16x32 against 1.62 with 32x32x16).
// NB: 16-column blocks per wave (16x16 form).  8 = the 256 x 256 tile; 7 = a 256 x 224 tile (waves of
// 128 x 112) for plain products with transposed-contiguous B whose 256-column tiles would leave a
// partial last round of compute units while 224-column tiles fill whole rounds (8192 x 3584: 448
// tiles = 1.75 rounds against 512 = 2).  Per flop the narrower tile reads 7 % more of A from LDS
// and L2, which two full rounds more than pay for.
template <bool B_NT, bool PEERS_FIRST, bool SPLIT = false, bool RAGGED = false, bool MI16 = false, int NB = 2 * TN, bool F8 = false>
__device__ __forceinline__ void gemm_dtl_tile(const GemmArgs& g, unsigned char* smem) {
    static_assert(NB == 2 * TN || (NB == 7 && MI16 && B_NT && !SPLIT && !RAGGED && !PEERS_FIRST), "224-column tile: plain NT products only");
    // F8: the operands are fp8 (e4m3fn) and g describes them as bf16 matrices of half the width (g.K, g.lda, g.ldb in
    // two-byte units), so a stage still holds 128-byte rows -- 128 k now -- and every load and LDS address below is unchanged;
    // only the k-step differs (k_step8: 16x16x128 MFMAs on the same 16 x 16 accumulator blocks).
    static_assert(!F8 || (MI16 && B_NT && !SPLIT && !RAGGED && !PEERS_FIRST && NB == 2 * TN), "fp8: plain NT products on whole tiles");
    constexpr int BNX = WN * NB * 16;                            // columns of the workgroup tile
    constexpr int WTNX = NB * 16;                                // columns of a wave
    constexpr int LOADS_B = BNX * BKD * 2 / 1024 / (WM * WN);    // LDS-DMA loads of B per wave per k-step: 8 or 7
    constexpr int LOADS_TILE = LOADS_A + LOADS_B;
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
    const int first_tile = g.tiles_m * g.tiles_n - g.tail_tiles;     // SPLIT: tiles the main launch took
    const int split = SPLIT ? (int)(blockIdx.x % (unsigned)g.k_splits) : 0;
    const int tail_index = SPLIT ? (int)(blockIdx.x / (unsigned)g.k_splits) : 0;
    tile_schedule(g, SPLIT ? schedule_position(g, tail_index, first_tile) : schedule_position(g, blockIdx.x), tile_m,
                  tile_n);
    const int m0 = tile_m * BM, n0 = tile_n * BNX;
    // k-steps of this workgroup: all of them, or the split's share
    const int kt_all = g.K / BKD;
    const int kt_begin = SPLIT ? (int)((int64_t)kt_all * split / g.k_splits) : 0;
    const int kt_total = SPLIT ? (int)((int64_t)kt_all * (split + 1) / g.k_splits) - kt_begin : kt_all;
    const int k_begin = kt_begin * BKD;
    const uint16_t* a_tile;   // first row of the tile's A panel (gathered matrix or local shard)
    int64_t lda;
    gathered_a_tile(g, m0, BM, a_tile, lda);
    // (the choice above is the same for the whole workgroup; the descriptor below wants it in
    // scalar registers)
    a_tile = (const uint16_t*)wave_uniform((int64_t)a_tile) + k_begin;
    lda = wave_uniform(lda);

    // ---- LDS-DMA addressing ----------------------------------------------------------------
    // A wave loads the 1 KiB chunks  wave, wave+4, ..., wave+28  of a stage.
    // A / transposed B: chunk = 8 rows of 128 B; lane l -> row l/8, slot l%8 holds the 16-byte
    // piece  slot ^ ((row >> 1) & 7)  of the row.  (row >> 1) & 7 = (4*chunk + l/16) & 7 and chunk
    // has the parity of the wave, so the per-lane byte offset is computed once; the wave-uniform
    // part (chunk row, k) goes to the scalar offset.
    const int dma_sw = (4 * (wave & 1) + (lane >> 4)) & 7;
    const uint32_t a_voff_lane = (uint32_t)(((int64_t)(lane >> 3) * lda + (((lane & 7) ^ dma_sw) << 3)) * 2);
    uint32_t b_voff_lane, b_voff_odd = 0;
    if (B_NT) {
        b_voff_lane = (uint32_t)(((int64_t)(lane >> 3) * g.ldb + (((lane & 7) ^ dma_sw) << 3)) * 2);
    } else {
        // row-major B: chunk = 2 k-rows of 512 B; lane l -> k-row l/32, piece slot l%32 holds piece
        // slot ^ 4*(k & 3); k & 3 = 2*(chunk & 1) + l/32 and chunk & 1 == wave & 1
        const int kq = ((wave & 1) << 1) | (lane >> 5);
        b_voff_lane = (uint32_t)(((int64_t)(lane >> 5) * g.ldb + (((lane & 31) ^ (kq << 2)) << 3)) * 2);
        // 16x16x32 blocks: all four 16-lane groups of a transposing read want the same 16 columns,
        // of k-rows 8 apart; a further XOR with 2*((k >> 3) & 1) puts groups 0/1 (2/3) on different
        // banks.  (k >> 3) & 1 = chunk parity of the load's index, a second offset for the odd ones.
        if (MI16) b_voff_odd = (uint32_t)(((int64_t)(lane >> 5) * g.ldb + (((lane & 31) ^ (kq << 2) ^ 2) << 3)) * 2);
    }
    // Buffer resource descriptor: 48-bit base, stride 0 (raw), 2^31-1 bytes, 32-bit data format.
    typedef int i32x4 __attribute__((ext_vector_type(4)));
    auto make_rsrc = [](const void* base, int64_t bytes = 0x7fffffff) {
        const uint64_t b = (uint64_t)base;
        return i32x4{(int)(uint32_t)b, (int)(uint32_t)((b >> 32) & 0xffff),
                     (int)(bytes < 0x7fffffff ? (bytes > 0 ? bytes : 0) : 0x7fffffff), 0x00020000};
    };
    // A tile at the lower or right edge of a ragged shape has fewer than 256 valid rows (columns):
    // its operand descriptors end with the last valid row, so the loads of the missing rows are
    // out of range (they fetch nothing) and the accumulators of those rows and columns, which
    // hold whatever the LDS stage held, are never stored (the epilogue masks them).
    const int rows_a = RAGGED ? min(BM, g.M - m0) : BM, rows_b = RAGGED ? min(BN, g.N - n0) : BN;
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
    const i32x4 a_rsrc = RAGGED ? make_rsrc(a_tile, ((int64_t)(rows_a - 1) * lda + (g.K - k_begin)) * 2) : make_rsrc(a_tile);
    const i32x4 bt_rsrc = RAGGED ? make_rsrc(g.B + (int64_t)n0 * g.ldb + (B_NT ? k_begin : 0),
                                             ((int64_t)(rows_b - 1) * g.ldb + (g.K - k_begin)) * 2)
                                 : make_rsrc(g.B + (int64_t)n0 * g.ldb + (B_NT ? k_begin : 0));

    // one LDS-DMA load of k-step t (clamped: the tail re-requests the last tile into a free stage)
    auto issue_load = [&](int t, uint32_t stage, int q) {
        // past the end nothing new is needed, but the per-step load count must not change (the
        // vmcnt arithmetic relies on it): every lane then re-reads the first 16 bytes of the
        // last tile's chunk into the free stage -- one cache line instead of a kilobyte
        const bool live = t < kt_total;
        const int tt = min(t, kt_total - 1);
        const int k0 = tt * BKD;
        const uint32_t a_voff = live ? a_voff_lane : 0u;
        const uint32_t b_voff = !live ? 0u : (MI16 && !B_NT && ((q % LOADS_A) & 1)) ? b_voff_odd : b_voff_lane;
        const int ch = wave + 4 * (q % LOADS_A);
        if (q < LOADS_A) {
            lds_dma_b128(a_rsrc, stage * A_ST + ch * 1024, a_voff, (int)(((int64_t)8 * ch * lda + k0) * 2));
        } else if (B_NT) {
            lds_dma_b128(bt_rsrc, B_BASE + stage * B_ST + ch * 1024, b_voff,
                         (int)(((int64_t)8 * ch * g.ldb + k0) * 2));
        } else {
            // re-based on the first k-row of the step: the scalar offset stays small for any K
            // (the descriptor ends with the matrix: columns past N of the last k-rows fetch nothing, those of
            // other k-rows read the next row's first columns -- neither reaches a stored element)
            lds_dma_b128(RAGGED ? make_rsrc(g.B + (int64_t)(k_begin + k0) * g.ldb + n0,
                                            ((int64_t)(g.K - 1 - (k_begin + k0)) * g.ldb + (g.N - n0)) * 2)
                                : make_rsrc(g.B + (int64_t)(k_begin + k0) * g.ldb + n0),
                         B_BASE + stage * B_ST + ch * 1024, b_voff,
                         (int)(((int64_t)2 * ch * g.ldb) * 2));
        }
    };

    // ---- fragment addressing -----------------------------------------------------------------
    // A (and transposed B): lane -> row (lane & 31) of the 32-row block, 8 k at piece 2*ks + (lane>>5)
    // of the row's eight, stored at piece ^ ((row >> 1) & 7) -- the same for all blocks (their rows
    // differ by 32); the sub-step enters as an XOR of bits 5..6
    const int frow = lane & 31, fkc = lane >> 5;
    const int fsw = (frow >> 1) & 7;
    uint32_t fa[4], fb[4];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) fa[ks] = (uint32_t)((wm * WTM + frow) * 128 + (((2 * ks + fkc) ^ fsw) << 4));
    if (B_NT) {
#pragma unroll
        for (int ks = 0; ks < 4; ++ks)
            fb[ks] = B_BASE + (uint32_t)((wn * WTN + frow) * 128 + (((2 * ks + fkc) ^ fsw) << 4));
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
        af[buf][i] = *(lds_frag)(size_t)(fa[ks] + stage_off + i * 4096);
    };
    auto read_b = [&](int buf, int j, int ks, uint32_t stage_off) {
        if (B_NT) {
            bfr[buf][j] = *(lds_frag)(size_t)(fb[ks] + stage_off + j * 4096);
        } else {
            const uint32_t a = fb[j] + stage_off + ks * 8192;
            const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_tr)(size_t)a);
            const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_tr)(size_t)(a + 2048));
            typedef short s16x8 __attribute__((ext_vector_type(8)));
            const s16x8 v = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
            bfr[buf][j] = __builtin_bit_cast(bf16x8, v);
        }
    };

    // 16x16x32 blocks: lane -> row (lane & 15) of a 16-row block, 8 k at piece 4*ks2 + (lane >> 4) of
    // the row's eight (ks2: the two 32-k halves of a stage); blocks are 2 KiB apart.  Row-major B:
    // the 16-lane group q = lane/16 reads k-rows 8q .. 8q+7 of the half with two transposing reads.
    uint32_t fa16[2], fb16[2 * TN];
    bf16x8 af16[2][2 * TM], bfr16[2][2 * TN];
    if constexpr (MI16) {
        const int p = lane & 15, gq = lane >> 4;
        const int sw16 = (p >> 1) & 7;
#pragma unroll
        for (int ks2 = 0; ks2 < 2; ++ks2) {
            fa16[ks2] = (uint32_t)((wm * WTM + p) * 128 + (((4 * ks2 + gq) ^ sw16) << 4));
            if (B_NT) fb16[ks2] = B_BASE + (uint32_t)((wn * WTNX + p) * 128 + (((4 * ks2 + gq) ^ sw16) << 4));
        }
        if (!B_NT) {
#pragma unroll
            for (int bj = 0; bj < 2 * TN; ++bj) {
                const int nl = wn * WTN + bj * 16 + 4 * (p & 3);
                const int kr = 8 * gq + (p >> 2);
                const int piece = (nl >> 3) ^ (((p >> 2) & 3) << 2) ^ ((gq & 1) << 1);
                fb16[bj] = B_BASE + (uint32_t)(kr * 512 + piece * 16 + (nl & 7) * 2);
            }
        }
    }
    auto read_a16 = [&](int buf, int bi, int ks2, uint32_t stage_off) {
        af16[buf][bi] = *(lds_frag)(size_t)(fa16[ks2] + stage_off + bi * 2048);
    };
    auto read_b16 = [&](int buf, int bj, int ks2, uint32_t stage_off) {
        if (B_NT) {
            bfr16[buf][bj] = *(lds_frag)(size_t)(fb16[ks2] + stage_off + bj * 2048);
        } else {
            const uint32_t a = fb16[bj] + stage_off + ks2 * 16384;
            const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_tr)(size_t)a);
            const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_tr)(size_t)(a + 2048));
            typedef short s16x8 __attribute__((ext_vector_type(8)));
            const s16x8 v = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
            bfr16[buf][bj] = __builtin_bit_cast(bf16x8, v);
        }
    };

    // fp8, 16x16x128 blocks: lane -> row (lane & 15) of a 16-row block and the 32 k at pieces q and 4 + q (q = lane >> 4) of
    // the row's eight -- two 16-byte reads, the halves of the operand's eight registers.  Both operands hand the matrix
    // cores their k in this same order, which is all the sum needs; each of the two reads then has the access pattern of a
    // 16x16x32 fragment read (pieces 2q and 2q+1 instead cost a two-way bank conflict on every read: LDS active 55.5 M
    // cycles per launch of 4096x6656x16384 with 27.7 M conflict cycles, against 27.5 M and none).
    typedef int i32x4 __attribute__((ext_vector_type(4)));
    typedef int i32x8 __attribute__((ext_vector_type(8)));
    typedef const __attribute__((address_space(3))) i32x4* lds_i32x4;
    uint32_t fa8[2], fb8[2];
    i32x8 af8[2][TM], bf8[2][2 * TN];   // A: blocks 0..3 and 4..7 of the current step; B: all blocks, this step's and the next one's
    if constexpr (F8) {
        const int p = lane & 15, gq = lane >> 4;
        const int sw8 = (p >> 1) & 7;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            fa8[h] = (uint32_t)((wm * WTM + p) * 128 + (((4 * h + gq) ^ sw8) << 4));
            fb8[h] = B_BASE + (uint32_t)((wn * WTN + p) * 128 + (((4 * h + gq) ^ sw8) << 4));
        }
    }
    // half h of fragment r of a stage: r = 0, 1: A block 0; 2 .. 17: B blocks 0 .. 7; 18 .. 23: A blocks 1 .. 3 (the order the
    // first MFMAs of a step need them in); A blocks 4 .. 7 are read_a8_late
    auto read_frag8 = [&](int buf, int r, uint32_t stage_off) __attribute__((always_inline)) {
        const int h = r & 1;
        if (r < 2 || r >= 18) {
            const int bi = r < 2 ? 0 : (r - 16) / 2;
            const i32x4 v = *(lds_i32x4)(size_t)(fa8[h] + stage_off + bi * 2048);
            if (h == 0) af8[0][bi].lo = v; else af8[0][bi].hi = v;
        } else {
            const int bj = (r - 2) / 2;
            const i32x4 v = *(lds_i32x4)(size_t)(fb8[h] + stage_off + bj * 2048);
            if (h == 0) bf8[buf][bj].lo = v; else bf8[buf][bj].hi = v;
        }
    };
    auto read_a8_late = [&](int r, uint32_t stage_off) __attribute__((always_inline)) {   // r = 0 .. 7: halves of A blocks 4 .. 7
        const i32x4 v = *(lds_i32x4)(size_t)(fa8[r & 1] + stage_off + (4 + r / 2) * 2048);
        if ((r & 1) == 0) af8[1][r / 2].lo = v; else af8[1][r / 2].hi = v;
    };

    // The accumulators start at the bias instead of zero when the whole tile lies in the reduce
    // band and nothing is left for the epilogue to add in bf16 (no peers, or peers added on the
    // matrix cores): product, partial sums and bias are then summed in fp32 and rounded once,
    // and the epilogue just converts and stores.  Lane holds row m; register v of block j is
    // column 32j + 8(v/4) + 4(lane/32) + v%4, so a lane needs 16 groups of 4 consecutive bias
    // values, the same for all four row blocks.
    const int band_lo = g.band_row0;
    const bool full_tile = !RAGGED || (m0 + BM <= g.M && n0 + BN <= g.N);
    const bool tile_in_band = full_tile && m0 >= band_lo && m0 + BM <= band_lo + g.band_rows;
    const bool mfma_peers = !SPLIT && NB == 2 * TN && g.peers_on_mfma && g.n_peers > 0 && tile_in_band;
    const bool bias_in_acc = !SPLIT && g.bias != nullptr && tile_in_band && (g.n_peers == 0 || mfma_peers);
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

    // the same for the 16x16 blocks: a lane holds row lane%16 and the columns 16j + 4(lane/16) .. +3
    f32x4 acc16[2 * TM][NB];
    if constexpr (MI16) {
        f32x4 init16[NB];
#pragma unroll
        for (int j = 0; j < NB; ++j) init16[j] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
        if (bias_in_acc) {
            typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
            const uint16_t* bp = g.bias + n0 + wn * WTNX + 4 * (lane >> 4);
#pragma unroll
            for (int j = 0; j < NB; ++j) {
                const u32x2 b4 = *(const u32x2*)(bp + j * 16);
                init16[j] = f32x4{bf16_lo(b4.x), bf16_hi(b4.x), bf16_lo(b4.y), bf16_hi(b4.y)};
            }
        }
#pragma unroll
        for (int i = 0; i < 2 * TM; ++i)
#pragma unroll
            for (int j = 0; j < NB; ++j) acc16[i][j] = init16[j];
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
        const int64_t wave_off = (int64_t)(m0 + wm * WTM - band_lo) * g.N + n0 + wn * WTN;
        auto issue_item = [&](int it, int stage) __attribute__((always_inline)) {
            // past the end: all lanes re-read 16 bytes of the last item (the load count per item
            // is fixed for the vmcnt arithmetic; the data is never used)
            const bool live = it < n_items;
            const int itc = min(it, n_items - 1);
            const i32x4 rs = make_rsrc((const uint16_t*)g.peer.p[itc >> 2] + wave_off + (int64_t)(itc & 3) * 32 * g.N);
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
    // The same on 16x16x32 blocks, where one MFMA takes the partial sums of TWO peers: with
    //   Y[m][k] = P_a[m][16j + k] (k < 16),  P_b[m][16j + k - 16] (k >= 16)   and   X[n][k] = (k % 16 == n),
    // acc16[n][m] += sum_{k<32} X[n][k] * Y[m][k] = P_a[m][16j + n] + P_b[m][16j + n].  The operand wants, per
    // lane, 8 consecutive columns of one row: lanes 0..31 take them from peer a, lanes 32..63 from
    // peer b.  An item is a pair's 16 rows x 128 columns of this wave (rows 0..15 of the stage: peer
    // a, rows 16..31: peer b; 8 KiB, eight LDS-DMA loads); half as many MFMA cycles per peer as the
    // 32x32x16 form.  An odd peer count repeats the last peer as b and masks it in X (a product
    // 0 * finite adds nothing).
    auto peer_phase16 = [&]() __attribute__((always_inline)) {
        if constexpr (NB == 2 * TN) {
        constexpr int kItemLoads = 8;
        constexpr int kItemBytes = kItemLoads * 1024;
        constexpr int kAhead = 4;
        constexpr int kSlabs = 2 * TM;         // 16-row slabs of the wave
        static_assert(kSlabs % kAhead == 0 && kAhead * kItemBytes * WM * WN <= LDS_BYTES, "peer stages must fit in the ring");
        typedef short s16x8 __attribute__((ext_vector_type(8)));
        bf16x8 xsel[2];   // [0]: both peers of the pair, [1]: peer a only
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            s16x8 x;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const int k = 8 * (lane >> 4) + e;
                x[e] = ((k & 15) == (lane & 15) && (h == 0 || k < 16)) ? (short)0x3f80 : (short)0;
            }
            xsel[h] = __builtin_bit_cast(bf16x8, x);
        }
        const uint32_t region = (uint32_t)wave * (kAhead * kItemBytes);
        // load r of an item fills stage rows 4r .. 4r+3 (r < 4: peer a, else peer b): lane l -> row
        // 4(r % 4) + l/16 of the slab, piece slot l%16 holds piece slot ^ row
        uint32_t pvoff[4];
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            const int row = 4 * b + (lane >> 4);
            pvoff[b] = (uint32_t)(((int64_t)row * g.N + (((lane & 15) ^ row) << 3)) * 2);
        }
        // fragment of column block bj: lane l -> stage row l%16 + 16(l/32), piece 2 bj + (l/16)%2
        uint32_t pa[2 * TN];
#pragma unroll
        for (int bj = 0; bj < 2 * TN; ++bj) {
            const int row = (lane & 15) + 16 * (lane >> 5);
            pa[bj] = region + (uint32_t)(row * 256 + (((2 * bj + ((lane >> 4) & 1)) ^ (row & 15)) << 4));
        }
        const int n_pairs = (g.n_peers + 1) >> 1;
        const int n_items = n_pairs * kSlabs;    // item = (pair, slab), pair-major
        const int64_t wave_off = (int64_t)(m0 + wm * WTM - band_lo) * g.N + n0 + wn * WTN;
        auto issue_item = [&](int it, int stage) __attribute__((always_inline)) {
            // past the end: all lanes re-read 16 bytes of the last item (the load count per item
            // is fixed for the vmcnt arithmetic; the data is never used)
            const bool live = it < n_items;
            const int itc = min(it, n_items - 1);
            const int qa = 2 * (itc / kSlabs), qb = min(qa + 1, g.n_peers - 1);
            const int64_t off = wave_off + (int64_t)(itc % kSlabs) * 16 * g.N;
            const i32x4 rs_a = make_rsrc((const uint16_t*)g.peer.p[qa] + off);
            const i32x4 rs_b = make_rsrc((const uint16_t*)g.peer.p[qb] + off);
#pragma unroll
            for (int r = 0; r < kItemLoads; ++r)
                lds_dma_b128_stream(r < 4 ? rs_a : rs_b, region + stage * kItemBytes + r * 1024, live ? pvoff[r & 3] : 0u, 0);
        };
#pragma unroll
        for (int it = 0; it < kAhead; ++it) issue_item(it, it);
#pragma nounroll
        for (int pr = 0; pr < n_pairs; ++pr) {
            const bf16x8 xs = (2 * pr + 1 < g.n_peers) ? xsel[0] : xsel[1];
#pragma unroll
            for (int i = 0; i < kSlabs; ++i) {
                // item (pr, i) has landed when at most the three younger items are outstanding; the
                // stages are private to the wave, so no barrier
                __builtin_amdgcn_s_waitcnt(vmcnt_imm((kAhead - 1) * kItemLoads));
                KR_SCHED_FENCE();
                bf16x8 y[2 * TN];
#pragma unroll
                for (int bj = 0; bj < 2 * TN; ++bj) y[bj] = *(lds_frag)(size_t)(pa[bj] + (i % kAhead) * kItemBytes);
                KR_SCHED_FENCE();   // all eight reads in flight before the first MFMA waits for one
#pragma unroll
                for (int bj = 0; bj < 2 * TN; ++bj)
                    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc16[i][bj]) : "v"(xs), "v"(y[bj]));
                // every fragment read has returned before the stage is handed back to the DMA
                __builtin_amdgcn_s_waitcnt(kLgkm0);
                KR_SCHED_FENCE();
                issue_item(pr * kSlabs + i + kAhead, i % kAhead);
                KR_SCHED_FENCE();
            }
        }
        __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
        __syncthreads();   // the ring is handed on (k loop or epilogue patches of other waves)
        }
    };
    // An empty statement that names every accumulator as an AGPR operand, placed between the
    // phases: with the live ranges cut here the register allocator keeps the accumulators
    // where the MFMAs left them instead of moving them to VGPRs and memory for the next phase.
    auto pin_accumulators = [&]() __attribute__((always_inline)) {
        if constexpr (MI16) {
#pragma unroll
            for (int i = 0; i < 2 * TM; ++i)
#pragma unroll
                for (int j = 0; j < NB; ++j) asm volatile("" : "+a"(acc16[i][j]));
        } else {
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j) asm volatile("" : "+a"(acc[i][j]));
        }
    };
    if (PEERS_FIRST && mfma_peers) {
        if constexpr (MI16 && NB == 2 * TN) peer_phase16();
        else if constexpr (!MI16) peer_phase();
    }
    pin_accumulators();

    // ---- prologue: request k-step 0 and the first loads of step 1; wait for step 0 ------------
    // How the LOADS_PER_TILE loads of a k-step are spread.  32x32x16 form: kEarly go out right behind the
    // barrier that frees their stage (rest of sub-step 3 of step t-2), the others during sub-steps 0 and
    // 1 of step t-1 -- every second MFMA.  One per MFMA from four waves is twice what the CU's
    // address unit takes (the waves then stall at issue).
    // 16x16x32 form: the stage is free early in the step (barrier (a) of k_step16, behind slot kBarA0 of
    // sub-step 0), and from there the loads of step t+2 go out evenly over a whole step's worth of
    // slots -- one per eight MFMAs (seven in the 224-column tile), 128 cycles apart; those that fall
    // behind the end of step t are the first thing step t+1 issues (kInStep counts the others).
    // fp8 form: see k_step8.
    constexpr int kEarly = 6;
    constexpr int kFrags16 = NB + 2 * TM;                              // fragments of a sub-step: 16 or 15
    constexpr int kBarA0 = 2 * (kFrags16 - 1) + (NB == 7 ? 8 : 10);    // slot of sub-step 0 behind which every read of the stage has returned
    constexpr int kLoadGap16 = NB == 7 ? 7 : 8;
    constexpr int kSlots16 = 2 * 2 * TM * NB;                          // MFMAs of a k-step: 128 or 112
    constexpr int kInStep = (kSlots16 - 1 - kBarA0 - 2) / kLoadGap16 + 1 < LOADS_TILE ? (kSlots16 - 1 - kBarA0 - 2) / kLoadGap16 + 1 : LOADS_TILE;
    constexpr int kBarA8 = 12, kBarB8 = 39, kLoadGap8 = 3;               // fp8 form (k_step8): barrier slots, slots between loads
    constexpr int kInStep8 = (63 - kBarA8 - 1) / kLoadGap8 + 1 < LOADS_TILE ? (63 - kBarA8 - 1) / kLoadGap8 + 1 : LOADS_TILE;
    constexpr int kFirst = F8 ? kInStep8 : MI16 ? kInStep : kEarly;   // loads of step 1 the prologue issues
    static_assert(NSTAGE == 2 && LOADS_PER_TILE == 16 && (LOADS_TILE == 16 || (NB == 7 && LOADS_TILE == 15)), "load schedules below");
#pragma unroll
    for (int q = 0; q < LOADS_TILE; ++q) issue_load(0, 0, q);
#pragma unroll
    for (int q = 0; q < kFirst; ++q) issue_load(1, 1, q);
    __builtin_amdgcn_s_waitcnt(vmcnt_imm(kFirst));
    __builtin_amdgcn_s_barrier();
    KR_SCHED_FENCE();
    if constexpr (F8) {
#pragma unroll
        for (int r = 0; r < 24; ++r) read_frag8(0, r, 0);
    } else if constexpr (MI16) {   // (A blocks 4..7 are read inside the first sub-step)
#pragma unroll
        for (int j = 0; j < NB; ++j) read_b16(0, j, 0, 0);
#pragma unroll
        for (int i = 0; i < TM; ++i) read_a16(0, i, 0, 0);
    } else {
#pragma unroll
        for (int i = 0; i < TM; ++i) read_a(0, i, 0, 0);
#pragma unroll
        for (int j = 0; j < TN; ++j) read_b(0, j, 0, 0);
    }

    // ---- main loop ---------------------------------------------------------------------------
    // k-step t (64 k): 4 sub-steps of 16 MFMAs on alternating fragment buffers; sub-step ks
    // computes on buffer ks&1 while the fragments of the next sub-step are read into the other.
    // The fragments of sub-step 3 are read during sub-step 2, so when a wave has issued the first
    // MFMAs of sub-step 3 every LDS read of the stage has returned: there it waits for its own
    // loads of step t+1 and meets the other waves.  From then on stage t+1 is complete (its first
    // fragments are read next) and stage t is free for the loads of step t+2.
    constexpr int NM = TM * TN;
    auto k_step = [&](int t, auto stage_c) __attribute__((always_inline)) {
        const uint32_t stage_cur = stage_c;
        const uint32_t stage_nxt = stage_cur ^ 1u;
        const uint32_t st_cur = stage_cur * A_ST, st_nxt = stage_nxt * A_ST;
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            const int cur = ks & 1, nxt = cur ^ 1;
#pragma unroll
            for (int s = 0; s < NM; ++s) {
                const int i = s / TN, j = s % TN;
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bfr[cur][j], af[cur][i], acc[i][j], 0, 0, 0);
                if (ks < 3) {
                    // fragments of the next sub-step, this stage: A blocks next to MFMAs 0..3, B 4..7
                    if (s < TM) read_a(nxt, s, ks + 1, st_cur);
                    else if (s < TM + TN) read_b(nxt, s - TM, ks + 1, st_cur);
                    // the later loads of step t+1
                    if (ks == 0 && s % 2 == 0) issue_load(t + 1, stage_nxt, kEarly + s / 2);
                    if (ks == 1 && s % 2 == 0 && s < 4) issue_load(t + 1, stage_nxt, kEarly + 8 + s / 2);
                } else {
                    if (s == 3) {
                        KR_SCHED_FENCE();
                        __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
                        __builtin_amdgcn_s_barrier();
                    }
                    // first fragments of k-step t+1
                    if (s >= 4 && s < 4 + TM) read_a(nxt, s - 4, 0, st_nxt);
                    else if (s >= 4 + TM && s < 4 + TM + TN) read_b(nxt, s - 4 - TM, 0, st_nxt);
                    // the first loads of step t+2, into the stage just vacated
                    if (s >= 4 && s % 2 == 0) issue_load(t + 2, stage_cur, (s - 4) / 2);
                }
                KR_SCHED_FENCE();
            }
        }
    };
    // The same k-step on 16x16x32 blocks: two sub-steps of 64 MFMAs (32 k each) on alternating
    // fragment buffers.  An MFMA lasts 16 cycles here, room for about three other instructions,
    // so fragment reads and loads get MFMA slots of their own.  Row i of MFMAs needs A block i and
    // all B blocks, so a sub-step can start on the B blocks and the first A blocks; the others
    // follow while it runs.
    //   sub-step 0: the fragments of sub-step 1 (every second slot), A blocks 4..7 of this
    //     sub-step (slots 1, 9, 17, 25), the last loads of step t+1;
    //   behind slot kBarA0 of sub-step 0: every LDS read of the stage has returned -- barrier (a):
    //     the stage is free, the loads of step t+2 start (one per eight MFMAs, through the rest of
    //     the step);
    //   sub-step 1, behind MFMA 47: wait for the loads of step t+1 (the younger ones of step t+2
    //     stay outstanding) -- barrier (b) -- and read the B blocks and A blocks 0..3 of step t+1.
    // The wait sits right in front of the first read that needs the data, not in front of the first
    // load that needs the room.  Reading sub-step 1's fragments in the first half of sub-step 0 (they
    // used to take all of it, with barrier (a) in sub-step 1 and the loads crowded into what was left
    // of the step, 64 cycles apart) is what makes room for the even spacing: same process, rotating
    // operands, 8192x8192x3584 row-major B with its band 356-357 -> 348-349 us, 8192x3584x8192
    // transposed B on 224-column tiles 326-327 -> 325-326 us, 4096x8192x1024 with seven peers
    // 118.2 -> 117.2 us; with the early barrier alone and the loads still 64 cycles apart nothing moves.
    // (224-column tile, NB = 7: 56 MFMAs per sub-step; barrier (b) behind MFMA 39, the same 16 slots
    // behind it for the 7 + 4 fragments of the next step; 15 fragments of sub-step 1 to read in sub-step 0)
    constexpr int NM16 = 2 * TM * NB;
    auto read_frag16 = [&](int buf, int r, int ks2, uint32_t stage_off) __attribute__((always_inline)) {
        if (r < NB) read_b16(buf, r, ks2, stage_off);
        else read_a16(buf, r - NB, ks2, stage_off);
    };
    constexpr int kBarB = NM16 - 17;
    // loads of step t+2 issued before the wait of barrier (b) (slots kBarA0 + 2, + kLoadGap16, ... <= NM16 + kBarB)
    constexpr int kLoadsBeforeB = (NM16 + kBarB - kBarA0 - 2) / kLoadGap16 + 1 < kInStep ? (NM16 + kBarB - kBarA0 - 2) / kLoadGap16 + 1 : kInStep;
    static_assert(!MI16 || (kBarA0 < NM16 && kBarA0 + 2 + kLoadGap16 * (LOADS_TILE - 1) - kSlots16 < kBarA0 + 2),
                  "a step's late loads go out before the next step's first ones");
    auto k_step16 = [&](int t, auto stage_c) __attribute__((always_inline)) {
        const uint32_t stage_cur = stage_c;
        const uint32_t stage_nxt = stage_cur ^ 1u;
        const uint32_t st_cur = stage_cur * A_ST, st_nxt = stage_nxt * A_ST;
#pragma unroll
        for (int ks2 = 0; ks2 < 2; ++ks2) {
            const int cur = ks2, nxt = cur ^ 1;
#pragma unroll
            for (int s = 0; s < NM16; ++s) {
                const int i = s / NB, j = s % NB;
                // (written out with the accumulator tied to the AGPRs it lives in: given the
                // builtin, the register allocator moves accumulators through VGPRs and other
                // AGPRs around the MFMAs, a copy or two per MFMA)
                asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0"
                             : "+a"(acc16[i][j])
                             : "v"(bfr16[cur][j]), "v"(af16[cur][i]));
                const int slot = ks2 * NM16 + s;               // slot of the step
                const int lq = slot - kBarA0 - 2;              // loads of step t+2: slots kBarA0 + 2 + kLoadGap16 * q
                const int lw = lq + kSlots16;                  // ... and those of step t+1 that fell behind the end of step t-1
                if (ks2 == 0) {
                    if (s % 2 == 0 && s / 2 < kFrags16) read_frag16(nxt, s / 2, 1, st_cur);
                    if (s % 8 == 1 && s / 8 + 4 < 2 * TM) read_a16(cur, s / 8 + 4, 0, st_cur);
                    if (s == kBarA0) {
                        KR_SCHED_FENCE();
                        __builtin_amdgcn_s_waitcnt(kLgkm0);
                        __builtin_amdgcn_s_barrier();
                    }
                }
                if (lq >= 0 && lq % kLoadGap16 == 0 && lq / kLoadGap16 < kInStep) issue_load(t + 2, stage_cur, lq / kLoadGap16);
                if (lw % kLoadGap16 == 0 && lw / kLoadGap16 >= kInStep && lw / kLoadGap16 < LOADS_TILE) issue_load(t + 1, stage_nxt, lw / kLoadGap16);
                if (ks2 == 1) {
                    if (s == kBarB) {
                        KR_SCHED_FENCE();
                        __builtin_amdgcn_s_waitcnt(vmcnt_imm(kLoadsBeforeB));
                        __builtin_amdgcn_s_barrier();
                    }
                    // B blocks and A blocks 0..3 of k-step t+1: slots 48, 50, ..., 62; 63; 51, 55, 59
                    if (s > kBarB && s % 2 == 0) read_frag16(nxt, (s - kBarB - 1) / 2, 0, st_nxt);
                    if (NB == 2 * TN && s == NM16 - 1) read_frag16(nxt, NB, 0, st_nxt);   // (NB = 7: A block 0 came with slot 54)
                    if (s > kBarB && s % 4 == 3 && s < NM16 - 1) read_frag16(nxt, NB + 1 + (s - kBarB - 4) / 4, 0, st_nxt);
                }
                KR_SCHED_FENCE();
            }
        }
    };
    // The k-step on fp8 operands: 64 MFMAs of 16x16x128 (32 cycles each), rows of blocks in order; a step's B fragments live
    // through the whole step, so B is double-buffered in registers (8 blocks x 8 registers x 2) and A in two halves of
    // four blocks.
    //   slots 0..7: A blocks 4..7 of this step (needed from slot 32 on);
    //   behind slot kBarA8: every LDS read of the stage has returned -- barrier (a): the stage is free, and the 16 loads of
    //     step t+2 go out, one per three MFMAs (96 cycles apart: measured 3-5 % faster than 64 cycles apart);
    //   behind slot kBarB8: wait for the loads of step t+1 (the younger ones of step t+2 stay outstanding) -- barrier (b) --
    //     and read all of B and A blocks 0..3 of step t+1, one half-fragment per slot (two per slot at first, were the
    //     barrier later than slot 39).
    // Same-process comparison of (kBarA8, kBarB8, gap) on 8192x4096x8192, 4096x6656x16384, 8192x8192x3584, rotating operands:
    // (16, 44, 2) 188 / 313-320 / 169-170 us, (16, 40, 2) 184 / 308-312 / 167, (16, 39, 3) 179 / 297-300 / 164-165,
    // (12, 39, 3) 174-176 / 296-298 / 164 (hipBLASLt's scaled fp8 product in the same runs: 168-172 / 304-305 / 160-165);
    // (12, 39, 4) and (12, 43, 4), whose last loads go out at the start of the next step, measure like (12, 39, 3).
    constexpr int kLoadsBeforeB8 = (kBarB8 - kBarA8 - 1) / kLoadGap8 + 1 < kInStep8 ? (kBarB8 - kBarA8 - 1) / kLoadGap8 + 1 : kInStep8;   // loads of step t+2 in slots <= kBarB8
    constexpr int kReadSlots8 = 63 - kBarB8, kDoubleReads8 = kReadSlots8 < 24 ? 24 - kReadSlots8 : 0;   // 24 fragment halves behind barrier (b): two per slot at first
    static_assert(kBarA8 >= 8 && kBarB8 > kBarA8 && kBarA8 + 1 + kLoadGap8 * (LOADS_PER_TILE - 1) - 64 < kBarA8 + 1 && kDoubleReads8 <= kReadSlots8, "fp8 k-step schedule");
    auto k_step8 = [&](int t, auto stage_c) __attribute__((always_inline)) {
        const uint32_t stage_cur = stage_c;
        const uint32_t stage_nxt = stage_cur ^ 1u;
        const uint32_t st_cur = stage_cur * A_ST, st_nxt = stage_nxt * A_ST;
        const int cur = stage_c, nxt = cur ^ 1;
#pragma unroll
        for (int s = 0; s < 64; ++s) {
            const int i = s / 8, j = s % 8;
            // (accumulator tied to its AGPRs, as in k_step16; formats left at their default, fp8 e4m3 for both operands)
            asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, %0"
                         : "+a"(acc16[i][j])
                         : "v"(bf8[cur][j]), "v"(af8[i >> 2][i & 3]));
            if (s < 8) read_a8_late(s, st_cur);
            if (s == kBarA8) {
                KR_SCHED_FENCE();
                __builtin_amdgcn_s_waitcnt(kLgkm0);
                __builtin_amdgcn_s_barrier();
            }
            if (s > kBarA8 && (s - kBarA8 - 1) % kLoadGap8 == 0 && (s - kBarA8 - 1) / kLoadGap8 < kInStep8)
                issue_load(t + 2, stage_cur, (s - kBarA8 - 1) / kLoadGap8);
            if ((s + 64 - kBarA8 - 1) % kLoadGap8 == 0 && (s + 64 - kBarA8 - 1) / kLoadGap8 >= kInStep8 && (s + 64 - kBarA8 - 1) / kLoadGap8 < LOADS_PER_TILE)
                issue_load(t + 1, stage_nxt, (s + 64 - kBarA8 - 1) / kLoadGap8);   // the loads of step t+1 that fell behind the end of step t-1
            if (s == kBarB8) {
                KR_SCHED_FENCE();
                __builtin_amdgcn_s_waitcnt(vmcnt_imm(kLoadsBeforeB8));
                __builtin_amdgcn_s_barrier();
            }
            if (s > kBarB8) {
                const int u = s - kBarB8 - 1;
                if (u < kDoubleReads8) {
                    read_frag8(nxt, 2 * u, st_nxt);
                    read_frag8(nxt, 2 * u + 1, st_nxt);
                } else if (kDoubleReads8 + u < 24) {
                    read_frag8(nxt, kDoubleReads8 + u, st_nxt);
                }
            }
            KR_SCHED_FENCE();
        }
    };
    // Main part: one trip = two k-steps, so every LDS stage offset is a compile-time constant
    // (immediate offsets on the fragment reads) and the loop branch is taken once per 128 MFMAs;
    // an odd last step follows.
    int t = 0;
    if constexpr (F8) {
#pragma nounroll
        for (; t + 2 <= kt_total; t += 2) {
            k_step8(t, std::integral_constant<uint32_t, 0>{});
            k_step8(t + 1, std::integral_constant<uint32_t, 1>{});
        }
        pin_accumulators();
        if (t < kt_total) k_step8(t, std::integral_constant<uint32_t, 0>{});
    } else if constexpr (MI16) {
#pragma nounroll
        for (; t + 2 <= kt_total; t += 2) {
            k_step16(t, std::integral_constant<uint32_t, 0>{});
            k_step16(t + 1, std::integral_constant<uint32_t, 1>{});
        }
        pin_accumulators();
        if (t < kt_total) k_step16(t, std::integral_constant<uint32_t, 0>{});
    } else {
#pragma nounroll
        for (; t + 2 <= kt_total; t += 2) {
            k_step(t, std::integral_constant<uint32_t, 0>{});
            k_step(t + 1, std::integral_constant<uint32_t, 1>{});
        }
        pin_accumulators();
        if (t < kt_total) k_step(t, std::integral_constant<uint32_t, 0>{});
    }
    // drain the tail's surplus loads before the LDS is reused
    __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
    __syncthreads();

    pin_accumulators();
    if constexpr (SPLIT) {
        // accumulators to the workspace in register order: quad q = (i, j, v/4) of thread tid at
        // [tail tile][split][q][tid], so that a wave's store is 1 KiB of consecutive addresses
        f32x4* part = (f32x4*)g.out + ((int64_t)tail_index * g.k_splits + split) * (TM * TN * 4 * WM * WN * 64) + tid;
        if constexpr (MI16) {   // quad q = block (i, j) of the 8 x 8
#pragma unroll
            for (int i = 0; i < 2 * TM; ++i)
#pragma unroll
                for (int j = 0; j < 2 * TN; ++j)
                    __builtin_nontemporal_store(acc16[i][j], part + (i * 2 * TN + j) * (WM * WN * 64));
            return;
        }
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int v = 0; v < 4; ++v)
                    __builtin_nontemporal_store(f32x4{acc[i][j][4 * v], acc[i][j][4 * v + 1], acc[i][j][4 * v + 2],
                                                      acc[i][j][4 * v + 3]},
                                                part + ((i * TN + j) * 4 + v) * (WM * WN * 64));
        return;
    }
    if (!PEERS_FIRST && mfma_peers) {
        if constexpr (MI16 && NB == 2 * TN) peer_phase16();
        else if constexpr (!MI16) peer_phase();
    }
    pin_accumulators();
    // peers and bias that are already in the accumulators are not added again
    if (F8 && g.out_fp8) {
        if constexpr (F8)
            store_tile_fp8_blocks(acc16, smem, (uint8_t*)g.out + (int64_t)(m0 + wm * WTM) * g.N + n0 + wn * WTN, g.N, lane, wave);
    } else if constexpr (NB != 2 * TN) {
        // 224-column tile of a plain product: every row goes to `out`
        store_tile_bf16_blocks<NB>(acc16, smem, (uint16_t*)g.out + (int64_t)(m0 + wm * WTM) * g.N + n0 + wn * WTNX, g.N, lane, wave);
    } else if constexpr (MI16) {
        if (full_tile) {
            gemm_epilogue<BM, WTM, WTN, TM, TN, true, EP_WAVE>(g, mfma_peers ? 0 : g.n_peers, bias_in_acc ? nullptr : g.bias, acc16,
                                                               smem, m0, n0, wm, wn, lane, wave);
        } else if constexpr (RAGGED) {
            gemm_epilogue<BM, WTM, WTN, TM, TN, false, EP_WAVE>(g, g.n_peers, g.bias, acc16, smem, m0, n0, wm, wn, lane, wave);
        }
    } else if (full_tile) {
        gemm_epilogue<BM, WTM, WTN, TM, TN, true, EP_WAVE>(g, mfma_peers ? 0 : g.n_peers, bias_in_acc ? nullptr : g.bias,
                                                           acc, smem, m0, n0, wm, wn, lane, wave);
    } else if constexpr (RAGGED) {   // edge tile: every access checked against M and N
        gemm_epilogue<BM, WTM, WTN, TM, TN, false, EP_WAVE>(g, g.n_peers, g.bias, acc, smem, m0, n0, wm, wn, lane, wave);
    }
}
#undef KR_SCHED_FENCE

// The two phase orders are two complete copies of the tile code under one uniform branch: each
// copy is straight-line (phase, phase, epilogue), which keeps the 256 accumulators in their
// registers; one copy with a run-time order has the register allocator move them through memory.
template <bool B_NT, bool RAGGED>
__global__ __launch_bounds__(WM* WN * 64) void gemm_dtl_kernel(const GemmArgs g) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];   // starts at LDS address 0
    if (g.peers_on_mfma && g.n_peers > 0 && (g.peers_on_mfma == 1 ? ((blockIdx.x >> 3) & 1) : g.peers_on_mfma == 2)) gemm_dtl_tile<B_NT, true, false, RAGGED>(g, smem);
    else gemm_dtl_tile<B_NT, false, false, RAGGED>(g, smem);
}

// The same on 16x16x32 blocks (k loop and peer phase).
template <bool B_NT, bool RAGGED>
__global__ __launch_bounds__(WM* WN * 64) void gemm_dtl16_kernel(const GemmArgs g) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    if (g.peers_on_mfma && g.n_peers > 0 && (g.peers_on_mfma == 1 ? ((blockIdx.x >> 3) & 1) : g.peers_on_mfma == 2)) gemm_dtl_tile<B_NT, true, false, RAGGED, true>(g, smem);
    else gemm_dtl_tile<B_NT, false, false, RAGGED, true>(g, smem);
}

// 256 x 224 tiles (plain products, transposed-contiguous B).
__global__ __launch_bounds__(WM* WN * 64) void gemm_dtl16n7_kernel(const GemmArgs g) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    gemm_dtl_tile<true, false, false, false, true, 7>(g, smem);
}

// fp8 (e4m3fn) operands, transposed-contiguous B, whole 256 x 256 tiles; the result is fp8, bf16 or fp32.
__global__ __launch_bounds__(WM* WN * 64) void gemm_dtl8_kernel(const GemmArgs g) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    gemm_dtl_tile<true, false, false, false, true, 2 * TN, true>(g, smem);
}

}  // namespace

// g as for the bf16 kernel with the fp8 operands described in two-byte units (K, lda, ldb halved).
hipError_t launch_gemm_dtl8(const GemmArgs& g, hipStream_t st) {
    static std::atomic<uint64_t> opted;
    if (hipError_t e = lds_opt_in((const void*)gemm_dtl8_kernel, LDS_BYTES, opted); e != hipSuccess) return e;
    hipLaunchKernelGGL(gemm_dtl8_kernel, dim3((unsigned)(g.tiles_m * g.tiles_n)), dim3(WM * WN * 64), LDS_BYTES, st, g);
    return hipGetLastError();
}

// Second launch of a call with a split tail: g.k_splits workgroups per tile of the last partial
// round (g.out = workspace).
template <bool B_NT, bool MI16>
__global__ __launch_bounds__(WM* WN * 64) void gemm_dtl_split_kernel(const GemmArgs g) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    gemm_dtl_tile<B_NT, false, true, false, MI16>(g, smem);
}

// Third launch: sums the parts of every tail tile in the order 0..S-1 and applies the epilogue
// of the one-pass kernel to it, with that kernel's rounding (spelled out at `tile_in_band` below:
// whole-band tiles sum product, peers and bias in fp32 and round once, every other tile of a bf16
// result rounds the product first).
// One thread per accumulator quad: block b = (tail tile, quad q), thread tid as in the GEMM
// kernel; the quad is row wm*128 + 32i + lane%32, columns wn*128 + 32j + 8(v/4) + 4(lane/32) .. +3.
__global__ __launch_bounds__(WM* WN * 64) void gemm_dtl_tail_finish_kernel(const GemmArgs g, const f32x4* __restrict__ parts) {
    constexpr int T = WM * WN * 64, NQ = TM * TN * 4;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int u = blockIdx.x / NQ, q = blockIdx.x % NQ;
    const int S = g.k_splits;
    const f32x4* p = parts + ((int64_t)u * S * NQ + q) * T + tid;
    f32x4 sum = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int sp = 0; sp < S; ++sp) {
        const f32x4 x = __builtin_nontemporal_load(p + (int64_t)sp * NQ * T);
        sum.x += x.x; sum.y += x.y; sum.z += x.z; sum.w += x.w;
    }
    int tile_m, tile_n;
    tile_schedule(g, schedule_position(g, u, g.tiles_m * g.tiles_n - g.tail_tiles), tile_m, tile_n);
    int m, n;
    if (g.mi16) {   // 16x16 blocks: quad q = block (q / 16, q % 16); row lane%16, columns 4(lane/16) .. +3
        m = tile_m * BM + (wave / WN) * WTM + (q / (2 * TN)) * 16 + (lane & 15);
        n = tile_n * BN + (wave % WN) * WTN + (q % (2 * TN)) * 16 + 4 * (lane >> 4);
    } else {
        const int i = q / (TN * 4), j = (q / 4) % TN, v4 = q % 4;
        m = tile_m * BM + (wave / WN) * WTM + i * 32 + (lane & 31);
        n = tile_n * BN + (wave % WN) * WTN + j * 32 + 8 * v4 + 4 * (lane >> 5);
    }
    typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
    const int mb = m - g.band_row0;
    if (mb < 0 || mb >= g.band_rows) {
        if (g.c_full != nullptr)
            *(u32x2*)(g.c_full + (int64_t)m * g.N + n) = u32x2{pack_bf16(sum.x, sum.y), pack_bf16(sum.z, sum.w)};
        return;
    }
    const int64_t off = (int64_t)mb * g.N + n;
    // The rounding of the main launch's tiles (gemm_dtl_tile): a tile that lies wholly in the band
    // and adds its peers on the matrix cores (or has none) sums product, peers and bias in fp32 and
    // rounds once; every other tile of a bf16 result rounds the product to bf16 first and adds the
    // peers and the bias to that.
    const bool tile_in_band = tile_m * BM >= g.band_row0 && tile_m * BM + BM <= g.band_row0 + g.band_rows;
    const bool peers_exact = g.peers_on_mfma && g.n_peers > 0 && tile_in_band;
    const bool bias_exact = g.bias != nullptr && tile_in_band && (g.n_peers == 0 || peers_exact);
    auto add_peers = [&]() {
        for (int pq = 0; pq < g.n_peers; ++pq) {
            const u32x2 w = *(const u32x2*)((const uint16_t*)g.peer.p[pq] + off);
            sum.x += bf16_lo(w.x); sum.y += bf16_hi(w.x); sum.z += bf16_lo(w.y); sum.w += bf16_hi(w.y);
        }
    };
    auto add_bias = [&]() {
        const u32x2 w = *(const u32x2*)(g.bias + n);
        sum.x += bf16_lo(w.x); sum.y += bf16_hi(w.x); sum.z += bf16_lo(w.y); sum.w += bf16_hi(w.y);
    };
    if (peers_exact) add_peers();
    if (bias_exact) add_bias();
    if (!g.out_is_fp32) {
        const uint32_t lo = pack_bf16(sum.x, sum.y), hi = pack_bf16(sum.z, sum.w);
        sum = f32x4{bf16_lo(lo), bf16_hi(lo), bf16_lo(hi), bf16_hi(hi)};
    }
    if (!peers_exact) add_peers();
    if (g.bias != nullptr && !bias_exact) add_bias();
    if (g.out_is_fp32) *(f32x4*)((float*)g.out + off) = sum;
    else *(u32x2*)((uint16_t*)g.out + off) = u32x2{pack_bf16(sum.x, sum.y), pack_bf16(sum.z, sum.w)};
}

bool gemm_dtl_supported(const GemmArgs& g) {
    return g.K % BKD == 0 && g.K >= BKD &&
           (int64_t)BM * g.lda * 2 < 0x7fffffffLL && (int64_t)(BN > 64 ? BN : 64) * g.ldb * 2 < 0x7fffffffLL;
}

hipError_t launch_gemm_dtl(const GemmArgs& g, bool b_nt, hipStream_t st, void* workspace) {
    const dim3 grid((unsigned)(g.tiles_m * g.tiles_n - g.tail_tiles)), block(WM * WN * 64);
    const bool ragged = g.M % BM != 0 || g.N % BN != 0;
    const void* kfn = b_nt ? (ragged ? (const void*)gemm_dtl_kernel<true, true> : (const void*)gemm_dtl_kernel<true, false>)
                           : (ragged ? (const void*)gemm_dtl_kernel<false, true> : (const void*)gemm_dtl_kernel<false, false>);
    if (g.mi16)
        kfn = b_nt ? (ragged ? (const void*)gemm_dtl16_kernel<true, true> : (const void*)gemm_dtl16_kernel<true, false>)
                   : (ragged ? (const void*)gemm_dtl16_kernel<false, true> : (const void*)gemm_dtl16_kernel<false, false>);
    static std::atomic<uint64_t> opted[8];
    if (hipError_t e = lds_opt_in(kfn, LDS_BYTES, opted[(g.mi16 ? 4 : 0) + (b_nt ? 2 : 0) + (ragged ? 1 : 0)]); e != hipSuccess)
        return e;
    if (g.n224) {
        static std::atomic<uint64_t> nopted;
        if (hipError_t e = lds_opt_in((const void*)gemm_dtl16n7_kernel, LDS_BYTES, nopted); e != hipSuccess) return e;
        hipLaunchKernelGGL(gemm_dtl16n7_kernel, grid, block, LDS_BYTES, st, g);
        return hipGetLastError();
    }
    if (grid.x == 0) {
        // every tile belongs to the split partial round
    } else if (g.mi16) {
        if (b_nt) {
            if (ragged) hipLaunchKernelGGL((gemm_dtl16_kernel<true, true>), grid, block, LDS_BYTES, st, g);
            else hipLaunchKernelGGL((gemm_dtl16_kernel<true, false>), grid, block, LDS_BYTES, st, g);
        } else {
            if (ragged) hipLaunchKernelGGL((gemm_dtl16_kernel<false, true>), grid, block, LDS_BYTES, st, g);
            else hipLaunchKernelGGL((gemm_dtl16_kernel<false, false>), grid, block, LDS_BYTES, st, g);
        }
    } else if (b_nt) {
        if (ragged) hipLaunchKernelGGL((gemm_dtl_kernel<true, true>), grid, block, LDS_BYTES, st, g);
        else hipLaunchKernelGGL((gemm_dtl_kernel<true, false>), grid, block, LDS_BYTES, st, g);
    } else {
        if (ragged) hipLaunchKernelGGL((gemm_dtl_kernel<false, true>), grid, block, LDS_BYTES, st, g);
        else hipLaunchKernelGGL((gemm_dtl_kernel<false, false>), grid, block, LDS_BYTES, st, g);
    }
    if (g.tail_tiles > 0) {
        // the tiles of the last partial round: k_splits workgroups each, parts to the workspace,
        // then the sum and the epilogue
        static std::atomic<uint64_t> split_opted[4];
        const void* sfn = g.mi16 ? (b_nt ? (const void*)gemm_dtl_split_kernel<true, true> : (const void*)gemm_dtl_split_kernel<false, true>)
                                 : (b_nt ? (const void*)gemm_dtl_split_kernel<true, false> : (const void*)gemm_dtl_split_kernel<false, false>);
        if (hipError_t e2 = lds_opt_in(sfn, LDS_BYTES, split_opted[(g.mi16 ? 2 : 0) + (b_nt ? 1 : 0)]); e2 != hipSuccess) return e2;
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
        GemmArgs gs = g;
        gs.out = workspace;
        const dim3 sgrid((unsigned)(g.tail_tiles * g.k_splits));
        if (g.mi16) {
            if (b_nt) hipLaunchKernelGGL((gemm_dtl_split_kernel<true, true>), sgrid, block, LDS_BYTES, st, gs);
            else hipLaunchKernelGGL((gemm_dtl_split_kernel<false, true>), sgrid, block, LDS_BYTES, st, gs);
        } else {
            if (b_nt) hipLaunchKernelGGL((gemm_dtl_split_kernel<true, false>), sgrid, block, LDS_BYTES, st, gs);
            else hipLaunchKernelGGL((gemm_dtl_split_kernel<false, false>), sgrid, block, LDS_BYTES, st, gs);
        }
        e = hipGetLastError();
        if (e != hipSuccess) return e;
        hipLaunchKernelGGL(gemm_dtl_tail_finish_kernel, dim3((unsigned)(g.tail_tiles * TM * TN * 4)), block, 0, st, g,
                           (const f32x4*)workspace);
    }
    return hipGetLastError();
}

}  // namespace kr
