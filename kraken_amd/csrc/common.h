// Shared device helpers for the gfx950 kernels: bf16 <-> fp32 packing, 128-bit
// vector access, wave64 reductions, host-side argument checks.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/kraken_amd.h"

namespace kr {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

constexpr int kWave = 64;

// ---- bf16 packing ---------------------------------------------------------
// A 32-bit word holds two bf16: element 2j in the low half, 2j+1 in the high half.
__device__ __forceinline__ float bf16_lo(uint32_t w) { return __builtin_bit_cast(float, w << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t w) { return __builtin_bit_cast(float, w & 0xffff0000u); }

// fp32 pair -> packed bf16 pair, round-to-nearest-even (v_cvt_pk_bf16_f32 on gfx950).
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
    bf16x2 p;
    p.x = (__bf16)lo;
    p.y = (__bf16)hi;
    return __builtin_bit_cast(uint32_t, p);
}

// 8 bf16 (one 128-bit vector) <-> 8 fp32
__device__ __forceinline__ void unpack8(const u32x4 v, float (&f)[8]) {
    f[0] = bf16_lo(v.x); f[1] = bf16_hi(v.x);
    f[2] = bf16_lo(v.y); f[3] = bf16_hi(v.y);
    f[4] = bf16_lo(v.z); f[5] = bf16_hi(v.z);
    f[6] = bf16_lo(v.w); f[7] = bf16_hi(v.w);
}
__device__ __forceinline__ void zero8(float (&f)[8]) {
#pragma unroll
    for (int j = 0; j < 8; ++j) f[j] = 0.0f;
}
// column (in 128-bit vectors) of flat vector index i in rows of d vectors
__device__ __forceinline__ uint32_t mod_vec(int64_t i, uint32_t d) {
    return (uint64_t)i <= 0xffffffffull ? (uint32_t)i % d : (uint32_t)((uint64_t)i % d);
}
__device__ __forceinline__ void add8(const u32x4 v, float (&f)[8]) {
    f[0] += bf16_lo(v.x); f[1] += bf16_hi(v.x);
    f[2] += bf16_lo(v.y); f[3] += bf16_hi(v.y);
    f[4] += bf16_lo(v.z); f[5] += bf16_hi(v.z);
    f[6] += bf16_lo(v.w); f[7] += bf16_hi(v.w);
}
__device__ __forceinline__ u32x4 pack8(const float (&f)[8]) {
    u32x4 v;
    v.x = pack_bf16(f[0], f[1]);
    v.y = pack_bf16(f[2], f[3]);
    v.z = pack_bf16(f[4], f[5]);
    v.w = pack_bf16(f[6], f[7]);
    return v;
}

// Streaming 128-bit accesses: every input byte of the reduce paths is used
// exactly once, so loads and stores carry the non-temporal hint.
__device__ __forceinline__ u32x4 ld_stream(const u32x4* p) { return __builtin_nontemporal_load(p); }
__device__ __forceinline__ void st_stream(u32x4* p, u32x4 v) { __builtin_nontemporal_store(v, p); }

// Streaming 128-bit load through a buffer descriptor: the address is the descriptor's base
// (uniform, in scalar registers) + a 32-bit byte offset per lane, so loads from many
// buffers share one offset register.  Bytes at or past `bytes` read as zero.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t stream_rsrc(const void* base, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);
}
__device__ __forceinline__ u32x4 ld_stream(__amdgpu_buffer_rsrc_t rs, uint32_t byte_off) {
    return __builtin_amdgcn_raw_buffer_load_b128(rs, (int)byte_off, 0, 2 /* non-temporal */);
}
// ---- wave64 sum -------------------------------------------------------------
// Sum over the 64 lanes of a wavefront; every lane returns the total.  The
// first four steps stay inside a row of 16 lanes and use DPP lane permutes
// (no LDS traffic); the four row totals are then combined through readlane.
template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v) {
    return __builtin_bit_cast(
        float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false));
}
__device__ __forceinline__ float wave_sum(float v) {
    v += dpp_f32<0xB1>(v);   // quad_perm [1,0,3,2]
    v += dpp_f32<0x4E>(v);   // quad_perm [2,3,0,1]
    v += dpp_f32<0x141>(v);  // row_half_mirror
    v += dpp_f32<0x140>(v);  // row_mirror
    const int b = __builtin_bit_cast(int, v);
    const float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 0));
    const float r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 16));
    const float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 32));
    const float r3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 48));
    return (r0 + r1) + (r2 + r3);
}

// ---- peer buffers ------------------------------------------------------------
// The W buffers a reduce reads, one device pointer per rank, passed to the kernels by
// value (kernel-argument memory, read through scalar loads): the pointer-table entry points
// copy the caller's table into it.
struct PeerTab {
    const u32x4* p[KR_MAX_WORLD];
    static constexpr bool kTable = true;
    __device__ __forceinline__ const u32x4* at(int r) const { return p[r]; }
};
// The same interface for the W slices of one stacked tensor, stride_v 128-bit vectors apart:
// the kernels are instantiated for both, so each form keeps its own address arithmetic.
struct StackedPeers {
    const u32x4* base;
    int64_t stride_v;
    static constexpr bool kTable = false;
    __device__ __forceinline__ const u32x4* at(int r) const { return base + r * stride_v; }
};

// ---- tuning switches ----------------------------------------------------------
// The KRAKEN_AMD_* environment variables (testing and tuning), read once per process and not on
// every launch; kr_reload_env() reads them again.  -1 = not set.
struct EnvSwitches {
    int reduce_unroll;   // KRAKEN_AMD_REDUCE_UNROLL=1|2|4
    int reduce_blocks;   // KRAKEN_AMD_REDUCE_BLOCKS=<n>
    int row_vpt;         // KRAKEN_AMD_ROW_VPT=1|2|4|8
    int row_lat;         // KRAKEN_AMD_ROW_LAT=0|1
    int row_split;       // KRAKEN_AMD_ROW_SPLIT=0|1
    int gemm_tile;       // KRAKEN_AMD_GEMM_TILE=128|256 -> 128, 256
    int gemm_peers;      // KRAKEN_AMD_GEMM_PEERS=epilogue|mfma|first|last -> 0, 1, 2, 3
    int gemm_mfma;       // KRAKEN_AMD_GEMM_MFMA=16|32 -> 16, 32
    int gemm_group;      // KRAKEN_AMD_GEMM_GROUP=<n>
    int gemm_splitk;     // KRAKEN_AMD_GEMM_SPLITK=<n>
    int gemm_tailsplit;  // KRAKEN_AMD_GEMM_TAILSPLIT=<n>
    int gemm_n224;       // KRAKEN_AMD_GEMM_N224=0|1
};
const EnvSwitches& env_switches();   // status.hip

// ---- host-side checks -------------------------------------------------------
static inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Table of the W slices of a stacked tensor (slice r at stack + r * stride elements of bf16).
// Entries past W repeat entry 0, so every entry can be dereferenced.
static inline void peer_tab_stacked(PeerTab& t, const void* stack, int W, int64_t stride_elems) {
    const uint16_t* b = static_cast<const uint16_t*>(stack);
    for (int r = 0; r < KR_MAX_WORLD; ++r)
        t.p[r] = reinterpret_cast<const u32x4*>(r < W ? b + (int64_t)r * stride_elems : b);
}

// Table copied from a caller's host array of W device pointers; KR_OK or the argument error.
static inline int peer_tab_from_ptrs(PeerTab& t, const void* const* bufs, int W) {
    if (bufs == nullptr) return KR_ERR_NULL_POINTER;
    for (int r = 0; r < W; ++r) {
        if (bufs[r] == nullptr) return KR_ERR_NULL_POINTER;
        if (!aligned16(bufs[r])) return KR_ERR_ALIGNMENT;
    }
    for (int r = 0; r < KR_MAX_WORLD; ++r) t.p[r] = static_cast<const u32x4*>(bufs[r < W ? r : 0]);
    return KR_OK;
}

}  // namespace kr
