// Stream-ordered flag write and flag wait, and the copy-engine copy they bracket: the pieces of
// the overlap of copies with a running GEMM (all-gather matmul, copy-engine reduce-scatter).
#include "common.h"

namespace kr {

// One store, written through to memory at system scope.  What the stream did before this
// kernel (the chunk copy) is complete and written back when this kernel starts -- the order
// of commands on a stream gives that -- so the store itself needs no cache write-back of its
// own (a release here would also flush whatever the concurrently running GEMM has written).
__global__ __launch_bounds__(kWave) void write_value32_kernel(uint32_t* addr, uint32_t value) {
    if (threadIdx.x == 0) __hip_atomic_store(addr, value, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

// Stream-ordered wait: ends once *addr == value.  One lane polls with system-scope loads and a
// short sleep; the wait is bounded by `ticks` of the 100 MHz constant clock, after which 1 is
// stored to *status (if given) and the kernel ends all the same, so the stream always drains.
// The acquire fence orders what follows on the stream behind the value seen.
__global__ __launch_bounds__(kWave) void wait_value32_kernel(const uint32_t* addr, uint32_t value, uint64_t ticks,
                                                             int* status) {
    if (threadIdx.x != 0) return;
    // a wait earlier on this stream that shares the status word has already run out: the flags are
    // not coming, and waiting for each of them in turn would only add the limit once per wait
    if (status != nullptr && __hip_atomic_load(status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM) != 0) return;
    const uint64_t t0 = __builtin_amdgcn_s_memrealtime();
    while (__hip_atomic_load(addr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM) != value) {
        if (__builtin_amdgcn_s_memrealtime() - t0 > ticks) {
            if (status != nullptr) __hip_atomic_store(status, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
            break;
        }
        __builtin_amdgcn_s_sleep(32);
    }
    __atomic_thread_fence(__ATOMIC_ACQUIRE);
}

// The two flag primitives the kernels of the all-gather matmul and of the producer GEMM use, in
// one launch: blocks 0 .. P-1 each set their flag (release exchange, as arrive_gmem_barrier with
// op = atomic_xchg), every other block waits for the flag of producer (block - P) / (C / P)
// (acquire load in a loop, as wait_gmem_barrier) -- bounded by `ticks`, after which the block
// stores 1 + flag index to *status and ends.
__global__ __launch_bounds__(kWave) void flag_arrive_wait_kernel(uint32_t* flags, int producers, int consumers,
                                                                uint64_t ticks, int* status) {
    const int b = blockIdx.x;
    if (b < producers) {
        if (threadIdx.x == 0) __hip_atomic_exchange(flags + b, 1u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
        return;
    }
    const int p = (b - producers) / (consumers / producers);
    const uint64_t t0 = __builtin_amdgcn_s_memrealtime();
    while (__hip_atomic_load(flags + p, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_AGENT) != 1u) {
        if (__builtin_amdgcn_s_memrealtime() - t0 > ticks) {
            if (status != nullptr && threadIdx.x == 0)
                __hip_atomic_store(status, 1 + p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            break;
        }
        __builtin_amdgcn_s_sleep(16);
    }
}

}  // namespace kr

extern "C" int kr_flag_arrive_wait(uint32_t* flags, int producers, int consumers, int64_t wait_limit_us, int* status,
                                   void* stream) {
    if (producers < 1 || consumers < 0 || producers > 4096 || consumers > 65536) return KR_ERR_BAD_DIM;
    if (consumers % producers != 0) return KR_ERR_STRIPE;
    if (flags == nullptr) return KR_ERR_NULL_POINTER;
    if ((reinterpret_cast<uintptr_t>(flags) & 3u) != 0 || (reinterpret_cast<uintptr_t>(status) & 3u) != 0)
        return KR_ERR_ALIGNMENT;
    if (wait_limit_us < 0) return KR_ERR_BAD_DIM;
    const uint64_t ticks = (uint64_t)(wait_limit_us > 0 ? wait_limit_us : 5000000) * 100u;
    hipLaunchKernelGGL(kr::flag_arrive_wait_kernel, dim3((unsigned)(producers + consumers)), dim3(kr::kWave), 0,
                       (hipStream_t)stream, flags, producers, consumers, ticks, status);
    return (int)hipGetLastError();
}

extern "C" int kr_stream_write_value32(uint32_t* addr, uint32_t value, void* stream) {
    if (addr == nullptr) return KR_ERR_NULL_POINTER;
    if ((reinterpret_cast<uintptr_t>(addr) & 3u) != 0) return KR_ERR_ALIGNMENT;
    hipLaunchKernelGGL(kr::write_value32_kernel, dim3(1), dim3(kr::kWave), 0, (hipStream_t)stream, addr, value);
    return (int)hipGetLastError();
}

extern "C" int kr_stream_wait_value32(const uint32_t* addr, uint32_t value, int64_t wait_limit_us, int* status,
                                      void* stream) {
    if (addr == nullptr) return KR_ERR_NULL_POINTER;
    if ((reinterpret_cast<uintptr_t>(addr) & 3u) != 0 || (reinterpret_cast<uintptr_t>(status) & 3u) != 0)
        return KR_ERR_ALIGNMENT;
    if (wait_limit_us < 0) return KR_ERR_BAD_DIM;
    const uint64_t ticks = (uint64_t)(wait_limit_us > 0 ? wait_limit_us : 5000000) * 100u;   // default 5 s
    hipLaunchKernelGGL(kr::wait_value32_kernel, dim3(1), dim3(kr::kWave), 0, (hipStream_t)stream, addr, value, ticks,
                       status);
    return (int)hipGetLastError();
}

extern "C" int kr_copy_engine_memcpy(void* dst, const void* src, int64_t bytes, void* stream) {
    if (bytes < 0) return KR_ERR_BAD_DIM;
    if (bytes == 0) return KR_OK;
    if (dst == nullptr || src == nullptr) return KR_ERR_NULL_POINTER;
    // a device-to-device copy that the runtime hands to the copy engines instead of a copy kernel:
    // it takes no CUs from the GEMM that runs beside it
    return (int)hipMemcpyAsync(dst, src, (size_t)bytes, hipMemcpyDeviceToDeviceNoCU, (hipStream_t)stream);
}
