// Stream-ordered 32-bit flag write: the arrival signal behind a chunk copy of the all-gather.
#include "common.h"

namespace kr {

// One store, written through to memory at system scope.  What the stream did before this
// kernel (the chunk copy) is complete and written back when this kernel starts -- the order
// of commands on a stream gives that -- so the store itself needs no cache write-back of its
// own (a release here would also flush whatever the concurrently running GEMM has written).
__global__ __launch_bounds__(kWave) void write_value32_kernel(uint32_t* addr, uint32_t value) {
    if (threadIdx.x == 0) __hip_atomic_store(addr, value, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

}  // namespace kr

extern "C" int kr_stream_write_value32(uint32_t* addr, uint32_t value, void* stream) {
    if (addr == nullptr) return KR_ERR_NULL_POINTER;
    if ((reinterpret_cast<uintptr_t>(addr) & 3u) != 0) return KR_ERR_ALIGNMENT;
    hipLaunchKernelGGL(kr::write_value32_kernel, dim3(1), dim3(kr::kWave), 0, (hipStream_t)stream, addr, value);
    return (int)hipGetLastError();
}
