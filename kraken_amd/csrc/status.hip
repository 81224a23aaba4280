// Version and error-text entry points of the C ABI.
#include "common.h"

#include <stdlib.h>

namespace kr {
static EnvSwitches read_env() {
    EnvSwitches e;
    auto num = [](const char* name) { const char* t = getenv(name); return t != nullptr && t[0] != 0 ? atoi(t) : -1; };
    e.reduce_unroll = num("KRAKEN_AMD_REDUCE_UNROLL");
    e.reduce_blocks = num("KRAKEN_AMD_REDUCE_BLOCKS");
    e.row_vpt = num("KRAKEN_AMD_ROW_VPT");
    e.row_lat = num("KRAKEN_AMD_ROW_LAT");
    e.row_split = num("KRAKEN_AMD_ROW_SPLIT");
    const char* t = getenv("KRAKEN_AMD_GEMM_TILE");
    e.gemm_tile = t == nullptr ? -1 : t[0] == '1' ? 128 : t[0] == '2' ? 256 : -1;
    t = getenv("KRAKEN_AMD_GEMM_PEERS");
    e.gemm_peers = t == nullptr ? -1 : t[0] == 'e' ? 0 : t[0] == 'f' ? 2 : t[0] == 'l' ? 3 : 1;
    t = getenv("KRAKEN_AMD_GEMM_MFMA");
    e.gemm_mfma = t == nullptr ? -1 : t[0] == '1' ? 16 : 32;
    e.gemm_group = num("KRAKEN_AMD_GEMM_GROUP");
    e.gemm_splitk = num("KRAKEN_AMD_GEMM_SPLITK");
    e.gemm_tailsplit = num("KRAKEN_AMD_GEMM_TAILSPLIT");
    e.gemm_n224 = num("KRAKEN_AMD_GEMM_N224");
    return e;
}
static EnvSwitches& env_storage() {
    static EnvSwitches e = read_env();
    return e;
}
const EnvSwitches& env_switches() { return env_storage(); }
}  // namespace kr

extern "C" void kr_reload_env(void) { kr::env_storage() = kr::read_env(); }

extern "C" int kr_version(void) { return 100; }  // 0.1.0

extern "C" const char* kr_strerror(int code) {
    switch (code) {
        case KR_OK: return "success";
        case KR_ERR_NULL_POINTER: return "a required pointer is NULL";
        case KR_ERR_ALIGNMENT: return "pointer or stride is not 16-byte (128-bit) aligned";
        case KR_ERR_NUMEL_MOD8: return "the number of elements must be 128-bit aligned (a multiple of 8 bf16)";
        case KR_ERR_BAD_DIM: return "negative, zero or inconsistent dimension";
        case KR_ERR_WORLD_SIZE: return "world size outside 1..16";
        case KR_ERR_BIAS_SHAPE: return "bias must have the shape of the input or be a vector of the last dimension";
        case KR_ERR_ROW_TOO_LONG: return "row length above 65536 is not supported by the row-resident kernels";
        case KR_ERR_BAND: return "row band outside [0, M)";
        case KR_ERR_LAYOUT: return "operand strides not supported (A must be k-contiguous; B row-major or transposed-contiguous)";
        case KR_ERR_STRIPE: return "stripe block must be a positive multiple of 8 and 0 <= rank < W";
        case KR_ERR_SCRATCH: return "the shape's split needs more scratch than the library's static device buffer (64 MiB) holds";
        default: break;
    }
    if (code > 0) return hipGetErrorString((hipError_t)code);
    return "unknown kraken_amd error code";
}
