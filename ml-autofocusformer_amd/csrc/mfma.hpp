// Helpers shared by the matrix-core gather kernels (gather_dot, gather_sum).
#pragma once

#include "common.hpp"

namespace clusten {

typedef float F32x4 __attribute__((ext_vector_type(4)));

// s_waitcnt immediate (gfx9 encoding) that waits until at most `vm` vector-memory operations are
// outstanding and leaves the LDS/scalar and export counters alone.
constexpr int waitcnt_vm(int vm) { return (vm & 15) | ((vm >> 4) << 14) | (7 << 4) | (15 << 8); }

// One LDS-direct load: every lane moves 16 bytes from its own global address `gptr` to LDS address
// `lptr` + 16 * lane (`lptr` is wave-uniform).  Completion is tracked by the vector-memory counter.
#define CLUSTEN_LDS_DMA16(gptr, lptr)                                                       \
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(gptr), \
                                     (__attribute__((address_space(3))) void*)(lptr), 16, 0, 0)

}  // namespace clusten
