// Helpers shared by the matrix-core gather kernels (gather_dot, gather_sum).
#pragma once

#include <type_traits>

#include "common.hpp"

namespace clusten {

typedef float F32x4 __attribute__((ext_vector_type(4)));

// CLUSTEN_REPLAY = 1 (set by replay_probe.hip alone, which compiles the forward kernels a second time under another
// namespace) turns every matrix instruction of the kernels into one integer operation on its operands: every global
// load, LDS access and store stays exactly where it is and the arithmetic goes.  What such a kernel takes is what the
// memory instruction stream of the real kernel costs on its own.
#ifndef CLUSTEN_REPLAY
#define CLUSTEN_REPLAY 0
#endif

__device__ __forceinline__ F32x4 replay_touch(uint32_t a, uint32_t b, F32x4 d) {
    d[0] = __uint_as_float(__float_as_uint(d[0]) ^ a ^ b);
    return d;
}

// D (16x16) += A (16x4) * B (4x16), fp32: `v_mfma_f32_16x16x4_f32`.
__device__ __forceinline__ F32x4 mfma_16x16x4(float a, float b, F32x4 d) {
    if constexpr (CLUSTEN_REPLAY != 0) {
        return replay_touch(__float_as_uint(a), __float_as_uint(b), d);
    } else {
        return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, d, 0, 0, 0);
    }
}

// Sixteen independent 4x4 blocks, D += A (4x1) * B (1x4), fp32: `v_mfma_f32_4x4x1_16b_f32`.
__device__ __forceinline__ F32x4 mfma_4x4x1(float a, float b, F32x4 d) {
    if constexpr (CLUSTEN_REPLAY != 0) {
        return replay_touch(__float_as_uint(a), __float_as_uint(b), d);
    } else {
        return __builtin_amdgcn_mfma_f32_4x4x1f32(a, b, d, 0, 0, 0);
    }
}

// Sixteen independent 4x4 blocks, D += A (4x4) * B (4x4) over four k steps of 16-bit operands, fp32 sums:
// `v_mfma_f32_4x4x4_16b_f16` / `_bf16`.  Lane t of a block holds row t of A (k = 0..3, two registers), column t of B
// (k = 0..3) and column t of D (rows 0..3).  Products of fp16 / bf16 values are exact in fp32.
template <typename T>
__device__ __forceinline__ F32x4 mfma_4x4x4_16b(const U32x2& a, const U32x2& b, F32x4 d) {
    static_assert(sizeof(T) == 2, "16-bit operands");
    typedef _Float16 H4 __attribute__((ext_vector_type(4)));
    typedef short S4 __attribute__((ext_vector_type(4)));
    if constexpr (CLUSTEN_REPLAY != 0) {
        return replay_touch(a[0] ^ a[1], b[0] ^ b[1], d);
    } else if constexpr (std::is_same<T, f16_t>::value) {
        return __builtin_amdgcn_mfma_f32_4x4x4f16(__builtin_bit_cast(H4, a), __builtin_bit_cast(H4, b), d, 0, 0, 0);
    } else {
        return __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(__builtin_bit_cast(S4, a), __builtin_bit_cast(S4, b), d, 0, 0, 0);
    }
}

// s_waitcnt immediate (gfx9 encoding) that waits until at most `vm` vector-memory operations are
// outstanding and leaves the LDS/scalar and export counters alone.
constexpr int waitcnt_vm(int vm) { return (vm & 15) | ((vm >> 4) << 14) | (7 << 4) | (15 << 8); }

// Orders the LDS traffic of a one-wave workgroup: every LDS access issued so far has completed, and the compiler
// moves no memory access across.  Unlike __syncthreads(), whose fence also waits for every vector-memory
// operation, it leaves LDS-direct loads, loads and stores in flight.
__device__ __forceinline__ void lds_sync() {
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
}
// The same, and at most `VM` vector-memory operations are still in flight.  They complete in the order of issue,
// so this waits for everything but the last `VM` of them (e.g. output stores issued after a prefetch).
template <int VM>
__device__ __forceinline__ void lds_sync_vm() {
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_s_waitcnt(waitcnt_vm(VM) & 0xF0FF);  // vmcnt(VM) lgkmcnt(0)
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
}

// Keeps a 32-bit byte offset a 32-bit register value at the place of use, so that the access it feeds is encoded
// as uniform base + lane offset instead of through a 64-bit address per lane held across the loops.
__device__ __forceinline__ uint32_t lane_offset(uint32_t off) {
    asm volatile("" : "+v"(off));
    return off;
}

// One LDS-direct load: every lane moves 16 bytes from its own global address `gptr` to LDS address
// `lptr` + 16 * lane (`lptr` is wave-uniform).  Completion is tracked by the vector-memory counter.
#define CLUSTEN_LDS_DMA16(gptr, lptr)                                                       \
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(gptr), \
                                     (__attribute__((address_space(3))) void*)(lptr), 16, 0, 0)
// The same for data that is read once, with the non-temporal hint when NT is set (a compile-time 0 / 1).
#define CLUSTEN_LDS_DMA16_STREAM(gptr, lptr, NT)                                            \
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(gptr), \
                                     (__attribute__((address_space(3))) void*)(lptr), 16, 0, (NT) ? 2 : 0)
template <bool NT, typename V>
__device__ __forceinline__ V load_stream(const V* p) {
    if constexpr (NT) return __builtin_nontemporal_load(p);
    else return *p;
}


// D(16x16) += A * B over the channels two lanes hold in one register group of 8 or 16 bytes each: `a` belongs to
// row lane % 16 of A, `b` to column lane % 16 of B, and lane / 16 selects which quarter of the channel range
// both cover.  fp32 data goes one channel (k = 4 per instruction) at a time; 16-bit data goes through the
// 16-bit matrix instructions with the register group as it came from memory (k = 16 or 32 per instruction):
// products of fp16 / bf16 values are exact in fp32 and the sums are fp32 either way.
template <typename T, typename Raw>
__device__ __forceinline__ F32x4 tile_mfma(const Raw& a, const Raw& b, F32x4 d) {
    if constexpr (sizeof(T) == 4) {
        constexpr int VEC = (int)sizeof(Raw) / 4;
#pragma unroll
        for (int e = 0; e < VEC; ++e) d = mfma_16x16x4(__uint_as_float(raw_word(a, e)), __uint_as_float(raw_word(b, e)), d);
        return d;
    } else if constexpr (CLUSTEN_REPLAY != 0) {
        return replay_touch(raw_word(a, 0) ^ raw_word(a, 1), raw_word(b, 0) ^ raw_word(b, 1), d);
    } else if constexpr (sizeof(Raw) == 16) {
        typedef _Float16 H8 __attribute__((ext_vector_type(8)));
        typedef __bf16 B8 __attribute__((ext_vector_type(8)));
        if constexpr (std::is_same<T, f16_t>::value) {
            return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(H8, a), __builtin_bit_cast(H8, b), d, 0, 0, 0);
        } else {
            return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(B8, a), __builtin_bit_cast(B8, b), d, 0, 0, 0);
        }
    } else {
        // 16x16x16.  Do not accumulate one of these onto the result of a 16x16x32 of the same tile (or the
        // reverse): in that chain of two different instructions the first two accumulator registers were read
        // back too early on gfx950 (wrong sums for tokens 4q, 4q+1).  Chains of one instruction are fine: pad
        // the short step to 16 bytes with zeros instead.
        static_assert(sizeof(Raw) == 8, "register groups of 8 or 16 bytes");
        typedef _Float16 H4 __attribute__((ext_vector_type(4)));
        typedef short S4 __attribute__((ext_vector_type(4)));
        if constexpr (std::is_same<T, f16_t>::value) {
            return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(H4, a), __builtin_bit_cast(H4, b), d, 0, 0, 0);
        } else {
            return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(S4, a), __builtin_bit_cast(S4, b), d, 0, 0, 0);
        }
    }
}

}  // namespace clusten
