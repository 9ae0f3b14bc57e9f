// Shared device/host helpers for the CLUSTEN gfx950 kernels.
//
// Conventions used by every kernel in this directory:
//   * one workgroup = one 64-lane wavefront, so __syncthreads() orders LDS traffic inside the wave
//     without an s_barrier between waves, and every value derived from blockIdx is wave-uniform;
//   * the flat workgroup id is remapped so that the workgroups the hardware deals round-robin to
//     one XCD (id % 8) cover one contiguous range of tiles: the rows a batch element gathers then
//     stay in that XCD's private L2;
//   * arithmetic is carried out in fp32 (fp64 for double) whatever the storage type.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/clusten_hip.h"

namespace clusten {

constexpr int kWave = 64;       // lanes per wavefront on CDNA
constexpr int kXcds = 8;        // accelerator dies of an MI355X, each with its own L2
constexpr int kTileTokens = 8;  // consecutive tokens handled by one wave (the model's cluster size)

// ---- storage types -----------------------------------------------------------------------------

struct bf16_t {
    uint16_t bits;
};
typedef _Float16 f16_t;

template <typename T>
struct Acc {
    typedef float type;
};
template <>
struct Acc<double> {
    typedef double type;
};

__device__ __forceinline__ float to_acc(float x) { return x; }
__device__ __forceinline__ double to_acc(double x) { return x; }
__device__ __forceinline__ float to_acc(f16_t x) { return (float)x; }
__device__ __forceinline__ float to_acc(bf16_t x) { return __uint_as_float(((uint32_t)x.bits) << 16); }

template <typename T>
__device__ __forceinline__ T from_acc(typename Acc<T>::type x);
template <>
__device__ __forceinline__ float from_acc<float>(float x) {
    return x;
}
template <>
__device__ __forceinline__ double from_acc<double>(double x) {
    return x;
}
template <>
__device__ __forceinline__ f16_t from_acc<f16_t>(float x) {
    return (f16_t)x;  // round to nearest even
}
template <>
__device__ __forceinline__ bf16_t from_acc<bf16_t>(float x) {
    // round to nearest even on the upper 16 bits; NaN stays NaN
    uint32_t u = __float_as_uint(x);
    bf16_t r;
    if ((u & 0x7fffffffu) > 0x7f800000u) {
        r.bits = (uint16_t)((u >> 16) | 0x0040u);
    } else {
        u += 0x7fffu + ((u >> 16) & 1u);
        r.bits = (uint16_t)(u >> 16);
    }
    return r;
}

// ---- 16-byte pieces ----------------------------------------------------------------------------

// A 16-byte piece of a row: what one lane moves with a single dwordx4 access.
typedef uint32_t Piece __attribute__((ext_vector_type(4)));

template <typename T>
struct PieceOf {
    static constexpr int kElems = 16 / (int)sizeof(T);
};

// Unpack the e-th element of a piece to the accumulation type.
template <typename T>
__device__ __forceinline__ typename Acc<T>::type piece_get(const Piece& p, int e);
template <>
__device__ __forceinline__ float piece_get<float>(const Piece& p, int e) {
    return __uint_as_float(p[e]);
}
template <>
__device__ __forceinline__ float piece_get<f16_t>(const Piece& p, int e) {
    uint32_t w = p[e >> 1];
    uint16_t h = (e & 1) ? (uint16_t)(w >> 16) : (uint16_t)(w & 0xffffu);
    f16_t v;
    __builtin_memcpy(&v, &h, 2);
    return (float)v;
}
template <>
__device__ __forceinline__ float piece_get<bf16_t>(const Piece& p, int e) {
    uint32_t w = p[e >> 1];
    return __uint_as_float((e & 1) ? (w & 0xffff0000u) : (w << 16));
}

// ---- short vectors of row elements -------------------------------------------------------------

typedef uint32_t U32x2 __attribute__((ext_vector_type(2)));

// The register type that moves BYTES contiguous bytes with one access.
template <int BYTES>
struct RawBytes;
template <>
struct RawBytes<2> {
    typedef uint16_t type;
};
template <>
struct RawBytes<4> {
    typedef uint32_t type;
};
template <>
struct RawBytes<8> {
    typedef U32x2 type;
};
template <>
struct RawBytes<16> {
    typedef Piece type;
};

__device__ __forceinline__ uint32_t raw_word(uint16_t r, int) { return r; }
__device__ __forceinline__ uint32_t raw_word(uint32_t r, int) { return r; }
__device__ __forceinline__ uint32_t raw_word(const U32x2& r, int k) { return r[k]; }
__device__ __forceinline__ uint32_t raw_word(const Piece& r, int k) { return r[k]; }
__device__ __forceinline__ void set_raw_word(uint16_t& r, int, uint32_t w) { r = (uint16_t)w; }
__device__ __forceinline__ void set_raw_word(uint32_t& r, int, uint32_t w) { r = w; }
__device__ __forceinline__ void set_raw_word(U32x2& r, int k, uint32_t w) { r[k] = w; }
__device__ __forceinline__ void set_raw_word(Piece& r, int k, uint32_t w) { r[k] = w; }

__device__ __forceinline__ uint32_t storage_bits(float x) { return __float_as_uint(x); }
__device__ __forceinline__ uint32_t storage_bits(f16_t x) {
    uint16_t h;
    __builtin_memcpy(&h, &x, 2);
    return h;
}
__device__ __forceinline__ uint32_t storage_bits(bf16_t x) { return x.bits; }

// VEC consecutive elements of storage type T (float, f16_t, bf16_t) as one register group,
// unpacked to / packed from fp32.
template <typename T, int VEC>
struct VecIO {
    static constexpr int kPerWord = 4 / (int)sizeof(T);  // elements per 32-bit word
    typedef typename RawBytes<(int)sizeof(T) * VEC>::type raw;

    static __device__ __forceinline__ void unpack(const raw& r, float (&x)[VEC]) {
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            const uint32_t w = raw_word(r, e / kPerWord);
            if constexpr (sizeof(T) == 4) {
                x[e] = __uint_as_float(w);
            } else {
                const uint16_t h = (e % kPerWord) ? (uint16_t)(w >> 16) : (uint16_t)(w & 0xffffu);
                T v;
                __builtin_memcpy(&v, &h, 2);
                x[e] = to_acc(v);
            }
        }
    }

    static __device__ __forceinline__ raw pack(const float (&x)[VEC]) {
        raw r = raw(0);
        constexpr int kWords = (VEC + kPerWord - 1) / kPerWord;
#pragma unroll
        for (int k = 0; k < kWords; ++k) {
            uint32_t w = storage_bits(from_acc<T>(x[k * kPerWord]));
            if constexpr (kPerWord == 2 && VEC > 1) w |= storage_bits(from_acc<T>(x[k * kPerWord + 1])) << 16;
            set_raw_word(r, k, w);
        }
        return r;
    }
};

// Four consecutive elements: the unit in which the lane-shared operands are loaded.
template <typename T>
using Quad = VecIO<T, 4>;

// ---- stores ---------------------------------------------------------------------------------------

// Store of output data that this kernel never reads again, with the non-temporal hint: the L2 streams the
// line to memory instead of keeping it, so that the outputs (a quarter to a third of a kernel's traffic) do
// not push the gathered rows, which are re-read many times, out of the cache.
template <typename V>
__device__ __forceinline__ void store_streaming(V* p, V v) {
    __builtin_nontemporal_store(v, p);
}

// ---- workgroup id -> tile ----------------------------------------------------------------------

// One short-lived one-wave workgroup per tile: on this device many small workgroups stream from HBM
// faster than few persistent ones (a plain copy loses 15-20 % of its bandwidth as a grid-stride loop).
//
// Workgroup `wg` of the grid runs on XCD wg % 8.  XCD x is given the contiguous tile range
// [x*per, (x+1)*per), so the waves that run at the same time on one XCD work on neighbouring tiles
// and the rows they gather are in that XCD's private L2.  Returns the tile index, or -1 for the
// padding workgroups of the last XCDs.
__device__ __forceinline__ int xcd_tile(int wg, int total) {
    const int per = (total + kXcds - 1) / kXcds;
    const int tile = (wg % kXcds) * per + wg / kXcds;
    return (wg / kXcds < per && tile < total) ? tile : -1;
}

// Grid size that xcd_tile() needs to cover `total` tiles.
inline int xcd_grid(int total) { return ((total + kXcds - 1) / kXcds) * kXcds; }

// Head groups per tile for the kernels in which one wave walks the heads of a tile: with few tiles and many
// heads (the late stages of a model) the device is short of waves, and the heads of a tile are dealt to two
// workgroups.  Measured at B = 128, fp32: 196 tokens x 8 heads 32 -> 27.6 us (QK), 33.4 -> 29.8 us (AV); 49 tokens x
// 16 heads 20.1 -> 16.1 us, 24.6 -> 17.4 us; four or eight groups are no faster, and at 784 tokens x 4 heads (12 544
// tiles) two groups cost AV 3 %.
inline int head_groups_for(int total_tiles, int H) { return (total_tiles < 8192 && H >= 4) ? 2 : 1; }

// ---- host-side argument checks ------------------------------------------------------------------

inline bool dtype_ok(int dtype) { return dtype >= CLUSTEN_F32 && dtype <= CLUSTEN_F64; }

inline size_t dtype_size(int dtype) {
    switch (dtype) {
        case CLUSTEN_F32: return 4;
        case CLUSTEN_F16: return 2;
        case CLUSTEN_BF16: return 2;
        default: return 8;
    }
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Strides of a (B,H,N,C) operand must be non-negative and the rows must not overlap.
inline bool strides_ok(const clusten_strides& s, int C) {
    return s.b >= 0 && s.h >= 0 && s.n >= C;
}

// True when every row of a strided (B,H,N,C) operand starts on a 16-byte boundary.
inline bool rows_aligned16(const void* p, const clusten_strides& s, size_t elem) {
    return aligned16(p) && (s.b * elem) % 16 == 0 && (s.h * elem) % 16 == 0 && (s.n * elem) % 16 == 0;
}

// True when every byte offset inside one batch element of a strided (B,H,N,C) operand with 8-byte
// elements at most fits an int, so that kernels may use 32-bit offsets from a per-batch base.
inline bool slice_fits_int32(const clusten_strides& s, int H, int N, int C) {
    return ((int64_t)(H - 1) * s.h + (int64_t)(N - 1) * s.n + C) * 8 < ((int64_t)1 << 31);
}

inline int check_attn_shape(const clusten_attn_shape& s) {
    if (s.B <= 0 || s.H <= 0 || s.N <= 0 || s.C <= 0 || s.M <= 0) return CLUSTEN_ERR_BAD_DIMS;
    // 32-bit indexing inside one batch element
    if ((int64_t)s.H * s.N * s.M >= (int64_t)1 << 31) return CLUSTEN_ERR_BAD_DIMS;
    if ((int64_t)s.H * s.N * s.C >= (int64_t)1 << 31) return CLUSTEN_ERR_BAD_DIMS;
    // workgroup counts stay below 2^31
    if ((int64_t)s.B * s.H * s.N >= ((int64_t)1 << 31) - 64) return CLUSTEN_ERR_BAD_DIMS;
    return CLUSTEN_OK;
}

inline int check_wf_shape(const clusten_wf_shape& s) {
    if (s.B <= 0 || s.N <= 0 || s.Nout <= 0 || s.C <= 0 || s.M <= 0 || s.IC <= 0) return CLUSTEN_ERR_BAD_DIMS;
    if ((int64_t)s.Nout * s.M * s.IC >= (int64_t)1 << 31) return CLUSTEN_ERR_BAD_DIMS;
    if ((int64_t)s.Nout * s.IC * s.C >= (int64_t)1 << 31) return CLUSTEN_ERR_BAD_DIMS;
    if ((int64_t)s.N * s.C >= (int64_t)1 << 31) return CLUSTEN_ERR_BAD_DIMS;
    if ((int64_t)s.B * s.Nout >= (int64_t)1 << 31) return CLUSTEN_ERR_BAD_DIMS;
    return CLUSTEN_OK;
}

inline int launch_status() { return hipGetLastError() == hipSuccess ? CLUSTEN_OK : CLUSTEN_ERR_LAUNCH; }

// Dispatch a generic lambda on the storage type named by a dtype code.
template <typename F>
inline int dispatch_dtype(int dtype, F&& f) {
    switch (dtype) {
        case CLUSTEN_F32: return f(float());
        case CLUSTEN_F16: return f(f16_t());
        case CLUSTEN_BF16: return f(bf16_t());
        case CLUSTEN_F64: return f(double());
        default: return CLUSTEN_ERR_BAD_DTYPE;
    }
}

}  // namespace clusten
