// Broadcast-operand FMAs on the DPP data path.
//
// The scatter kernel multiplies a small operand that is the same for every lane (a row of upstream
// gradients) with data that differs per lane (rows of the other operand); the down-sampling kernel
// spreads every token's list over the 16-lane rows of that token the same way.  Keeping the shared operand in LDS would make the LDS the bottleneck: every
// FMA would need 4 bytes per lane from it.  Instead the shared operand is loaded so that each row
// of 16 lanes holds the same 16 values of it in one VGPR, and the FMA reads lane `L` of its own
// row through the DPP `row_newbcast:L` control.  One VALU instruction, no LDS, no scalar loads.
//
// The compiler does not fold a DPP move into an FMA for this control, so the FMAs are written as
// inline assembly.  Two hardware rules then become this file's responsibility:
//   * a VGPR written by a VALU instruction may be read through DPP only 2 wait states later —
//     every block below opens with `s_nop 1`;
//   * DPP reads lanes that EXEC disables as invalid — the kernels call these helpers only in
//     wave-uniform control flow with all 64 lanes enabled (stores are the only masked operations).
// The blocks are `volatile` so that the compiler keeps them where they are written instead of
// sinking them into a lane-masked region next to a store.
#pragma once

#include <hip/hip_runtime.h>

namespace clusten {

// acc += b0[L]*x0 + b1[L]*x1 + b2[L]*x2 + b3[L]*x3, where b[L] is lane L of the caller's row of 16.
template <int L>
__device__ __forceinline__ void fma4_rowlane(float& acc, float b0, float b1, float b2, float b3, float x0, float x1,
                                             float x2, float x3) {
    static_assert(L >= 0 && L < 16, "row lane");
    asm volatile(
        "s_nop 1\n\t"
        "v_fmac_f32_dpp %0, %1, %5 row_newbcast:%9 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f32_dpp %0, %2, %6 row_newbcast:%9 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f32_dpp %0, %3, %7 row_newbcast:%9 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f32_dpp %0, %4, %8 row_newbcast:%9 row_mask:0xf bank_mask:0xf"
        : "+v"(acc)
        : "v"(b0), "v"(b1), "v"(b2), "v"(b3), "v"(x0), "v"(x1), "v"(x2), "v"(x3), "n"(L));
}

// acc += b[L] * x
template <int L>
__device__ __forceinline__ void fma1_rowlane(float& acc, float b, float x) {
    static_assert(L >= 0 && L < 16, "row lane");
    asm volatile(
        "s_nop 1\n\t"
        "v_fmac_f32_dpp %0, %1, %2 row_newbcast:%3 row_mask:0xf bank_mask:0xf"
        : "+v"(acc)
        : "v"(b), "v"(x), "n"(L));
}

// Lane L of the caller's row of 16 lanes, in every lane of that row.
template <int L>
__device__ __forceinline__ int rowlane_bcast(int x) {
    static_assert(L >= 0 && L < 16, "row lane");
    int r;
    asm volatile(
        "s_nop 1\n\t"
        "v_mov_b32_dpp %0, %1 row_newbcast:%2 row_mask:0xf bank_mask:0xf"
        : "=v"(r)
        : "v"(x), "n"(L));
    return r;
}

// Compile-time loop: f(std::integral_constant<int, I>) for I in [0, N).
template <int I>
struct Index {
    static constexpr int value = I;
};
template <int I, int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (I < N) {
        f(Index<I>{});
        static_for<I + 1, N>(f);
    }
}

// Software pipeline over SLOTS items in groups of GS: the loads of group g+1 are issued before
// group g is consumed.  The volatile FMA blocks keep memory operations in program order, so the
// order written here is the order the hardware sees: at most 2*GS loads are in flight.
template <int SLOTS, int GS, typename LoadF, typename UseF>
__device__ __forceinline__ void slot_pipeline(LoadF&& load, UseF&& use) {
    static_assert(SLOTS % GS == 0, "whole groups");
    constexpr int NG = SLOTS / GS;
    static_for<0, GS>(load);
    static_for<0, NG>([&](auto gi) {
        constexpr int g = decltype(gi)::value;
        if constexpr (g + 1 < NG) static_for<(g + 1) * GS, (g + 2) * GS>(load);
        static_for<g * GS, (g + 1) * GS>(use);
    });
}

}  // namespace clusten
