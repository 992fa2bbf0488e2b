// Reductions over lanes of a wavefront without LDS, for the gfx950 kernels.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>

namespace saetta {

// Steps inside a 16-lane row are DPP moves (quad permutes, then the two mirrors: once the quads
// agree, mirroring the half row and the row brings in the other quads).  Rows are joined by
// v_permlane16_swap / v_permlane32_swap, which exchange 16- and 32-lane rows of two registers;
// they may not read a register a vector instruction wrote in the two cycles before.
template <int CTRL>
__device__ __forceinline__ float dpp(float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xf, 0xf, false));
}
__device__ __forceinline__ void swap_rows16(uint32_t &u, uint32_t &v) {
    asm volatile("s_nop 1\nv_permlane16_swap_b32 %0, %1\n" : "+v"(u), "+v"(v));
}
__device__ __forceinline__ void swap_rows32(uint32_t &u, uint32_t &v) {
    asm volatile("s_nop 1\nv_permlane32_swap_b32 %0, %1\n" : "+v"(u), "+v"(v));
}
struct MaxOp {
    __device__ __forceinline__ float operator()(float a, float b) const { return fmaxf(a, b); }
};
struct SumOp {
    __device__ __forceinline__ float operator()(float a, float b) const { return a + b; }
};
// x combined over the lanes l ^ 16 (FROM <= 16 < WIDTH) and l ^ 32 (FROM <= 32 < WIDTH)
template <int FROM, int WIDTH, typename Op>
__device__ __forceinline__ float across_rows(float x, Op op) {
    if constexpr (FROM <= 16 && WIDTH > 16) {
        uint32_t u = __builtin_bit_cast(uint32_t, x), v = u;
        swap_rows16(u, v);  // u = rows (0, 0, 2, 2), v = rows (1, 1, 3, 3)
        x = op(__builtin_bit_cast(float, u), __builtin_bit_cast(float, v));
    }
    if constexpr (FROM <= 32 && WIDTH > 32) {
        uint32_t u = __builtin_bit_cast(uint32_t, x), v = u;
        swap_rows32(u, v);  // u = (lower half, lower half), v = (upper, upper)
        x = op(__builtin_bit_cast(float, u), __builtin_bit_cast(float, v));
    }
    return x;
}
// x combined over aligned groups of WIDTH lanes (1, 2, 4, ... 64); every lane gets the result
template <int WIDTH, typename Op>
__device__ __forceinline__ float group_reduce(float x, Op op) {
    if constexpr (WIDTH > 1) x = op(x, dpp<0xb1>(x));   // quad_perm [1, 0, 3, 2]
    if constexpr (WIDTH > 2) x = op(x, dpp<0x4e>(x));   // quad_perm [2, 3, 0, 1]
    if constexpr (WIDTH > 4) x = op(x, dpp<0x141>(x));  // row_half_mirror
    if constexpr (WIDTH > 8) x = op(x, dpp<0x140>(x));  // row_mirror
    return across_rows<16, WIDTH>(x, op);
}

}  // namespace saetta
