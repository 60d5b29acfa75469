// gfx950 (CDNA4) building blocks shared by the bf16 attention kernels: MFMA fragment types, the
// swizzled LDS tile layout, and the row-wise / transposed LDS fragment reads.
//
// MFMA v_mfma_f32_32x32x16_bf16, wave64, lane l, r = l % 32, hh = l / 32:
//   A (32 x 16): lane holds A[r][8*hh .. 8*hh+7]          (8 bf16)
//   B (16 x 32): lane holds B[8*hh .. 8*hh+7][r]          (8 bf16)
//   C (32 x 32): lane holds C[8*(v/4) + 4*hh + v%4][r]    (v = 0..15, fp32)
// Because the C layout of one product has the shape of a B operand (a lane owns one column and
// 16 of its rows), the kernels compute transposed products (S^T = K Q^T, then O^T = V^T P^T) so
// that P never leaves registers; the only thing to arrange is that the other operand enumerates
// the contraction index in the order 16t + 8*(e/4) + 4*hh + e%4 (e = 0..7), see tr_frag().
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ma {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

#define MA_LDS __attribute__((address_space(3)))
typedef MA_LDS char* lds_ptr;

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

// Byte offset of 16-byte chunk `chunk` of row `row` in a [rows][D] bf16 tile.  Chunks are XOR-ed
// with a function of the row chosen so that (a) 16 consecutive rows at one chunk index and (b) 4
// consecutive rows x 4 consecutive chunks both spread over all 64 LDS banks.
template <int D>
__device__ __forceinline__ int swz(int row, int chunk) {
    constexpr int CH = D / 8;
    constexpr int M = CH >= 16 ? 15 : CH - 1;
    const int f = (((row & 3) << 2) | ((row >> 2) & 3)) & M;
    return row * (D * 2) + ((chunk ^ f) << 4);
}

// Row-wise fragment: 8 consecutive elements of one row (A or B operand whose contraction index
// is the contiguous one).
template <int D>
__device__ __forceinline__ bf16x8 row_frag(lds_ptr tile, int row, int chunk) {
    return *(MA_LDS bf16x8*)(tile + swz<D>(row, chunk));
}

// Transposed fragment through ds_read_b64_tr_b16.  Within each group of 16 lanes, lane i supplies
// the address of 4 consecutive elements and receives element i%4 of the rows supplied by lanes
// i/4, 4+i/4, 8+i/4, 12+i/4.  With lane i pointing at (row = row0 + i/4, col = col0 + 4*(i%4))
// lane i ends up with column col0 + i of rows row0 .. row0+3.
template <int D>
__device__ __forceinline__ bf16x4 tr_read4(lds_ptr tile, int row0, int col0, int lane) {
    const int i = lane & 15;
    const int row = row0 + (i >> 2);
    const int col = col0 + ((i & 3) << 2);
    const int off = swz<D>(row, col >> 3) + ((col & 7) << 1);
    return __builtin_amdgcn_ds_read_tr16_b64_v4bf16((MA_LDS bf16x4*)(tile + off));
}

// A operand (M = tile column, K = tile row) for one 32-column x 16-row block whose partner is a
// C-layout fragment: lane (r, hh) gets column c0 + r and rows r0 + 4*hh + {0..3}, r0 + 8 + 4*hh + {0..3}.
template <int D>
__device__ __forceinline__ bf16x8 tr_frag(lds_ptr tile, int r0, int c0, int lane) {
    const int hh = lane >> 5;
    const int cb = c0 + (((lane >> 4) & 1) << 4);
    const bf16x4 lo = tr_read4<D>(tile, r0 + 4 * hh, cb, lane);
    const bf16x4 hi = tr_read4<D>(tile, r0 + 8 + 4 * hh, cb, lane);
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
}

__device__ __forceinline__ f32x16 mfma32(bf16x8 a, bf16x8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}

// Copy ROWS rows of D bf16 from global (row stride in elements) into a swizzled LDS tile; rows at
// or beyond `rows_valid` are zero-filled.  All NT threads of the block take part.
template <int D, int ROWS, int NT>
__device__ __forceinline__ void stage_tile(lds_ptr tile, const __bf16* g, int64_t stride, int rows_valid, int tid) {
    constexpr int CH = D / 8;
    constexpr int N = ROWS * CH;
    static_assert(N % NT == 0, "tile chunks must divide evenly over the block");
#pragma unroll
    for (int n = 0; n < N / NT; ++n) {
        const int id = tid + n * NT;
        const int row = id / CH, c = id % CH;
        u32x4 val = {0, 0, 0, 0};
        if (row < rows_valid) val = *(const u32x4*)(g + (int64_t)row * stride + c * 8);
        *(MA_LDS u32x4*)(tile + swz<D>(row, c)) = val;
    }
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

__device__ __forceinline__ float xor32(float x) { return __shfl_xor(x, 32, 64); }

}  // namespace ma
