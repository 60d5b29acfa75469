// gfx950 (CDNA4) building blocks shared by the bf16 attention kernels: MFMA fragment types, the
// LDS tile layout, and the row-wise / transposed LDS fragment reads.
//
// MFMA v_mfma_f32_32x32x16_bf16, wave64, lane l, r = l % 32, hh = l / 32:
//   A (32 x 16): lane holds A[r][8*hh .. 8*hh+7]          (8 bf16)
//   B (16 x 32): lane holds B[8*hh .. 8*hh+7][r]          (8 bf16)
//   C (32 x 32): lane holds C[8*(v/4) + 4*hh + v%4][r]    (v = 0..15, fp32)
// Because the C layout of one product has the shape of a B operand (a lane owns one column and
// 16 of its rows), the kernels compute transposed products (S^T = K Q^T, then O^T = V^T P^T) so
// that P never leaves registers; the only thing to arrange is that the other operand enumerates
// the contraction index in the order 16t + 8*(e/4) + 4*hh + e%4 (e = 0..7), see tr_frag().
//
// LDS tile layout ("permuted rows, padded"): a tile of R rows x D bf16 keeps logical row
// 16a + 4m + e at physical row 16a + 4e + m, with a row pitch of D*2 + 16 bytes.  The pitch is
// 4 banks (mod 64) so 16 consecutive physical rows start in 16 distinct 4-bank groups -- a
// row-wise b128 read by 16 lanes with consecutive rows is conflict free -- and the row
// permutation puts the 4 consecutive logical rows a transposed read touches 16 banks apart, so
// that one is conflict free too.  Every access is lane_base + compile-time offset: no address
// arithmetic in the loops.
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

template <int D>
struct Tile {
    static constexpr int kPitch = D * 2 + 16;  // bytes per physical row
    static constexpr int kChunks = D / 8;      // 16-byte chunks per row
    static constexpr int bytes(int rows) { return rows * kPitch; }

    // physical row of a logical row (swap the two 2-bit fields inside each group of 16)
    __device__ __forceinline__ static int prow(int row) {
        return (row & ~15) | ((row & 3) << 2) | ((row >> 2) & 3);
    }
    __device__ __forceinline__ static int off(int row, int col) { return prow(row) * kPitch + col * 2; }

    // ---- row-wise fragments (contraction index contiguous in memory) -------------------------
    // lane (r, hh) reads row row0 + r, elements 16*kk + 8*hh .. +7.  row0 must be a multiple of 32.
    __device__ __forceinline__ static int row_base(int lane) {
        return prow(lane & 31) * kPitch + (lane >> 5) * 16;
    }
    __device__ __forceinline__ static bf16x8 row_frag(lds_ptr tile, int base, int row0, int kk) {
        return *(MA_LDS bf16x8*)(tile + base + row0 * kPitch + kk * 32);
    }

    // ---- transposed fragments through ds_read_b64_tr_b16 -----------------------------------------
    // Within each group of 16 lanes, lane i supplies the address of 4 consecutive elements and
    // receives element i%4 of the rows supplied by lanes i/4, 4+i/4, 8+i/4, 12+i/4.  Lane i of a
    // group points at (row = g + i/4, col = c + 4*(i%4)) and ends up with column c + i of rows
    // g..g+3.  For an A operand (M = tile column, K = tile row) over columns c0..c0+31 and rows
    // r0..r0+15 paired with a C-layout fragment, lane (r, hh) needs column c0 + r and rows
    // r0 + 4*hh + {0..3} and r0 + 8 + 4*hh + {0..3}: two reads, 8 rows apart.
    // r0 must be a multiple of 16, c0 a multiple of 32.
    __device__ __forceinline__ static int tr_base(int lane) {
        const int i = lane & 15, hh = lane >> 5;
        const int row = 4 * hh + (i >> 2);                       // logical row within the group of 16
        const int col = (((lane >> 4) & 1) << 4) + ((i & 3) << 2);
        return prow(row) * kPitch + col * 2;
    }
    __device__ __forceinline__ static bf16x8 tr_frag(lds_ptr tile, int base, int r0, int c0) {
        // logical rows +8 inside a group of 16 are physical rows +2
        const bf16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((MA_LDS bf16x4*)(tile + base + r0 * kPitch + c0 * 2));
        const bf16x4 hi =
            __builtin_amdgcn_ds_read_tr16_b64_v4bf16((MA_LDS bf16x4*)(tile + base + (r0 + 2) * kPitch + c0 * 2));
        return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    }
};

__device__ __forceinline__ f32x16 mfma32(bf16x8 a, bf16x8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}

// Global -> registers -> LDS staging of a ROWS x D bf16 tile by NT threads.  load() issues all the
// global loads of the thread back to back (rows past the end are clamped to the last valid row so
// that the loads need no branches; their data is zeroed in store()), store() writes them to LDS.
// Splitting the two lets the loads of the next tile fly while the current one is being consumed.
template <int D, int ROWS, int NT>
struct Stager {
    static constexpr int CH = D / 8;
    static constexpr int N = ROWS * CH / NT;  // chunks per thread
    static constexpr int RPP = NT / CH;       // rows covered per pass
    static_assert((ROWS * CH) % NT == 0 && NT % CH == 0, "staging shape");
    u32x4 v[N];

    __device__ __forceinline__ void load(const __bf16* g, int64_t stride, int rows_valid, int tid) {
        const int c = tid % CH, r0 = tid / CH;
#pragma unroll
        for (int n = 0; n < N; ++n) {
            const int row = min(r0 + n * RPP, rows_valid - 1);
            v[n] = *(const u32x4*)(g + (int64_t)row * stride + c * 8);
        }
    }
    __device__ __forceinline__ void store(lds_ptr tile, int rows_valid, int tid) {
        const int c = tid % CH, r0 = tid / CH;
        if (rows_valid < ROWS) {
#pragma unroll
            for (int n = 0; n < N; ++n)
                if (r0 + n * RPP >= rows_valid) v[n] = u32x4{0, 0, 0, 0};
        }
#pragma unroll
        for (int n = 0; n < N; ++n) *(MA_LDS u32x4*)(tile + Tile<D>::off(r0 + n * RPP, c * 8)) = v[n];
    }
};

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

__device__ __forceinline__ float xor32(float x) { return __shfl_xor(x, 32, 64); }

}  // namespace ma
