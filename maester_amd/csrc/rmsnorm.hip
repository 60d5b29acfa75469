// Gemma's sandwich RMSNorms over the model dimension, forward and backward, with the residual add
// of the post-norms fused in.
//
// Stands in for RMSNorm.forward (maester/models/gemma/model.py:135-172: fp32 math,
// y = x * rsqrt(mean(x^2) + eps) * (1 + w), cast back to the dtype of x) as it is used by
// Gemma2DecoderLayer.forward (model.py:488-508): input_layernorm and pre_feedforward_layernorm
// feed a GEMM, post_attention_layernorm and post_feedforward_layernorm are followed by
// `residual + hidden_states`.  With a residual the kernel adds it to the rounded norm output (the
// reference rounds the norm output to the IO dtype before the add, and so does this), so one pass
// reads x and the residual and writes the sum: HBM-bound, one read and one write per element.
//
// One wave per row; a lane owns every 64th group of 8 consecutive elements, which stay in registers
// between the two uses (sum of squares, scaling).  dW of the backward is summed per workgroup in
// registers, written as one partial row per workgroup and reduced by a second kernel in a fixed
// order: no atomics, bit-identical from run to run.
#include <hip/hip_runtime.h>

#include "common.h"
#include "rowio.h"

namespace ma {

namespace {

constexpr int kNormWaves = 4;

// NCH: groups of 8 elements per lane (dim <= 512 * NCH)
template <typename T, int NCH>
__global__ __launch_bounds__(64 * kNormWaves) void rmsnorm_fwd_kernel(const T* __restrict__ x, const T* __restrict__ residual,
                                                                      const float* __restrict__ weight, T* __restrict__ out,
                                                                      float* __restrict__ rstd, int64_t rows, int dim, float eps,
                                                                      int unit) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * kNormWaves + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int groups = dim / 8;
    const T* xr = x + row * dim;
    float v[NCH][8];
    float ss = 0.f;
#pragma unroll
    for (int c = 0; c < NCH; ++c) {
        const int g = lane + 64 * c;
        if (g < groups) {
            ld8<T>(xr + g * 8, v[c]);
#pragma unroll
            for (int i = 0; i < 8; ++i) ss += v[c][i] * v[c][i];
        }
    }
    const float r = rsqrtf(wave_sum(ss) / (float)dim + eps);
    if (rstd && lane == 0) rstd[row] = r;
#pragma unroll
    for (int c = 0; c < NCH; ++c) {
        const int g = lane + 64 * c;
        if (g < groups) {
            float w[8], y[8];
            ld8<float>(weight + g * 8, w);
#pragma unroll
            for (int i = 0; i < 8; ++i) y[i] = v[c][i] * r * (unit ? 1.0f + w[i] : w[i]);
            if (residual) {
                float res[8];
                ld8<T>(residual + row * dim + g * 8, res);
#pragma unroll
                for (int i = 0; i < 8; ++i) y[i] = res[i] + through<T>(y[i]);
            }
            st8<T>(out + row * dim + g * 8, y);
        }
    }
}

// dx = r * (g*(1+w) - xhat * mean(g*(1+w) * xhat)), xhat = x * r.  A workgroup takes up to four rows at
// a time; a thread owns the same (up to NG) groups of 8 columns in every row, so its dW sums stay in
// registers for the whole launch and the only exchange is the row means (one LDS round per batch of
// rows).  Few registers per thread: many waves per SIMD to cover the HBM latency.
constexpr int kNormRowsMax = 4;
constexpr int norm_rows(int ng) { return kNormRowsMax / ng; }  // rows per batch: 16 registers per row and group
template <typename T, int NG>
__global__ __launch_bounds__(256) void rmsnorm_bwd_kernel(const T* __restrict__ x, const float* __restrict__ weight,
                                                          const float* __restrict__ rstd, const T* __restrict__ dout,
                                                          T* __restrict__ dx, float* __restrict__ dw_partial, int64_t rows, int dim,
                                                          int unit) {
    constexpr int kNormRows = norm_rows(NG);
    __shared__ float s_red[2][4][kNormRows];
    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
    const int groups = dim / 8;
    float wv[NG][8], acc[NG][8];
#pragma unroll
    for (int c = 0; c < NG; ++c) {
        const int g = tid + 256 * c;
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[c][i] = wv[c][i] = 0.f;
        if (g < groups) {
            ld8<float>(weight + g * 8, wv[c]);
#pragma unroll
            for (int i = 0; i < 8; ++i) wv[c][i] = unit ? 1.0f + wv[c][i] : wv[c][i];
        }
    }
    int flip = 0;
    for (int64_t row0 = (int64_t)blockIdx.x * kNormRows; row0 < rows; row0 += (int64_t)gridDim.x * kNormRows, flip ^= 1) {
        float xh[kNormRows][NG][8], gv[kNormRows][NG][8], rr[kNormRows], dot[kNormRows];
#pragma unroll
        for (int k = 0; k < kNormRows; ++k) {
            const int64_t row = row0 + k < rows ? row0 + k : rows - 1;  // rows past the end repeat the last one (not stored)
            rr[k] = rstd[row];
            dot[k] = 0.f;
#pragma unroll
            for (int c = 0; c < NG; ++c) {
                const int g = tid + 256 * c;
                if (g < groups) {
                    ld8<T>(x + row * dim + g * 8, xh[k][c]);
                    ld8<T>(dout + row * dim + g * 8, gv[k][c]);
                }
            }
        }
#pragma unroll
        for (int k = 0; k < kNormRows; ++k) {
#pragma unroll
            for (int c = 0; c < NG; ++c) {
                if (tid + 256 * c < groups) {
#pragma unroll
                    for (int i = 0; i < 8; ++i) {
                        xh[k][c][i] *= rr[k];
                        dot[k] += gv[k][c][i] * wv[c][i] * xh[k][c][i];
                    }
                }
            }
            dot[k] = wave_sum(dot[k]);
            if (lane == 0) s_red[flip][w][k] = dot[k];
        }
        __syncthreads();  // (two sets of slots: the next batch writes the other one, so one barrier per batch is enough)
#pragma unroll
        for (int k = 0; k < kNormRows; ++k) {
            const float m = ((s_red[flip][0][k] + s_red[flip][1][k]) + (s_red[flip][2][k] + s_red[flip][3][k])) / (float)dim;
            const bool live = row0 + k < rows;
#pragma unroll
            for (int c = 0; c < NG; ++c) {
                const int g = tid + 256 * c;
                if (g < groups && live) {
                    float o[8];
#pragma unroll
                    for (int i = 0; i < 8; ++i) {
                        o[i] = rr[k] * (gv[k][c][i] * wv[c][i] - xh[k][c][i] * m);
                        acc[c][i] += gv[k][c][i] * xh[k][c][i];
                    }
                    st8<T>(dx + (row0 + k) * dim + g * 8, o);
                }
            }
        }
    }
#pragma unroll
    for (int c = 0; c < NG; ++c) {
        const int g = tid + 256 * c;
        if (g < groups) st8<float>(dw_partial + (size_t)blockIdx.x * dim + g * 8, acc[c]);
    }
}

// dw[e] = sum over the partial rows, in a fixed order: a workgroup takes 32 columns, its 8 groups of 32
// threads each sum every 8th partial row (loads of many rows in flight), then the 8 sums are added in order.
__global__ __launch_bounds__(256) void rmsnorm_dw_reduce_kernel(const float* __restrict__ partial, int n_partial, int dim,
                                                                float* __restrict__ dw) {
    __shared__ float s_part[8][32];
    const int col = blockIdx.x * 32 + (threadIdx.x & 31), slice = threadIdx.x >> 5;
    float s = 0.f;
    if (col < dim) {
        float t[4] = {0.f, 0.f, 0.f, 0.f};
        int k = slice;
        for (; k + 24 < n_partial; k += 32) {
#pragma unroll
            for (int u = 0; u < 4; ++u) t[u] += partial[(size_t)(k + 8 * u) * dim + col];
        }
        for (; k < n_partial; k += 8) t[0] += partial[(size_t)k * dim + col];
        s = (t[0] + t[1]) + (t[2] + t[3]);
    }
    s_part[slice][threadIdx.x & 31] = s;
    __syncthreads();
    if (slice == 0 && col < dim) {
        float r = 0.f;
#pragma unroll
        for (int j = 0; j < 8; ++j) r += s_part[j][threadIdx.x];
        dw[col] = r;
    }
}

template <typename T, int NCH>
int fwd_launch(const void* x, const void* residual, const float* weight, void* out, float* rstd, int64_t rows, int dim, float eps,
               int unit, hipStream_t st) {
    hipLaunchKernelGGL((rmsnorm_fwd_kernel<T, NCH>), dim3((unsigned)((rows + kNormWaves - 1) / kNormWaves)), dim3(64 * kNormWaves), 0,
                       st, (const T*)x, (const T*)residual, weight, (T*)out, rstd, rows, dim, eps, unit);
    return check_launch("rmsnorm_fwd_kernel");
}
template <typename T, int NG>
int bwd_launch(const void* x, const float* weight, const float* rstd, const void* dout, void* dx, float* dw, float* partial,
               int n_blocks, int64_t rows, int dim, int unit, hipStream_t st) {
    hipLaunchKernelGGL((rmsnorm_bwd_kernel<T, NG>), dim3(n_blocks), dim3(256), 0, st, (const T*)x, weight, rstd, (const T*)dout,
                       (T*)dx, partial, rows, dim, unit);
    int rc = check_launch("rmsnorm_bwd_kernel");
    if (rc) return rc;
    hipLaunchKernelGGL(rmsnorm_dw_reduce_kernel, dim3((dim + 31) / 32), dim3(256), 0, st, partial, n_blocks, dim, dw);
    return check_launch("rmsnorm_dw_reduce_kernel");
}

}  // namespace

int rmsnorm_bwd_blocks(int64_t rows) {
    const int64_t want = rows;
    const int64_t cap = (int64_t)compute_units() * 4;
    return (int)(want < cap ? want : cap);
}

int launch_rmsnorm_fwd(const void* x, const void* residual, const float* weight, void* out, float* rstd, int64_t rows, int dim,
                       float eps, int unit, int dtype, hipStream_t st) {
    const bool bf = dtype == MA_DTYPE_BF16;
    if (dim <= 2048) return bf ? fwd_launch<uint16_t, 4>(x, residual, weight, out, rstd, rows, dim, eps, unit, st)
                               : fwd_launch<float, 4>(x, residual, weight, out, rstd, rows, dim, eps, unit, st);
    if (dim <= 4096) return bf ? fwd_launch<uint16_t, 8>(x, residual, weight, out, rstd, rows, dim, eps, unit, st)
                               : fwd_launch<float, 8>(x, residual, weight, out, rstd, rows, dim, eps, unit, st);
    return bf ? fwd_launch<uint16_t, 16>(x, residual, weight, out, rstd, rows, dim, eps, unit, st)
              : fwd_launch<float, 16>(x, residual, weight, out, rstd, rows, dim, eps, unit, st);
}

int launch_rmsnorm_bwd(const void* x, const float* weight, const float* rstd, const void* dout, void* dx, float* dw, void* ws,
                       int64_t rows, int dim, int unit, int dtype, hipStream_t st) {
    const bool bf = dtype == MA_DTYPE_BF16;
    const int nb = rmsnorm_bwd_blocks(rows);
    float* partial = (float*)ws;
    if (dim <= 2048) return bf ? bwd_launch<uint16_t, 1>(x, weight, rstd, dout, dx, dw, partial, nb, rows, dim, unit, st)
                               : bwd_launch<float, 1>(x, weight, rstd, dout, dx, dw, partial, nb, rows, dim, unit, st);
    if (dim <= 4096) return bf ? bwd_launch<uint16_t, 2>(x, weight, rstd, dout, dx, dw, partial, nb, rows, dim, unit, st)
                               : bwd_launch<float, 2>(x, weight, rstd, dout, dx, dw, partial, nb, rows, dim, unit, st);
    return bf ? bwd_launch<uint16_t, 4>(x, weight, rstd, dout, dx, dw, partial, nb, rows, dim, unit, st)
              : bwd_launch<float, 4>(x, weight, rstd, dout, dx, dw, partial, nb, rows, dim, unit, st);
}

}  // namespace ma
