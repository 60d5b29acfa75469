// Softmax cross entropy over rows of logits, loss and gradient in one launch, for the fused
// linear + cross-entropy loss that ends the model's forward.
//
// Stands in for the elementwise half of `linear_cross_entropy(hidden, embedder_weight, labels)`
// (maester/models/gemma/model.py:762-769; the loss is cut-cross-entropy 25.9.3's, pinned in the
// reference's uv.lock) and of `F.cross_entropy(pred.float(), labels)` (train.py:258-259): per row
//   lse = log sum_j exp(x_j),  nll = lse - x_label,  dx_j = (exp(x_j - lse) - [j == label]) * scale,
// rows whose label is `ignore_index` contribute neither loss nor gradient.  With a soft cap the
// logits are first replaced by cap * tanh(x / cap) and the gradient carries its derivative.  The host
// side forms the logits a block of rows at a time with a library GEMM (the full [tokens, vocab]
// matrix never exists), hands the block to this kernel, which leaves the gradient in its place, and
// feeds that to the two gradient GEMMs.
//
// One workgroup per row.  A Gemma row is 262 208 logits, half a megabyte: the row is read twice
// (running maximum and sum, then the gradient) and written once, three passes at the HBM rate.  All
// arithmetic is fp32 in the exp2 domain; the reduction order is fixed, so results are identical from
// run to run.
#include <hip/hip_runtime.h>

#include "common.h"
#include "rowio.h"

namespace ma {

namespace {

constexpr int kCeThreads = 512;
constexpr int kCeWaves = kCeThreads / 64;
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

__device__ __forceinline__ float wave_max(float x) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) x = fmaxf(x, __shfl_xor(x, off, 64));
    return x;
}

template <typename T>
__device__ __forceinline__ float ld1(const T* p);
template <>
__device__ __forceinline__ float ld1<float>(const float* p) { return *p; }
template <>
__device__ __forceinline__ float ld1<uint16_t>(const uint16_t* p) { return __uint_as_float((uint32_t)*p << 16); }
template <typename T>
__device__ __forceinline__ void st1(T* p, float v);
template <>
__device__ __forceinline__ void st1<float>(float* p, float v) { *p = v; }
template <>
__device__ __forceinline__ void st1<uint16_t>(uint16_t* p, float v) {
    const __bf16 b = (__bf16)v;
    *p = *(const uint16_t*)&b;
}

// ---- arithmetic on 8 logits ------------------------------------------------------------------------
// Everything is kept in log2 units so that an exponential is one fused multiply-add and one exp2:
// exp(x - lse) * scale = exp2(x * log2e - (lse2 - log2 scale)).
template <bool CAP>
__device__ __forceinline__ void soft_cap8(float* v, float* dcap, float cap, float inv_cap) {
    if (CAP) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const float t = tanhf(v[i] * inv_cap);
            v[i] = cap * t;
            dcap[i] = 1.f - t * t;
        }
    }
}

// running maximum m (log2 units) and sum l of exp2(y - m)
template <bool CAP>
__device__ __forceinline__ void fold8(float* v, float cap, float inv_cap, float& m, float& l) {
    float dcap[8];
    soft_cap8<CAP>(v, dcap, cap, inv_cap);
    float vm = fmaxf(fmaxf(v[0], v[1]), fmaxf(v[2], v[3]));
    vm = fmaxf(vm, fmaxf(fmaxf(v[4], v[5]), fmaxf(v[6], v[7])));
    const float mn = fmaxf(m, vm * kLog2e);
    float add = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) add += exp2f(fmaf(v[i], kLog2e, -mn));
    l = l * exp2f(m - mn) + add;
    m = mn;
}
__device__ __forceinline__ void fold1(float y, float& m, float& l) {
    const float mn = fmaxf(m, y);
    l = l * exp2f(m - mn) + exp2f(y - mn);
    m = mn;
}

// v <- (softmax - onehot) * scale; shift = lse2 - log2(scale); label_elem < 0: the label is elsewhere
template <bool CAP>
__device__ __forceinline__ void grad8(float* v, float cap, float inv_cap, float shift, float scale, int label_elem) {
    float dcap[8];
    soft_cap8<CAP>(v, dcap, cap, inv_cap);
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = exp2f(fmaf(v[i], kLog2e, -shift));
    if (label_elem >= 0) {
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] -= i == label_elem ? scale : 0.f;
    }
    if (CAP) {
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] *= dcap[i];
    }
}

template <bool CAP>
__device__ __forceinline__ float capped(float x, float cap, float inv_cap) {
    return CAP ? cap * tanhf(x * inv_cap) : x;
}

// combines the (m, l) of the threads of a workgroup; s_m / s_l: one slot per wave
template <int WAVES>
__device__ __forceinline__ float workgroup_lse2(float m, float l, float* s_m, float* s_l) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    // a thread without elements holds (-inf, 0); in a wave of such threads m - mw would be inf - inf
    const float mw = wave_max(m);
    float lw = m == -INFINITY ? 0.f : l * exp2f(m - mw);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) lw += __shfl_xor(lw, off, 64);
    if (lane == 0) {
        s_m[wave] = mw;
        s_l[wave] = lw;
    }
    __syncthreads();
    float big = s_m[0];
#pragma unroll
    for (int w = 1; w < WAVES; ++w) big = fmaxf(big, s_m[w]);
    float sum = 0.f;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) sum += s_l[w] * exp2f(s_m[w] - big);
    return big + log2f(sum);
}

// ---- rows read twice ---------------------------------------------------------------------------------
// VEC: the row pitch and the vocabulary allow 8-element accesses
template <typename T, bool CAP, bool VEC>
__global__ __launch_bounds__(kCeThreads) void ce_rows_kernel(T* __restrict__ logits, int64_t pitch,
                                                             const int64_t* __restrict__ targets, int vocab,
                                                             int64_t ignore_index, float cap,
                                                             const float* __restrict__ grad_scale, float* __restrict__ lse_out,
                                                             float* __restrict__ nll_out, int write_grad) {
    __shared__ float s_m[kCeWaves], s_l[kCeWaves];
    const int tid = threadIdx.x;
    const int64_t row = blockIdx.x;
    T* xr = logits + row * pitch;
    const int64_t label = targets[row];
    const bool valid = label != ignore_index && label >= 0 && label < vocab;
    const float inv_cap = CAP ? 1.f / cap : 0.f;
    // read before the second pass overwrites the row
    float x_label = 0.f;
    if (valid && tid == 0) x_label = ld1<T>(xr + label);

    const int groups = VEC ? vocab / 8 : 0;
    float m = -INFINITY, l = 0.f;
    for (int g = tid; g < groups; g += kCeThreads) {
        float v[8];
        ld8<T>(xr + (int64_t)g * 8, v);
        fold8<CAP>(v, cap, inv_cap, m, l);
    }
    for (int j = groups * 8 + tid; j < vocab; j += kCeThreads) fold1(capped<CAP>(ld1<T>(xr + j), cap, inv_cap) * kLog2e, m, l);
    const float lse2 = workgroup_lse2<kCeWaves>(m, l, s_m, s_l);

    if (tid == 0) {
        if (lse_out) lse_out[row] = lse2 * kLn2;
        if (nll_out) nll_out[row] = valid ? (lse2 - capped<CAP>(x_label, cap, inv_cap) * kLog2e) * kLn2 : 0.f;
    }
    if (!write_grad) return;

    const float scale = valid ? (grad_scale ? *grad_scale : 1.f) : 0.f;
    const float shift = lse2 - log2f(scale);
    const int label_group = valid ? (int)(label >> 3) : -1, label_elem = (int)(label & 7);
    for (int g = tid; g < groups; g += kCeThreads) {
        float v[8];
        if (valid) {
            ld8<T>(xr + (int64_t)g * 8, v);
            grad8<CAP>(v, cap, inv_cap, shift, scale, g == label_group ? label_elem : -1);
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) v[i] = 0.f;
        }
        st8<T>(xr + (int64_t)g * 8, v);
    }
    for (int j = groups * 8 + tid; j < vocab; j += kCeThreads) {
        float d = 0.f;
        if (valid) {
            const float x = ld1<T>(xr + j);
            float t = 0.f;
            if (CAP) t = tanhf(x * inv_cap);
            d = exp2f(fmaf(CAP ? cap * t : x, kLog2e, -shift));
            if (j == label) d -= scale;
            if (CAP) d *= 1.f - t * t;
        }
        st1<T>(xr + j, d);
    }
}

constexpr int kCeReduceThreads = 1024;

// stats[0] = number of rows that count, stats[1] = its reciprocal (inf when there is none)
__global__ __launch_bounds__(kCeReduceThreads) void ce_valid_count_kernel(const int64_t* __restrict__ targets, int64_t n,
                                                                          int64_t ignore_index, int vocab,
                                                                          float* __restrict__ stats) {
    __shared__ int s_cnt[kCeReduceThreads / 64];
    int cnt = 0;
    for (int64_t i = threadIdx.x; i < n; i += kCeReduceThreads) {
        const int64_t t = targets[i];
        cnt += (t != ignore_index && t >= 0 && t < vocab) ? 1 : 0;
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) cnt += __shfl_xor(cnt, off, 64);
    if ((threadIdx.x & 63) == 0) s_cnt[threadIdx.x >> 6] = cnt;
    __syncthreads();
    if (threadIdx.x == 0) {
        int total = 0;
        for (int w = 0; w < kCeReduceThreads / 64; ++w) total += s_cnt[w];
        stats[0] = (float)total;
        stats[1] = 1.f / (float)total;
    }
}

// loss = (sum of nll in a fixed order, fp64) * scale
__global__ __launch_bounds__(kCeReduceThreads) void ce_loss_reduce_kernel(const float* __restrict__ nll, int64_t n,
                                                                          const float* __restrict__ scale,
                                                                          float* __restrict__ loss) {
    __shared__ double s_sum[kCeReduceThreads];
    double acc = 0.0;
    for (int64_t i = threadIdx.x; i < n; i += kCeReduceThreads) acc += (double)nll[i];
    s_sum[threadIdx.x] = acc;
    __syncthreads();
    for (int half = kCeReduceThreads / 2; half > 0; half >>= 1) {
        if ((int)threadIdx.x < half) s_sum[threadIdx.x] += s_sum[threadIdx.x + half];
        __syncthreads();
    }
    if (threadIdx.x == 0) loss[0] = (float)(s_sum[0] * (scale ? (double)*scale : 1.0));
}

// ---- [rows, cols] -> [cols, rows] -----------------------------------------------------------------
// The gradient GEMM d hidden = d logits . C runs more than twice as fast in the library when both
// operands are contiguous along the vocabulary, so the host keeps a transposed copy of C for one call.
// 64 x 64 tiles through LDS, 16-byte accesses on both sides where the shape allows.
constexpr int kTrTile = 64;

template <typename TO, typename TI>
__device__ __forceinline__ TO convert_elem(TI x);
template <>
__device__ __forceinline__ uint16_t convert_elem<uint16_t, uint16_t>(uint16_t x) { return x; }
template <>
__device__ __forceinline__ float convert_elem<float, float>(float x) { return x; }
template <>
__device__ __forceinline__ uint16_t convert_elem<uint16_t, float>(float x) {  // round to nearest even, like torch's cast
    const __bf16 b = (__bf16)x;
    return *(const uint16_t*)&b;
}

// TI -> TO: same type, or fp32 in and bf16 out (the weight gradient summed in fp32, handed back in bf16)
template <typename TI, typename TO>
__global__ __launch_bounds__(256) void transpose_kernel(const TI* __restrict__ src, TO* __restrict__ dst, int64_t rows, int64_t cols) {
    constexpr int VI = 16 / sizeof(TI), VO = 16 / sizeof(TO);      // elements per 16-byte access
    constexpr int kInPerRow = kTrTile / VI, kOutPerRow = kTrTile / VO;
    __shared__ TO tile[kTrTile][kTrTile + 2];
    const int64_t r0 = (int64_t)blockIdx.y * kTrTile, c0 = (int64_t)blockIdx.x * kTrTile;
    const bool vec_in = cols % VI == 0 && ((uintptr_t)src & 15) == 0, vec_out = rows % VO == 0 && ((uintptr_t)dst & 15) == 0;
    for (int a = threadIdx.x; a < kTrTile * kInPerRow; a += 256) {
        const int r = a / kInPerRow, c = (a % kInPerRow) * VI;
        if (r0 + r >= rows) continue;
        const TI* p = src + (r0 + r) * cols + c0 + c;
        if (vec_in && c0 + c + VI <= cols) {
            const uint4 q = *(const uint4*)p;
            const TI* e = (const TI*)&q;
#pragma unroll
            for (int i = 0; i < VI; ++i) tile[r][c + i] = convert_elem<TO, TI>(e[i]);
        } else {
            for (int i = 0; i < VI && c0 + c + i < cols; ++i) tile[r][c + i] = convert_elem<TO, TI>(p[i]);
        }
    }
    __syncthreads();
    for (int a = threadIdx.x; a < kTrTile * kOutPerRow; a += 256) {
        const int c = a / kOutPerRow, r = (a % kOutPerRow) * VO;    // dst row c0 + c, dst columns r0 + r ..
        if (c0 + c >= cols) continue;
        TO* p = dst + (c0 + c) * rows + r0 + r;
        if (vec_out && r0 + r + VO <= rows) {
            uint4 q;
            TO* e = (TO*)&q;
#pragma unroll
            for (int i = 0; i < VO; ++i) e[i] = tile[r + i][c];
            *(uint4*)p = q;
        } else {
            for (int i = 0; i < VO && r0 + r + i < rows; ++i) p[i] = tile[r + i][c];
        }
    }
}

template <typename T>
int launch_rows(void* logits, int64_t pitch, const int64_t* targets, int64_t rows, int vocab, int64_t ignore_index, float cap,
                const float* grad_scale, float* lse, float* nll, int write_grad, hipStream_t stream) {
    const bool vec = vocab >= 8 && pitch % 8 == 0 && ((uintptr_t)logits & 15) == 0;
    const dim3 grid((unsigned)rows), block(kCeThreads);
    T* x = (T*)logits;
    if (cap > 0.f) {
        if (vec)
            ce_rows_kernel<T, true, true><<<grid, block, 0, stream>>>(x, pitch, targets, vocab, ignore_index, cap, grad_scale, lse, nll, write_grad);
        else
            ce_rows_kernel<T, true, false><<<grid, block, 0, stream>>>(x, pitch, targets, vocab, ignore_index, cap, grad_scale, lse, nll, write_grad);
    } else {
        if (vec)
            ce_rows_kernel<T, false, true><<<grid, block, 0, stream>>>(x, pitch, targets, vocab, ignore_index, cap, grad_scale, lse, nll, write_grad);
        else
            ce_rows_kernel<T, false, false><<<grid, block, 0, stream>>>(x, pitch, targets, vocab, ignore_index, cap, grad_scale, lse, nll, write_grad);
    }
    return check_launch("ce_rows_kernel");
}

}  // namespace

int launch_ce_rows(void* logits, int64_t pitch, const int64_t* targets, int64_t rows, int vocab, int64_t ignore_index,
                   float softcap, const float* grad_scale, float* lse, float* nll, int write_grad, int dtype, hipStream_t stream) {
    if (dtype == MA_DTYPE_BF16)
        return launch_rows<uint16_t>(logits, pitch, targets, rows, vocab, ignore_index, softcap, grad_scale, lse, nll, write_grad, stream);
    return launch_rows<float>(logits, pitch, targets, rows, vocab, ignore_index, softcap, grad_scale, lse, nll, write_grad, stream);
}

int launch_transpose(const void* src, void* dst, int64_t rows, int64_t cols, int src_dtype, int dst_dtype, hipStream_t stream) {
    const dim3 grid((unsigned)((cols + kTrTile - 1) / kTrTile), (unsigned)((rows + kTrTile - 1) / kTrTile));
    if (src_dtype == MA_DTYPE_BF16)
        transpose_kernel<uint16_t, uint16_t><<<grid, 256, 0, stream>>>((const uint16_t*)src, (uint16_t*)dst, rows, cols);
    else if (dst_dtype == MA_DTYPE_BF16)
        transpose_kernel<float, uint16_t><<<grid, 256, 0, stream>>>((const float*)src, (uint16_t*)dst, rows, cols);
    else
        transpose_kernel<float, float><<<grid, 256, 0, stream>>>((const float*)src, (float*)dst, rows, cols);
    return check_launch("transpose_kernel");
}

int launch_ce_valid_count(const int64_t* targets, int64_t n, int64_t ignore_index, int vocab, float* stats, hipStream_t stream) {
    ce_valid_count_kernel<<<1, kCeReduceThreads, 0, stream>>>(targets, n, ignore_index, vocab, stats);
    return check_launch("ce_valid_count_kernel");
}

int launch_ce_loss_reduce(const float* nll, int64_t n, const float* scale, float* loss, hipStream_t stream) {
    ce_loss_reduce_kernel<<<1, kCeReduceThreads, 0, stream>>>(nll, n, scale, loss);
    return check_launch("ce_loss_reduce_kernel");
}

}  // namespace ma
