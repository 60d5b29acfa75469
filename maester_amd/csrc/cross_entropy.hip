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
// One workgroup per row.  A Gemma row is 262 208 logits, half a megabyte, too long to keep in
// registers: the row is read twice (running maximum and sum, then the gradient) and written once.
// All arithmetic is fp32 in the exp2 domain; the reduction order is fixed, so results are identical
// from run to run.
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

// soft-capped logit in log2 units; t receives tanh(x / cap) (unused without a cap)
template <bool CAP>
__device__ __forceinline__ float to_log2(float x, float cap, float inv_cap, float& t) {
    if (CAP) {
        t = tanhf(x * inv_cap);
        return cap * t * kLog2e;
    }
    t = 0.f;
    return x * kLog2e;
}

// VEC: the row pitch and the vocabulary allow 8-element accesses
template <typename T, bool CAP, bool VEC>
__global__ __launch_bounds__(kCeThreads) void ce_rows_kernel(T* __restrict__ logits, int64_t pitch,
                                                             const int64_t* __restrict__ targets, int vocab,
                                                             int64_t ignore_index, float cap,
                                                             const float* __restrict__ grad_scale, float* __restrict__ lse_out,
                                                             float* __restrict__ nll_out, int write_grad) {
    __shared__ float s_m[kCeWaves], s_l[kCeWaves];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
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
        float v[8], t;
        ld8<T>(xr + (int64_t)g * 8, v);
        float vm = -INFINITY;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            v[i] = to_log2<CAP>(v[i], cap, inv_cap, t);
            vm = fmaxf(vm, v[i]);
        }
        const float mn = fmaxf(m, vm);
        float add = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) add += exp2f(v[i] - mn);
        l = l * exp2f(m - mn) + add;
        m = mn;
    }
    for (int j = groups * 8 + tid; j < vocab; j += kCeThreads) {
        float t;
        const float y = to_log2<CAP>(ld1<T>(xr + j), cap, inv_cap, t);
        const float mn = fmaxf(m, y);
        l = l * exp2f(m - mn) + exp2f(y - mn);
        m = mn;
    }
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
    for (int w = 1; w < kCeWaves; ++w) big = fmaxf(big, s_m[w]);
    float sum = 0.f;
#pragma unroll
    for (int w = 0; w < kCeWaves; ++w) sum += s_l[w] * exp2f(s_m[w] - big);
    const float lse2 = big + log2f(sum);

    if (tid == 0) {
        float t;
        if (lse_out) lse_out[row] = lse2 * kLn2;
        if (nll_out) nll_out[row] = valid ? (lse2 - to_log2<CAP>(x_label, cap, inv_cap, t)) * kLn2 : 0.f;
    }
    if (!write_grad) return;

    const float scale = valid ? (grad_scale ? *grad_scale : 1.f) : 0.f;
    const int label_group = valid ? (int)(label >> 3) : -1, label_elem = (int)(label & 7);
    for (int g = tid; g < groups; g += kCeThreads) {
        float v[8];
        if (valid) {
            ld8<T>(xr + (int64_t)g * 8, v);
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                float t;
                const float y = to_log2<CAP>(v[i], cap, inv_cap, t);
                float d = exp2f(y - lse2);
                if (g == label_group && i == label_elem) d -= 1.f;
                v[i] = d * scale * (CAP ? 1.f - t * t : 1.f);
            }
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) v[i] = 0.f;
        }
        st8<T>(xr + (int64_t)g * 8, v);
    }
    for (int j = groups * 8 + tid; j < vocab; j += kCeThreads) {
        float d = 0.f;
        if (valid) {
            float t;
            const float y = to_log2<CAP>(ld1<T>(xr + j), cap, inv_cap, t);
            d = exp2f(y - lse2);
            if (j == label) d -= 1.f;
            d *= scale * (CAP ? 1.f - t * t : 1.f);
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

int launch_ce_valid_count(const int64_t* targets, int64_t n, int64_t ignore_index, int vocab, float* stats, hipStream_t stream) {
    ce_valid_count_kernel<<<1, kCeReduceThreads, 0, stream>>>(targets, n, ignore_index, vocab, stats);
    return check_launch("ce_valid_count_kernel");
}

int launch_ce_loss_reduce(const float* nll, int64_t n, const float* scale, float* loss, hipStream_t stream) {
    ce_loss_reduce_kernel<<<1, kCeReduceThreads, 0, stream>>>(nll, n, scale, loss);
    return check_launch("ce_loss_reduce_kernel");
}

}  // namespace ma
