// Fused QK-RMSNorm + RoPE prologue over per-document position_ids, forward and backward.
//
// Stands in for query_norm/key_norm (maester/models/gemma/model.py:135-172, 366-368) followed by
// apply_rotary_emb (model.py:97-106, 371-372) and the per-token table gather (model.py:744-747).
// One pass over q and k: every element is read once and written once (HBM-bound); cos/sin rows
// are read once per token and shared by all heads.
//
// Work split: a group of LPH = D/16 lanes owns one head vector; each lane holds 8 contiguous
// elements of the first half and the 8 elements of the second half that RoPE pairs them with, so
// the rotation is lane-local and the RMS reduction is a butterfly over LPH lanes.  A wave owns one
// token and walks its Hq+Hkv heads 64/LPH at a time.
#include "common.h"

namespace ma {

__device__ __forceinline__ float bf16_bits_to_f32(uint16_t b) { return __uint_as_float((uint32_t)b << 16); }
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
    // round to nearest even, as torch's float -> bfloat16 cast
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);  // quiet NaN
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

template <typename T>
__device__ __forceinline__ void load8(const T* p, float* v);
template <>
__device__ __forceinline__ void load8<float>(const float* p, float* v) {
    const float4 a = *(const float4*)p, b = *(const float4*)(p + 4);
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}
template <>
__device__ __forceinline__ void load8<uint16_t>(const uint16_t* p, float* v) {
    const uint4 a = *(const uint4*)p;
    const uint32_t w[4] = {a.x, a.y, a.z, a.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        v[2 * i] = __uint_as_float(w[i] << 16);
        v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    }
}
// The same in two halves -- the load, and the conversion of what it returned -- so that a kernel can have
// the next head's elements on their way while it works on the current one's.
template <typename T>
struct Raw8;
template <>
struct Raw8<float> {
    float4 a, b;
    __device__ __forceinline__ void load(const float* p) { a = *(const float4*)p; b = *(const float4*)(p + 4); }
    __device__ __forceinline__ void get(float* v) const { v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w; }
};
template <>
struct Raw8<uint16_t> {
    uint4 a;
    __device__ __forceinline__ void load(const uint16_t* p) { a = *(const uint4*)p; }
    __device__ __forceinline__ void get(float* v) const {
        const uint32_t w[4] = {a.x, a.y, a.z, a.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            v[2 * i] = __uint_as_float(w[i] << 16);
            v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
        }
    }
};
template <typename T>
__device__ __forceinline__ void store8(T* p, const float* v);
template <>
__device__ __forceinline__ void store8<float>(float* p, const float* v) {
    *(float4*)p = make_float4(v[0], v[1], v[2], v[3]);
    *(float4*)(p + 4) = make_float4(v[4], v[5], v[6], v[7]);
}
template <>
__device__ __forceinline__ void store8<uint16_t>(uint16_t* p, const float* v) {
    // the hardware conversion (v_cvt_pk_bf16_f32) rounds to nearest even like torch's cast
    typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
    bf16x8_t o;
#pragma unroll
    for (int i = 0; i < 8; ++i) o[i] = (__bf16)v[i];
    *(bf16x8_t*)p = o;
}

template <int LPH>
__device__ __forceinline__ float group_sum(float x) {
#pragma unroll
    for (int off = LPH / 2; off > 0; off >>= 1) x += __shfl_xor(x, off, 64);
    return x;
}

constexpr int kWavesPerBlock = 4;

// A position outside the table would be an out-of-bounds read; the reference's gather raises an
// index error instead (model.py:744-747).  Clamp so that a bad id cannot fault the GPU.
__device__ __forceinline__ int64_t clamp_pos(int64_t p, int64_t n_pos) {
    return p < 0 ? 0 : (p >= n_pos ? n_pos - 1 : p);
}

template <typename T, int D>
__global__ __launch_bounds__(64 * kWavesPerBlock) void prologue_fwd_kernel(
    ma_tensor4 qi, ma_tensor4 ki, ma_tensor4 qo, ma_tensor4 ko, const float* __restrict__ qw,
    const float* __restrict__ kw, const float* __restrict__ cs, const float* __restrict__ sn,
    const int64_t* __restrict__ pos, int64_t n_pos, float eps, int unit, float* __restrict__ q_rstd,
    float* __restrict__ k_rstd, int B, int S, int Hq, int Hkv) {
    constexpr int LPH = D / 16;       // lanes per head vector
    constexpr int HPW = 64 / LPH;     // heads per wave pass
    const int lane = threadIdx.x & 63;
    const int tok = blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
    if (tok >= B * S) return;
    const int b = tok / S, s = tok - b * S;
    const int sub = lane % LPH, hsel = lane / LPH;
    const int H = Hq + Hkv;
    // where head h of this token lives (a lane group past the last head re-reads the last one and stores nothing)
    auto src_of = [&](int h) {
        const int hc = min(h, H - 1);
        const bool is_q = hc < Hq;
        const ma_tensor4& ti = is_q ? qi : ki;
        return (const T*)ti.ptr + b * ti.stride_b + s * ti.stride_s + (is_q ? hc : hc - Hq) * ti.stride_h;
    };
    // The first heads' elements are requested before anything else: the position, and then the table rows
    // that hang on it, are two dependent round trips the elements do not have to wait behind.  After that
    // the next heads' elements are always on their way while the current ones are worked on.
    Raw8<T> r1, r2;
    {
        const T* src = src_of(hsel);
        r1.load(src + sub * 8);
        r2.load(src + D / 2 + sub * 8);
    }
    const int64_t p = clamp_pos(pos ? pos[tok] : (int64_t)s, n_pos);
    float c[8], sv[8];
    load8<float>(cs + p * (D / 2) + sub * 8, c);
    load8<float>(sn + p * (D / 2) + sub * 8, sv);
    for (int h0 = 0; h0 < H; h0 += HPW) {
        const int h = h0 + hsel;
        float x1[8], x2[8];
        r1.get(x1);
        r2.get(x2);
        if (h0 + HPW < H) {  // (wave-uniform)
            const T* nsrc = src_of(h + HPW);
            r1.load(nsrc + sub * 8);
            r2.load(nsrc + D / 2 + sub * 8);
        }
        if (h >= H) break;  // whole lane groups drop out together
        const bool is_q = h < Hq;
        const int hh = is_q ? h : h - Hq;
        const ma_tensor4& to = is_q ? qo : ko;
        const float* w = is_q ? qw : kw;
        T* dst = (T*)to.ptr + b * to.stride_b + s * to.stride_s + hh * to.stride_h;
        if (w) {
            float ss = 0.f;
#pragma unroll
            for (int i = 0; i < 8; ++i) ss += x1[i] * x1[i] + x2[i] * x2[i];
            ss = group_sum<LPH>(ss);
            const float r = rsqrtf(ss * (1.0f / D) + eps);
            float g1[8], g2[8];
            load8<float>(w + sub * 8, g1);
            load8<float>(w + D / 2 + sub * 8, g2);
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                x1[i] = x1[i] * r * (unit ? 1.0f + g1[i] : g1[i]);
                x2[i] = x2[i] * r * (unit ? 1.0f + g2[i] : g2[i]);
            }
            float* rs = is_q ? q_rstd : k_rstd;
            if (rs && sub == 0) rs[(size_t)tok * (is_q ? Hq : Hkv) + hh] = r;
        }
        float o1[8], o2[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            o1[i] = x1[i] * c[i] - x2[i] * sv[i];
            o2[i] = x1[i] * sv[i] + x2[i] * c[i];
        }
        store8<T>(dst + sub * 8, o1);
        store8<T>(dst + D / 2 + sub * 8, o2);
    }
}

// Backward.  Each wave walks tokens with a grid stride and keeps the dW partial sums of its lanes in
// registers; at the end lanes that own the same elements are combined (butterfly across the head
// selector bits, then across the waves of the block through LDS) and each block writes one row of
// partials; a second kernel sums the rows.  No atomics, fixed summation order.
template <typename T, int D>
__global__ __launch_bounds__(64 * kWavesPerBlock) void prologue_bwd_kernel(
    ma_tensor4 qi, ma_tensor4 ki, ma_tensor4 dqo, ma_tensor4 dko, ma_tensor4 dqi, ma_tensor4 dki,
    const float* __restrict__ qw, const float* __restrict__ kw, const float* __restrict__ cs,
    const float* __restrict__ sn, const int64_t* __restrict__ pos, int64_t n_pos, int unit,
    const float* __restrict__ q_rstd, const float* __restrict__ k_rstd, float* __restrict__ partials, int B, int S,
    int Hq, int Hkv) {
    constexpr int LPH = D / 16;
    constexpr int HPW = 64 / LPH;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int sub = lane % LPH, hsel = lane / LPH;
    const int H = Hq + Hkv;
    float accq[16], acck[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) accq[i] = acck[i] = 0.f;
    float gq1[8], gq2[8], gk1[8], gk2[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) gq1[i] = gq2[i] = gk1[i] = gk2[i] = 1.f;
    if (qw) {
        load8<float>(qw + sub * 8, gq1);
        load8<float>(qw + D / 2 + sub * 8, gq2);
        if (unit)
#pragma unroll
            for (int i = 0; i < 8; ++i) { gq1[i] += 1.f; gq2[i] += 1.f; }
    }
    if (kw) {
        load8<float>(kw + sub * 8, gk1);
        load8<float>(kw + D / 2 + sub * 8, gk2);
        if (unit)
#pragma unroll
            for (int i = 0; i < 8; ++i) { gk1[i] += 1.f; gk2[i] += 1.f; }
    }
    const int ntok = B * S;
    // what a head of a token needs from memory: requested as one group, a head ahead of the arithmetic.
    // No load hangs on a condition: a lane group past the last head re-reads the last one, and a tensor
    // without norm weight -- whose forward input and rstd are not passed at all (null) -- reads the incoming
    // gradient a second time and the cos table instead; those values are never used.
    Raw8<T> rg1, rg2, rx1, rx2;
    float rr = 0.f;
    auto request = [&](int tok, int b, int s, int h) {
        const int hc = min(h, H - 1);
        const bool is_q = hc < Hq;
        const int hh = is_q ? hc : hc - Hq;
        const ma_tensor4& tx = is_q ? qi : ki;
        const ma_tensor4& tg = is_q ? dqo : dko;
        const bool normed = (is_q ? qw : kw) != nullptr;  // then tx and the rstd array are there (checked by the caller)
        const T* gsrc = (const T*)tg.ptr + b * tg.stride_b + s * tg.stride_s + hh * tg.stride_h;
        const T* xsrc = normed ? (const T*)tx.ptr + b * tx.stride_b + s * tx.stride_s + hh * tx.stride_h : gsrc;
        rg1.load(gsrc + sub * 8);
        rg2.load(gsrc + D / 2 + sub * 8);
        rx1.load(xsrc + sub * 8);
        rx2.load(xsrc + D / 2 + sub * 8);
        rr = *(normed ? (is_q ? q_rstd : k_rstd) + (size_t)tok * (is_q ? Hq : Hkv) + hh : cs);
    };
    for (int tok = blockIdx.x * kWavesPerBlock + wave; tok < ntok; tok += gridDim.x * kWavesPerBlock) {
        const int b = tok / S, s = tok - b * S;
        request(tok, b, s, hsel);  // (before the position and the table rows that hang on it)
        const int64_t p = clamp_pos(pos ? pos[tok] : (int64_t)s, n_pos);
        float c[8], sv[8];
        load8<float>(cs + p * (D / 2) + sub * 8, c);
        load8<float>(sn + p * (D / 2) + sub * 8, sv);
        for (int h0 = 0; h0 < H; h0 += HPW) {
            const int h = h0 + hsel;
            float g1[8], g2[8], x1[8], x2[8], dy1[8], dy2[8];
            rg1.get(g1);
            rg2.get(g2);
            rx1.get(x1);
            rx2.get(x2);
            const float r = rr;
            if (h0 + HPW < H) request(tok, b, s, h + HPW);  // (wave-uniform)
            if (h >= H) break;
            const bool is_q = h < Hq;
            const int hh = is_q ? h : h - Hq;
            const ma_tensor4& td = is_q ? dqi : dki;
            const float* w = is_q ? qw : kw;
            T* dst = (T*)td.ptr + b * td.stride_b + s * td.stride_s + hh * td.stride_h;
#pragma unroll
            for (int i = 0; i < 8; ++i) {  // transpose of the rotation
                dy1[i] = g1[i] * c[i] + g2[i] * sv[i];
                dy2[i] = -g1[i] * sv[i] + g2[i] * c[i];
            }
            if (w) {
                float dot = 0.f;
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const float n1 = x1[i] * r, n2 = x2[i] * r;
                    if (is_q) { accq[i] += dy1[i] * n1; accq[8 + i] += dy2[i] * n2; }
                    else      { acck[i] += dy1[i] * n1; acck[8 + i] += dy2[i] * n2; }
                    const float dn1 = dy1[i] * (is_q ? gq1[i] : gk1[i]);
                    const float dn2 = dy2[i] * (is_q ? gq2[i] : gk2[i]);
                    dy1[i] = dn1; dy2[i] = dn2;
                    x1[i] = n1; x2[i] = n2;
                    dot += dn1 * n1 + dn2 * n2;
                }
                dot = group_sum<LPH>(dot) * (1.0f / D);
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    dy1[i] = r * (dy1[i] - x1[i] * dot);
                    dy2[i] = r * (dy2[i] - x2[i] * dot);
                }
            }
            store8<T>(dst + sub * 8, dy1);
            store8<T>(dst + D / 2 + sub * 8, dy2);
        }
    }
    if (!partials) return;
    // combine lanes that own the same elements (different head selectors)
#pragma unroll
    for (int i = 0; i < 16; ++i) {
#pragma unroll
        for (int off = LPH; off < 64; off <<= 1) {
            accq[i] += __shfl_xor(accq[i], off, 64);
            acck[i] += __shfl_xor(acck[i], off, 64);
        }
    }
    __shared__ float red[kWavesPerBlock][2][D];
    if (hsel == 0) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            red[wave][0][sub * 8 + i] = accq[i];
            red[wave][0][D / 2 + sub * 8 + i] = accq[8 + i];
            red[wave][1][sub * 8 + i] = acck[i];
            red[wave][1][D / 2 + sub * 8 + i] = acck[8 + i];
        }
    }
    __syncthreads();
    for (int e = threadIdx.x; e < 2 * D; e += blockDim.x) {
        float t = 0.f;
        for (int w = 0; w < kWavesPerBlock; ++w) t += red[w][e / D][e % D];
        partials[(size_t)blockIdx.x * 2 * D + e] = t;
    }
}

// Sums the per-block partial rows: a block owns 16 columns, 16 lanes per column stride over the rows
// (fixed order, no atomics), then a tree over the 16 lanes in LDS.
__global__ __launch_bounds__(256) void prologue_dw_reduce_kernel(const float* __restrict__ partials, int nblocks, int D,
                                                                 float* __restrict__ dqw, float* __restrict__ dkw) {
    __shared__ float red[16][17];
    const int c = threadIdx.x & 15, rl = threadIdx.x >> 4;
    const int e = blockIdx.x * 16 + c;
    float t = 0.f;
    if (e < 2 * D)
        for (int r = rl; r < nblocks; r += 16) t += partials[(size_t)r * 2 * D + e];
    red[rl][c] = t;
    __syncthreads();
    if (rl == 0 && e < 2 * D) {
        float sum = 0.f;
#pragma unroll
        for (int i = 0; i < 16; ++i) sum += red[i][c];
        if (e < D) { if (dqw) dqw[e] = sum; }
        else       { if (dkw) dkw[e - D] = sum; }
    }
}

int prologue_bwd_blocks(int B, int S) {
    const long ntok = (long)B * S;
    const long need = (ntok + kWavesPerBlock - 1) / kWavesPerBlock;
    return (int)(need < 1024 ? need : 1024);
}

template <typename T, int D>
static int fwd_t(const ma_tensor4& qi, const ma_tensor4& ki, const ma_tensor4& qo, const ma_tensor4& ko,
                 const float* qw, const float* kw, const float* cs, const float* sn, const int64_t* pos, int64_t n_pos,
                 float eps, int unit, float* q_rstd, float* k_rstd, int B, int S, int Hq, int Hkv, hipStream_t st) {
    const int ntok = B * S;
    const int grid = (ntok + kWavesPerBlock - 1) / kWavesPerBlock;
    hipLaunchKernelGGL((prologue_fwd_kernel<T, D>), dim3(grid), dim3(64 * kWavesPerBlock), 0, st, qi, ki, qo, ko, qw,
                       kw, cs, sn, pos, n_pos, eps, unit, q_rstd, k_rstd, B, S, Hq, Hkv);
    return check_launch("prologue_fwd_kernel");
}

int launch_prologue_fwd(const ma_tensor4& qi, const ma_tensor4& ki, const ma_tensor4& qo, const ma_tensor4& ko,
                        const float* qw, const float* kw, const float* cs, const float* sn, int64_t n_pos,
                        const int64_t* pos, float eps, int unit, float* q_rstd, float* k_rstd, int dtype, int B,
                        int S, int Hq, int Hkv, int D, hipStream_t st) {
#define MA_PF(TT, DD) \
    return fwd_t<TT, DD>(qi, ki, qo, ko, qw, kw, cs, sn, pos, n_pos, eps, unit, q_rstd, k_rstd, B, S, Hq, Hkv, st)
    if (dtype == MA_DTYPE_BF16) {
        if (D == 64) MA_PF(uint16_t, 64);
        if (D == 128) MA_PF(uint16_t, 128);
        if (D == 256) MA_PF(uint16_t, 256);
    } else {
        if (D == 64) MA_PF(float, 64);
        if (D == 128) MA_PF(float, 128);
        if (D == 256) MA_PF(float, 256);
    }
#undef MA_PF
    return fail(MA_ERR_UNSUPPORTED, "prologue: head_dim %d not in {64,128,256}", D);
}

template <typename T, int D>
static int bwd_t(const ma_tensor4& qi, const ma_tensor4& ki, const ma_tensor4& dqo, const ma_tensor4& dko,
                 const ma_tensor4& dqi, const ma_tensor4& dki, const float* qw, const float* kw, const float* cs,
                 const float* sn, const int64_t* pos, int64_t n_pos, int unit, const float* q_rstd,
                 const float* k_rstd, float* dqw, float* dkw, void* ws, int B, int S, int Hq, int Hkv, hipStream_t st) {
    // One resident wave set: the kernel walks tokens with a grid stride, so a grid larger than what
    // the device holds at once only adds a ragged second round (the workspace is sized for the cap).
    int grid = prologue_bwd_blocks(B, S);
    {
        static int resident = 0;  // blocks of this instantiation the current device holds at once
        if (resident == 0) {
            int dev = 0, cus = 0, per_cu = 0;
            if (hipGetDevice(&dev) == hipSuccess &&
                hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess &&
                hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, prologue_bwd_kernel<T, D>, 64 * kWavesPerBlock, 0) == hipSuccess)
                resident = cus * per_cu;
            if (resident <= 0) resident = 1024;
        }
        if (grid > resident) grid = resident;
    }
    float* partials = (qw || kw) ? (float*)ws : nullptr;
    hipLaunchKernelGGL((prologue_bwd_kernel<T, D>), dim3(grid), dim3(64 * kWavesPerBlock), 0, st, qi, ki, dqo, dko,
                       dqi, dki, qw, kw, cs, sn, pos, n_pos, unit, q_rstd, k_rstd, partials, B, S, Hq, Hkv);
    int rc = check_launch("prologue_bwd_kernel");
    if (rc || !partials) return rc;
    hipLaunchKernelGGL(prologue_dw_reduce_kernel, dim3((2 * D + 15) / 16), dim3(256), 0, st, partials, grid, D,
                       qw ? dqw : nullptr, kw ? dkw : nullptr);
    return check_launch("prologue_dw_reduce_kernel");
}

int launch_prologue_bwd(const ma_tensor4& qi, const ma_tensor4& ki, const ma_tensor4& dqo, const ma_tensor4& dko,
                        const ma_tensor4& dqi, const ma_tensor4& dki, const float* qw, const float* kw,
                        const float* cs, const float* sn, int64_t n_pos, const int64_t* pos, int unit,
                        const float* q_rstd, const float* k_rstd, float* dqw, float* dkw, void* ws, int dtype,
                        int B, int S, int Hq, int Hkv, int D, hipStream_t st) {
#define MA_PB(TT, DD)                                                                                      \
    return bwd_t<TT, DD>(qi, ki, dqo, dko, dqi, dki, qw, kw, cs, sn, pos, n_pos, unit, q_rstd, k_rstd, dqw, dkw, \
                         ws, B, S, Hq, Hkv, st)
    if (dtype == MA_DTYPE_BF16) {
        if (D == 64) MA_PB(uint16_t, 64);
        if (D == 128) MA_PB(uint16_t, 128);
        if (D == 256) MA_PB(uint16_t, 256);
    } else {
        if (D == 64) MA_PB(float, 64);
        if (D == 128) MA_PB(float, 128);
        if (D == 256) MA_PB(float, 256);
    }
#undef MA_PB
    return fail(MA_ERR_UNSUPPORTED, "prologue: head_dim %d not in {64,128,256}", D);
}

}  // namespace ma
