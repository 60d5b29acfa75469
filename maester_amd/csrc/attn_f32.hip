// Full-precision (fp32 arithmetic, no matrix cores) document-masked GQA attention.
//
// This is the path for fp32 activations, where the result has to agree with torch's eager
// FlexAttention math (torch/_higher_order_ops/flex_attention.py:159-267, 825-993) to ~1e-6; the
// bf16 training path uses the MFMA kernels in attn_fwd_bf16.hip / attn_bwd_bf16.hip instead.
// Layout: one thread owns one q row (forward, dQ) or one kv row (dK/dV); K/V (or Q/dO) chunks are
// staged in LDS and read as wave-wide broadcasts.  Only the tiles named by the tile map are
// visited; elements of partial tiles are masked with the document/causal/window predicate.
#include "common.h"

namespace ma {

constexpr int kRows = 64;  // rows per workgroup (one wave)

template <int D>
struct F32Cfg {
    static constexpr int KC = D >= 256 ? 16 : 32;  // kv rows staged per step
    static constexpr int LDQ = D + 1;              // padded row stride of per-thread rows in LDS
};

__device__ __forceinline__ bool elem_allowed(int q, int kv, int S, int causal, int64_t window, int64_t dq,
                                             const int64_t* kdoc, int c, bool has_doc) {
    if (kv >= S) return false;
    bool ok = pair_allowed(q, kv, causal, window);
    if (has_doc) ok = ok && (kdoc[c] == dq);
    return ok;
}

template <int D>
__global__ __launch_bounds__(kRows) void attn_fwd_f32_kernel(AttnArgs a) {
    using C = F32Cfg<D>;
    extern __shared__ float smem[];
    float* qs = smem;                         // [kRows][LDQ]
    float* ks = qs + kRows * C::LDQ;          // [KC][D]
    float* vs = ks + C::KC * D;               // [KC][D]
    int64_t* kdoc = (int64_t*)(vs + C::KC * D);  // [KC]

    const int t = threadIdx.x;
    const int half = blockIdx.x & 1, i = blockIdx.x >> 1, h = blockIdx.y, b = blockIdx.z;
    const int hk = h / (a.Hq / a.Hkv);
    const int q = i * kTile + half * kRows + t;
    const bool qvalid = q < a.S;
    const float* qp = (const float*)a.q.ptr + b * a.q.stride_b + h * a.q.stride_h;
    const float* kp = (const float*)a.k.ptr + b * a.k.stride_b + hk * a.k.stride_h;
    const float* vp = (const float*)a.v.ptr + b * a.v.stride_b + hk * a.v.stride_h;
    const int64_t* drow = a.doc ? a.doc + (size_t)b * a.S : nullptr;

    // stage the 64 q rows (coalesced), then each thread reads its own padded row
    for (int e = t; e < kRows * D; e += kRows) {
        const int r = e / D, d = e - r * D;
        const int qq = i * kTile + half * kRows + r;
        qs[r * C::LDQ + d] = qq < a.S ? qp[(int64_t)qq * a.q.stride_s + d] : 0.f;
    }
    const int64_t dq = (drow && qvalid) ? drow[q] : 0;
    float o[D];
#pragma unroll
    for (int d = 0; d < D; ++d) o[d] = 0.f;
    float m = -INFINITY, l = 0.f;

    const int32_t* plist = a.map.kv_indices + ((size_t)b * a.T + i) * a.T;
    const int32_t* flist = a.map.full_kv_indices + ((size_t)b * a.T + i) * a.T;
    const int np = a.map.kv_num_blocks[(size_t)b * a.T + i];
    const int nf = a.map.full_kv_num_blocks[(size_t)b * a.T + i];
    for (int it = 0; it < np + nf; ++it) {
        const bool partial = it < np;
        const int j = partial ? plist[it] : flist[it - np];
        for (int c0 = 0; c0 < kTile; c0 += C::KC) {
            const int k0 = j * kTile + c0;
            __syncthreads();
            for (int e = t; e < C::KC * D; e += kRows) {
                const int r = e / D, d = e - r * D;
                const int kv = k0 + r;
                ks[e] = kv < a.S ? kp[(int64_t)kv * a.k.stride_s + d] : 0.f;
                vs[e] = kv < a.S ? vp[(int64_t)kv * a.v.stride_s + d] : 0.f;
            }
            if (drow && t < C::KC) kdoc[t] = (k0 + t < a.S) ? drow[k0 + t] : 0;
            __syncthreads();
            float sc[C::KC];
            float cmax = -INFINITY;
#pragma unroll
            for (int c = 0; c < C::KC; ++c) {
                float acc = 0.f;
#pragma unroll
                for (int d = 0; d < D; ++d) acc += qs[t * C::LDQ + d] * ks[c * D + d];
                acc *= a.scale;
                bool ok = qvalid;
                if (partial) ok = ok && elem_allowed(q, k0 + c, a.S, a.causal, a.window, dq, kdoc, c, drow != nullptr);
                sc[c] = ok ? acc : -INFINITY;
                cmax = fmaxf(cmax, sc[c]);
            }
            const float mn = fmaxf(m, cmax);
            if (mn == -INFINITY) continue;  // nothing visible for this row yet
            const float corr = __expf(m - mn);
            l *= corr;
#pragma unroll
            for (int d = 0; d < D; ++d) o[d] *= corr;
#pragma unroll
            for (int c = 0; c < C::KC; ++c) {
                const float p = __expf(sc[c] - mn);
                l += p;
#pragma unroll
                for (int d = 0; d < D; ++d) o[d] += p * vs[c * D + d];
            }
            m = mn;
        }
    }
    if (qvalid) {
        const float inv = l > 0.f ? 1.0f / l : 0.f;
        float* op = (float*)a.o.ptr + b * a.o.stride_b + (int64_t)q * a.o.stride_s + h * a.o.stride_h;
#pragma unroll
        for (int d = 0; d < D; ++d) op[d] = o[d] * inv;
        a.lse[((size_t)b * a.Hq + h) * a.S + q] = l > 0.f ? m + __logf(l) : -INFINITY;
    }
}

// delta[b,h,q] = sum_d O * dO   (fp32 inputs)
__global__ void attn_delta_f32_kernel(AttnArgs a) {
    const int64_t row = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t nrows = (int64_t)a.B * a.Hq * a.S;
    if (row >= nrows) return;
    const int q = row % a.S;
    const int h = (row / a.S) % a.Hq;
    const int b = row / ((int64_t)a.S * a.Hq);
    const float* op = (const float*)a.o.ptr + b * a.o.stride_b + (int64_t)q * a.o.stride_s + h * a.o.stride_h;
    const float* gp = (const float*)a.dout.ptr + b * a.dout.stride_b + (int64_t)q * a.dout.stride_s + h * a.dout.stride_h;
    float acc = 0.f;
    for (int d = 0; d < a.D; ++d) acc += op[d] * gp[d];
    a.delta[row] = acc;
}

template <int D>
__global__ __launch_bounds__(kRows) void attn_bwd_dq_f32_kernel(AttnArgs a) {
    using C = F32Cfg<D>;
    extern __shared__ float smem[];
    float* qs = smem;                          // [kRows][LDQ]
    float* gs = qs + kRows * C::LDQ;           // [kRows][LDQ]  dO rows
    float* ks = gs + kRows * C::LDQ;           // [KC][D]
    float* vs = ks + C::KC * D;                // [KC][D]
    int64_t* kdoc = (int64_t*)(vs + C::KC * D);

    const int t = threadIdx.x;
    const int half = blockIdx.x & 1, i = blockIdx.x >> 1, h = blockIdx.y, b = blockIdx.z;
    const int hk = h / (a.Hq / a.Hkv);
    const int q = i * kTile + half * kRows + t;
    const bool qvalid = q < a.S;
    const float* qp = (const float*)a.q.ptr + b * a.q.stride_b + h * a.q.stride_h;
    const float* gp = (const float*)a.dout.ptr + b * a.dout.stride_b + h * a.dout.stride_h;
    const float* kp = (const float*)a.k.ptr + b * a.k.stride_b + hk * a.k.stride_h;
    const float* vp = (const float*)a.v.ptr + b * a.v.stride_b + hk * a.v.stride_h;
    const int64_t* drow = a.doc ? a.doc + (size_t)b * a.S : nullptr;
    for (int e = t; e < kRows * D; e += kRows) {
        const int r = e / D, d = e - r * D;
        const int qq = i * kTile + half * kRows + r;
        qs[r * C::LDQ + d] = qq < a.S ? qp[(int64_t)qq * a.q.stride_s + d] : 0.f;
        gs[r * C::LDQ + d] = qq < a.S ? gp[(int64_t)qq * a.dout.stride_s + d] : 0.f;
    }
    const int64_t dqid = (drow && qvalid) ? drow[q] : 0;
    const size_t rowi = ((size_t)b * a.Hq + h) * a.S + (qvalid ? q : 0);
    const float lse = a.lse[rowi], delta = a.delta[rowi];
    float acc[D];
#pragma unroll
    for (int d = 0; d < D; ++d) acc[d] = 0.f;

    const int32_t* plist = a.map.kv_indices + ((size_t)b * a.T + i) * a.T;
    const int32_t* flist = a.map.full_kv_indices + ((size_t)b * a.T + i) * a.T;
    const int np = a.map.kv_num_blocks[(size_t)b * a.T + i];
    const int nf = a.map.full_kv_num_blocks[(size_t)b * a.T + i];
    for (int it = 0; it < np + nf; ++it) {
        const bool partial = it < np;
        const int j = partial ? plist[it] : flist[it - np];
        for (int c0 = 0; c0 < kTile; c0 += C::KC) {
            const int k0 = j * kTile + c0;
            __syncthreads();
            for (int e = t; e < C::KC * D; e += kRows) {
                const int r = e / D, d = e - r * D;
                const int kv = k0 + r;
                ks[e] = kv < a.S ? kp[(int64_t)kv * a.k.stride_s + d] : 0.f;
                vs[e] = kv < a.S ? vp[(int64_t)kv * a.v.stride_s + d] : 0.f;
            }
            if (drow && t < C::KC) kdoc[t] = (k0 + t < a.S) ? drow[k0 + t] : 0;
            __syncthreads();
#pragma unroll 4
            for (int c = 0; c < C::KC; ++c) {
                bool ok = qvalid;
                if (partial) ok = ok && elem_allowed(q, k0 + c, a.S, a.causal, a.window, dqid, kdoc, c, drow != nullptr);
                float s = 0.f, dp = 0.f;
#pragma unroll
                for (int d = 0; d < D; ++d) {
                    s += qs[t * C::LDQ + d] * ks[c * D + d];
                    dp += gs[t * C::LDQ + d] * vs[c * D + d];
                }
                const float p = ok ? __expf(s * a.scale - lse) : 0.f;
                const float ds = p * (dp - delta);
#pragma unroll
                for (int d = 0; d < D; ++d) acc[d] += ds * ks[c * D + d];
            }
        }
    }
    if (qvalid) {
        float* op = (float*)a.dq.ptr + b * a.dq.stride_b + (int64_t)q * a.dq.stride_s + h * a.dq.stride_h;
#pragma unroll
        for (int d = 0; d < D; ++d) op[d] = acc[d] * a.scale;
    }
}

template <int D>
__global__ __launch_bounds__(kRows) void attn_bwd_dkv_f32_kernel(AttnArgs a) {
    constexpr int QC = 16;          // q rows staged per step
    constexpr int LDK = D + 1;
    extern __shared__ float smem[];
    float* ks = smem;                  // [kRows][LDK]
    float* vs = ks + kRows * LDK;      // [kRows][LDK]
    float* qs = vs + kRows * LDK;      // [QC][D]
    float* gs = qs + QC * D;           // [QC][D]
    float* ls = gs + QC * D;           // [QC] lse
    float* dl = ls + QC;               // [QC] delta
    int64_t* qdoc = (int64_t*)(dl + QC);

    const int t = threadIdx.x;
    const int half = blockIdx.x & 1, j = blockIdx.x >> 1, hk = blockIdx.y, b = blockIdx.z;
    const int G = a.Hq / a.Hkv;
    const int kv = j * kTile + half * kRows + t;
    const bool kvalid = kv < a.S;
    const float* kp = (const float*)a.k.ptr + b * a.k.stride_b + hk * a.k.stride_h;
    const float* vp = (const float*)a.v.ptr + b * a.v.stride_b + hk * a.v.stride_h;
    const int64_t* drow = a.doc ? a.doc + (size_t)b * a.S : nullptr;
    for (int e = t; e < kRows * D; e += kRows) {
        const int r = e / D, d = e - r * D;
        const int kk = j * kTile + half * kRows + r;
        ks[r * LDK + d] = kk < a.S ? kp[(int64_t)kk * a.k.stride_s + d] : 0.f;
        vs[r * LDK + d] = kk < a.S ? vp[(int64_t)kk * a.v.stride_s + d] : 0.f;
    }
    const int64_t dk_id = (drow && kvalid) ? drow[kv] : 0;
    float dk[D], dv[D];
#pragma unroll
    for (int d = 0; d < D; ++d) dk[d] = dv[d] = 0.f;

    const int32_t* plist = a.map.q_indices + ((size_t)b * a.T + j) * a.T;
    const int32_t* flist = a.map.full_q_indices + ((size_t)b * a.T + j) * a.T;
    const int np = a.map.q_num_blocks[(size_t)b * a.T + j];
    const int nf = a.map.full_q_num_blocks[(size_t)b * a.T + j];
    for (int g = 0; g < G; ++g) {
        const int h = hk * G + g;
        const float* qp = (const float*)a.q.ptr + b * a.q.stride_b + h * a.q.stride_h;
        const float* gp = (const float*)a.dout.ptr + b * a.dout.stride_b + h * a.dout.stride_h;
        const size_t rowbase = ((size_t)b * a.Hq + h) * a.S;
        for (int it = 0; it < np + nf; ++it) {
            const bool partial = it < np;
            const int i = partial ? plist[it] : flist[it - np];
            for (int c0 = 0; c0 < kTile; c0 += QC) {
                const int q0 = i * kTile + c0;
                __syncthreads();
                for (int e = t; e < QC * D; e += kRows) {
                    const int r = e / D, d = e - r * D;
                    const int qq = q0 + r;
                    qs[e] = qq < a.S ? qp[(int64_t)qq * a.q.stride_s + d] : 0.f;
                    gs[e] = qq < a.S ? gp[(int64_t)qq * a.dout.stride_s + d] : 0.f;
                }
                if (t < QC) {
                    const int qq = q0 + t;
                    ls[t] = qq < a.S ? a.lse[rowbase + qq] : 0.f;
                    dl[t] = qq < a.S ? a.delta[rowbase + qq] : 0.f;
                    if (drow) qdoc[t] = qq < a.S ? drow[qq] : 0;
                }
                __syncthreads();
#pragma unroll 2
                for (int c = 0; c < QC; ++c) {
                    const int qq = q0 + c;
                    bool ok = kvalid && qq < a.S;
                    if (partial) {
                        ok = ok && pair_allowed(qq, kv, a.causal, a.window);
                        if (drow) ok = ok && (qdoc[c] == dk_id);
                    }
                    float s = 0.f, dp = 0.f;
#pragma unroll
                    for (int d = 0; d < D; ++d) {
                        s += qs[c * D + d] * ks[t * LDK + d];
                        dp += gs[c * D + d] * vs[t * LDK + d];
                    }
                    const float p = ok ? __expf(s * a.scale - ls[c]) : 0.f;
                    const float ds = p * (dp - dl[c]);
#pragma unroll
                    for (int d = 0; d < D; ++d) {
                        dv[d] += p * gs[c * D + d];
                        dk[d] += ds * qs[c * D + d];
                    }
                }
            }
        }
    }
    if (kvalid) {
        float* okp = (float*)a.dk.ptr + b * a.dk.stride_b + (int64_t)kv * a.dk.stride_s + hk * a.dk.stride_h;
        float* ovp = (float*)a.dv.ptr + b * a.dv.stride_b + (int64_t)kv * a.dv.stride_s + hk * a.dv.stride_h;
#pragma unroll
        for (int d = 0; d < D; ++d) {
            okp[d] = dk[d] * a.scale;
            ovp[d] = dv[d];
        }
    }
}

template <typename K>
static int set_lds(K kernel, size_t bytes) {
    if (bytes <= 64 * 1024) return MA_OK;
    hipError_t e = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
    if (e != hipSuccess) return fail(MA_ERR_LAUNCH, "hipFuncSetAttribute(%zu bytes of LDS): %s", bytes, hipGetErrorString(e));
    return MA_OK;
}

template <int D>
static int fwd_d(const AttnArgs& a, hipStream_t st) {
    using C = F32Cfg<D>;
    const size_t lds = (size_t)(kRows * C::LDQ + 2 * C::KC * D) * 4 + C::KC * 8;
    int rc = set_lds(attn_fwd_f32_kernel<D>, lds);
    if (rc) return rc;
    hipLaunchKernelGGL(attn_fwd_f32_kernel<D>, dim3(2 * a.T, a.Hq, a.B), dim3(kRows), lds, st, a);
    return check_launch("attn_fwd_f32_kernel");
}

int launch_attn_fwd_f32(const AttnArgs& a, hipStream_t st) {
    switch (a.D) {
        case 64: return fwd_d<64>(a, st);
        case 128: return fwd_d<128>(a, st);
        case 256: return fwd_d<256>(a, st);
    }
    return fail(MA_ERR_UNSUPPORTED, "attn_fwd fp32: head_dim %d not in {64,128,256}", a.D);
}

template <int D>
static int bwd_d(const AttnArgs& a, hipStream_t st) {
    using C = F32Cfg<D>;
    const int64_t nrows = (int64_t)a.B * a.Hq * a.S;
    int rc = MA_OK;
    if (a.stages & MA_BWD_DELTA) {
        hipLaunchKernelGGL(attn_delta_f32_kernel, dim3((unsigned)((nrows + 255) / 256)), dim3(256), 0, st, a);
        rc = check_launch("attn_delta_f32_kernel");
        if (rc) return rc;
    }
    const size_t lds_q = (size_t)(2 * kRows * C::LDQ + 2 * C::KC * D) * 4 + C::KC * 8;
    rc = set_lds(attn_bwd_dq_f32_kernel<D>, lds_q);
    if (rc) return rc;
    if (a.stages & MA_BWD_DQ) {
        hipLaunchKernelGGL(attn_bwd_dq_f32_kernel<D>, dim3(2 * a.T, a.Hq, a.B), dim3(kRows), lds_q, st, a);
        rc = check_launch("attn_bwd_dq_f32_kernel");
        if (rc) return rc;
    }
    if (!(a.stages & MA_BWD_DKV)) return MA_OK;
    const size_t lds_k = (size_t)(2 * kRows * (D + 1) + 2 * 16 * D + 32) * 4 + 16 * 8;
    rc = set_lds(attn_bwd_dkv_f32_kernel<D>, lds_k);
    if (rc) return rc;
    hipLaunchKernelGGL(attn_bwd_dkv_f32_kernel<D>, dim3(2 * a.T, a.Hkv, a.B), dim3(kRows), lds_k, st, a);
    return check_launch("attn_bwd_dkv_f32_kernel");
}

int launch_attn_bwd_f32(const AttnArgs& a, hipStream_t st) {
    switch (a.D) {
        case 64: return bwd_d<64>(a, st);
        case 128: return bwd_d<128>(a, st);
    }
    return fail(MA_ERR_UNSUPPORTED, "attn_bwd fp32: head_dim %d not in {64,128}", a.D);
}

}  // namespace ma
