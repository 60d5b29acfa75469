// GQA flash-style backward for bf16 activations on gfx950 matrix cores.
//
// Stands in for the FlexAttention backward autograd runs for GemmaAttention
// (torch/_higher_order_ops/flex_attention.py:825-993):
//   delta = rowsum(O * dO);  P = exp(S - lse);  dV = P^T dO;  dS = P * (dO V^T - delta);
//   dQ = scale * dS K;  dK = scale * dS^T Q;  dK/dV summed over the query heads of a kv head.
// Three kernels, no atomics anywhere (results are run-to-run identical):
//   1. delta                      -- one pass over O and dO;
//   2. dK/dV: one workgroup owns a 128-row kv tile of one (batch row, kv head), wave w its rows
//      32w..32w+31 (K, V fragments and the fp32 dK^T/dV^T accumulators in registers); it walks
//      the q-side lists of the tile map for each of the G query heads, 64 q rows per step
//      through LDS, recomputing S and dP;
//   3. dQ: the forward's decomposition (128-row q tile per workgroup, 32 rows per wave, K/V
//      64 rows per step through LDS), recomputing S^T and dP^T.
// All products are arranged so that P and dS stay in registers between the two MFMAs that
// produce and consume them (see mfma.h).
#include "common.h"
#include "mfma.h"

namespace ma {

constexpr int kBwdThreads = 256;
constexpr int kStep = 64;  // rows staged per step

// ------------------------------------------------------------------------------------------------
// delta[b,h,q] = sum_d O[b,q,h,d] * dO[b,q,h,d]
// ------------------------------------------------------------------------------------------------
template <int D>
__global__ __launch_bounds__(256) void attn_delta_bf16_kernel(AttnArgs a) {
    constexpr int LPR = D / 8;  // lanes per row
    constexpr int RPB = 256 / LPR;
    const int64_t row = (int64_t)blockIdx.x * RPB + threadIdx.x / LPR;
    const int sub = threadIdx.x % LPR;
    const int64_t nrows = (int64_t)a.B * a.Hq * a.S;
    float acc = 0.f;
    if (row < nrows) {
        const int q = row % a.S;
        const int h = (row / a.S) % a.Hq;
        const int b = row / ((int64_t)a.S * a.Hq);
        const __bf16* op = (const __bf16*)a.o.ptr + b * a.o.stride_b + (int64_t)q * a.o.stride_s + h * a.o.stride_h;
        const __bf16* gp = (const __bf16*)a.dout.ptr + b * a.dout.stride_b + (int64_t)q * a.dout.stride_s + h * a.dout.stride_h;
        const bf16x8 x = *(const bf16x8*)(op + sub * 8), y = *(const bf16x8*)(gp + sub * 8);
#pragma unroll
        for (int e = 0; e < 8; ++e) acc += (float)x[e] * (float)y[e];
    }
#pragma unroll
    for (int off = LPR / 2; off > 0; off >>= 1) acc += __shfl_xor(acc, off, 64);
    if (row < nrows && sub == 0) a.delta[row] = acc;
}

// ------------------------------------------------------------------------------------------------
// dK / dV
// ------------------------------------------------------------------------------------------------
template <int D>
__global__ __launch_bounds__(kBwdThreads) void attn_bwd_dkv_bf16_kernel(AttnArgs a) {
    using TL = Tile<D>;
    constexpr int KK = D / 16;
    constexpr int DB = D / 32;
    constexpr int BM = kStep;
    extern __shared__ __align__(16) char smem_raw[];
    lds_ptr Qs = (lds_ptr)smem_raw;
    lds_ptr Gs = Qs + TL::bytes(BM);  // dO rows
    MA_LDS float* lse2s = (MA_LDS float*)(Gs + TL::bytes(BM));
    MA_LDS float* dls = lse2s + BM;
    MA_LDS int64_t* qdoc = (MA_LDS int64_t*)(dls + BM);

    const int tid = threadIdx.x, lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 31, hh = lane >> 5;
    const int j = blockIdx.y, hk = blockIdx.x % a.Hkv, b = blockIdx.x / a.Hkv;
    const int rbase = TL::row_base(lane), tbase = TL::tr_base(lane);
    const int G = a.Hq / a.Hkv;
    const int kw_lo = j * kTile + 32 * w, kw_hi = kw_lo + 31;
    const int kv = kw_lo + r;
    const bool kvalid = kv < a.S;
    const bool bounded = a.causal || a.window >= 0;
    const float sl2 = a.scale * kLog2e;

    const __bf16* kp = (const __bf16*)a.k.ptr + b * a.k.stride_b + hk * a.k.stride_h;
    const __bf16* vp = (const __bf16*)a.v.ptr + b * a.v.stride_b + hk * a.v.stride_h;
    const int64_t* drow = a.doc ? a.doc + (size_t)b * a.S : nullptr;

    // rows past the end of the sequence read the last valid row; their results are masked / not stored
    const int kvc = min(kv, a.S - 1);
    bf16x8 kf[KK], vf[KK];
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
        kf[kk] = *(const bf16x8*)(kp + (int64_t)kvc * a.k.stride_s + 16 * kk + 8 * hh);
        vf[kk] = *(const bf16x8*)(vp + (int64_t)kvc * a.v.stride_s + 16 * kk + 8 * hh);
    }
    const int64_t dock = drow ? drow[kvc] : 0;
    const int wlim = a.window >= 0 ? (int)min(a.window, (int64_t)0x3fffffff) : 0x7fffffff;

    f32x16 dkacc[DB], dvacc[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int v = 0; v < 16; ++v) dkacc[db][v] = dvacc[db][v] = 0.f;

    const size_t mrow = (size_t)b * a.T + j;
    const int32_t* plist = a.map.q_indices + mrow * a.T;
    const int32_t* flist = a.map.full_q_indices + mrow * a.T;
    const int np = a.map.q_num_blocks[mrow];
    const int nf = a.map.full_q_num_blocks[mrow];

    for (int g = 0; g < G; ++g) {
        const int h = hk * G + g;
        const __bf16* qp = (const __bf16*)a.q.ptr + b * a.q.stride_b + h * a.q.stride_h;
        const __bf16* gp = (const __bf16*)a.dout.ptr + b * a.dout.stride_b + h * a.dout.stride_h;
        const size_t rowbase = ((size_t)b * a.Hq + h) * a.S;
        for (int it = 0; it < np + nf; ++it) {
            const bool partial = it < np;
            const int i = partial ? plist[it] : flist[it - np];
            for (int half = 0; half < kTile / BM; ++half) {
                const int q0 = i * kTile + half * BM;
                if (q0 >= a.S) continue;
                if (partial && bounded && q0 + BM - 1 < j * kTile) continue;
                if (partial && a.window >= 0 && (int64_t)q0 - (j * kTile + kTile - 1) > a.window) continue;

                __syncthreads();
                const int rows_valid = min(BM, a.S - q0);
                {
                    Stager<D, BM, kBwdThreads> sq, sg;
                    sq.load(qp + (int64_t)q0 * a.q.stride_s, a.q.stride_s, rows_valid, tid);
                    sg.load(gp + (int64_t)q0 * a.dout.stride_s, a.dout.stride_s, rows_valid, tid);
                    sq.store(Qs, rows_valid, tid);
                    sg.store(Gs, rows_valid, tid);
                }
                if (tid < BM) {
                    const bool ok = q0 + tid < a.S;
                    lse2s[tid] = ok ? a.lse[rowbase + q0 + tid] * kLog2e : 0.f;
                    dls[tid] = ok ? a.delta[rowbase + q0 + tid] : 0.f;
                    if (partial && drow) qdoc[tid] = ok ? drow[q0 + tid] : 0;
                }
                __syncthreads();

#pragma unroll 1
                for (int mb = 0; mb < BM / 32; ++mb) {
                    const int qb0 = q0 + 32 * mb;
                    if (qb0 >= a.S) continue;
                    if (partial && bounded && qb0 + 31 < kw_lo) continue;
                    if (partial && a.window >= 0 && (int64_t)qb0 - kw_hi > a.window) continue;

                    f32x16 s, dp;
#pragma unroll
                    for (int v = 0; v < 16; ++v) s[v] = dp[v] = 0.f;
#pragma unroll
                    for (int kk = 0; kk < KK; ++kk) s = mfma32(TL::row_frag(Qs, rbase, 32 * mb, kk), kf[kk], s);
#pragma unroll
                    for (int kk = 0; kk < KK; ++kk) dp = mfma32(TL::row_frag(Gs, rbase, 32 * mb, kk), vf[kk], dp);

                    bf16x8 pf[2], dsf[2];
                    // d = q - kv for element v is drel + 8*(v/4) + v%4; all tests are branch-free
                    const int drel = q0 + 32 * mb + 4 * hh - kv;
                    const int dmin = bounded ? 0 : -0x40000000;
                    const int dend = a.S - kv;                    // q < S  <=>  d < S - kv
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        const int qc = 8 * (v >> 2) + (v & 3);
                        const int ql = 32 * mb + qc + 4 * hh;
                        float p = fast_exp2(s[v] * sl2 - lse2s[ql]);
                        if (partial) {
                            const int d = drel + qc;
                            bool ok = (d >= dmin) & (d <= wlim) & (d < dend) & kvalid;
                            if (drow) ok = ok & (qdoc[ql] == dock);
                            p = ok ? p : 0.f;
                        }
                        const float ds = p * (dp[v] - dls[ql]);
                        pf[v >> 3][v & 7] = (__bf16)p;
                        dsf[v >> 3][v & 7] = (__bf16)ds;
                    }
#pragma unroll
                    for (int t = 0; t < 2; ++t) {
#pragma unroll
                        for (int db = 0; db < DB; ++db) {
                            dvacc[db] = mfma32(TL::tr_frag(Gs, tbase, 32 * mb + 16 * t, 32 * db), pf[t], dvacc[db]);
                            dkacc[db] = mfma32(TL::tr_frag(Qs, tbase, 32 * mb + 16 * t, 32 * db), dsf[t], dkacc[db]);
                        }
                    }
                }
            }
        }
    }

    if (kvalid) {
        __bf16* okp = (__bf16*)a.dk.ptr + b * a.dk.stride_b + (int64_t)kv * a.dk.stride_s + hk * a.dk.stride_h;
        __bf16* ovp = (__bf16*)a.dv.ptr + b * a.dv.stride_b + (int64_t)kv * a.dv.stride_s + hk * a.dv.stride_h;
#pragma unroll
        for (int db = 0; db < DB; ++db) {
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4) {
                bf16x4 pk, pv;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    pk[e] = (__bf16)(dkacc[db][4 * g4 + e] * a.scale);
                    pv[e] = (__bf16)dvacc[db][4 * g4 + e];
                }
                *(bf16x4*)(okp + 32 * db + 8 * g4 + 4 * hh) = pk;
                *(bf16x4*)(ovp + 32 * db + 8 * g4 + 4 * hh) = pv;
            }
        }
    }
}

// ------------------------------------------------------------------------------------------------
// dQ
// ------------------------------------------------------------------------------------------------
template <int D>
__global__ __launch_bounds__(kBwdThreads) void attn_bwd_dq_bf16_kernel(AttnArgs a) {
    using TL = Tile<D>;
    constexpr int KK = D / 16;
    constexpr int DB = D / 32;
    constexpr int BN = kStep;
    extern __shared__ __align__(16) char smem_raw[];
    lds_ptr Ks = (lds_ptr)smem_raw;
    lds_ptr Vs = Ks + TL::bytes(BN);
    MA_LDS int64_t* kdoc = (MA_LDS int64_t*)(Vs + TL::bytes(BN));

    const int tid = threadIdx.x, lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 31, hh = lane >> 5;
    const int i = gridDim.y - 1 - blockIdx.y;
    const int h = blockIdx.x % a.Hq, b = blockIdx.x / a.Hq;
    const int rbase = TL::row_base(lane), tbase = TL::tr_base(lane);
    const int hk = h / (a.Hq / a.Hkv);
    const int qw_lo = i * kTile + 32 * w, qw_hi = qw_lo + 31;
    const int q = qw_lo + r;
    const bool qvalid = q < a.S;
    const bool bounded = a.causal || a.window >= 0;
    const float sl2 = a.scale * kLog2e;

    const __bf16* qp = (const __bf16*)a.q.ptr + b * a.q.stride_b + h * a.q.stride_h;
    const __bf16* gp = (const __bf16*)a.dout.ptr + b * a.dout.stride_b + h * a.dout.stride_h;
    const __bf16* kp = (const __bf16*)a.k.ptr + b * a.k.stride_b + hk * a.k.stride_h;
    const __bf16* vp = (const __bf16*)a.v.ptr + b * a.v.stride_b + hk * a.v.stride_h;
    const int64_t* drow = a.doc ? a.doc + (size_t)b * a.S : nullptr;

    const int qc = min(q, a.S - 1);  // rows past the end read the last valid row; never stored
    bf16x8 qf[KK], gf[KK];
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
        qf[kk] = *(const bf16x8*)(qp + (int64_t)qc * a.q.stride_s + 16 * kk + 8 * hh);
        gf[kk] = *(const bf16x8*)(gp + (int64_t)qc * a.dout.stride_s + 16 * kk + 8 * hh);
    }
    const int64_t docq = drow ? drow[qc] : 0;
    const int wlim = a.window >= 0 ? (int)min(a.window, (int64_t)0x3fffffff) : 0x7fffffff;
    const size_t rowi = ((size_t)b * a.Hq + h) * a.S + qc;
    const float lse2 = a.lse[rowi] * kLog2e;
    const float delta = a.delta[rowi];

    f32x16 acc[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[db][v] = 0.f;

    const size_t mrow = (size_t)b * a.T + i;
    const int32_t* plist = a.map.kv_indices + mrow * a.T;
    const int32_t* flist = a.map.full_kv_indices + mrow * a.T;
    const int np = a.map.kv_num_blocks[mrow];
    const int nf = a.map.full_kv_num_blocks[mrow];

    for (int it = 0; it < np + nf; ++it) {
        const bool partial = it < np;
        const int j = partial ? plist[it] : flist[it - np];
        for (int half = 0; half < kTile / BN; ++half) {
            const int k0 = j * kTile + half * BN;
            if (k0 >= a.S) continue;
            if (partial && bounded && k0 > i * kTile + kTile - 1) continue;
            if (partial && a.window >= 0 && (int64_t)(i * kTile) - (k0 + BN - 1) > a.window) continue;

            __syncthreads();
            const int rows_valid = min(BN, a.S - k0);
            {
                Stager<D, BN, kBwdThreads> sk, sv;
                sk.load(kp + (int64_t)k0 * a.k.stride_s, a.k.stride_s, rows_valid, tid);
                sv.load(vp + (int64_t)k0 * a.v.stride_s, a.v.stride_s, rows_valid, tid);
                sk.store(Ks, rows_valid, tid);
                sv.store(Vs, rows_valid, tid);
            }
            if (partial && drow && tid < BN) kdoc[tid] = (k0 + tid < a.S) ? drow[k0 + tid] : 0;
            __syncthreads();

#pragma unroll 1
            for (int nb = 0; nb < BN / 32; ++nb) {
                const int kb0 = k0 + 32 * nb;
                if (kb0 >= a.S) continue;
                if (partial && bounded && kb0 > qw_hi) continue;
                if (partial && a.window >= 0 && (int64_t)qw_lo - (kb0 + 31) > a.window) continue;

                f32x16 s, dp;
#pragma unroll
                for (int v = 0; v < 16; ++v) s[v] = dp[v] = 0.f;
#pragma unroll
                for (int kk = 0; kk < KK; ++kk) s = mfma32(TL::row_frag(Ks, rbase, 32 * nb, kk), qf[kk], s);
#pragma unroll
                for (int kk = 0; kk < KK; ++kk) dp = mfma32(TL::row_frag(Vs, rbase, 32 * nb, kk), gf[kk], dp);

                bf16x8 dsf[2];
                const int qrel = q - k0 - 32 * nb - 4 * hh;   // d = q - kv = qrel - (8*(v/4) + v%4)
                const int dmin = bounded ? 0 : -0x40000000;
                const int dend = q - a.S;                       // kv < S  <=>  d > q - S
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    float p = fast_exp2(s[v] * sl2 - lse2);
                    if (partial) {
                        const int kc = 8 * (v >> 2) + (v & 3);
                        const int d = qrel - kc;
                        bool ok = (d >= dmin) & (d <= wlim) & (d > dend) & qvalid;
                        if (drow) ok = ok & (kdoc[32 * nb + kc + 4 * hh] == docq);
                        p = ok ? p : 0.f;
                    }
                    dsf[v >> 3][v & 7] = (__bf16)(p * (dp[v] - delta));
                }
#pragma unroll
                for (int t = 0; t < 2; ++t) {
#pragma unroll
                    for (int db = 0; db < DB; ++db)
                        acc[db] = mfma32(TL::tr_frag(Ks, tbase, 32 * nb + 16 * t, 32 * db), dsf[t], acc[db]);
                }
            }
        }
    }

    if (qvalid) {
        __bf16* op = (__bf16*)a.dq.ptr + b * a.dq.stride_b + (int64_t)q * a.dq.stride_s + h * a.dq.stride_h;
#pragma unroll
        for (int db = 0; db < DB; ++db) {
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4) {
                bf16x4 pk;
#pragma unroll
                for (int e = 0; e < 4; ++e) pk[e] = (__bf16)(acc[db][4 * g4 + e] * a.scale);
                *(bf16x4*)(op + 32 * db + 8 * g4 + 4 * hh) = pk;
            }
        }
    }
}

template <typename K>
static int opt_in_lds(K kernel, size_t bytes, const char* name) {
    if (bytes <= 64 * 1024) return MA_OK;
    hipError_t e = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
    if (e != hipSuccess) return fail(MA_ERR_LAUNCH, "hipFuncSetAttribute(%s, %zu): %s", name, bytes, hipGetErrorString(e));
    return MA_OK;
}

template <int D>
static int bwd_d(const AttnArgs& a, hipStream_t st) {
    constexpr int RPB = 256 / (D / 8);
    const int64_t nrows = (int64_t)a.B * a.Hq * a.S;
    int rc = MA_OK;
    if (a.stages & MA_BWD_DELTA) {
        hipLaunchKernelGGL(attn_delta_bf16_kernel<D>, dim3((unsigned)((nrows + RPB - 1) / RPB)), dim3(256), 0, st, a);
        rc = check_launch("attn_delta_bf16_kernel");
        if (rc) return rc;
    }

    const size_t lds_kv = (size_t)2 * Tile<D>::bytes(kStep) + kStep * (4 + 4 + 8);
    rc = opt_in_lds(attn_bwd_dkv_bf16_kernel<D>, lds_kv, "attn_bwd_dkv_bf16");
    if (rc) return rc;
    if (a.stages & MA_BWD_DKV) {
        hipLaunchKernelGGL(attn_bwd_dkv_bf16_kernel<D>, dim3(a.B * a.Hkv, a.T, 1), dim3(kBwdThreads), lds_kv, st, a);
        rc = check_launch("attn_bwd_dkv_bf16_kernel");
        if (rc) return rc;
    }
    if (!(a.stages & MA_BWD_DQ)) return MA_OK;

    const size_t lds_q = (size_t)2 * Tile<D>::bytes(kStep) + kStep * 8;
    rc = opt_in_lds(attn_bwd_dq_bf16_kernel<D>, lds_q, "attn_bwd_dq_bf16");
    if (rc) return rc;
    hipLaunchKernelGGL(attn_bwd_dq_bf16_kernel<D>, dim3(a.B * a.Hq, a.T, 1), dim3(kBwdThreads), lds_q, st, a);
    return check_launch("attn_bwd_dq_bf16_kernel");
}

int launch_attn_bwd_bf16(const AttnArgs& a, hipStream_t st) {
    switch (a.D) {
        case 64: return bwd_d<64>(a, st);
        case 128: return bwd_d<128>(a, st);
        case 256: return bwd_d<256>(a, st);
    }
    return fail(MA_ERR_UNSUPPORTED, "attn_bwd bf16: head_dim %d not in {64,128,256}", a.D);
}

}  // namespace ma
