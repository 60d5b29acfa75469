// GQA flash-style forward for bf16 activations on gfx950 matrix cores.
//
// Stands in for the FlexAttention forward GemmaAttention.forward calls
// (maester/models/gemma/model.py:384-396; semantics torch/_higher_order_ops/flex_attention.py:159-267).
//
// One workgroup (4 waves) owns a 128-row q tile of one (batch row, q head); wave w owns rows
// 32w..32w+31 and keeps their Q fragments, the fp32 O^T accumulator and the online-softmax state in
// registers.  K/V are walked 64 rows at a time through swizzled LDS tiles, following the kv lists
// of the tile map (partial tiles first, then full tiles -- fully masked tiles are never touched).
// Per step:  S^T = K Q^T (MFMA 32x32x16, K row fragments x Q registers), fp32 online softmax in
// the exp2 domain with the lane owning one q row (row max/sum = in-lane reduction + one 32-lane
// exchange), P^T cast to bf16 in place, O^T += V^T P^T (MFMA, V through transposed LDS reads).
// Inside partial tiles the 32-row kv blocks a wave cannot see under the causal/window bound are
// skipped, the rest is masked element-wise with the document/causal/window predicate.
#include "common.h"
#include "mfma.h"

namespace ma {

constexpr int kFwdThreads = 256;
constexpr int kFwdBN = 64;  // kv rows per step

template <int D>
__global__ __launch_bounds__(kFwdThreads) void attn_fwd_bf16_kernel(AttnArgs a) {
    constexpr int KK = D / 16;  // contraction steps of S^T
    constexpr int DB = D / 32;  // 32-row blocks of O^T
    constexpr int BN = kFwdBN;
    extern __shared__ __align__(16) char smem_raw[];
    lds_ptr Ks = (lds_ptr)smem_raw;
    lds_ptr Vs = Ks + BN * D * 2;
    MA_LDS int64_t* kdoc = (MA_LDS int64_t*)(Vs + BN * D * 2);

    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
    const int r = lane & 31, hh = lane >> 5;
    const int i = gridDim.x - 1 - blockIdx.x;  // late q tiles see the most keys: start them first
    const int h = blockIdx.y, b = blockIdx.z;
    const int hk = h / (a.Hq / a.Hkv);
    const int qw_lo = i * kTile + 32 * w, qw_hi = qw_lo + 31;
    const int q = qw_lo + r;
    const bool qvalid = q < a.S;
    const bool bounded = a.causal || a.window >= 0;  // kv <= q is part of the predicate

    const __bf16* qp = (const __bf16*)a.q.ptr + b * a.q.stride_b + h * a.q.stride_h;
    const __bf16* kp = (const __bf16*)a.k.ptr + b * a.k.stride_b + hk * a.k.stride_h;
    const __bf16* vp = (const __bf16*)a.v.ptr + b * a.v.stride_b + hk * a.v.stride_h;
    const int64_t* drow = a.doc ? a.doc + (size_t)b * a.S : nullptr;

    bf16x8 qf[KK];
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
        bf16x8 val = {0, 0, 0, 0, 0, 0, 0, 0};
        if (qvalid) val = *(const bf16x8*)(qp + (int64_t)q * a.q.stride_s + 16 * kk + 8 * hh);
        qf[kk] = val;
    }
    const int64_t docq = (drow && qvalid) ? drow[q] : 0;

    f32x16 o[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int v = 0; v < 16; ++v) o[db][v] = 0.f;
    float m = -INFINITY, lsum = 0.f;
    const float sl2 = a.scale * kLog2e;

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
            // steps no row of the workgroup can see (uniform over the workgroup)
            if (k0 >= a.S) continue;
            if (partial && bounded && k0 > i * kTile + kTile - 1) continue;
            if (partial && a.window >= 0 && (int64_t)(i * kTile) - (k0 + BN - 1) > a.window) continue;

            __syncthreads();
            const int rows_valid = min(BN, a.S - k0);
            stage_tile<D, BN, kFwdThreads>(Ks, kp + (int64_t)k0 * a.k.stride_s, a.k.stride_s, rows_valid, tid);
            stage_tile<D, BN, kFwdThreads>(Vs, vp + (int64_t)k0 * a.v.stride_s, a.v.stride_s, rows_valid, tid);
            if (partial && drow && tid < BN) kdoc[tid] = (k0 + tid < a.S) ? drow[k0 + tid] : 0;
            __syncthreads();

            bool act[2];
#pragma unroll
            for (int nb = 0; nb < 2; ++nb) {
                const int kb0 = k0 + 32 * nb;
                bool on = kb0 < a.S;
                if (partial && bounded && kb0 > qw_hi) on = false;
                if (partial && a.window >= 0 && (int64_t)qw_lo - (kb0 + 31) > a.window) on = false;
                act[nb] = on;
            }
            if (!act[0] && !act[1]) continue;

            // S^T blocks (kv x q), already in log2 units after the scale
            f32x16 s[2];
#pragma unroll
            for (int nb = 0; nb < 2; ++nb) {
#pragma unroll
                for (int v = 0; v < 16; ++v) s[nb][v] = 0.f;
                if (act[nb]) {
#pragma unroll
                    for (int kk = 0; kk < KK; ++kk)
                        s[nb] = mfma32(row_frag<D>(Ks, 32 * nb + r, 2 * kk + hh), qf[kk], s[nb]);
                }
            }
            float mx = -INFINITY;
#pragma unroll
            for (int nb = 0; nb < 2; ++nb) {
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    float x = s[nb][v] * sl2;
                    bool ok = act[nb];
                    if (partial) {
                        const int kl = 32 * nb + 8 * (v >> 2) + 4 * hh + (v & 3);
                        const int kv = k0 + kl;
                        ok = ok && kv < a.S && pair_allowed(q, kv, a.causal, a.window);
                        if (drow) ok = ok && (kdoc[kl] == docq);
                    }
                    x = ok ? x : -INFINITY;
                    s[nb][v] = x;
                    mx = fmaxf(mx, x);
                }
            }
            mx = fmaxf(mx, xor32(mx));
            const float mn = fmaxf(m, mx);
            const float mu = mn == -INFINITY ? 0.f : mn;
            const float alpha = fast_exp2(m - mu);
            float rs = 0.f;
            bf16x8 pf[2][2];
#pragma unroll
            for (int nb = 0; nb < 2; ++nb) {
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const float p = fast_exp2(s[nb][v] - mu);
                    rs += p;
                    pf[nb][v >> 3][v & 7] = (__bf16)p;
                }
            }
            rs += xor32(rs);
            lsum = lsum * alpha + rs;
            m = mn;
#pragma unroll
            for (int db = 0; db < DB; ++db)
#pragma unroll
                for (int v = 0; v < 16; ++v) o[db][v] *= alpha;

            // O^T += V^T P^T
#pragma unroll
            for (int nb = 0; nb < 2; ++nb) {
                if (!act[nb]) continue;
#pragma unroll
                for (int t = 0; t < 2; ++t) {
#pragma unroll
                    for (int db = 0; db < DB; ++db)
                        o[db] = mfma32(tr_frag<D>(Vs, 32 * nb + 16 * t, 32 * db, lane), pf[nb][t], o[db]);
                }
            }
        }
    }

    if (qvalid) {
        const float inv = lsum > 0.f ? 1.0f / lsum : 0.f;
        __bf16* op = (__bf16*)a.o.ptr + b * a.o.stride_b + (int64_t)q * a.o.stride_s + h * a.o.stride_h;
#pragma unroll
        for (int db = 0; db < DB; ++db) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                bf16x4 pk;
#pragma unroll
                for (int e = 0; e < 4; ++e) pk[e] = (__bf16)(o[db][4 * g + e] * inv);
                *(bf16x4*)(op + 32 * db + 8 * g + 4 * hh) = pk;
            }
        }
        if (hh == 0)
            a.lse[((size_t)b * a.Hq + h) * a.S + q] = lsum > 0.f ? (m + __log2f(lsum)) * kLn2 : -INFINITY;
    }
}

template <int D>
static int fwd_d(const AttnArgs& a, hipStream_t st) {
    const size_t lds = (size_t)2 * kFwdBN * D * 2 + kFwdBN * 8;
    if (lds > 64 * 1024) {
        hipError_t e = hipFuncSetAttribute((const void*)attn_fwd_bf16_kernel<D>,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return fail(MA_ERR_LAUNCH, "hipFuncSetAttribute(attn_fwd_bf16, %zu): %s", lds, hipGetErrorString(e));
    }
    hipLaunchKernelGGL(attn_fwd_bf16_kernel<D>, dim3(a.T, a.Hq, a.B), dim3(kFwdThreads), lds, st, a);
    return check_launch("attn_fwd_bf16_kernel");
}

int launch_attn_fwd_bf16(const AttnArgs& a, hipStream_t st) {
    switch (a.D) {
        case 64: return fwd_d<64>(a, st);
        case 128: return fwd_d<128>(a, st);
        case 256: return fwd_d<256>(a, st);
    }
    return fail(MA_ERR_UNSUPPORTED, "attn_fwd bf16: head_dim %d not in {64,128,256}", a.D);
}

}  // namespace ma
